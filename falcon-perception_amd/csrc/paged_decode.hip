// Split-K paged decode attention (one query token per sequence) and its merge.
//
// Replaces the reference's compiled_flex_attn_decode call (attention.py:17,
// model.py:156-162) on the pool views that PagedKVCache.assign returns
// (paged_attention.py:232), and the block-mask conversion that call depends on
// (paged_attention.py:234-333, paged_inference.py:783-826): the kernel reads
// page_table[batch_idx[b], t / P] itself and bounds the context by input_pos[b].
//
// HBM-bound: every cached K and V row of every sequence is read exactly once.
//   grid  = (cache heads, batch, splits); a workgroup of 4 wavefronts owns one
//           (sequence, cache head, token range) and serves all G = Hq / Hc query
//           heads of that cache head from a single read of K and V.  A launch
//           larger than the GPU holds at once runs as (cache heads, chunks)
//           instead: the contexts laid end to end and cut into equal chunks, a
//           workgroup working through the sequences its chunk touches.
//   loads = a row (D elements) is covered by TPR = D * elem / 16 lanes holding
//           16 bytes each, so a wavefront load instruction moves 64 / TPR whole
//           rows, contiguous inside a page; U such loads of K and of V are in
//           flight per lane before the arithmetic starts.
//   math  = each lane group keeps its own online-softmax state (m, l, acc) in
//           log2 space; q.k partial sums are combined across the TPR lanes with
//           DPP adds; lane groups, then wavefronts (through LDS), then splits
//           (through the workspace, by the merge kernel) are combined at the end.
#include "fp_common.h"

#include <atomic>

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <math.h>

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kMaxSplitPages = 1024;  // page ids of one split held in LDS
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct DecodeArgs {
  const char* q;
  int64_t qs_b, qs_h;  // bytes
  const char* pool_k;
  const char* pool_v;
  const int64_t* page_table;
  int64_t pt_row_stride;
  const int64_t* batch_idx;
  const void* input_pos;
  int pos_i64;
  char* out;
  int64_t os_b, os_h;  // bytes
  float* lse;
  const float* sinks;  // optional [Hq]: out is multiplied by sigmoid(lse - sinks[h])
  float* ws_acc;  // [B, Hq, n_splits, D]
  float* ws_ml;   // [B, Hq, n_splits, 2]
  int Hq, Hc;
  fp::PageDiv pd;
  int n_pages, max_batch;
  int64_t n_slots;
  int max_context;
  int split_tokens;
  int n_splits;
  float qscale;  // scale * log2(e)
  // fused append (optional): the row of the newest token of every sequence, [B, Hc, 1, D]
  const char* k_new;
  const char* v_new;
  int64_t kn_b, kn_h, vn_b, vn_h;  // bytes
  int B;         // sequences of the launch
  int n_chunks;  // even cut (kFlat): workgroups per cache head
  int* plan;     // optional: the step's plan of the even cut (fp_paged_decode_plan), kPlanInts ints per chunk
};

// The plan of a decode step: what every workgroup of the even cut needs before it can ask for its first K row,
// computed once per step instead of once per layer and workgroup.  Per chunk (workgroup of a cache head):
//   rec[0]            pieces of the chunk, or -1: no plan for this chunk (more pieces or pages than a record
//                     holds), the workgroup works everything out itself
//   rec[1 .. 3]       B, n_chunks, max_context of the launch the plan was made for: a workgroup that finds other
//                     values ignores the plan
//   rec[4 + 6 k ..]   piece k: sequence, first token, tokens, raw length (position + 1), row of the page table
//                     (-1: not a valid slot), offset of its page ids in the chunk's list
//   pages[..]         page ids of the pieces, piece after piece (unmapped or foreign pages as 0, like the kernel
//                     stages them)
//   chunk 0, rec[126]  a hash of the positions and slots the plan was made from (plan_hash_term)
// The positions, the slots and the page table must not change between the plan and the launches that use it.
// What the launches do if they did: the merge pass recomputes the hash from the step's positions and slots
// (it reads them anyway) and stores NaN in every row of out and lse when it differs, so a stale plan fails
// loudly.  The split-K pass itself does not look (a check of its own position before the fused append's store
// measured 1.2 us per launch): with a stale plan the fresh rows of the sequences that moved land where the plan
// says.
constexpr int kPlanPieces = 20;
constexpr int kPlanHashAt = 126;
constexpr int kPlanRec = 128;            // 4 + 6 * kPlanPieces, rounded up
constexpr int kPlanPages = kMaxSplitPages;
constexpr int kPlanInts = kPlanRec + kPlanPages;
static_assert(4 + 6 * kPlanPieces <= kPlanHashAt && kPlanHashAt < kPlanRec, "a record holds its pieces and the hash");

// Contribution of sequence b to the hash of a step's positions and slots (summed over the sequences, mod 2^32).
__device__ __forceinline__ uint32_t plan_hash_term(int b, int64_t L, int64_t trow) {
  const uint32_t w = 2u * static_cast<uint32_t>(b) + 1u;
  return (static_cast<uint32_t>(L) + static_cast<uint32_t>(trow) * 0x9E3779B1u) * w;
}

// ---- element access: 16 bytes of a row -----------------------------------
// A lane holds 16 bytes of a K or V row as four 32-bit words.  `Q` is the lane's
// share of a query row, `dot` its contribution to q.k, `unpack` the V values as floats.
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

struct F32 {
  using type = float;
  static constexpr int kEpl = 4;
  struct Q { float f[4]; };
  static __device__ __forceinline__ Q load_q(const v4u& r) {
    return Q{{__uint_as_float(r.x), __uint_as_float(r.y), __uint_as_float(r.z), __uint_as_float(r.w)}};
  }
  static __device__ __forceinline__ float dot(const Q& q, const v4u& k) {
    float p = q.f[0] * __uint_as_float(k.x);
    p = fmaf(q.f[1], __uint_as_float(k.y), p);
    p = fmaf(q.f[2], __uint_as_float(k.z), p);
    return fmaf(q.f[3], __uint_as_float(k.w), p);
  }
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
    f[0] = __uint_as_float(r.x);
    f[1] = __uint_as_float(r.y);
    f[2] = __uint_as_float(r.z);
    f[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ void store(char* p, float v) { *reinterpret_cast<float*>(p) = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
// bf16 / f16: q.k on the packed pairs with v_dot2 (fp32 accumulate), no conversion of K
struct BF16 {
  using type = __hip_bfloat16;
  static constexpr int kEpl = 8;
  struct Q { v4u w; };
  static __device__ __forceinline__ Q load_q(const v4u& r) { return Q{r}; }
  static __device__ __forceinline__ float dot(const Q& q, const v4u& k) {
    float p = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // the words go through scalars: bit_cast applied directly to a vector element reads element 0
      const uint32_t qw = q.w[i], kw = k[i];
      p = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, qw), __builtin_bit_cast(bf16x2_t, kw), p, false);
    }
    return p;
  }
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(r[i] << 16);
      f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(char* p, float v) {
    *reinterpret_cast<__hip_bfloat16*>(p) = __float2bfloat16(v);
  }
  static __device__ __forceinline__ float round(float v) { return __bfloat162float(__float2bfloat16(v)); }
};
struct F16 {
  using type = __half;
  static constexpr int kEpl = 8;
  struct Q { v4u w; };
  static __device__ __forceinline__ Q load_q(const v4u& r) { return Q{r}; }
  static __device__ __forceinline__ float dot(const Q& q, const v4u& k) {
    float p = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t qw = q.w[i], kw = k[i];
      p = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, qw), __builtin_bit_cast(f16x2_t, kw), p, false);
    }
    return p;
  }
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = r[i];
      const f16x2_t h = __builtin_bit_cast(f16x2_t, w);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  static __device__ __forceinline__ void store(char* p, float v) { *reinterpret_cast<__half*>(p) = __float2half(v); }
  static __device__ __forceinline__ float round(float v) { return __half2float(__float2half(v)); }
};

// K and V are streamed once: non-temporal loads keep them from displacing the caches
__device__ __forceinline__ v4u stream_load(const char* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
}

// Attention-sink gate of the caller's post-attention step (model.py:122-128), applied where the
// output row and its lse are final: the reference multiplies the attention output, already rounded
// to the model dtype, by sigmoid(lse - sinks[h]) in fp32 and rounds again.
template <typename E>
__device__ __forceinline__ float sink_gate(float o, float lse_nat, const float* sinks, int hq) {
  if (sinks == nullptr) return o;
  const float g = 1.f / (1.f + __expf(sinks[hq] - lse_nat));
  return E::round(o) * g;
}

// ---- cross-lane helpers ---------------------------------------------------
template <int kCtrl>
__device__ __forceinline__ float dpp(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), kCtrl, 0xf, 0xf, true));
}

// Sum over the kLanes consecutive lanes that share a row; every lane gets the total.
// All kN values advance one butterfly step at a time, so back-to-back DPP
// instructions are independent of each other.
template <int kLanes, int kN>
__device__ __forceinline__ void row_sum(float (&x)[kN]) {
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 2) x[i] += dpp<0xB1>(x[i]);   // quad_perm [1,0,3,2]
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 4) x[i] += dpp<0x4E>(x[i]);   // quad_perm [2,3,0,1]
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 8) x[i] += dpp<0x141>(x[i]);  // row_half_mirror
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 16) x[i] += dpp<0x140>(x[i]); // row_mirror
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 32) x[i] += __shfl_xor(x[i], 16);
#pragma unroll
  for (int i = 0; i < kN; ++i) if (kLanes >= 64) x[i] += __shfl_xor(x[i], 32);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float safe_max(float m) { return m == -INFINITY ? 0.f : m; }

// tokens per split of a context of L tokens: L is divided evenly over ceil(L / split_tokens)
// splits, rounded up to 64 tokens (so every split starts on a wavefront-iteration boundary)
__device__ __forceinline__ int split_part(int L, int split_tokens) {
  if (L <= 0) return split_tokens;
  const int n = (L + split_tokens - 1) / split_tokens;
  const int even = (L + n - 1) / n;
  return (even + 63) & ~63;
}

// One wavefront iteration: U row loads of K and V per lane are already in registers;
// fold them into the lane group's online-softmax state.  kMasked: rows at or past
// `t1` (only in the last iteration of a split) get a score of -inf.
// GK = 1: the G query heads share one K row; GK = G: every query head has its own K row (a cache
// that stores one K head per query head) while V is still shared.
template <typename E, int TPR, int G, int GK, int U, int RPW, bool kMasked>
__device__ __forceinline__ void fold_rows(const v4u (&kreg)[GK][U], const v4u (&vreg)[U], const typename E::Q (&q)[G],
                                          float qscale, int row0, int t1, float (&m)[G], float (&l)[G],
                                          float (&acc)[G][E::kEpl]) {
  constexpr int EPL = E::kEpl;
  float s[G][U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int g = 0; g < G; ++g) s[g][u] = E::dot(q[g], kreg[GK == 1 ? 0 : g][u]);
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    row_sum<TPR, U>(s[g]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float tot = s[g][u] * qscale;
      s[g][u] = (!kMasked || row0 + u * RPW < t1) ? tot : -INFINITY;
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mx = m[g];
#pragma unroll
    for (int u = 0; u < U; ++u) mx = fmaxf(mx, s[g][u]);
    const float ms = safe_max(mx);
    const float alpha = fast_exp2(m[g] - ms);
    m[g] = mx;
    float ps = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      s[g][u] = fast_exp2(s[g][u] - ms);
      ps += s[g][u];
    }
    l[g] = l[g] * alpha + ps;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][e] *= alpha;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float vf[EPL];
    E::unpack(vreg[u], vf);
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][e] = fmaf(s[g][u], vf[e], acc[g][e]);
    }
  }
}

// ---- main kernel ------------------------------------------------------------
// kAligned: the page size is a power of two and a multiple of the rows one
// wavefront iteration covers, so those rows share one page and one base address.
//
// kPerHeadK serves a cache that holds one K head per QUERY head (the reference stores K and V
// expanded to n_heads because the 2D rotary angles differ per head, model.py:112-114) whose V heads
// are n_rep identical copies: a workgroup takes the G = n_rep query heads of one group, reads their G
// K rows and ONE V row (the first copy), i.e. (G + 1) / 2G of the bytes an expanded read costs.
constexpr int decode_loads_in_flight(int G, bool per_head_k) { return per_head_k && G >= 4 ? 4 : 8; }

// Four workgroups per CU instead of three (at most 128 registers) where the kernel fits without spilling:
// one query head per cache head, and two in fp32 (the 16-bit kernels keep twice the elements per lane).  Not for
// the even cut, which runs two workgroups per CU.
template <typename E, int D, int G, bool kPerHeadK, bool kFlat>
constexpr int decode_waves_per_simd() {
  return (!kFlat && !kPerHeadK && (G == 1 || (G == 2 && sizeof(typename E::type) == 4))) ? 4 : 1;
}

// Even cut of a launch (kFlat): the contexts of the launch, each rounded up to 64 tokens, are laid end
// to end and cut into n_chunks pieces of equal length.  Sequence b starts at flat_start[b]; chunk c covers
// [c * len, (c + 1) * len); a chunk that spans several sequences works through them one after another.
constexpr int kFlatMaxB = 1024;

// Start of every sequence on the flat axis -> s_start[0 .. B] (s_start[B] = total), by one wavefront.
__device__ __forceinline__ void flat_starts(const DecodeArgs& a, int* s_start) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    const int per = (a.B + 63) / 64;  // consecutive sequences per lane
    int sum = 0;
    for (int i = 0; i < per; ++i) {
      const int b = lane * per + i;
      int Lr = 0;
      if (b < a.B) {
        int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
        const int64_t trow = a.batch_idx[b];
        if (trow < 0 || trow >= a.max_batch || L < 0) L = 0;
        if (L > a.max_context) L = a.max_context;
        Lr = (static_cast<int>(L) + 63) & ~63;
      }
      sum += Lr;
    }
    int incl = sum;  // inclusive scan over the lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    int run = incl - sum;
    for (int i = 0; i < per; ++i) {
      const int b = lane * per + i;
      if (b > a.B) break;
      s_start[b] = run;
      if (b < a.B) {
        int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
        const int64_t trow = a.batch_idx[b];
        if (trow < 0 || trow >= a.max_batch || L < 0) L = 0;
        if (L > a.max_context) L = a.max_context;
        run += (static_cast<int>(L) + 63) & ~63;
      }
    }
    if (lane == 63 && a.B == 64 * per) s_start[a.B] = incl;
  }
}

// tokens per chunk of the even cut
__device__ __forceinline__ int flat_chunk_len(int total, int n_chunks) {
  const int len = (total + n_chunks - 1) / n_chunks;
  return len < 64 ? 64 : (len + 63) & ~63;
}

template <typename E, int D, int G, bool kDirect, bool kAligned, bool kPerHeadK = false, bool kFlat = false>
__global__ __launch_bounds__(kThreads, (decode_waves_per_simd<E, D, G, kPerHeadK, kFlat>())) void paged_decode_kernel(const DecodeArgs a) {
  constexpr int EPL = E::kEpl;          // elements per lane
  constexpr int TPR = D / EPL;          // lanes per row
  constexpr int RPW = 64 / TPR;         // rows per wavefront load
  constexpr int GK = kPerHeadK ? G : 1; // K rows per token a workgroup reads
  constexpr int U = decode_loads_in_flight(G, kPerHeadK);  // loads of K (per K head) and of V in flight per lane
  constexpr int CH = RPW * U;           // rows per wavefront iteration
  constexpr int ROWB = D * sizeof(typename E::type);

  __shared__ int s_pages[kMaxSplitPages];
  __shared__ float s_acc[kWaves][G][D];
  __shared__ float s_ml[kWaves][G][2];

  // Workgroups are dealt to the 8 XCDs round-robin by linear id.  Heads run fastest:
  // every head of a sequence has the same amount of work, so each XCD gets an equal
  // share of the non-empty workgroups whatever the context lengths are.
  // The workgroup dispatcher deals consecutive workgroups of an XCD to its four shader engines in turn
  // and starts them in order, so with grid y = sequence every split of a sequence would land on the
  // same engine and an engine's load would be the lengths of "its" sequences (12 % apart at 64
  // sequences of 1 k to 4 k tokens).  Rotating the sequences by the split index spreads each sequence
  // over the engines.
  const int hc = blockIdx.x;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int grp = lane / TPR;  // row of this lane inside a wavefront load
  const int col = lane % TPR;  // 16-byte chunk of the row

  // Tokens [t0, t0 + part) of sequence b; a partial result goes to row hq * part_mul + part_add of the
  // workspace.
  auto piece = [&](const int b, const int t0, const int part, const bool first, const int64_t part_mul,
                   const int64_t part_add, const int* pre = nullptr, const int* pre_pages = nullptr) {
  int64_t L = pre ? static_cast<int64_t>(pre[3]) : fp::load_index(a.input_pos, b, a.pos_i64) + 1;
  const int64_t trow = pre ? static_cast<int64_t>(pre[4]) : a.batch_idx[b];
  const int* pages_lds = pre_pages ? pre_pages : s_pages;
  if (trow < 0 || trow >= a.max_batch) L = 0;
  // A position at or beyond max_context is outside what the launch was sized for: the context is read
  // up to max_context from the pool, and the fresh row of a fused append is neither folded nor stored
  // (it must not land on the slot of position max_context - 1, which holds a valid row).
  const bool beyond = L > a.max_context;
  if (beyond) L = a.max_context;
  auto lse_at = [&](int hq) -> float& {
    return a.lse[static_cast<int64_t>(b) * a.Hq + hq];
  };
  if (t0 >= L) {
    if (kDirect && first) {
      // no visible key at all: out = 0, lse = -inf
      for (int i = tid; i < G * D; i += kThreads) {
        const int g = i / D, d = i - g * D;
        E::store(a.out + b * a.os_b + (hc * G + g) * a.os_h + d * sizeof(typename E::type), 0.f);
      }
      if (tid < G) lse_at(hc * G + tid) = -INFINITY;
    }
    return;
  }
  const int t1 = static_cast<int>(L < t0 + part ? L : t0 + part);
  // Fused append: the newest token (position L - 1) is not in the pool yet.  The workgroup whose
  // range holds it reads that row from k_new / v_new, folds it in and writes it to its slot; the
  // pool is only read up to L - 2.
  const bool owns_new = a.k_new != nullptr && !beyond && L - 1 >= t0;  // t1 == L whenever L - 1 lies in this split
  const int t1_pool = (owns_new && t1 == L) ? t1 - 1 : t1;

  // this lane's 16 bytes of the query row of every head of the group
  typename E::Q q[G];
#pragma unroll
  for (int g = 0; g < G; ++g)
    q[g] = E::load_q(*reinterpret_cast<const v4u*>(a.q + b * a.qs_b + (hc * G + g) * a.qs_h + col * 16));

  float m[G], l[G], acc[G][EPL];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
  }

  // cache head of the workgroup's first K row and of its V row; with kPerHeadK the group's K heads
  // follow at head_stride
  const int64_t head_stride = a.n_slots * ROWB;
  const char* kbase = a.pool_k + static_cast<int64_t>(kPerHeadK ? hc * G : hc) * head_stride + col * 16;
  const char* vbase = a.pool_v + static_cast<int64_t>(kPerHeadK ? hc * G : hc) * head_stride + col * 16;

  // page ids of the split -> LDS, then the rows
  int64_t blk0;
  {
    int off_unused;
    a.pd.split(t0, blk0, off_unused);
    int64_t blk_last;
    a.pd.split(t1 - 1, blk_last, off_unused);
    const int nblk = pre_pages ? 0 : static_cast<int>(blk_last - blk0) + 1;
    for (int i = tid; i < nblk; i += kThreads) {
      int64_t page = 0;
      if (blk0 + i < a.n_pages) page = a.page_table[trow * a.pt_row_stride + blk0 + i];
      if (page < 0 || page >= a.n_slots / a.pd.page_size) page = 0;  // not a page of the pool
      s_pages[i] = static_cast<int>(page);
    }
  }
  __syncthreads();
  const int c_end = t1_pool;

#pragma nounroll
  for (int c0 = t0 + wave * CH; c0 < c_end; c0 += kWaves * CH) {
    v4u kreg[GK][U], vreg[U];
    if (kAligned) {
      // the CH rows of this iteration lie in one page: one base, constant offsets
      const int page = pages_lds[(c0 >> a.pd.shift) - static_cast<int>(blk0)];
      const int64_t slot = static_cast<int64_t>(page) * a.pd.page_size + (c0 & (a.pd.page_size - 1)) + grp;
      const char* kp = kbase + slot * ROWB;
      const char* vp = vbase + slot * ROWB;
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int gk = 0; gk < GK; ++gk) kreg[gk][u] = stream_load(kp + gk * head_stride + u * RPW * ROWB);
        vreg[u] = stream_load(vp + u * RPW * ROWB);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int t = c0 + u * RPW + grp;
        if (t >= c_end) t = c_end - 1;
        int64_t blk;
        int off;
        a.pd.split(t, blk, off);
        const int64_t slot = static_cast<int64_t>(pages_lds[blk - blk0]) * a.pd.page_size + off;
#pragma unroll
        for (int gk = 0; gk < GK; ++gk) kreg[gk][u] = stream_load(kbase + gk * head_stride + slot * ROWB);
        vreg[u] = stream_load(vbase + slot * ROWB);
      }
    }
    if (c0 + CH <= c_end)
      fold_rows<E, TPR, G, GK, U, RPW, false>(kreg, vreg, q, a.qscale, c0 + grp, c_end, m, l, acc);
    else
      fold_rows<E, TPR, G, GK, U, RPW, true>(kreg, vreg, q, a.qscale, c0 + grp, c_end, m, l, acc);
  }

  if (t1_pool != t1 && wave == 0) {
    // the newest token: one row, held by lane group 0; every other row of this pass is masked
    v4u kreg[GK][U], vreg[U];
    const int h0 = kPerHeadK ? hc * G : hc;  // first cache head of this workgroup
    v4u kn[GK];
#pragma unroll
    for (int gk = 0; gk < GK; ++gk)
      kn[gk] = *reinterpret_cast<const v4u*>(a.k_new + b * a.kn_b + (h0 + gk) * a.kn_h + col * 16);
    const v4u vn = *reinterpret_cast<const v4u*>(a.v_new + b * a.vn_b + h0 * a.vn_h + col * 16);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int gk = 0; gk < GK; ++gk) kreg[gk][u] = kn[gk];
      vreg[u] = vn;
    }
    fold_rows<E, TPR, G, GK, U, RPW, true>(kreg, vreg, q, a.qscale, t1 - 1 + grp, t1, m, l, acc);
    if (grp == 0) {
      int64_t blk;
      int off;
      a.pd.split(t1 - 1, blk, off);
      const int64_t slot = static_cast<int64_t>(pages_lds[blk - blk0]) * a.pd.page_size + off;
#pragma unroll
      for (int gk = 0; gk < GK; ++gk) {
        // every cached head gets its K row; V is written to every copy so the pool stays what the
        // reference's append leaves (the copies are read by the prefill kernel and by other callers)
        __builtin_nontemporal_store(kn[gk], reinterpret_cast<v4u*>(const_cast<char*>(kbase) + gk * head_stride + slot * ROWB));
        const v4u vrow = kPerHeadK ? *reinterpret_cast<const v4u*>(a.v_new + b * a.vn_b + (h0 + gk) * a.vn_h + col * 16) : vn;
        __builtin_nontemporal_store(vrow, reinterpret_cast<v4u*>(const_cast<char*>(vbase) + gk * head_stride + slot * ROWB));
      }
    }
  }

  // combine the lane groups of this wavefront
#pragma unroll
  for (int off = TPR; off < 64; off <<= 1) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float mo = __shfl_xor(m[g], off);
      const float lo = __shfl_xor(l[g], off);
      const float mn = fmaxf(m[g], mo);
      const float ms = safe_max(mn);
      const float wa = fast_exp2(m[g] - ms);
      const float wb = fast_exp2(mo - ms);
      l[g] = l[g] * wa + lo * wb;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][e] = acc[g][e] * wa + __shfl_xor(acc[g][e], off) * wb;
      m[g] = mn;
    }
  }
  if (lane < TPR) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) s_acc[wave][g][col * EPL + e] = acc[g][e];
      if (lane == 0) {
        s_ml[wave][g][0] = m[g];
        s_ml[wave][g][1] = l[g];
      }
    }
  }
  __syncthreads();

  // combine the wavefronts; one thread per (head of the group, element)
  for (int i = tid; i < G * D; i += kThreads) {
    const int g = i / D, d = i - g * D;
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) mn = fmaxf(mn, s_ml[w][g][0]);
    const float ms = safe_max(mn);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float wgt = fast_exp2(s_ml[w][g][0] - ms);
      num += s_acc[w][g][d] * wgt;
      den += s_ml[w][g][1] * wgt;
    }
    const int hq = hc * G + g;
    if (kDirect) {
      const float lse_nat = (mn + log2f(den)) * kLn2;
      E::store(a.out + b * a.os_b + hq * a.os_h + d * sizeof(typename E::type), sink_gate<E>(num / den, lse_nat, a.sinks, hq));
      if (d == 0) lse_at(hq) = lse_nat;
    } else {
      const int64_t p = hq * part_mul + part_add;
      a.ws_acc[p * D + d] = num;
      if (d == 0) {
        a.ws_ml[p * 2] = mn;
        a.ws_ml[p * 2 + 1] = den;
      }
    }
  }
  };  // piece

  if constexpr (!kFlat) {
    // grid (Hc, B, splits).  A context of L tokens is cut into ceil(L / split_tokens) parts of equal
    // size (a multiple of 64 tokens), so the workgroups of one sequence carry the same load instead of
    // leaving a short tail split.
    // The workgroup dispatcher deals consecutive workgroups of an XCD to its four shader engines in turn
    // and starts them in order, so with grid y = sequence every split of a sequence would land on the
    // same engine and an engine's load would be the lengths of "its" sequences (12 % apart at 64
    // sequences of 1 k to 4 k tokens).  Rotating the sequences by the split index spreads each sequence
    // over the engines.
    const int split = blockIdx.z;
    const int b = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
    int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
    if (L > a.max_context) L = a.max_context;
    const int part = split_part(static_cast<int>(L < 0 ? 0 : L), a.split_tokens);
    piece(b, split * part, part, split == 0, a.n_splits, static_cast<int64_t>(b) * a.Hq * a.n_splits + split);
  } else {
    // grid (Hc, n_chunks): every workgroup streams the same number of rows, whatever the lengths are
    __shared__ int s_start[kFlatMaxB + 1];
    if (a.plan) {
      // the chunk's record goes where the sequence starts would go, its page ids where a piece stages its own:
      // one trip to memory instead of positions -> cut -> page table
      const int* src = a.plan + static_cast<int64_t>(blockIdx.y) * kPlanInts;
      if (tid < kPlanRec) s_start[tid] = src[tid];
      s_pages[tid] = src[kPlanRec + tid];  // the first kThreads page ids; more only for very long chunks
      __syncthreads();
      const int n = s_start[0];
      if (n >= 0 && n <= kPlanPieces && s_start[1] == a.B && s_start[2] == a.n_chunks && s_start[3] == a.max_context) {
        int n_pages_used = 0;
        if (n > 0) {
          const int* last = s_start + 4 + 6 * (n - 1);
          n_pages_used = last[5] + last[2] / a.pd.page_size + 2;  // an upper bound of the list's length
        }
        if (n_pages_used > kThreads) {
          for (int i = kThreads + tid; i < n_pages_used && i < kPlanPages; i += kThreads) s_pages[i] = src[kPlanRec + i];
          __syncthreads();
        }
        const int c = blockIdx.y;
        // the records are read from registers of a copy: a piece reuses s_start's LDS for nothing, but keeps s_pages
        for (int k = 0; k < n; ++k) {
          int r[6];
#pragma unroll
          for (int j = 0; j < 6; ++j) r[j] = s_start[4 + 6 * k + j];
          piece(r[0], r[1], r[2], false, 1, static_cast<int64_t>(c + r[0]) * a.Hq, r, s_pages + r[5]);
          __syncthreads();  // the LDS of the piece is free again
        }
        return;
      }
      __syncthreads();  // no usable plan: s_start and s_pages are written anew below
    }
    flat_starts(a, s_start);
    __syncthreads();
    const int total = s_start[a.B];
    const int len = flat_chunk_len(total, a.n_chunks);
    const int c = blockIdx.y;
    const int64_t lo = static_cast<int64_t>(c) * len;
    const int64_t hi = lo + len < total ? lo + len : total;
    if (lo >= total) return;
    // first sequence that ends after lo
    int b = 0;
    {
      int left = 0, right = a.B - 1;
      while (left < right) {
        const int mid = (left + right) >> 1;
        if (s_start[mid + 1] > lo) right = mid; else left = mid + 1;
      }
      b = left;
    }
    for (; b < a.B && s_start[b] < hi; ++b) {
      const int begin = s_start[b], end = s_start[b + 1];
      if (end == begin) continue;  // a sequence without keys has no piece; the merge pass writes its zeros
      const int t0 = lo > begin ? static_cast<int>(lo - begin) : 0;
      const int t1 = static_cast<int>((hi < end ? hi : end) - begin);
      piece(b, t0, t1 - t0, false, 1, static_cast<int64_t>(c + b) * a.Hq);
      __syncthreads();  // the LDS of the piece is free again
    }
  }
}

// Writes the plan of a step (see kPlanInts): one wavefront per chunk of the even cut repeats the cut the
// main kernel would make and looks the page ids of its pieces up.
__global__ __launch_bounds__(64) void paged_decode_plan_kernel(const DecodeArgs a) {
  __shared__ int s_start[kFlatMaxB + 1];
  flat_starts(a, s_start);
  __syncthreads();
  const int c = blockIdx.x;
  int* rec = a.plan + static_cast<int64_t>(c) * kPlanInts;
  int* pages = rec + kPlanRec;
  const int total = s_start[a.B];
  const int len = flat_chunk_len(total, a.n_chunks);
  const int64_t lo = static_cast<int64_t>(c) * len;
  const int64_t hi = lo + len < total ? lo + len : total;
  const int lane = threadIdx.x;
  const int64_t pool_pages = a.n_slots / a.pd.page_size;
  int n = 0, page_off = 0;
  bool ok = true;
  if (lo < total) {
    int b = 0;  // first sequence that ends after lo
    {
      int left = 0, right = a.B - 1;
      while (left < right) {
        const int mid = (left + right) >> 1;
        if (s_start[mid + 1] > lo) right = mid; else left = mid + 1;
      }
      b = left;
    }
    for (; b < a.B && s_start[b] < hi; ++b) {
      const int begin = s_start[b], end = s_start[b + 1];
      if (end == begin) continue;
      const int t0 = lo > begin ? static_cast<int>(lo - begin) : 0;
      const int part = static_cast<int>((hi < end ? hi : end) - begin) - t0;
      int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
      int64_t trow = a.batch_idx[b];
      const int64_t L_raw = L > INT32_MAX ? INT32_MAX : L < INT32_MIN ? INT32_MIN : L;
      if (trow < 0 || trow >= a.max_batch) {
        trow = -1;
        L = 0;
      }
      if (L > a.max_context) L = a.max_context;
      if (n >= kPlanPieces) {
        ok = false;
        break;
      }
      int nblk = 0;
      if (t0 < L) {  // the pages of tokens t0 .. min(L, t0 + part) - 1, as the main kernel stages them
        const int t1 = static_cast<int>(L < t0 + part ? L : t0 + part);
        int64_t blk0, blk_last;
        int off_unused;
        a.pd.split(t0, blk0, off_unused);
        a.pd.split(t1 - 1, blk_last, off_unused);
        nblk = static_cast<int>(blk_last - blk0) + 1;
        if (page_off + nblk > kPlanPages) {
          ok = false;
          break;
        }
        for (int i = lane; i < nblk; i += 64) {
          int64_t page = 0;
          if (blk0 + i < a.n_pages) page = a.page_table[trow * a.pt_row_stride + blk0 + i];
          if (page < 0 || page >= pool_pages) page = 0;  // not a page of the pool
          pages[page_off + i] = static_cast<int>(page);
        }
      }
      if (lane == 0) {
        int* r = rec + 4 + 6 * n;
        r[0] = b;
        r[1] = t0;
        r[2] = part;
        r[3] = static_cast<int>(L_raw);
        r[4] = static_cast<int>(trow);
        r[5] = page_off;
      }
      page_off += nblk;
      ++n;
    }
  }
  if (lane == 0) {
    rec[0] = ok ? n : -1;
    rec[1] = a.B;
    rec[2] = a.n_chunks;
    rec[3] = a.max_context;
  }
  if (c == 0) {
    uint32_t hash = 0;
    for (int i = lane; i < a.B; i += 64)
      hash += plan_hash_term(i, fp::load_index(a.input_pos, i, a.pos_i64) + 1, a.batch_idx[i]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) hash += __shfl_xor(hash, off);
    if (lane == 0) rec[kPlanHashAt] = static_cast<int>(hash);
  }
}

// ---- cross-split merge ------------------------------------------------------
// One batch of kBatch consecutive splits of a partial row, as this lane holds it.
template <int D, int kBatch>
struct SplitBatch {
  float m[kBatch], l[kBatch], acc[kBatch][(D + 63) / 64];
};

// Requests the splits base .. base + kBatch - 1 (those below `limit`) of partial row p0.
template <int D, int kBatch>
__device__ __forceinline__ void load_batch(const DecodeArgs& a, int64_t p0, int base, int limit, int64_t row_stride,
                                           SplitBatch<D, kBatch>& t) {
  constexpr int DPL = (D + 63) / 64;
#pragma unroll
  for (int s = 0; s < kBatch; ++s) {
    const bool on = base + s < limit;
    const int64_t p = p0 + (on ? base + s : 0) * row_stride;
    t.m[s] = on ? a.ws_ml[p * 2] : -INFINITY;
    t.l[s] = on ? a.ws_ml[p * 2 + 1] : 0.f;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
      const int d = (threadIdx.x & 63) + j * 64;
      t.acc[s][j] = (on && d < D) ? a.ws_acc[p * D + d] : 0.f;
    }
  }
}

// Folds the splits of a batch that lie below ns into the running state (m_run, den, num) of this lane.  A batch
// that was requested before ns was known may hold rows of splits the sequence does not have (whatever the
// workspace held): they are dropped here by selects and never enter the arithmetic.
template <int D, int kBatch>
__device__ __forceinline__ void fold_batch(SplitBatch<D, kBatch>& t, int base, int ns, float& m_run, float& den,
                                           float (&num)[(D + 63) / 64]) {
  constexpr int DPL = (D + 63) / 64;
  float mn = m_run;
#pragma unroll
  for (int s = 0; s < kBatch; ++s) {
    if (base + s >= ns) {
      t.m[s] = -INFINITY;
      t.l[s] = 0.f;
#pragma unroll
      for (int j = 0; j < DPL; ++j) t.acc[s][j] = 0.f;
    }
    mn = fmaxf(mn, t.m[s]);
  }
  const float ms = safe_max(mn);
  const float keep = fast_exp2(m_run - ms);  // 0 while the state is empty
  den *= keep;
#pragma unroll
  for (int j = 0; j < DPL; ++j) num[j] *= keep;
#pragma unroll
  for (int s = 0; s < kBatch; ++s) {
    const float wgt = fast_exp2(t.m[s] - ms);
    den += t.l[s] * wgt;
#pragma unroll
    for (int j = 0; j < DPL; ++j) num[j] += t.acc[s][j] * wgt;
  }
  m_run = mn;
}

// Folds the splits first, first + stride, ... (kBatch consecutive splits each time, below ns) of partial
// row p0 into the running state (m_run, den, num) of this lane; scores are in log2 units.
template <int D, int kBatch>
__device__ __forceinline__ void merge_batches(const DecodeArgs& a, int64_t p0, int first, int stride, int ns, float& m_run,
                                              float& den, float (&num)[(D + 63) / 64], int64_t row_stride = 1) {
  for (int base = first; base < ns; base += stride) {
    SplitBatch<D, kBatch> t;
    load_batch<D, kBatch>(a, p0, base, ns, row_stride, t);
    fold_batch<D, kBatch>(t, base, ns, m_run, den, num);
  }
}

// Normalises, gates and stores one merged row (lane = output elements lane, lane + 64, ...).
template <typename E, int D>
__device__ __forceinline__ void finish_merge(const DecodeArgs& a, int b, int hq, bool any, float mn, float den,
                                             const float (&num)[(D + 63) / 64]) {
  const float lse_nat = any ? (mn + log2f(den)) * kLn2 : -INFINITY;
#pragma unroll
  for (int j = 0; j < (D + 63) / 64; ++j) {
    const int d = (threadIdx.x & 63) + j * 64;
    if (d >= D) continue;
    const float o = any ? num[j] / den : 0.f;
    E::store(a.out + b * a.os_b + hq * a.os_h + d * sizeof(typename E::type), sink_gate<E>(o, lse_nat, a.sinks, hq));
  }
  if ((threadIdx.x & 63) == 0) a.lse[static_cast<int64_t>(b) * a.Hq + hq] = lse_nat;
}

template <typename E, int D>
__global__ __launch_bounds__(64) void paged_decode_merge_kernel(const DecodeArgs a) {
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int64_t p0 = (static_cast<int64_t>(b) * a.Hq + hq) * a.n_splits;

  // The kernel is a chain of memory latencies, so the first kBatch splits are requested together with the
  // sequence's position, by the launch's split count: the partials of splits this sequence does not have
  // are dropped by selects once its length is known and never enter the arithmetic.
  constexpr int kBatch = 8;
  constexpr int DPL = (D + 63) / 64;  // output elements per lane
  int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
  const int64_t trow = a.batch_idx[b];
  SplitBatch<D, kBatch> first;
  load_batch<D, kBatch>(a, p0, 0, a.n_splits, 1, first);
  if (trow < 0 || trow >= a.max_batch) L = 0;
  if (L > a.max_context) L = a.max_context;
  const int part = split_part(static_cast<int>(L), a.split_tokens);
  const int ns = L <= 0 ? 0 : static_cast<int>((L + part - 1) / part);

  // The same lane keeps a running (maximum, denominator, numerator) over batches of kBatch splits, every load
  // of a batch requested at once.  The wide variant of this kernel spreads the batches over several wavefronts.
  float m_run = -INFINITY, den = 0.f, num[DPL];
#pragma unroll
  for (int j = 0; j < DPL; ++j) num[j] = 0.f;
  if (ns > 0) fold_batch<D, kBatch>(first, 0, ns, m_run, den, num);
  merge_batches<D, kBatch>(a, p0, kBatch, kBatch, ns, m_run, den, num);
  finish_merge<E, D>(a, b, hq, ns > 0, m_run, den, num);
}

// Cross-split merge after the even cut: sequence b has one partial result per chunk it touches, in
// workspace rows (chunk + b) * Hq + hq.
template <typename E, int D>
__global__ __launch_bounds__(64) void paged_decode_merge_flat_kernel(const DecodeArgs a) {
  constexpr int DPL = (D + 63) / 64;
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int lane = threadIdx.x;
  int before = 0, total = 0, mine = 0;  // rounded lengths: of the sequences before b, of all, of b
  // the plan's launch values and hash, if the split-K pass had a plan: requested with the positions
  int planned[4] = {0, 0, 0, 0};
  if (a.plan) {
    planned[0] = a.plan[1];
    planned[1] = a.plan[2];
    planned[2] = a.plan[3];
    planned[3] = a.plan[kPlanHashAt];
  }
  uint32_t hash = 0;
  for (int i = lane; i < a.B; i += 64) {
    int64_t L = fp::load_index(a.input_pos, i, a.pos_i64) + 1;
    const int64_t trow = a.batch_idx[i];
    hash += plan_hash_term(i, L, trow);
    if (trow < 0 || trow >= a.max_batch || L < 0) L = 0;
    if (L > a.max_context) L = a.max_context;
    const int Lr = (static_cast<int>(L) + 63) & ~63;
    total += Lr;
    if (i < b) before += Lr;
    if (i == b) mine = Lr;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    total += __shfl_xor(total, off);
    before += __shfl_xor(before, off);
    mine += __shfl_xor(mine, off);
    hash += __shfl_xor(hash, off);
  }
  // the split-K pass followed a plan (same acceptance test as there) that was made from other positions or slots
  const bool stale = a.plan && planned[0] == a.B && planned[1] == a.n_chunks && planned[2] == a.max_context &&
                     static_cast<uint32_t>(planned[3]) != hash;
  const int len = flat_chunk_len(total, a.n_chunks);
  const int c_first = before / len;
  const int ns = mine > 0 ? (before + mine - 1) / len - c_first + 1 : 0;
  float m_run = -INFINITY, den = 0.f, num[DPL];
#pragma unroll
  for (int j = 0; j < DPL; ++j) num[j] = 0.f;
  merge_batches<D, 8>(a, static_cast<int64_t>(c_first + b) * a.Hq + hq, 0, 8, ns, m_run, den, num, a.Hq);
  if (stale) den = __builtin_nanf("");  // every row of out and lse: not a result
  finish_merge<E, D>(a, b, hq, ns > 0 || stale, m_run, den, num);
}

// Cross-split merge for launches with many splits per sequence: kMergeWideWaves wavefronts per
// (sequence, query head) take the batches of splits round-robin and combine their states through LDS.
constexpr int kMergeWideWaves = 8;
constexpr int kMergeWideSplits = 16;  // launches with more splits than this use it

template <typename E, int D>
__global__ __launch_bounds__(kMergeWideWaves * 64) void paged_decode_merge_wide_kernel(const DecodeArgs a) {
  constexpr int kBatch = 8;
  constexpr int DPL = (D + 63) / 64;
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t p0 = (static_cast<int64_t>(b) * a.Hq + hq) * a.n_splits;
  __shared__ float s_m[kMergeWideWaves], s_den[kMergeWideWaves], s_num[kMergeWideWaves][DPL * 64];

  // The kernel is a chain of memory latencies: the position of the sequence and this wavefront's first batch of
  // partial rows are requested together (the batch by the launch's split count; what the sequence does not
  // have is dropped once its length is known), the later batches of a launch of more than 64 splits after it.
  int64_t L = fp::load_index(a.input_pos, b, a.pos_i64) + 1;
  const int64_t trow = a.batch_idx[b];
  SplitBatch<D, kBatch> first;
  load_batch<D, kBatch>(a, p0, wave * kBatch, a.n_splits, 1, first);
  if (trow < 0 || trow >= a.max_batch) L = 0;
  if (L > a.max_context) L = a.max_context;
  const int part = split_part(static_cast<int>(L), a.split_tokens);
  const int ns = L <= 0 ? 0 : static_cast<int>((L + part - 1) / part);

  float m_run = -INFINITY, den = 0.f, num[DPL];
#pragma unroll
  for (int j = 0; j < DPL; ++j) num[j] = 0.f;
  if (wave * kBatch < ns) fold_batch<D, kBatch>(first, wave * kBatch, ns, m_run, den, num);
  merge_batches<D, kBatch>(a, p0, (wave + kMergeWideWaves) * kBatch, kMergeWideWaves * kBatch, ns, m_run, den, num);
  if (lane == 0) {
    s_m[wave] = m_run;
    s_den[wave] = den;
  }
#pragma unroll
  for (int j = 0; j < DPL; ++j) s_num[wave][j * 64 + lane] = num[j];
  __syncthreads();
  if (wave != 0) return;
  float mn = -INFINITY;
#pragma unroll
  for (int w = 0; w < kMergeWideWaves; ++w) mn = fmaxf(mn, s_m[w]);
  const float ms = safe_max(mn);
  den = 0.f;
#pragma unroll
  for (int j = 0; j < DPL; ++j) num[j] = 0.f;
#pragma unroll
  for (int w = 0; w < kMergeWideWaves; ++w) {
    const float wgt = fast_exp2(s_m[w] - ms);  // 0 for a wavefront that had no split
    den += s_den[w] * wgt;
#pragma unroll
    for (int j = 0; j < DPL; ++j) num[j] += s_num[w][j * 64 + lane] * wgt;
  }
  finish_merge<E, D>(a, b, hq, ns > 0, mn, den, num);
}

constexpr int kPhasePartial = 1;
constexpr int kPhaseMerge = 2;
constexpr int kPhasePlan = 4;  // alone: write the step's plan instead of launching the passes

// Workgroups of the even-cut kernel the current device holds at once (asked once per kernel and device).
template <typename E, int D, int G, bool kAligned, bool kPerHeadK>
int resident_workgroups() {
  const auto kernel = paged_decode_kernel<E, D, G, false, kAligned, kPerHeadK, true>;
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, 0) != hipSuccess || per_cu <= 0) {
      (void)hipGetLastError();  // not an error of the launch that follows: the launch goes split by split
      cached[dev] = -1;
    } else
      cached[dev] = per_cu * fp::compute_units();
  }
  return cached[dev] > 0 ? cached[dev] : 0;
}

template <typename E, int D, int G, bool kPerHeadK = false>
void launch_decode(const DecodeArgs& a, int B, int phases, hipStream_t st) {
  dim3 grid(a.Hc, B, a.n_splits);  // a.Hc = workgroups per sequence and split: cache heads, or groups of G heads
  // rows per wavefront iteration: the loads in flight times 64 / (D * elem / 16) rows each
  const int chunk_rows = decode_loads_in_flight(G, kPerHeadK) * 64 / (D * static_cast<int>(sizeof(typename E::type)) / 16);
  const bool aligned = a.pd.shift >= 0 && a.pd.page_size % chunk_rows == 0;
  if (a.n_splits == 1) {
    // one split covers every context: the partial pass writes out and lse itself
    if (!(phases & kPhasePartial)) return;  // also the plan phase: such a launch has no even cut
    if (aligned)
      hipLaunchKernelGGL((paged_decode_kernel<E, D, G, true, true, kPerHeadK>), grid, dim3(kThreads), 0, st, a);
    else
      hipLaunchKernelGGL((paged_decode_kernel<E, D, G, true, false, kPerHeadK>), grid, dim3(kThreads), 0, st, a);
  } else {
    // A launch with more workgroups than the GPU holds at once is cut evenly instead: two chunks
    // per CU, all of the same length, all resident from the start, so that every CU streams the same
    // number of rows (split by split, the CUs end up with loads 25 % apart at 64 sequences of 1 k to
    // 4 k tokens, and workgroups queue behind busy shader engines).  Measured at 64 sequences of 16 q /
    // 8 kv heads, bf16, % of 8 TB/s for the step with 1 / 2 / 3 / 4 chunks per CU and split by split:
    // D 128: 75.5 / 75.4 / 73.8 / 73.1 and 73.0; D 64: 67.2 / 68.3 / 68.1 / 63.7 and 67.1; 32 q heads:
    // 63.9 / 70.6 / 64.2 / 67.9 and 67.2; 16-token pages: 70.0 / 74.4 / 73.9 / 68.9 and 72.6.  fp32 with
    // two chunks per CU: D 128 80.7 against 78.4 split by split, D 64 76.9 against 76.1, 32 q heads 77.4
    // against 73.4 (the even-cut kernels are not held to 128 registers: two workgroups per CU do not need
    // it, and in fp32 it made them spill).  With the step's plan read by every workgroup the same sweep gives, in us per
    // step for 1 / 2 / 3 chunks per CU: D 128 110.4 / 111.3 / 112.2; D 64 61.7 / 61.3 / 62.1; page size 64, 32
    // sequences 89.2 / 90.9 / 90.4: two stays.  The even cut needs the lengths of at most kFlatMaxB sequences in LDS, a workspace row per (chunk + sequence),
    // and chunks within the page-id table.
    int n_chunks = 0;
    {
      const int resident = aligned ? resident_workgroups<E, D, G, true, kPerHeadK>()
                                   : resident_workgroups<E, D, G, false, kPerHeadK>();
      const int64_t wgs = static_cast<int64_t>(a.Hc) * B * a.n_splits;
      const int chunks = 2 * fp::compute_units() / a.Hc;
      const bool rows_fit = chunks + B <= static_cast<int64_t>(B) * a.n_splits;  // workspace rows: one per (chunk + sequence)
      const bool positions_fit = static_cast<int64_t>(B) * (a.max_context + 64) < (1ll << 30);  // the flat axis is int
      if (chunks >= 1 && wgs > resident && B <= kFlatMaxB && rows_fit && positions_fit &&
          (static_cast<int64_t>(B) * (a.max_context + 64) / chunks + 128) / a.pd.page_size + 2 <= kMaxSplitPages)
        n_chunks = chunks;
    }
    DecodeArgs af = a;
    af.B = B;
    af.n_chunks = n_chunks;
    if (phases & kPhasePlan) {
      // the plan of a step serves the even cut only; a launch that goes split by split needs none
      if (a.plan && n_chunks > 0) hipLaunchKernelGGL(paged_decode_plan_kernel, dim3(n_chunks), dim3(64), 0, st, af);
      return;
    }
    if (phases & kPhasePartial) {
      if (n_chunks > 0) {
        if (aligned)
          hipLaunchKernelGGL((paged_decode_kernel<E, D, G, false, true, kPerHeadK, true>), dim3(a.Hc, n_chunks), dim3(kThreads), 0, st, af);
        else
          hipLaunchKernelGGL((paged_decode_kernel<E, D, G, false, false, kPerHeadK, true>), dim3(a.Hc, n_chunks), dim3(kThreads), 0, st, af);
      } else if (aligned) {
        hipLaunchKernelGGL((paged_decode_kernel<E, D, G, false, true, kPerHeadK>), grid, dim3(kThreads), 0, st, a);
      } else {
        hipLaunchKernelGGL((paged_decode_kernel<E, D, G, false, false, kPerHeadK>), grid, dim3(kThreads), 0, st, a);
      }
    }
    if (phases & kPhaseMerge) {
      if (n_chunks > 0)
        hipLaunchKernelGGL((paged_decode_merge_flat_kernel<E, D>), dim3(a.Hq, B), dim3(64), 0, st, af);
      else if (a.n_splits > kMergeWideSplits)
        hipLaunchKernelGGL((paged_decode_merge_wide_kernel<E, D>), dim3(a.Hq, B), dim3(kMergeWideWaves * 64), 0, st, a);
      else
        hipLaunchKernelGGL((paged_decode_merge_kernel<E, D>), dim3(a.Hq, B), dim3(64), 0, st, a);
    }
  }
}

template <typename E, int D>
int dispatch_group(const DecodeArgs& a, int B, int phases, int kv_rep, hipStream_t st) {
  if (kv_rep > 1) {  // a.Hc already counts groups of kv_rep heads
    switch (kv_rep) {
      case 2: launch_decode<E, D, 2, true>(a, B, phases, st); return FP_OK;
      case 4: launch_decode<E, D, 4, true>(a, B, phases, st); return FP_OK;
      default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: kv_rep = %d (supported: 1, 2, 4)", kv_rep);
    }
  }
  switch (a.Hq / a.Hc) {
    case 1: launch_decode<E, D, 1>(a, B, phases, st); return FP_OK;
    case 2: launch_decode<E, D, 2>(a, B, phases, st); return FP_OK;
    case 4: launch_decode<E, D, 4>(a, B, phases, st); return FP_OK;
    case 8: launch_decode<E, D, 8>(a, B, phases, st); return FP_OK;
    default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: Hq/Hc = %d (supported: 1, 2, 4, 8)", a.Hq / a.Hc);
  }
}

template <typename E>
int dispatch_dim(const DecodeArgs& a, int B, int D, int phases, int kv_rep, hipStream_t st) {
  switch (D) {
    case 64: return dispatch_group<E, 64>(a, B, phases, kv_rep, st);
    case 128: return dispatch_group<E, 128>(a, B, phases, kv_rep, st);
    default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: head_dim %d (supported: 64, 128)", D);
  }
}

// Largest split (fewest partials to merge, least per-workgroup overhead) that still yields enough
// workgroups when every sequence is at max_context.  Enough is about 2048 (8 per CU) for a batch whose
// sequences alone give every CU two workgroups: their lengths differ, and small pieces even that out.
// A small batch wants larger pieces: from 512 workgroups (4 * B * Hc in between) the pass no longer gets
// faster, and every further split is one more partial result to merge.
int default_split_tokens(int B, int Hc, int max_context, int page_size) {
  int64_t target = 4 * static_cast<int64_t>(B) * Hc;
  target = target < 512 ? 512 : target > 2048 ? 2048 : target;
  int split = 2048;
  while (split > 128 && static_cast<int64_t>(B) * Hc * ((max_context + split - 1) / split) < target) split >>= 1;
  while (split / page_size + 2 > kMaxSplitPages) split >>= 1;
  return split < 64 ? 64 : split;
}

int n_splits_for(int max_context, int split_tokens) {
  const int n = (max_context + split_tokens - 1) / split_tokens;
  return n < 1 ? 1 : n;
}

}  // namespace

extern "C" int32_t fp_paged_decode_default_split(int32_t B, int32_t Hc, int32_t max_context, int32_t page_size) {
  if (B <= 0 || Hc <= 0 || max_context < 0 || page_size <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_default_split: bad dimension");
  return default_split_tokens(B, Hc, max_context, page_size);
}

extern "C" int64_t fp_paged_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t D, int32_t max_context,
                                                   int32_t split_tokens) {
  if (B < 0 || Hq <= 0 || D <= 0 || max_context < 0 || split_tokens <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_workspace_bytes: bad dimension");
  if (split_tokens % 64) return fp::fail(FP_ERR_INVALID_ARGUMENT, "split_tokens must be a multiple of 64");
  const int64_t ns = n_splits_for(max_context, split_tokens);
  if (ns == 1) return 0;
  return static_cast<int64_t>(B) * Hq * ns * (D + 2) * static_cast<int64_t>(sizeof(float));
}

namespace {

// A plan has a record per chunk of the even cut; a launch has at most two chunks per CU and cache head.
int64_t plan_buffer_bytes() { return 2LL * fp::compute_units() * kPlanInts * static_cast<int64_t>(sizeof(int)); }

struct NewRows {
  const void* k;
  const void* v;
  int64_t k_stride_b, k_stride_h, v_stride_b, v_stride_h;  // elements
};

int decode_entry(int phases, const NewRows* fresh, const void* q, int64_t q_stride_b, int64_t q_stride_h, const void* pool_k,
                 const void* pool_v, const int64_t* page_table, int64_t pt_row_stride,
                 const int64_t* batch_idx, const void* input_pos, int pos_index_type,
                 void* out, int64_t out_stride_b, int64_t out_stride_h, float* lse, const float* sinks,
                 void* workspace, int64_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep,
                 int32_t D, int32_t page_size, int32_t n_pages, int32_t max_batch,
                 int64_t n_slots, int32_t max_context, int32_t split_tokens, float scale,
                 int dtype, void* plan, int64_t plan_bytes, void* stream) {
  const bool plan_only = phases == kPhasePlan;  // q, out, lse and the workspace are not touched then
  const int eb = fp::elem_bytes(dtype);
  if (eb == 0) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: unknown dtype %d", dtype);
  if (B < 0 || Hq <= 0 || Hc <= 0 || D <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 ||
      n_slots <= 0 || max_context < 0 || split_tokens < 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: bad dimension");
  if (Hq % Hc) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: Hq=%d not a multiple of Hc=%d", Hq, Hc);
  if (kv_rep < 1) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: kv_rep must be at least 1");
  if (kv_rep > 1 && (Hc != Hq || Hq % kv_rep))
    return fp::fail(FP_ERR_INVALID_ARGUMENT,
                    "fp_paged_decode: kv_rep = %d needs a cache with one head per query head (Hc = Hq = %d here %d) "
                    "and Hq a multiple of kv_rep", kv_rep, Hq, Hc);
  const int wg_heads = kv_rep > 1 ? Hq / kv_rep : Hc;  // workgroups per sequence and split
  if (n_slots < page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: n_slots smaller than one page");
  if (max_context > static_cast<int64_t>(n_pages) * page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: max_context exceeds the page table width");
  if (pos_index_type != FP_INDEX_I32 && pos_index_type != FP_INDEX_I64)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: bad pos_index_type");
  if (B > 65535 || Hc > 65535 || Hq > 65535)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: B, Hq or Hc exceeds 65535");
  if (B == 0) return FP_OK;
  if (!page_table || !batch_idx || !input_pos) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: null pointer");
  if (plan_only) {
    if (!plan) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_plan: null plan");
  } else {
    if (!q || !pool_k || !pool_v || !out || !lse) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: null pointer");
    if (!fp::aligned(q, 16) || !fp::aligned(pool_k, 16) || !fp::aligned(pool_v, 16) ||
        (q_stride_b * eb) % 16 || (q_stride_h * eb) % 16)
      return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: q and pool rows must be 16-byte aligned");
    if (!fp::aligned(out, eb)) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: out misaligned");
  }
  if (plan && (!fp::aligned(plan, 4) || plan_bytes < plan_buffer_bytes()))
    return fp::fail(FP_ERR_WORKSPACE, "fp_paged_decode: the plan buffer needs %lld bytes (fp_paged_decode_plan_bytes), %lld given",
                    static_cast<long long>(plan_buffer_bytes()), static_cast<long long>(plan_bytes));

  if (split_tokens == 0) split_tokens = default_split_tokens(B, wg_heads, max_context, page_size);
  if (split_tokens % 64) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode: split_tokens must be a multiple of 64");
  if (split_tokens / page_size + 2 > kMaxSplitPages)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: split of %d tokens spans more than %d pages", split_tokens,
                    kMaxSplitPages - 2);
  const int ns = n_splits_for(max_context, split_tokens);
  if (ns > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_decode: more than 65535 splits");

  DecodeArgs a{static_cast<const char*>(q), q_stride_b * eb, q_stride_h * eb,
               static_cast<const char*>(pool_k), static_cast<const char*>(pool_v),
               page_table, pt_row_stride, batch_idx, input_pos, pos_index_type == FP_INDEX_I64,
               static_cast<char*>(out), out_stride_b * eb, out_stride_h * eb, lse, sinks,
               nullptr, nullptr, Hq, wg_heads, fp::PageDiv(page_size), n_pages, max_batch, n_slots,
               max_context, split_tokens, ns, scale * kLog2e,  // scores are kept in log2 units
               nullptr, nullptr, 0, 0, 0, 0, B, 0, static_cast<int*>(plan)};
  if (fresh) {
    if (!fresh->k || !fresh->v) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_append: null k_new / v_new");
    if (!fp::aligned(fresh->k, 16) || !fp::aligned(fresh->v, 16) || (fresh->k_stride_b * eb) % 16 ||
        (fresh->k_stride_h * eb) % 16 || (fresh->v_stride_b * eb) % 16 || (fresh->v_stride_h * eb) % 16)
      return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_append: k_new / v_new rows must be 16-byte aligned");
    a.k_new = static_cast<const char*>(fresh->k);
    a.v_new = static_cast<const char*>(fresh->v);
    a.kn_b = fresh->k_stride_b * eb;
    a.kn_h = fresh->k_stride_h * eb;
    a.vn_b = fresh->v_stride_b * eb;
    a.vn_h = fresh->v_stride_h * eb;
  }
  if (ns > 1 && !plan_only) {
    const int64_t need = static_cast<int64_t>(B) * Hq * ns * (D + 2) * static_cast<int64_t>(sizeof(float));
    if (!workspace || workspace_bytes < need || !fp::aligned(workspace, 16))
      return fp::fail(FP_ERR_WORKSPACE, "fp_paged_decode: workspace of %lld bytes needed, %lld given",
                      static_cast<long long>(need), static_cast<long long>(workspace_bytes));
    a.ws_acc = static_cast<float*>(workspace);
    a.ws_ml = a.ws_acc + static_cast<int64_t>(B) * Hq * ns * D;
  }

  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
  switch (dtype) {
    case FP_DTYPE_F32: rc = dispatch_dim<F32>(a, B, D, phases, kv_rep, st); break;
    case FP_DTYPE_BF16: rc = dispatch_dim<BF16>(a, B, D, phases, kv_rep, st); break;
    default: rc = dispatch_dim<F16>(a, B, D, phases, kv_rep, st); break;
  }
  if (rc != FP_OK) return rc;
  return fp::check_launch("fp_paged_decode");
}

}  // namespace

#define FP_DECODE_PARAMS                                                                                   \
  const void *q, int64_t q_stride_b, int64_t q_stride_h, const void *pool_k, const void *pool_v,          \
      const int64_t *page_table, int64_t pt_row_stride, const int64_t *batch_idx, const void *input_pos,  \
      int pos_index_type, void *out, int64_t out_stride_b, int64_t out_stride_h, float *lse,              \
      const float *sinks,                                                                                 \
      void *workspace, int64_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep,        \
      int32_t D,                                                                                          \
      int32_t page_size, int32_t n_pages, int32_t max_batch, int64_t n_slots, int32_t max_context,        \
      int32_t split_tokens, float scale, int dtype, void *plan, int64_t plan_bytes, void *stream
#define FP_DECODE_ARGS                                                                                     \
  q, q_stride_b, q_stride_h, pool_k, pool_v, page_table, pt_row_stride, batch_idx, input_pos,             \
      pos_index_type, out, out_stride_b, out_stride_h, lse, sinks, workspace, workspace_bytes, B, Hq, Hc, kv_rep, D, \
      page_size, n_pages, max_batch, n_slots, max_context, split_tokens, scale, dtype, plan, plan_bytes, stream

extern "C" int64_t fp_paged_decode_plan_bytes(void) { return plan_buffer_bytes(); }
extern "C" int fp_paged_decode_plan(FP_DECODE_PARAMS) { return decode_entry(kPhasePlan, nullptr, FP_DECODE_ARGS); }
extern "C" int fp_paged_decode(FP_DECODE_PARAMS) {
  return decode_entry(kPhasePartial | kPhaseMerge, nullptr, FP_DECODE_ARGS);
}
extern "C" int fp_paged_decode_partial(FP_DECODE_PARAMS) { return decode_entry(kPhasePartial, nullptr, FP_DECODE_ARGS); }
extern "C" int fp_paged_decode_merge(FP_DECODE_PARAMS) { return decode_entry(kPhaseMerge, nullptr, FP_DECODE_ARGS); }
extern "C" int fp_paged_decode_append(const void* k_new, const void* v_new, int64_t k_stride_b, int64_t k_stride_h,
                                      int64_t v_stride_b, int64_t v_stride_h, FP_DECODE_PARAMS) {
  const NewRows fresh{k_new, v_new, k_stride_b, k_stride_h, v_stride_b, v_stride_h};
  return decode_entry(kPhasePartial | kPhaseMerge, &fresh, FP_DECODE_ARGS);
}


// ---------------------------------------------------------------------------------------------
// fp_paged_decode for callers that cannot allocate: the split-K partial results go to an array that
// lives in the library's device image instead of a caller-owned workspace.
//
// `scratch` below is, in host code, only a handle of the device symbol: its device address differs
// per GPU and is asked for once per device with hipGetSymbolAddress, on the entry point's first call
// on that device (with that device current).  Only that address is ever handed to a kernel.  Every
// launch on a GPU shares the GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race on it.  The partial pass writes every row the merge pass reads, so the contents left
// by an earlier call never need clearing.
constexpr int64_t kScratchBytes = FP_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device, nullptr + error message on failure
void* scratch_address() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fp::fail(FP_ERR_LAUNCH, "fp_paged_decode_noalloc: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    (void)hipGetLastError();
    fp::fail(FP_ERR_LAUNCH, "fp_paged_decode_noalloc: hipGetSymbolAddress(scratch) on device %d: %s", dev,
             hipGetErrorString(e));
    return nullptr;
  }
  g_scratch_ptr[dev].store(p, std::memory_order_release);  // two first calls racing store the same address
  return p;
}
}  // namespace

extern "C" int fp_paged_decode_noalloc(const void* q, int64_t q_stride_b, int64_t q_stride_h, const void* pool_k,
                                       const void* pool_v, const int64_t* page_table, int64_t pt_row_stride,
                                       const int64_t* batch_idx, const void* input_pos, int pos_index_type,
                                       void* out, int64_t out_stride_b, int64_t out_stride_h, float* lse,
                                       const float* sinks, int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep,
                                       int32_t D, int32_t page_size, int32_t n_pages, int32_t max_batch,
                                       int64_t n_slots, int32_t max_context, int32_t split_tokens, float scale,
                                       int dtype, void* stream) {
  // size the partial results exactly as decode_entry will, and refuse what the array cannot hold
  if (B < 0 || Hq <= 0 || Hc <= 0 || D <= 0 || page_size <= 0 || max_context < 0 || split_tokens < 0 || kv_rep < 1)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_noalloc: bad dimension");
  int st = split_tokens;
  if (st == 0) st = default_split_tokens(B, kv_rep > 1 ? Hq / kv_rep : Hc, max_context, page_size);
  if (st % 64) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_decode_noalloc: split_tokens must be a multiple of 64");
  const int64_t ns = n_splits_for(max_context, st);
  const int64_t need = ns > 1 ? static_cast<int64_t>(B) * Hq * ns * (D + 2) * static_cast<int64_t>(sizeof(float)) : 0;
  if (need > kScratchBytes)
    return fp::fail(FP_ERR_WORKSPACE,
                    "fp_paged_decode_noalloc: this launch needs %lld bytes of split-K partial results, the library's "
                    "array holds %lld; use fp_paged_decode with a caller-owned workspace, or a larger split_tokens",
                    static_cast<long long>(need), static_cast<long long>(kScratchBytes));
  void* ws = nullptr;
  if (need) {
    ws = scratch_address();
    if (!ws) return FP_ERR_LAUNCH;
  }
  return decode_entry(kPhasePartial | kPhaseMerge, nullptr, q, q_stride_b, q_stride_h, pool_k, pool_v, page_table,
                      pt_row_stride, batch_idx, input_pos, pos_index_type, out, out_stride_b, out_stride_h, lse, sinks,
                      ws, need ? kScratchBytes : 0, B, Hq, Hc, kv_rep, D, page_size, n_pages, max_batch, n_slots,
                      max_context, st, scale, dtype, nullptr, 0, stream);
}
