// QK RMS-norm + 3D rotary embedding + KV append in one pass.
//
// Restates the tail of Attention._pre_attention (reference model.py:110-119) together with
// the cache insert that follows it (model.py:150-153 -> paged_attention.py:184-232, 364-393):
//   xq = rms_norm(xq), xk = rms_norm(xk) over head_dim, no weight          (model.py:110-111)
//   xk, xv repeated n_rep times along the head axis                        (model.py:112-113, :74-83)
//   first half of head_dim: 1D rotary, complex pairs (2i, 2i+1) times freqs_cis[t, i]
//                                                                           (rope.py:31-46, :88-97)
//   second half: "golden" 2D rotary with per-head freqs_cis_2d[t, h, f]    (rope.py:71-86, :98-100),
//                left as it is when freqs_cis_2d is absent
//   q to [.., H, .., D] layout, K and V rows to pool[h, slot(batch_idx, pos), :]
// Rounding follows the reference: the norm result is rounded to the model dtype (rms_norm
// returns that dtype), the rotation is computed in fp32 from the rounded value (xq.float())
// and rounded again (type_as).
//
// HBM / launch bound.  A group of D * elem / 16 lanes holds a row in one 16-byte vector per lane.  For the
// model's shapes (Hq / Hkv in {1, 2, 4, 8}, head_dim 64 or 128) a group owns one (token, kv head): the query
// rows of the kv head, its K row and its V row, so that the per-head angles are fetched once for the query
// row and the K replica that share them (32768 tokens, 16 q / 8 kv heads: 134 us against 154 us row by
// row, where the angle table was fetched twice); the groups run over the source in its memory order.  Other
// shapes go row by row: one group per source row (token, head), token-fastest inside a head.  A K row is
// normalised once and rotated once per replica (the 2D angles differ per head), a V row is stored n_rep times.
#include "fp_common.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

namespace {

typedef uint32_t v4u __attribute__((ext_vector_type(4)));

struct RopeArgs {
  const char* xq;
  const char* xk;
  const char* xv;
  int64_t qs_t, qs_h, ks_t, ks_h, vs_t, vs_h;  // bytes
  const float* freqs;     // [T, D/4, 2] cos, sin
  const float* freqs_2d;  // [T, Hq, D/4, 2] or null
  char* q_out;
  int64_t qo_t, qo_h;  // bytes
  char* pool_k;
  char* pool_v;
  const int64_t* page_table;
  int64_t pt_row_stride;
  const int64_t* batch_idx;
  const void* input_pos;
  int pos_i64;
  int T, Hq, Hkv, n_rep;
  fp::PageDiv pd;
  int n_pages, max_batch;
  int64_t n_slots;
  float eps;
  int clamp_negative;
  int order;  // groups of the (token, kv head) kernel: 1 = kv heads of a token fastest, 0 = tokens of a kv head fastest
};

struct F32 {
  static constexpr int kEpv = 4;
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r[i]);
  }
  static __device__ __forceinline__ v4u pack(const float* f) {
    return v4u{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
  }
  static __device__ __forceinline__ float round(float v) { return v; }
};
struct BF16 {
  static constexpr int kEpv = 8;
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = r[i];
      f[2 * i] = __uint_as_float(w << 16);
      f[2 * i + 1] = __uint_as_float(w & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint32_t bits(float v) {
    return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, __float2bfloat16(v)));
  }
  static __device__ __forceinline__ v4u pack(const float* f) {
    v4u r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = bits(f[2 * i]) | (bits(f[2 * i + 1]) << 16);
    return r;
  }
  static __device__ __forceinline__ float round(float v) { return __bfloat162float(__float2bfloat16(v)); }
};
struct F16 {
  static constexpr int kEpv = 8;
  static __device__ __forceinline__ void unpack(const v4u& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w = r[i];
      f[2 * i] = __half2float(__builtin_bit_cast(__half, static_cast<unsigned short>(w & 0xffffu)));
      f[2 * i + 1] = __half2float(__builtin_bit_cast(__half, static_cast<unsigned short>(w >> 16)));
    }
  }
  static __device__ __forceinline__ uint32_t bits(float v) {
    return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, __float2half(v)));
  }
  static __device__ __forceinline__ v4u pack(const float* f) {
    v4u r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = bits(f[2 * i]) | (bits(f[2 * i + 1]) << 16);
    return r;
  }
  static __device__ __forceinline__ float round(float v) { return __half2float(__float2half(v)); }
};

constexpr int kThreads = 256;

// TPR = lanes per row (a power of two between 1 and 64)
template <typename E, int TPR>
__global__ __launch_bounds__(kThreads) void qkv_rope_append_kernel(const RopeArgs a) {
  constexpr int EPV = E::kEpv;
  constexpr int D = TPR * EPV;
  constexpr int kRowBytes = TPR * 16;
  constexpr int kRows = kThreads / TPR;
  const int sub = threadIdx.x % TPR;  // this lane's 16-byte vector inside the row
  const int64_t rid = static_cast<int64_t>(blockIdx.x) * kRows + threadIdx.x / TPR;
  const int n_src = a.Hq + 2 * a.Hkv;
  // source rows: head-major, tokens fastest inside a head
  const int j = static_cast<int>(rid / a.T);  // source head: q heads, then k heads, then v heads
  const int t = static_cast<int>(rid - static_cast<int64_t>(j) * a.T);
  const bool live = j < n_src;  // lanes of one row agree; dead rows still take part in the shuffles
  const int kind = !live ? 3 : j < a.Hq ? 0 : j < a.Hq + a.Hkv ? 1 : 2;
  const int hsrc = kind == 0 ? j : kind == 1 ? j - a.Hq : j - a.Hq - a.Hkv;

  float x[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) x[e] = 0.f;
  if (live) {
    const char* src = kind == 0   ? a.xq + t * a.qs_t + hsrc * a.qs_h
                      : kind == 1 ? a.xk + t * a.ks_t + hsrc * a.ks_h
                                  : a.xv + t * a.vs_t + hsrc * a.vs_h;
    E::unpack(__builtin_nontemporal_load(reinterpret_cast<const v4u*>(src + sub * 16)), x);
  }

  // pool slot of this token (K and V rows)
  int64_t slot = -1;
  if (kind == 1 || kind == 2) {
    const int64_t b = a.batch_idx[t];
    const int64_t pos = fp::load_index(a.input_pos, t, a.pos_i64);
    if (b >= 0 && b < a.max_batch && pos >= 0) {
      int64_t blk;
      int off;
      a.pd.split(pos, blk, off);
      if (blk < a.n_pages) {
        int64_t page = a.page_table[b * a.pt_row_stride + blk];
        if (a.clamp_negative && page < 0) page = 0;
        slot = page * a.pd.page_size + off;
        if (slot < 0) slot += a.n_slots;  // negative index counts from the end of the slot axis
        if (slot >= a.n_slots) slot = -1;
      }
    }
  }

  if (kind == 2) {  // V: plain copies to the n_rep heads of its group
    if (slot >= 0) {
      const v4u raw = E::pack(x);
      for (int r = 0; r < a.n_rep; ++r) {
        const int64_t h = static_cast<int64_t>(hsrc) * a.n_rep + r;
        __builtin_nontemporal_store(raw, reinterpret_cast<v4u*>(a.pool_v + (h * a.n_slots + slot) * kRowBytes + sub * 16));
      }
    }
  }

  // RMS norm over the row: x * rsqrt(mean(x^2) + eps), rounded to the dtype
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPV; ++e) ss += x[e] * x[e];
#pragma unroll
  for (int off = TPR / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
  if (kind >= 2) return;
  const float rstd = rsqrtf(ss / D + a.eps);
#pragma unroll
  for (int e = 0; e < EPV; ++e) x[e] = E::round(x[e] * rstd);

  // rotation: this lane's elements lie in one half of the row
  const int e0 = sub * EPV;
  const bool second = e0 >= D / 2;
  const int f0 = (second ? e0 - D / 2 : e0) / 2;  // first complex pair of this lane inside its half
  const float* f1d = a.freqs + (static_cast<int64_t>(t) * (D / 4) + f0) * 2;
  const int reps = kind == 1 ? a.n_rep : 1;
  for (int r = 0; r < reps; ++r) {
    const int h = kind == 1 ? hsrc * a.n_rep + r : hsrc;  // head of the output row
    float y[EPV];
    if (second && a.freqs_2d == nullptr) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) y[e] = x[e];
    } else {
      // with 2D angles the head index of freqs_2d is the query head; K replicas use their own head
      const float* cs = second ? a.freqs_2d + ((static_cast<int64_t>(t) * a.Hq + h) * (D / 4) + f0) * 2 : f1d;
#pragma unroll
      for (int p = 0; p < EPV / 2; ++p) {
        const float c = cs[2 * p], s = cs[2 * p + 1];
        const float re = x[2 * p], im = x[2 * p + 1];
        y[2 * p] = E::round(re * c - im * s);
        y[2 * p + 1] = E::round(re * s + im * c);
      }
    }
    const v4u raw = E::pack(y);
    if (kind == 0) {
      *reinterpret_cast<v4u*>(a.q_out + t * a.qo_t + h * a.qo_h + sub * 16) = raw;
    } else if (slot >= 0) {
      __builtin_nontemporal_store(raw, reinterpret_cast<v4u*>(a.pool_k + (static_cast<int64_t>(h) * a.n_slots + slot) * kRowBytes + sub * 16));
    }
  }
}

// The same work, one group of TPR lanes per (token, kv head): the NQ = Hq / Hkv query rows of the group,
// its K row and its V row.  With per-head 2D angles, the K replica of head h and the query row of head h
// rotate by the same angles, so a group fetches every angle row ONCE (the row-per-group kernel above reads
// the [T, Hq, D/4] table twice, 134 MB of 814 MB at 32768 tokens x 16 heads, because query rows and K rows
// of a head are handled by workgroups far apart in time).  Groups run over the source in its memory order
// (a.order): for the projection output [T, heads, D] the kv heads of a token run fastest, so a workgroup reads
// whole 8 KiB token rows.  Tokens fastest inside a kv head measured 129 us or 141 us at 32768 tokens depending
// on where the allocator had placed the buffers, kv heads fastest 134 us either way.
template <typename E, int TPR, int NQ>
__global__ __launch_bounds__(kThreads) void qkv_rope_group_kernel(const RopeArgs a) {
  constexpr int EPV = E::kEpv;
  constexpr int D = TPR * EPV;
  constexpr int kRowBytes = TPR * 16;
  constexpr int kRows = kThreads / TPR;
  const int sub = threadIdx.x % TPR;  // this lane's 16-byte vector inside a row
  const int64_t uid = static_cast<int64_t>(blockIdx.x) * kRows + threadIdx.x / TPR;
  const int g = a.order ? static_cast<int>(uid % a.Hkv) : static_cast<int>(uid / a.T);  // kv head
  const int t = a.order ? static_cast<int>(uid / a.Hkv) : static_cast<int>(uid - static_cast<int64_t>(g) * a.T);
  const bool live = a.order ? t < a.T : g < a.Hkv;  // lanes of one group agree; dead groups still take part in the shuffles

  // every load of the group is requested before the first use
  v4u rq[NQ];
  v4u rk = v4u{0, 0, 0, 0}, rv = v4u{0, 0, 0, 0};
#pragma unroll
  for (int r = 0; r < NQ; ++r) rq[r] = v4u{0, 0, 0, 0};
  const int e0 = sub * EPV;
  const bool second = e0 >= D / 2;  // this lane's elements lie in one half of the row
  const int f0 = (second ? e0 - D / 2 : e0) / 2;  // first complex pair of this lane inside its half
  const bool rot2d = second && a.freqs_2d != nullptr;
  const bool identity = second && a.freqs_2d == nullptr;
  float ang[NQ][EPV];  // (cos, sin) of this lane's pairs: row 0 alone unless the angles are per head
  if (live) {
#pragma unroll
    for (int r = 0; r < NQ; ++r)
      rq[r] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(a.xq + t * a.qs_t + (g * NQ + r) * a.qs_h + sub * 16));
    rk = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(a.xk + t * a.ks_t + g * a.ks_h + sub * 16));
    rv = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(a.xv + t * a.vs_t + g * a.vs_h + sub * 16));
    if (rot2d) {
#pragma unroll
      for (int r = 0; r < NQ; ++r) {
        const float* cs = a.freqs_2d + ((static_cast<int64_t>(t) * a.Hq + g * NQ + r) * (D / 4) + f0) * 2;
#pragma unroll
        for (int e = 0; e < EPV; ++e) ang[r][e] = __builtin_nontemporal_load(cs + e);
      }
    } else if (!identity) {
      const float* cs = a.freqs + (static_cast<int64_t>(t) * (D / 4) + f0) * 2;
#pragma unroll
      for (int e = 0; e < EPV; ++e) ang[0][e] = cs[e];
    }
  }

  // pool slot of this token
  int64_t slot = -1;
  if (live) {
    const int64_t b = a.batch_idx[t];
    const int64_t pos = fp::load_index(a.input_pos, t, a.pos_i64);
    if (b >= 0 && b < a.max_batch && pos >= 0) {
      int64_t blk;
      int off;
      a.pd.split(pos, blk, off);
      if (blk < a.n_pages) {
        int64_t page = a.page_table[b * a.pt_row_stride + blk];
        if (a.clamp_negative && page < 0) page = 0;
        slot = page * a.pd.page_size + off;
        if (slot < 0) slot += a.n_slots;  // negative index counts from the end of the slot axis
        if (slot >= a.n_slots) slot = -1;
      }
    }
  }

  // V: plain copies to the n_rep cached heads of the group
  if (slot >= 0) {
    for (int r = 0; r < a.n_rep; ++r) {
      const int64_t h = static_cast<int64_t>(g) * a.n_rep + r;
      __builtin_nontemporal_store(rv, reinterpret_cast<v4u*>(a.pool_v + (h * a.n_slots + slot) * kRowBytes + sub * 16));
    }
  }

  // RMS norm over a row, x * rsqrt(mean(x^2) + eps) rounded to the dtype
  auto normed = [&](const v4u& raw, float* x) {
    E::unpack(raw, x);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPV; ++e) ss += x[e] * x[e];
#pragma unroll
    for (int off = TPR / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
    const float rstd = rsqrtf(ss / D + a.eps);
#pragma unroll
    for (int e = 0; e < EPV; ++e) x[e] = E::round(x[e] * rstd);
  };
  // rotation of this lane's pairs by one row of angles (fp32 from the rounded value, rounded again)
  auto rotated = [&](const float* x, const float* cs) -> v4u {
    float y[EPV];
    if (identity) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) y[e] = x[e];
    } else {
#pragma unroll
      for (int p = 0; p < EPV / 2; ++p) {
        const float c = cs[2 * p], sn = cs[2 * p + 1];
        const float re = x[2 * p], im = x[2 * p + 1];
        y[2 * p] = E::round(re * c - im * sn);
        y[2 * p + 1] = E::round(re * sn + im * c);
      }
    }
    return E::pack(y);
  };

  float x[EPV];
  normed(rk, x);
  if (a.freqs_2d != nullptr) {  // one rotation per replica: n_rep == NQ, replica r is cached head g * NQ + r
#pragma unroll
    for (int r = 0; r < NQ; ++r) {
      const v4u raw = rotated(x, second ? ang[r] : ang[0]);
      if (slot >= 0)
        __builtin_nontemporal_store(raw, reinterpret_cast<v4u*>(a.pool_k + ((static_cast<int64_t>(g) * NQ + r) * a.n_slots + slot) * kRowBytes + sub * 16));
    }
  } else {
    const v4u raw = rotated(x, ang[0]);
    if (slot >= 0) {
      for (int r = 0; r < a.n_rep; ++r) {
        const int64_t h = static_cast<int64_t>(g) * a.n_rep + r;
        __builtin_nontemporal_store(raw, reinterpret_cast<v4u*>(a.pool_k + (h * a.n_slots + slot) * kRowBytes + sub * 16));
      }
    }
  }
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
    normed(rq[r], x);
    const v4u raw = rotated(x, rot2d ? ang[r] : ang[0]);
    if (live) *reinterpret_cast<v4u*>(a.q_out + t * a.qo_t + (g * NQ + r) * a.qo_h + sub * 16) = raw;
  }
}

template <typename E, int TPR>
bool launch_groups(const RopeArgs& a, hipStream_t st) {
  const int64_t units = static_cast<int64_t>(a.T) * a.Hkv;
  const int per_block = kThreads / TPR;
  const dim3 grid(static_cast<unsigned>((units + per_block - 1) / per_block));
  switch (a.Hq / a.Hkv) {
    case 1: hipLaunchKernelGGL((qkv_rope_group_kernel<E, TPR, 1>), grid, dim3(kThreads), 0, st, a); return true;
    case 2: hipLaunchKernelGGL((qkv_rope_group_kernel<E, TPR, 2>), grid, dim3(kThreads), 0, st, a); return true;
    case 4: hipLaunchKernelGGL((qkv_rope_group_kernel<E, TPR, 4>), grid, dim3(kThreads), 0, st, a); return true;
    case 8: hipLaunchKernelGGL((qkv_rope_group_kernel<E, TPR, 8>), grid, dim3(kThreads), 0, st, a); return true;
    default: return false;
  }
}

template <typename E>
int launch(const RopeArgs& a, int D, hipStream_t st) {
  const int tpr = D / E::kEpv;
  // the model's shapes (query heads a power-of-two multiple of the kv heads, head_dim 64 or 128) go by groups
  if (a.Hq % a.Hkv == 0) {
    if (tpr == 8 && launch_groups<E, 8>(a, st)) return FP_OK;
    if (tpr == 16 && launch_groups<E, 16>(a, st)) return FP_OK;
    if (tpr == 32 && launch_groups<E, 32>(a, st)) return FP_OK;
  }
  const int64_t rows = static_cast<int64_t>(a.T) * (a.Hq + 2 * a.Hkv);
  const int per_block = kThreads / tpr;
  const dim3 grid(static_cast<unsigned>((rows + per_block - 1) / per_block));
  switch (tpr) {
    case 4: hipLaunchKernelGGL((qkv_rope_append_kernel<E, 4>), grid, dim3(kThreads), 0, st, a); return FP_OK;
    case 8: hipLaunchKernelGGL((qkv_rope_append_kernel<E, 8>), grid, dim3(kThreads), 0, st, a); return FP_OK;
    case 16: hipLaunchKernelGGL((qkv_rope_append_kernel<E, 16>), grid, dim3(kThreads), 0, st, a); return FP_OK;
    case 32: hipLaunchKernelGGL((qkv_rope_append_kernel<E, 32>), grid, dim3(kThreads), 0, st, a); return FP_OK;
    case 64: hipLaunchKernelGGL((qkv_rope_append_kernel<E, 64>), grid, dim3(kThreads), 0, st, a); return FP_OK;
    default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_qkv_norm_rope_append: head_dim %d", D);
  }
}

}  // namespace

extern "C" int fp_qkv_norm_rope_append(const void* xq, const void* xk, const void* xv,
                                       int64_t q_stride_t, int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_h,
                                       int64_t v_stride_t, int64_t v_stride_h, const float* freqs_cis,
                                       const float* freqs_cis_2d, void* q_out, int64_t qo_stride_t,
                                       int64_t qo_stride_h, void* pool_k, void* pool_v, const int64_t* page_table,
                                       int64_t pt_row_stride, const int64_t* batch_idx, const void* input_pos,
                                       int pos_index_type, int32_t T, int32_t Hq, int32_t Hkv, int32_t H_pool,
                                       int32_t D, int32_t page_size, int32_t n_pages, int32_t max_batch,
                                       int64_t n_slots, float eps, int dtype, int clamp_negative, void* stream) {
  const int eb = fp::elem_bytes(dtype);
  if (eb == 0) return fp::fail(FP_ERR_UNSUPPORTED, "fp_qkv_norm_rope_append: unknown dtype %d", dtype);
  if (T < 0 || Hq <= 0 || Hkv <= 0 || H_pool <= 0 || D <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 ||
      n_slots <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: non-positive dimension");
  if (H_pool % Hkv) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: pool heads %d not a multiple of Hkv=%d", H_pool, Hkv);
  if (freqs_cis_2d && H_pool != Hq)
    return fp::fail(FP_ERR_INVALID_ARGUMENT,
                    "fp_qkv_norm_rope_append: per-head 2D angles need one cached K head per query head (pool %d, Hq %d)",
                    H_pool, Hq);
  const int epv = 16 / eb;
  const int tpr = D / epv;
  if (D % (2 * epv) || (tpr & (tpr - 1)) || tpr > 64)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_qkv_norm_rope_append: head_dim %d for %d-byte elements", D, eb);
  if (n_slots < page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: n_slots smaller than one page");
  if (pos_index_type != FP_INDEX_I32 && pos_index_type != FP_INDEX_I64)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: bad pos_index_type");
  if (T == 0) return FP_OK;
  if (!xq || !xk || !xv || !freqs_cis || !q_out || !pool_k || !pool_v || !page_table || !batch_idx || !input_pos)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: null pointer");
  const int64_t strides[] = {q_stride_t, q_stride_h, k_stride_t, k_stride_h, v_stride_t, v_stride_h, qo_stride_t, qo_stride_h};
  for (int64_t s : strides)
    if ((s * eb) % 16) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: rows must be 16-byte aligned");
  if (!fp::aligned(xq, 16) || !fp::aligned(xk, 16) || !fp::aligned(xv, 16) || !fp::aligned(q_out, 16) ||
      !fp::aligned(pool_k, 16) || !fp::aligned(pool_v, 16) || !fp::aligned(freqs_cis, 8) ||
      (freqs_cis_2d && !fp::aligned(freqs_cis_2d, 8)))
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_qkv_norm_rope_append: rows must be 16-byte aligned");
  // a dispatch holds fewer than 2^32 lanes
  if ((static_cast<int64_t>(T) * (Hq + 2 * Hkv) + kThreads) * tpr >= (1ll << 32))
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_qkv_norm_rope_append: too many rows for one launch (%lld lanes)",
                    static_cast<long long>(T) * (Hq + 2 * Hkv) * tpr);

  RopeArgs a{static_cast<const char*>(xq), static_cast<const char*>(xk), static_cast<const char*>(xv),
             q_stride_t * eb, q_stride_h * eb, k_stride_t * eb, k_stride_h * eb, v_stride_t * eb, v_stride_h * eb,
             freqs_cis, freqs_cis_2d, static_cast<char*>(q_out), qo_stride_t * eb, qo_stride_h * eb,
             static_cast<char*>(pool_k), static_cast<char*>(pool_v), page_table, pt_row_stride, batch_idx, input_pos,
             pos_index_type == FP_INDEX_I64, T, Hq, Hkv, H_pool / Hkv, fp::PageDiv(page_size), n_pages, max_batch,
             n_slots, eps, clamp_negative,
             // the groups run over the source in its memory order: the kv heads of a token next to each other for the
             // [T, heads, D] projection output
             (q_stride_h <= q_stride_t && k_stride_h <= k_stride_t && v_stride_h <= v_stride_t) ? 1 : 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
  if (dtype == FP_DTYPE_F32) rc = launch<F32>(a, D, st);
  else if (dtype == FP_DTYPE_BF16) rc = launch<BF16>(a, D, st);
  else rc = launch<F16>(a, D, st);
  if (rc != FP_OK) return rc;
  return fp::check_launch("fp_qkv_norm_rope_append");
}
