// Chunked-prefill attention over the paged cache under the hybrid mask (bf16 / f16 MFMA).
//
// Replaces the reference's compiled_flex_attn_prefill call (attention.py:18,
// model.py:156-162) and extends it to read the prefix from pages: the reference
// attends over the packed fresh K/V only (paged_attention.py:393), here every key
// of a row's sequence, prefix and chunk alike, is fetched through the page table.
// The hybrid mask (attention.py:75-96 OR document-causal, paged_attention.py:353-359)
// arrives as one number per query row: keys 0..row_limit-1 of the row's own
// sequence are visible.
//
// MFMA-bound.  A workgroup of 4 wavefronts owns kRowBlocks * 128 consecutive packed
// query rows of one query head; a wavefront owns kRowBlocks blocks of 32 rows.
//   S^T = K Q^T  (v_mfma_f32_32x32x16): keys are the M rows, queries the N columns, so a
//         lane holds scores of ONE query and softmax row reductions stay in registers
//         (plus one exchange between the two lane halves).
//   O^T = V^T P^T: P^T is already in B-operand layout in the S^T accumulators; V^T
//         comes out of LDS through ds_read_b64_tr_b16, so V is staged row-major like K.
//   K/V tiles of 64 keys are fetched page by page with 16-byte loads one tile ahead
//   (registers), page ids two tiles ahead, and double-buffered in LDS.
// Rows of one 128-row tile may belong to several sequences: the tile is processed one
// run of equal batch_idx at a time; rows of slot 0 are padding (out 0, lse -inf).
#include "fp_common.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <math.h>

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kTileN = 64;  // keys per tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

struct PrefillArgs {
  const char* q;
  int64_t qs_row, qs_h;  // bytes
  const char* pool_k;
  const char* pool_v;
  const int64_t* page_table;
  int64_t pt_row_stride;
  const int64_t* batch_idx;
  const int32_t* row_limit;
  char* out;
  int64_t os_row, os_h;  // bytes
  float* lse;            // [Hq, Lq]
  int Lq, Hq, Hc;
  fp::PageDiv pd;
  int n_pages, max_batch;
  int64_t n_slots;
  float qscale;  // scale * log2(e)
  int n_tiles;   // query tiles
};

struct BF16 {
  using vec8 = bf16x8;
  static __device__ __forceinline__ f32x16 mfma(const s16x8& a, const s16x8& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ short from_float(float x) {
    return __builtin_bit_cast(short, static_cast<__bf16>(x));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};
struct F16 {
  using vec8 = f16x8;
  static __device__ __forceinline__ f32x16 mfma(const s16x8& a, const s16x8& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ short from_float(float x) {
    return __builtin_bit_cast(short, static_cast<_Float16>(x));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
  }
};

constexpr f32x16 kZero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// LDS transpose read: the 16 lanes of a block each name 4 consecutive 16-bit elements;
// lane i receives, for j = 0..3, element (i % 4) of the chunk named by lane 4 * j + i / 4.
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p));
}

template <typename E, int D, int MB, bool kPow2>
__global__ __launch_bounds__(kThreads, 2) void paged_prefill_kernel(const PrefillArgs a) {
  constexpr int BM = kWaves * 32 * MB;     // query rows per workgroup
  constexpr int RS = D * 2 + 16;           // LDS row stride in bytes (16-byte pad: no bank conflicts)
  constexpr int CPR = D * 2 / 16;          // 16-byte chunks per K/V row
  constexpr int NI = kTileN * CPR / kThreads;  // chunks per thread per tile and tensor
  constexpr int DS = D / 16;               // MFMA k-steps over head_dim
  constexpr int DB = D / 32;               // 32-wide blocks of head_dim in O^T
  constexpr int TILE_BYTES = kTileN * RS;

  __shared__ __attribute__((aligned(16))) char s_k[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_v[2][TILE_BYTES];
  __shared__ int s_bidx[BM];
  __shared__ int s_red[kWaves];

  // linear id = cache head + Hc * (head in group + G * tile): all query heads and tiles that
  // read one cache head run on the XCD that already holds its K/V in L2
  const int G = a.Hq / a.Hc;
  const int hc = blockIdx.x;
  const int g = blockIdx.y % G;
  const int tile = a.n_tiles - 1 - blockIdx.y / G;  // longest key ranges first
  const int hq = hc * G + g;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int half = lane >> 5;   // which 8 of 16 k-values / which 4 of 8 rows this lane holds
  const int ln = lane & 31;     // query column (S^T, O^T) or key row (K operand)
  const int tile0 = tile * BM;

  for (int i = tid; i < BM; i += kThreads) {
    const int r = tile0 + i;
    int64_t bi = r < a.Lq ? a.batch_idx[r] : 0;
    if (bi < 0 || bi >= a.max_batch) bi = 0;
    s_bidx[i] = static_cast<int>(bi);
  }
  __syncthreads();

  const char* kplane = a.pool_k + static_cast<int64_t>(hc) * a.n_slots * (D * 2);
  const char* vplane = a.pool_v + static_cast<int64_t>(hc) * a.n_slots * (D * 2);

  int run0 = 0;
  while (run0 < BM) {
    // values every lane agrees on are moved to scalar registers so the control flow that
    // depends on them stays uniform
    const int sq = __builtin_amdgcn_readfirstlane(s_bidx[run0]);
    int run1 = run0 + 1;
    while (run1 < BM && __builtin_amdgcn_readfirstlane(s_bidx[run1]) == sq) ++run1;

    // rows of this wavefront: block mb covers tile rows wave*32*MB + mb*32 + ln
    int row[MB], lim[MB];
    bool active[MB];
    int my_max = 0;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int tr = wave * 32 * MB + mb * 32 + ln;
      row[mb] = tile0 + tr;
      active[mb] = tr >= run0 && tr < run1 && row[mb] < a.Lq;
      lim[mb] = (active[mb] && sq != 0) ? a.row_limit[row[mb]] : 0;
      if (lim[mb] < 0) lim[mb] = 0;
      my_max = max(my_max, lim[mb]);
    }

    if (sq == 0) {
      // padding rows: out = 0, lse = -inf
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (!active[mb]) continue;
        // a row is 2 * D bytes; each lane half clears D of them
        char* o = a.out + row[mb] * a.os_row + hq * a.os_h + half * D;
#pragma unroll
        for (int c = 0; c < D / 8; ++c) *reinterpret_cast<uint2*>(o + c * 8) = uint2{0, 0};
        if (half == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row[mb]] = -INFINITY;
      }
      run0 = run1;
      continue;
    }

    // key range of the run: wavefront maximum, then workgroup maximum
    int wave_max = my_max;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, off));
    wave_max = __builtin_amdgcn_readfirstlane(wave_max);
    int wave_min = 0x7fffffff;  // smallest limit among the active rows (tiles below it need no masking)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      if (active[mb]) wave_min = min(wave_min, lim[mb]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) wave_min = min(wave_min, __shfl_xor(wave_min, off));
    wave_min = __builtin_amdgcn_readfirstlane(wave_min);
    __syncthreads();  // s_red and the LDS tiles of the previous run are free
    if (lane == 0) s_red[wave] = wave_max;
    __syncthreads();
    int kv_max = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) kv_max = max(kv_max, s_red[w]);
    kv_max = __builtin_amdgcn_readfirstlane(kv_max);
    const int n_kv_tiles = (kv_max + kTileN - 1) / kTileN;

    // Q^T operands: lane (query ln, half) holds d = 16*ds + 8*half .. +8 for every k-step
    s16x8 qreg[MB][DS];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        v4u w = {0, 0, 0, 0};
        if (active[mb])
          w = *reinterpret_cast<const v4u*>(a.q + row[mb] * a.qs_row + hq * a.qs_h + (16 * ds + 8 * half) * 2);
        qreg[mb][ds] = __builtin_bit_cast(s16x8, w);
      }
    }

    f32x16 o_acc[MB][DB];
    float m_run[MB], l_run[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      m_run[mb] = -INFINITY;
      l_run[mb] = 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db) o_acc[mb][db] = kZero16;
    }

    // ---- K/V fetch pipeline: page ids two tiles ahead, rows one tile ahead ----
    const int64_t* pt_row = a.page_table + static_cast<int64_t>(sq) * a.pt_row_stride;
    // pool slot of this thread's rows in the tile about to be fetched; -1 = no such key.
    // Lookups and loads are branch-free: an absent row reads slot 0 and is zeroed afterwards.
    int slot_next[NI];
    v4u kst[NI], vst[NI];
    bool fetched[NI];  // whether the row held in kst/vst exists

    auto lookup = [&](int kt, int (&slot)[NI]) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int c = tid + i * kThreads;
        const int kpos = kt * kTileN + c / CPR;
        int blk, off;
        if (kPow2) {  // page size is a power of two: shift and mask, no branch on the page size
          blk = kpos >> a.pd.shift;
          off = kpos & (a.pd.page_size - 1);
        } else {
          blk = kpos / a.pd.page_size;
          off = kpos - blk * a.pd.page_size;
        }
        const bool in_range = kpos < kv_max && blk < a.n_pages;
        const int64_t page = pt_row[in_range ? blk : 0];
        const bool ok = in_range && page >= 0 && page < a.n_pages;
        slot[i] = ok ? static_cast<int>(page) * a.pd.page_size + off : -1;
      }
    };
    auto fetch = [&](const int (&slot)[NI]) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int cc = (tid + i * kThreads) % CPR;
        fetched[i] = slot[i] >= 0;
        const int64_t byte = (static_cast<int64_t>(fetched[i] ? slot[i] : 0) * (D * 2)) + cc * 16;
        kst[i] = *reinterpret_cast<const v4u*>(kplane + byte);
        vst[i] = *reinterpret_cast<const v4u*>(vplane + byte);
      }
    };
    auto stage = [&](int buf) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int c = tid + i * kThreads;
        const int off = (c / CPR) * RS + (c % CPR) * 16;
        *reinterpret_cast<v4u*>(&s_k[buf][off]) = fetched[i] ? kst[i] : v4u{0, 0, 0, 0};
        *reinterpret_cast<v4u*>(&s_v[buf][off]) = fetched[i] ? vst[i] : v4u{0, 0, 0, 0};
      }
    };

    if (n_kv_tiles > 0) {
      lookup(0, slot_next);
      fetch(slot_next);
      lookup(1, slot_next);
      stage(0);
    }
    __syncthreads();

    for (int kt = 0; kt < n_kv_tiles; ++kt) {
      const int buf = kt & 1;
      const bool more = kt + 1 < n_kv_tiles;
      if (more) fetch(slot_next);          // rows of tile kt+1 (their slots were looked up a tile ago)
      int slot_after[NI];
      if (more) lookup(kt + 2, slot_after);

      const int key0 = kt * kTileN;
      if (key0 < wave_max) {
        // ---- S^T = K Q^T for the two 32-key blocks of the tile ----
        f32x16 s_acc[MB][2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int kb = 0; kb < 2; ++kb) s_acc[mb][kb] = kZero16;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
          for (int ds = 0; ds < DS; ++ds) {
            const v4u kw = *reinterpret_cast<const v4u*>(&s_k[buf][(kb * 32 + ln) * RS + (16 * ds + 8 * half) * 2]);
            const s16x8 ka = __builtin_bit_cast(s16x8, kw);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) s_acc[mb][kb] = E::mfma(ka, qreg[mb][ds], s_acc[mb][kb]);
          }
        }

        // ---- online softmax, one query per lane ----
        // Scores are handled as plain scalars (element writes into the MFMA vector types
        // make the compiler copy whole vectors), P is packed two values per register.
        const bool need_mask = key0 + kTileN > wave_min;
        s16x8 p_op[MB][4];  // P^T as B operands of the 4 k-steps (16 keys each)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          float sc[32];
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) sc[kb * 16 + i] = s_acc[mb][kb][i];
          if (need_mask) {
            // register i of block kb is key kb*32 + (i/4)*8 + half*4 + i%4 of the tile
            const int rel = lim[mb] - key0 - half * 4;
#pragma unroll
            for (int x = 0; x < 32; ++x) {
              const int key = (x >> 4) * 32 + ((x & 15) >> 2) * 8 + (x & 3);
              sc[x] = key < rel ? sc[x] : -INFINITY;
            }
          }
          float mx = sc[0];
#pragma unroll
          for (int x = 1; x < 32; ++x) mx = fmaxf(mx, sc[x]);
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          const float m_new = fmaxf(m_run[mb], mx * a.qscale);
          const float m_safe = m_new == -INFINITY ? 0.f : m_new;
          const float alpha = fast_exp2(m_run[mb] - m_safe);
          m_run[mb] = m_new;
          float psum = 0.f;
          uint32_t pw[16];
#pragma unroll
          for (int x = 0; x < 32; x += 2) {
            const float p0 = fast_exp2(fmaf(sc[x], a.qscale, -m_safe));
            const float p1 = fast_exp2(fmaf(sc[x + 1], a.qscale, -m_safe));
            psum += p0 + p1;
            pw[x >> 1] = E::pack2(p0, p1);
          }
          // k-step j takes registers 8j .. 8j+7 of the 32 scores = words 4j .. 4j+3
#pragma unroll
          for (int j = 0; j < 4; ++j)
            p_op[mb][j] = __builtin_bit_cast(s16x8, v4u{pw[4 * j], pw[4 * j + 1], pw[4 * j + 2], pw[4 * j + 3]});
          l_run[mb] = l_run[mb] * alpha + psum;
          if (__any(alpha != 1.f)) {
#pragma unroll
            for (int db = 0; db < DB; ++db) o_acc[mb][db] *= alpha;
          }
        }

        // ---- O^T += V^T P^T ----
        const int blk = lane >> 4;   // 16-lane block of the transpose read
        const int bi = lane & 15;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            // this lane supplies the chunk (key = base + bi / 4, d = dblock + 4 * (bi % 4)) and receives
            // d = dblock + bi for keys base .. base + 3
            const int keyb = (j >> 1) * 32 + (j & 1) * 16 + half * 4 + (bi >> 2);
            const int dcol = db * 32 + (blk & 1) * 16 + (bi & 3) * 4;
            const char* p0 = &s_v[buf][keyb * RS + dcol * 2];
            const s16x4 lo = lds_read_tr(p0);
            const s16x4 hi = lds_read_tr(p0 + 8 * RS);
            const s16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) o_acc[mb][db] = E::mfma(va, p_op[mb][j], o_acc[mb][db]);
          }
        }
      }

      if (more) {
        stage(buf ^ 1);
#pragma unroll
        for (int i = 0; i < NI; ++i) slot_next[i] = slot_after[i];
      }
      __syncthreads();
    }

    // ---- finish the run: normalise and store ----
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const float l_tot = l_run[mb] + __shfl_xor(l_run[mb], 32);
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
      if (!active[mb]) continue;
      char* o = a.out + row[mb] * a.os_row + hq * a.os_h;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          // registers 4*i4 .. 4*i4+3 hold d = db*32 + i4*8 + half*4 + 0..3
          const int d = db * 32 + i4 * 8 + half * 4;
          s16x4 pk;
#pragma unroll
          for (int e = 0; e < 4; ++e) pk[e] = E::from_float(o_acc[mb][db][i4 * 4 + e] * inv);
          *reinterpret_cast<s16x4*>(o + d * 2) = pk;
        }
      }
      if (half == 0)
        a.lse[static_cast<int64_t>(hq) * a.Lq + row[mb]] = l_tot > 0.f ? (m_run[mb] + log2f(l_tot)) * kLn2 : -INFINITY;
    }
    run0 = run1;
  }
}

template <typename E, int D>
void launch(const PrefillArgs& a0, hipStream_t st) {
  PrefillArgs a = a0;
  constexpr int MB = 1;
  constexpr int BM = kWaves * 32 * MB;
  a.n_tiles = (a.Lq + BM - 1) / BM;
  const int G = a.Hq / a.Hc;
  dim3 grid(a.Hc, G * a.n_tiles);
  if (a.pd.shift >= 0)
    hipLaunchKernelGGL((paged_prefill_kernel<E, D, MB, true>), grid, dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((paged_prefill_kernel<E, D, MB, false>), grid, dim3(kThreads), 0, st, a);
}

}  // namespace

extern "C" int fp_paged_prefill(const void* q, int64_t q_stride_row, int64_t q_stride_h, const void* pool_k,
                                const void* pool_v, const int64_t* page_table, int64_t pt_row_stride,
                                const int64_t* batch_idx, const int32_t* row_limit, void* out,
                                int64_t out_stride_row, int64_t out_stride_h, float* lse, int32_t Lq, int32_t Hq,
                                int32_t Hc, int32_t D, int32_t page_size, int32_t n_pages, int32_t max_batch,
                                int64_t n_slots, float scale, int dtype, void* stream) {
  if (dtype != FP_DTYPE_BF16 && dtype != FP_DTYPE_F16)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: dtype %d (supported: bf16, f16)", dtype);
  if (D != 64 && D != 128) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: head_dim %d (supported: 64, 128)", D);
  if (Lq < 0 || Hq <= 0 || Hc <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 || n_slots <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: bad dimension");
  if (Hq % Hc) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: Hq=%d not a multiple of Hc=%d", Hq, Hc);
  if (n_slots < static_cast<int64_t>(n_pages) * page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: n_slots smaller than n_pages * page_size");
  if (Hc > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: Hc exceeds 65535");
  if (n_slots > INT32_MAX) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: more than 2^31-1 slots per head");
  if (Lq == 0) return FP_OK;
  if (!q || !pool_k || !pool_v || !page_table || !batch_idx || !row_limit || !out || !lse)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: null pointer");
  if (!fp::aligned(q, 16) || !fp::aligned(pool_k, 16) || !fp::aligned(pool_v, 16) || !fp::aligned(out, 8) ||
      (q_stride_row * 2) % 16 || (q_stride_h * 2) % 16 || (out_stride_row * 2) % 8 || (out_stride_h * 2) % 8)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: q rows must be 16-byte and out rows 8-byte aligned");
  const int64_t tiles = (static_cast<int64_t>(Lq) + 127) / 128;
  if (tiles * (Hq / Hc) > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: too many query tiles");

  PrefillArgs a{static_cast<const char*>(q), q_stride_row * 2, q_stride_h * 2,
                static_cast<const char*>(pool_k), static_cast<const char*>(pool_v),
                page_table, pt_row_stride, batch_idx, row_limit,
                static_cast<char*>(out), out_stride_row * 2, out_stride_h * 2, lse,
                Lq, Hq, Hc, fp::PageDiv(page_size), n_pages, max_batch, n_slots, scale * kLog2e, 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == FP_DTYPE_BF16) {
    if (D == 64) launch<BF16, 64>(a, st); else launch<BF16, 128>(a, st);
  } else {
    if (D == 64) launch<F16, 64>(a, st); else launch<F16, 128>(a, st);
  }
  return fp::check_launch("fp_paged_prefill");
}
