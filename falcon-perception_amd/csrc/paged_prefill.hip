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
// MFMA-bound.  A workgroup of 8 wavefronts owns one cache head and 256 / G consecutive packed
// query rows of each of its G query heads; a wavefront owns 32 rows of one query head.  (Large launches
// at head_dim 64 use workgroups of 4 wavefronts and 128 / G rows, three to a CU.)
//   S^T = K Q^T  (v_mfma_f32_32x32x16): keys are the M rows, queries the N columns, so a
//         lane holds scores of ONE query and softmax row reductions stay in registers
//         (plus one exchange between the two lane halves).
//   O^T = V^T P^T: P^T is already in B-operand layout in the S^T accumulators; V^T
//         comes out of LDS through ds_read_b64_tr_b16, so V is staged row-major like K.
//   K/V tiles of 64 keys go straight from global memory into LDS with global_load_lds
//   (16 bytes per lane, no staging registers), into double buffers whose rows are
//   chunk-permuted against bank conflicts; the first pool slot of every tile of a run is
//   looked up once, so a staging load is a scalar base plus a fixed lane offset.
//   The two wavefronts that share a SIMD run half a step apart (two barriers per tile): one is
//   in its MFMA phase (O^T of the previous tile, S^T of the current one) while the other is in
//   its softmax.
// Rows of one tile may belong to several sequences: the tile is processed one
// run of equal batch_idx at a time; rows of slot 0 are padding (out 0, lse -inf).
#include "fp_common.h"
#include "prefill_common.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <math.h>

#include <type_traits>

namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kTileN = 64;  // keys per tile
constexpr int kSlotTable = 2048;  // tiles of a run whose first pool slot is looked up ahead of the tile loop
constexpr float kMaxSlack = 6.f;  // the running maximum may lag a row's true maximum by this much (log2)
constexpr int kPrefetchK = 4; // K operand reads in flight ahead of the MFMA that uses them
constexpr int kPrefetchV = 4; // V^T operand read pairs in flight ahead of their MFMA
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
  const float* sinks;    // optional [Hq]: out is multiplied by sigmoid(lse - sinks[h])
  int Lq, Hq, Hc;
  fp::PageDiv pd;
  int n_pages, max_batch;
  int64_t n_slots;
  float qscale;  // scale * log2(e)
  int n_tiles;   // query tiles
  // key split: grid z = n_key_splits workgroups share a query tile, each taking an equal share of every
  // run's key tiles and leaving unnormalised partial results for the merge pass
  // key shares: a share's result for a row, normalised by its own denominator, in the model dtype (half
  // the bytes of fp32 partials; the merge pass is bound by this traffic), with its maximum and denominator
  short* ws_acc;  // [n_key_splits, Lq, Hq, D] elements of the model dtype
  float* ws_ml;   // [n_key_splits, Lq, Hq, 2]: running maximum (log2 units), denominator
  // optional (fp_paged_prefill_tile_order): the query tile workgroup row y works on, longest key range first
  const int* order;
  int order_rows;  // rows per query tile the order was made for; another tile size ignores it
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
  static __device__ __forceinline__ float round(float x) { return static_cast<float>(static_cast<__bf16>(x)); }
  static __device__ __forceinline__ float to_float(short x) { return static_cast<float>(__builtin_bit_cast(__bf16, x)); }
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
  static __device__ __forceinline__ float round(float x) { return static_cast<float>(static_cast<_Float16>(x)); }
  static __device__ __forceinline__ float to_float(short x) { return static_cast<float>(__builtin_bit_cast(_Float16, x)); }
};

constexpr f32x16 kZero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// LDS transpose read: the 16 lanes of a block each name 4 consecutive 16-bit elements;
// lane i receives, for j = 0..3, element (i % 4) of the chunk named by lane 4 * j + i / 4.
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p));
}

template <int N>
struct IntC {
  static constexpr int value = N;
};

using fp::load_to_lds;

// K/V tiles in LDS are 64 unpadded rows of D * 2 bytes, filled by global_load_lds (each lane's
// 16 bytes land at base + lane * 16).  Bank conflicts are avoided by permuting the 16-byte chunks
// of a row on the GLOBAL side of the load:
//   K: chunk c of row r sits at position c ^ kswz(r).  The MFMA operand read takes the same chunk
//      of 16 consecutive rows, which then fall into 16 different positions.
//   V: the 32-byte region c32 of row r sits at region (c32 + vrot(r)) mod regions.  The transpose
//      read takes 4 consecutive rows x 32 bytes per 16-lane block, two blocks side by side.
template <int D>
struct Swizzle {
  static constexpr int CPR = D * 2 / 16;  // 16-byte chunks per row
  static constexpr int R32 = CPR / 2;     // 32-byte regions per row
  static __device__ __forceinline__ int kswz(int r) { return (r / (16 / CPR)) % CPR; }
  static __device__ __forceinline__ int vrot(int r) { return (2 * ((r / (8 / R32)) & 3)) % R32; }
};

// G = query heads per cache head.  The 8 wavefronts of a workgroup are G heads x 8 / G blocks of
// 32 query rows: every head of the group works from the same staged K/V tile, so the bytes that
// travel from L2 into LDS (64 B per cycle and CU, and a wavefront waits at its load instructions
// while that path is busy) are shared by all of them.
template <typename E, int D, int G, bool kPow2, int W = kWaves, bool kBounded = false>
__global__ __launch_bounds__(W * 64, (W == 4 && D == 64 ? 3 : 2)) void paged_prefill_kernel(const PrefillArgs a) {
  constexpr int kThreads = W * 64;  // shadows the file-scope constant: W wavefronts per workgroup
  using SW = Swizzle<D>;
  constexpr int MB = 1;                    // 32-row blocks per wavefront
  constexpr int RB = W / G;                // 32-row blocks per workgroup
  constexpr int BM = RB * 32;              // query rows per workgroup
  constexpr int ROWB = D * 2;              // bytes of a K/V row
  constexpr int CPR = SW::CPR;
  constexpr int R32 = SW::R32;
  constexpr int RPI = 64 / CPR;            // rows one wavefront load instruction brings in
  constexpr int NI = kTileN / (RPI * W);   // load instructions per wavefront, tile and tensor
  constexpr int DS = D / 16;               // MFMA k-steps over head_dim
  constexpr int DB = D / 32;               // 32-wide blocks of head_dim in O^T
  constexpr int TILE_BYTES = kTileN * ROWB;

  // four separate arrays (not one indexed array) so that a load into one buffer is known not to
  // alias the reads of the other
  __shared__ __attribute__((aligned(1024))) char s_k0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_k1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_v0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_v1[TILE_BYTES];
  __shared__ int s_bidx[BM];
  __shared__ int s_red[W];
  __shared__ int s_tslot[kSlotTable];

  // linear id = cache head + Hc * tile: all tiles that read one cache head run on the XCD that
  // already holds its K/V in L2
  const int hc = blockIdx.x;
  // Workgroups are handed out in the order of their ids, so the ids should run from the longest key range to the
  // shortest.  Without an order from the caller: descending tile index, which is that inside a sequence (later
  // rows see more keys) but not across a packed row of several.
  int tile = a.n_tiles - 1 - blockIdx.y;
  if (a.order) {
    tile = a.order[blockIdx.y];
    tile = tile < 0 ? 0 : tile >= a.n_tiles ? a.n_tiles - 1 : tile;  // whatever the buffer holds, no row outside the launch
  }
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hq = hc * G + wave % G;  // query head of this wavefront
  const int rblock = wave / G;       // its block of 32 rows inside the tile
  const int lane = tid & 63;
  const int half = lane >> 5;   // which 8 of 16 k-values / which 4 of 8 rows this lane holds
  const int ln = lane & 31;     // query column (S^T, O^T) or key row (K operand)
  const int blk = lane >> 4;    // 16-lane block of the transpose read
  const int bi = lane & 15;
  const int tile0 = tile * BM;

  // Everything the set-up needs from global memory is requested at once, so the loads travel
  // together: the sequence of each row of the tile, then this wavefront's row limits and Q rows.
  // Rows outside a run keep their Q values: what such a row computes is never stored.
  int64_t bx_raw[(BM + kThreads - 1) / kThreads];
#pragma unroll
  for (int j = 0; j < (BM + kThreads - 1) / kThreads; ++j) {
    const int r = tile0 + j * kThreads + tid;
    bx_raw[j] = (j * kThreads + tid < BM && r < a.Lq) ? a.batch_idx[r] : 0;
  }
  int row[MB], lim_raw[MB];
  s16x8 qreg[MB][DS];  // Q^T operands: lane (query ln, half) holds d = 16*ds + 8*half .. +8 for every k-step
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    row[mb] = tile0 + (rblock * MB + mb) * 32 + ln;
    const bool in = row[mb] < a.Lq;
    lim_raw[mb] = in ? a.row_limit[row[mb]] : 0;
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) {
      v4u w = {0, 0, 0, 0};
      if (in) w = *reinterpret_cast<const v4u*>(a.q + row[mb] * a.qs_row + hq * a.qs_h + (16 * ds + 8 * half) * 2);
      if constexpr (kBounded) {
        // bounded scores: Q carries scale * log2(e), so that the matrix product leaves the exponent itself
#pragma unroll
        for (int c = 0; c < 4; ++c)
          w[c] = E::pack2(E::to_float(static_cast<short>(w[c] & 0xffffu)) * a.qscale,
                          E::to_float(static_cast<short>(w[c] >> 16)) * a.qscale);
      }
      qreg[mb][ds] = __builtin_bit_cast(s16x8, w);
    }
  }
#pragma unroll
  for (int j = 0; j < (BM + kThreads - 1) / kThreads; ++j) {
    int64_t bx = bx_raw[j];
    if (bx < 0 || bx >= a.max_batch) bx = 0;
    if (j * kThreads + tid < BM) s_bidx[j * kThreads + tid] = static_cast<int>(bx);
  }
  __syncthreads();

  const char* kplane = a.pool_k + static_cast<int64_t>(hc) * a.n_slots * ROWB;
  const char* vplane = a.pool_v + static_cast<int64_t>(hc) * a.n_slots * ROWB;

  // ---- per-lane constants of the staging loads and of the operand reads ----
  // load instruction i of this wavefront fills LDS rows (i * W + wave) * RPI .. + RPI; this lane
  // fills position lp of row lrow in that group.  kswz / vrot of the row do not depend on i.
  const int lrow = lane / CPR;
  const int lp = lane % CPR;
  const int st_row0 = wave * RPI + lrow;  // row of load instruction 0; instruction i adds i * W * RPI
  const int k_src_off = (lp ^ SW::kswz(st_row0)) * 16;
  const int v_src_off = ((((lp >> 1) + R32 - SW::vrot(st_row0)) % R32) * 2 + (lp & 1)) * 16;
  // K operand: row kb * 32 + ln, chunk 2 * ds + half at position (2 * ds) ^ ksel
  const int ksel = half ^ SW::kswz(ln);
  // V operand: rows keyb .. , region (2 * db + vsel) % R32, 8 bytes (bi & 3) inside it
  const int vsel = (blk & 1) + SW::vrot(half * 4 + (bi >> 2));

  int run0 = 0;
  while (run0 < BM) {
    // values every lane agrees on are moved to scalar registers so the control flow that
    // depends on them stays uniform
    const int sq = __builtin_amdgcn_readfirstlane(s_bidx[run0]);
    // end of the run: the first row of another sequence, found 64 rows at a time
    int run1 = BM;
    for (int base = run0; base < BM; base += 64) {
      const int idx = base + lane;
      const unsigned long long other = __ballot(idx < BM && s_bidx[idx] != sq);
      if (other != 0) {
        run1 = base + __builtin_ctzll(other);
        break;
      }
    }
    run1 = __builtin_amdgcn_readfirstlane(run1);

    // rows of this wavefront: tile rows rblock * 32 + ln
    int lim[MB];
    bool active[MB];
    int my_max = 0;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int tr = (rblock * MB + mb) * 32 + ln;
      active[mb] = tr >= run0 && tr < run1 && row[mb] < a.Lq;
      lim[mb] = (active[mb] && sq != 0) ? lim_raw[mb] : 0;
      if (lim[mb] < 0) lim[mb] = 0;
      my_max = max(my_max, lim[mb]);
    }

    if (sq == 0) {
      // padding rows: out = 0, lse = -inf
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (!active[mb]) continue;
        if (gridDim.z > 1) {  // an empty share; the merge pass then writes out = 0, lse = -inf
          const int64_t p = (static_cast<int64_t>(blockIdx.z) * a.Lq + row[mb]) * a.Hq + hq;
#pragma unroll
          for (int c = 0; c < D / 8; ++c) *reinterpret_cast<uint2*>(a.ws_acc + p * D + half * (D / 2) + c * 4) = uint2{0, 0};
          if (half == 0) *reinterpret_cast<float2*>(a.ws_ml + p * 2) = float2{-INFINITY, 0.f};
          continue;
        }
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
    for (int w = 0; w < W; ++w) kv_max = max(kv_max, s_red[w]);
    kv_max = __builtin_amdgcn_readfirstlane(kv_max);
    const int n_run_tiles = (kv_max + kTileN - 1) / kTileN;
    // this workgroup's share of the run's key tiles: [kt_lo, n_kv_tiles)
    const int kt_lo = static_cast<int>(static_cast<int64_t>(n_run_tiles) * blockIdx.z / gridDim.z);
    const int n_kv_tiles = static_cast<int>(static_cast<int64_t>(n_run_tiles) * (blockIdx.z + 1) / gridDim.z);
    const int n_my = n_kv_tiles - kt_lo;

    f32x16 o_acc[MB][DB];
    float m_run[MB], l_run[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      m_run[mb] = kBounded ? 0.f : -INFINITY;  // bounded scores: the reference point of the exponentials is 0 throughout
      l_run[mb] = 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db) o_acc[mb][db] = kZero16;
    }

    // ---- K/V fetch pipeline ----
    // Every wavefront stages NI groups of RPI rows of each tile.  Where a page holds whole tiles
    // (page size a power of two, at least the tile), a tile that lies before the run's last key in a
    // mapped page is contiguous in the pool: its first slot is looked up once per run into s_tslot,
    // and a staging load is then a scalar base plus a fixed offset per lane.  Any other tile (the
    // last one of a run, small or odd page sizes, unmapped pages, runs longer than the table) is
    // staged row by row: a key that does not exist (past the run's last key, or an unmapped page)
    // reads slot 0, finite bytes, and every such key is masked.
    const int64_t* pt_row = a.page_table + static_cast<int64_t>(sq) * a.pt_row_stride;
    const int64_t pool_pages = a.n_slots / a.pd.page_size;
    const bool page_holds_tile = kPow2 && a.pd.page_size % kTileN == 0;
    for (int t = kt_lo + tid; t < n_kv_tiles && t - kt_lo < kSlotTable; t += kThreads) {
      int slot = -1;
      if (page_holds_tile && (t + 1) * kTileN <= kv_max) {
        const int key0 = t * kTileN;
        const int blk = key0 >> a.pd.shift;
        if (blk < a.n_pages) {
          const int64_t pg = pt_row[blk];
          if (pg >= 0 && pg < pool_pages) slot = static_cast<int>(pg) * a.pd.page_size + (key0 & (a.pd.page_size - 1));
        }
      }
      s_tslot[t - kt_lo] = slot;
    }
    __syncthreads();
    // first pool slot of tile kt, or -1: wavefront-uniform
    auto tile_slot = [&](int kt) {
      return __builtin_amdgcn_readfirstlane((kt >= kt_lo && kt < n_kv_tiles && kt - kt_lo < kSlotTable) ? s_tslot[kt - kt_lo] : -1);
    };

    auto key_block = [&](int kpos, int& blkid, int& off) {
      if (kPow2) {  // page size is a power of two: shift and mask, no branch on the page size
        blkid = kpos >> a.pd.shift;
        off = kpos & (a.pd.page_size - 1);
      } else {
        blkid = kpos / a.pd.page_size;
        off = kpos - blkid * a.pd.page_size;
      }
    };
    const char* ksrc = kplane + k_src_off;
    const char* vsrc = vplane + v_src_off;
    uint32_t lane_k[NI], lane_v[NI];  // byte offset of this lane's 16 bytes from the first row of a tile
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      lane_k[i] = (i * W * RPI + st_row0) * ROWB + k_src_off;
      lane_v[i] = (i * W * RPI + st_row0) * ROWB + v_src_off;
    }
    // One staging load of tile kt, whose first slot is ts (or -1): pieces 0 .. NI - 1 are the V loads
    // of the row groups, NI .. 2 NI - 1 the K loads.  Tiles past the run's last one are not staged.
    auto fetch_piece = [&](int piece, int kt, int ts, char* dst) {
      if (kt >= n_kv_tiles) return;
      const int i = piece % NI;
      const bool is_k = piece >= NI;
      char* lds = dst + (i * W + wave) * RPI * ROWB;  // wavefront-uniform
      if (ts >= 0) {
        load_to_lds((is_k ? kplane : vplane) + static_cast<int64_t>(ts) * ROWB, is_k ? lane_k[i] : lane_v[i], lds);
      } else {
        asm volatile("");  // rare: keep it out of the way as a branch
        const int kpos = kt * kTileN + i * W * RPI + st_row0;
        int blkid, off;
        key_block(kpos, blkid, off);
        const bool in_range = kpos < kv_max && blkid < a.n_pages;
        const int64_t pg = pt_row[in_range ? blkid : 0];
        const bool ok = in_range && pg >= 0 && pg < pool_pages;
        const int slot = ok ? static_cast<int>(pg) * a.pd.page_size + off : 0;
        load_to_lds((is_k ? ksrc : vsrc) + static_cast<int64_t>(slot) * ROWB, lds);
      }
    };

    // per-lane LDS offsets of the operand reads, the same for every tile and buffer
    int kofs[DS], vofs[DB];
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) kofs[ds] = ln * ROWB + (((2 * ds) ^ ksel) * 16);
#pragma unroll
    for (int db = 0; db < DB; ++db)
      vofs[db] = (half * 4 + (bi >> 2)) * ROWB + (bi & 3) * 8 + ((2 * db + vsel) % R32) * 32;

    // ---- schedule ----
    // Step i of a wavefront is M(i) = { O^T += V^T P^T of tile i - 1;  S^T = K Q^T of tile i } on the
    // matrix pipe, then X(i) = softmax of tile i on the vector pipe.  The two wavefronts that share a
    // SIMD (w and w + 4) run half a step apart: between two barriers the first half does M(i) then
    // X(i), the second half X(i - 1) then M(i), so that one is in M while the other is in X and the
    // matrix and the vector pipe of the SIMD work at the same time.  One barrier per step (B(i), at the
    // start of the first half's step and in the middle of the second half's) is all the data needs:
    // staging step i (K of tile i + 1, V of tile i) is issued after B(i), when M(i - 1) is over
    // everywhere, and every wavefront has waited for its loads before B(i + 1), after which M(i + 1)
    // begins.  (A second barrier between the two parts of the interval kept the halves in step more
    // strictly and cost 2 %.)  K(i) lives in K buffer i % 2, V(i) in V buffer i % 2.
    {
      const int ts0 = tile_slot(kt_lo);
#pragma unroll
      for (int piece = NI; piece < 2 * NI; ++piece) fetch_piece(piece, kt_lo, ts0, s_k0);  // K of the first tile
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's rows have landed in LDS

    s16x8 p_op[MB][4];  // P^T as B operands of the 4 k-steps (16 keys each), from X(i) to M(i + 1)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 4; ++j) p_op[mb][j] = s16x8{0, 0, 0, 0, 0, 0, 0, 0};

    float alpha_next[MB];  // factor the accumulators still have to take before tile i - 1 is added
    bool moved_next[MB];   // whether it differs from 1 (uniform over the wavefront)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      alpha_next[mb] = 1.f;
      moved_next[mb] = false;
    }
    auto step = [&](auto second_c, auto parity, int i) {
      constexpr bool kSecond = decltype(second_c)::value != 0;
      constexpr int kBuf = decltype(parity)::value;
      const char* kcur = kBuf ? s_k1 : s_k0;   // K(i)
      const char* vprev = kBuf ? s_v0 : s_v1;  // V(i - 1)
      char* knext = kBuf ? s_k0 : s_k1;        // K(i + 1) goes here
      char* vcur = kBuf ? s_v1 : s_v0;         // V(i) goes here
      const int key0 = (kt_lo + i) * kTileN;  // step i works on key tile kt_lo + i
      const bool work_cur = i < n_my && key0 < wave_max;
      const bool work_prev = i > 0 && key0 - kTileN < wave_max;

      // the staging step this wavefront issues during the step: K of tile kt_k, V of tile kt_k - 1.
      // The table is read ahead of the barrier, whose wait hides the LDS latency.
      const int kt_k = kt_lo + (kSecond ? i + 2 : i + 1);
      const int ts_k = tile_slot(kt_k);
      const int ts_v = tile_slot(kt_k - 1);
      if (!kSecond) __builtin_amdgcn_s_waitcnt(0x0F70);  // staging step i - 1 of this wavefront has landed
      if (!kSecond) __builtin_amdgcn_s_barrier();

      // ---- M(i), first part: O^T += V^T P^T of tile i - 1 ----
      f32x16 s_acc[MB][2];  // written by the first MFMA of each block, which starts from zero
      constexpr int kPvEvery = 4 * DB / NI;  // MFMA steps between two staging loads
      constexpr int kSEvery = 2 * DS / NI;
      if (work_prev) {
        asm volatile("");
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          if (moved_next[mb]) {
            asm volatile("");  // the rescale is rare and must not run unconditionally
#pragma unroll
            for (int db = 0; db < DB; ++db) o_acc[mb][db] *= alpha_next[mb];
          }
        }
        // step t = (j, db): this lane names the chunk (key = base + bi / 4, d = dblock + 4 * (bi % 4))
        // and receives d = dblock + bi for keys base .. base + 3, once for each half of the 16 keys
        auto read_v = [&](int t, s16x4& lo, s16x4& hi) {
          const int j = t / DB, db = t % DB;
          const char* p0 = vprev + vofs[db] + ((j >> 1) * 32 + (j & 1) * 16) * ROWB;
          lo = lds_read_tr(p0);
          hi = lds_read_tr(p0 + 8 * ROWB);
        };
        s16x4 rlo[kPrefetchV], rhi[kPrefetchV];
#pragma unroll
        for (int t = 0; t < kPrefetchV; ++t) read_v(t, rlo[t], rhi[t]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4 * DB; ++t) {
          const s16x4 lo = rlo[t % kPrefetchV], hi = rhi[t % kPrefetchV];
          const s16x8 va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          if (!kSecond && t % kPvEvery == 0) fetch_piece(t / kPvEvery, kt_k - 1, ts_v, vcur);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) o_acc[mb][t % DB] = E::mfma(va, p_op[mb][t / DB], o_acc[mb][t % DB]);
          if (t + kPrefetchV < 4 * DB) read_v(t + kPrefetchV, rlo[t % kPrefetchV], rhi[t % kPrefetchV]);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else if (!kSecond) {
#pragma unroll
        for (int piece = 0; piece < NI; ++piece) fetch_piece(piece, kt_k - 1, ts_v, vcur);
      }

      // ---- M(i), second part: S^T = K Q^T for the two 32-key blocks of tile i ----
      // LDS operands are read kPrefetchK steps ahead of the MFMA that consumes them; the two 32-key
      // blocks alternate so that consecutive MFMAs are independent.  The scheduling barriers pin this
      // order: left alone, the compiler gathers the reads and waits for all of them before every MFMA.
      if (work_cur) {
        asm volatile("");
        auto read_k = [&](int t) {
          const int kb = t & 1, ds = t >> 1;
          return *reinterpret_cast<const v4u*>(kcur + kofs[ds] + kb * 32 * ROWB);
        };
        v4u ring[kPrefetchK];
#pragma unroll
        for (int t = 0; t < kPrefetchK; ++t) ring[t] = read_k(t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2 * DS; ++t) {
          const s16x8 ka = __builtin_bit_cast(s16x8, ring[t % kPrefetchK]);
          if (!kSecond && t % kSEvery == 0) fetch_piece(NI + t / kSEvery, kt_k, ts_k, knext);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            s_acc[mb][t & 1] = E::mfma(ka, qreg[mb][t >> 1], (t >> 1) == 0 ? kZero16 : s_acc[mb][t & 1]);
          if (t + kPrefetchK < 2 * DS) ring[t % kPrefetchK] = read_k(t + kPrefetchK);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else if (!kSecond) {
#pragma unroll
        for (int piece = NI; piece < 2 * NI; ++piece) fetch_piece(piece, kt_k, ts_k, knext);
      }

      if (kSecond) __builtin_amdgcn_s_waitcnt(0x0F70);  // staging step i of this wavefront has landed
      if (kSecond) __builtin_amdgcn_s_barrier();
      if (kSecond) {
        // staging step i + 1: K(i + 2) into the buffer of K(i), V(i + 1) into that of V(i - 1)
#pragma unroll
        for (int piece = 0; piece < 2 * NI; ++piece)
          fetch_piece(piece, piece < NI ? kt_k - 1 : kt_k, piece < NI ? ts_v : ts_k,
                      const_cast<char*>(piece < NI ? vprev : kcur));
      }

      // ---- X(i): online softmax of tile i, one query per lane ----
      // Scores are handled as plain scalars (element writes into the MFMA vector types
      // make the compiler copy whole vectors), P is packed two values per register.
      if (work_cur) {
        asm volatile("");
        const bool need_mask = key0 + kTileN > wave_min;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          float sc[32];
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int x = 0; x < 16; ++x) sc[kb * 16 + x] = s_acc[mb][kb][x];
          if (need_mask) {
            asm volatile("");  // keeps this a branch: turned into selects it would run on every tile
            // register x of block kb is key kb*32 + (x/4)*8 + half*4 + x%4 of the tile
            const int rel = lim[mb] - key0 - half * 4;
#pragma unroll
            for (int x = 0; x < 32; ++x) {
              const int key = (x >> 4) * 32 + ((x & 15) >> 2) * 8 + (x & 3);
              sc[x] = key < rel ? sc[x] : -INFINITY;
            }
          }
          if constexpr (kBounded) {
            // |score| is bounded by the caller's declaration: exp2 of the score itself neither overflows nor
            // vanishes in fp32 / bf16, so there is no running maximum, no exchange between the lane halves,
            // no vote and no rescale: exponential, pack, row sum
            float part[4] = {0.f, 0.f, 0.f, 0.f};
            uint32_t pw[16];
#pragma unroll
            for (int x = 0; x < 32; x += 2) {
              const float p0 = fast_exp2(sc[x]);
              const float p1 = fast_exp2(sc[x + 1]);
              pw[x >> 1] = E::pack2(p0, p1);
              part[(x >> 1) & 3] += p0 + p1;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
              p_op[mb][j] = __builtin_bit_cast(s16x8, v4u{pw[4 * j], pw[4 * j + 1], pw[4 * j + 2], pw[4 * j + 3]});
            l_run[mb] += (part[0] + part[1]) + (part[2] + part[3]);
            continue;
          }
          // four independent chains: one wavefront alone issues a dependent instruction every ~8 cycles
          float mx4[4] = {sc[0], sc[1], sc[2], sc[3]};
#pragma unroll
          for (int x = 4; x < 32; ++x) mx4[x & 3] = fmaxf(mx4[x & 3], sc[x]);
          float mx = fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3]));
          mx = fp::max_across_lane_halves(mx);
          // Lazy running maximum: the reference point m_run only moves when some row's maximum has
          // grown by more than kMaxSlack (log2 units); until then exp2(s - m_run) may reach
          // 2^kMaxSlack, harmless in bf16/f16 P and fp32 sums, and the accumulators need no rescale.
          const float m_cand = mx * a.qscale;
          const bool moved = __any(m_cand > m_run[mb] + kMaxSlack);
          const float m_new = moved ? fmaxf(m_run[mb], m_cand) : m_run[mb];
          const float m_safe = m_new == -INFINITY ? 0.f : m_new;
          const float alpha = moved ? fast_exp2(m_run[mb] - m_safe) : 1.f;
          m_run[mb] = m_new;
          // Stage by stage (scale, exponential, pack and sum) with scheduling barriers between: left alone,
          // the compiler pairs every exponential with the multiply-add right before it, and a wavefront
          // that runs alone on the vector pipe waits out the latency of each pair.
          float part[4] = {0.f, 0.f, 0.f, 0.f};
          uint32_t pw[16];
#pragma unroll
          for (int x = 0; x < 32; x += 2) {
            const float p0 = fast_exp2(fmaf(sc[x], a.qscale, -m_safe));
            const float p1 = fast_exp2(fmaf(sc[x + 1], a.qscale, -m_safe));
            pw[x >> 1] = E::pack2(p0, p1);
            part[(x >> 1) & 3] += p0 + p1;
          }
          const float psum = (part[0] + part[1]) + (part[2] + part[3]);
          // k-step j takes registers 8j .. 8j+7 of the 32 scores = words 4j .. 4j+3
#pragma unroll
          for (int j = 0; j < 4; ++j)
            p_op[mb][j] = __builtin_bit_cast(s16x8, v4u{pw[4 * j], pw[4 * j + 1], pw[4 * j + 2], pw[4 * j + 3]});
          l_run[mb] = fmaf(l_run[mb], alpha, psum);  // alpha is 1 unless the reference point moved
          // the accumulators are rescaled where they are next used, at the start of M(i + 1)
          alpha_next[mb] = alpha;
          moved_next[mb] = moved;
        }
      }
    };

    // steps 0 .. n_my (the last one only has the O^T part of the last tile)
    if (wave < W / 2) {
      for (int i = 0; i <= n_my; i += 2) {
        step(IntC<0>{}, IntC<0>{}, i);
        if (i + 1 <= n_my) step(IntC<0>{}, IntC<1>{}, i + 1);
      }
      __builtin_amdgcn_s_barrier();  // the second half's last barrier, B(n_my + 1)
    } else {
      __builtin_amdgcn_s_barrier();  // B(0): the first half starts M(0)
      {  // staging step 0: K(1), V(0)
        const int ts1 = tile_slot(kt_lo + 1), ts0 = tile_slot(kt_lo);
#pragma unroll
        for (int piece = 0; piece < 2 * NI; ++piece)
          fetch_piece(piece, piece < NI ? kt_lo : kt_lo + 1, piece < NI ? ts0 : ts1, piece < NI ? s_v0 : s_k1);
      }
      for (int i = 0; i <= n_my; i += 2) {
        step(IntC<1>{}, IntC<0>{}, i);
        if (i + 1 <= n_my) step(IntC<1>{}, IntC<1>{}, i + 1);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // no staging load is in flight when the LDS tiles are reused

    // ---- finish the run: normalise and store ----
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const float l_tot = l_run[mb] + __shfl_xor(l_run[mb], 32);
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
      if (!active[mb]) continue;
      if (gridDim.z > 1) {
        // one of several key shares: the unnormalised state goes to the merge pass
        const int64_t p = (static_cast<int64_t>(blockIdx.z) * a.Lq + row[mb]) * a.Hq + hq;
        short* po = a.ws_acc + p * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            *reinterpret_cast<uint2*>(po + db * 32 + i4 * 8 + half * 4) =
                uint2{E::pack2(o_acc[mb][db][i4 * 4] * inv, o_acc[mb][db][i4 * 4 + 1] * inv),
                      E::pack2(o_acc[mb][db][i4 * 4 + 2] * inv, o_acc[mb][db][i4 * 4 + 3] * inv)};
        if (half == 0) *reinterpret_cast<float2*>(a.ws_ml + p * 2) = float2{m_run[mb], l_tot};
        continue;
      }
      char* o = a.out + row[mb] * a.os_row + hq * a.os_h;
      const float lse_nat = l_tot > 0.f ? (m_run[mb] + log2f(l_tot)) * kLn2 : -INFINITY;
      // attention-sink gate of the caller's post-attention step (model.py:122-128): the output,
      // rounded to the model dtype, times sigmoid(lse - sinks[h]) in fp32, rounded again
      const bool gated = a.sinks != nullptr;
      const float gate = gated ? 1.f / (1.f + __expf(a.sinks[hq] - lse_nat)) : 1.f;
      auto fin = [&](float x) { return gated ? E::round(x * inv) * gate : x * inv; };
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          // registers 4*i4 .. 4*i4+3 hold d = db*32 + i4*8 + half*4 + 0..3
          const int d = db * 32 + i4 * 8 + half * 4;
          const uint32_t w0 = E::pack2(fin(o_acc[mb][db][i4 * 4 + 0]), fin(o_acc[mb][db][i4 * 4 + 1]));
          const uint32_t w1 = E::pack2(fin(o_acc[mb][db][i4 * 4 + 2]), fin(o_acc[mb][db][i4 * 4 + 3]));
          *reinterpret_cast<uint2*>(o + d * 2) = uint2{w0, w1};
        }
      }
      if (half == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row[mb]] = lse_nat;
    }
    run0 = run1;
  }
}

// ---- merge of the key shares ----
// One wavefront per (query row, query head): combines the shares' results, each weighted by its
// denominator at the common maximum, applies the sink gate, stores out and lse.
constexpr int kMergeRows = 4;  // (row, head) pairs per workgroup

template <typename E, int D>
__global__ __launch_bounds__(kMergeRows * 64) void paged_prefill_merge_kernel(const PrefillArgs a, int n_shares) {
  constexpr int EPL = D / 64;  // output elements per lane
  const int lane = threadIdx.x & 63;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kMergeRows + (threadIdx.x >> 6);
  if (item >= static_cast<int64_t>(a.Lq) * a.Hq) return;
  const int row = static_cast<int>(item / a.Hq), hq = static_cast<int>(item % a.Hq);
  const int64_t share_stride = static_cast<int64_t>(a.Lq) * a.Hq;
  constexpr int kBatch = 8;  // the launcher never makes more shares
  float m_s[kBatch], l_s[kBatch], acc_s[kBatch][EPL];
#pragma unroll
  for (int s = 0; s < kBatch; ++s) {
    const bool on = s < n_shares;
    const int64_t p = s * share_stride + item;
    m_s[s] = on ? a.ws_ml[p * 2] : -INFINITY;
    l_s[s] = on ? a.ws_ml[p * 2 + 1] : 0.f;
    if (EPL == 2) {
      const uint32_t w = on ? *reinterpret_cast<const uint32_t*>(a.ws_acc + p * D + lane * 2) : 0u;
      acc_s[s][0] = E::to_float(static_cast<short>(w & 0xffffu));
      acc_s[s][EPL - 1] = E::to_float(static_cast<short>(w >> 16));
    } else {
      acc_s[s][0] = on ? E::to_float(a.ws_acc[p * D + lane]) : 0.f;
    }
  }
  float mn = -INFINITY;
#pragma unroll
  for (int s = 0; s < kBatch; ++s) mn = fmaxf(mn, m_s[s]);
  const float ms = mn == -INFINITY ? 0.f : mn;
  float den = 0.f, num[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) num[e] = 0.f;
#pragma unroll
  for (int s = 0; s < kBatch; ++s) {
    const float wgt = l_s[s] * fast_exp2(m_s[s] - ms);  // 0 for a share that saw no key
    den += wgt;
#pragma unroll
    for (int e = 0; e < EPL; ++e) num[e] += acc_s[s][e] * wgt;
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const float lse_nat = den > 0.f ? (mn + log2f(den)) * kLn2 : -INFINITY;
  const bool gated = a.sinks != nullptr;
  const float gate = gated ? 1.f / (1.f + __expf(a.sinks[hq] - lse_nat)) : 1.f;
  auto fin = [&](float x) { return gated ? E::round(x * inv) * gate : x * inv; };
  char* o = a.out + row * a.os_row + hq * a.os_h + lane * EPL * 2;
  if (EPL == 2)
    *reinterpret_cast<uint32_t*>(o) = E::pack2(fin(num[0]), fin(num[EPL - 1]));
  else
    *reinterpret_cast<short*>(o) = E::from_float(fin(num[0]));
  if (lane == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row] = lse_nat;
}

constexpr int kMaxKeyShares = 8;

// Key shares for a launch of `wgs` workgroups.  bf16 / f16: a launch that would leave at least half of the
// CUs idle is cut along the keys until every CU has a workgroup.  (With about one workgroup per CU
// already, a cut in two costs more in partial results and their merge than the shorter critical path
// saves: 138 us against 111 us at 8 sequences x 512 rows.)  fp32: the kernel takes about eight times as
// long over the same partial results, so the cut pays until there are about four workgroups per CU to
// even out sequences of different lengths and the last, partly filled round of workgroups (8 sequences
// x 512 rows: 962 us uncut, 838 us in four shares; one sequence of 4608 rows: 1992 us and 1315 us).
int key_shares_for(int64_t wgs, int dtype) {
  if (wgs < 1) wgs = 1;
  const int64_t n = dtype == FP_DTYPE_F32 ? (4 * fp::compute_units() + wgs / 2) / wgs : fp::compute_units() / wgs;
  return static_cast<int>(n < 1 ? 1 : n > kMaxKeyShares ? kMaxKeyShares : n);
}

// workspace of `shares` key shares: per row and head D results of elem bytes, and two floats
int64_t share_bytes(int shares, int Lq, int Hq, int D, int elem) {
  return shares <= 1 ? 0 : static_cast<int64_t>(shares) * Lq * Hq * (static_cast<int64_t>(D) * elem + 8);
}

// Scores the caller bounds (|scale * q.k| <= score_bound, natural units) take the kernel instance without a
// running maximum.  bf16 only: the probabilities span 2^(+-bound * log2 e), which bf16 (fp32's exponent
// range) holds and f16 does not; the limit keeps row sums over 2^31 keys and the accumulators inside fp32.
constexpr float kMaxScoreBound = 40.f;

template <typename E>
bool bounded_path(float score_bound) {
  return std::is_same<E, BF16>::value && score_bound > 0.f && score_bound <= kMaxScoreBound;
}

template <typename E, int D, int G, bool kPow2, int W, bool kBounded>
void launch_instance(const PrefillArgs& a, dim3 grid, hipStream_t st) {
  hipLaunchKernelGGL((paged_prefill_kernel<E, D, G, kPow2, W, kBounded>), grid, dim3(W * 64), 0, st, a);
}

template <typename E, int D, int G, int W>
void launch_main(const PrefillArgs& a, dim3 grid, bool bounded, hipStream_t st) {
  const bool pow2 = a.pd.shift >= 0;
  if constexpr (std::is_same<E, BF16>::value) {
    if (bounded) {
      if (pow2) launch_instance<E, D, G, true, W, true>(a, grid, st);
      else launch_instance<E, D, G, false, W, true>(a, grid, st);
      return;
    }
  }
  if (pow2) launch_instance<E, D, G, true, W, false>(a, grid, st);
  else launch_instance<E, D, G, false, W, false>(a, grid, st);
}

template <typename E, int D, int G>
void launch_group(const PrefillArgs& a0, float score_bound, void* workspace, int64_t workspace_bytes, hipStream_t st) {
  PrefillArgs a = a0;
  const bool bounded = bounded_path<E>(score_bound);
  constexpr int BM = (kWaves / G) * 32;
  a.n_tiles = (a.Lq + BM - 1) / BM;
  int shares = workspace ? key_shares_for(static_cast<int64_t>(a.Hc) * a.n_tiles, FP_DTYPE_BF16) : 1;  // f16 alike
  while (shares > 1 && share_bytes(shares, a.Lq, a.Hq, D, 2) > workspace_bytes) --shares;  // what the workspace holds
  if (shares > 1) {
    a.ws_ml = static_cast<float*>(workspace);
    a.ws_acc = reinterpret_cast<short*>(a.ws_ml + static_cast<int64_t>(shares) * a.Lq * a.Hq * 2);
  }
  // head_dim 64: a launch that is not cut along the keys goes out as workgroups of four wavefronts, up to
  // three to a CU.  A staged K/V tile then serves half as many query rows, but at 128-byte rows the staging is
  // cheap, the softmax (which does not shrink with head_dim) is what a step waits for, and independent
  // workgroups on a CU fill each other's barrier and set-up gaps: 8 x 512-row chunks 85 us against 91 us, the
  // same 8 sequences whole 350 us against 370 us with two per CU and 316 us with three (the instance is
  // compiled for 168 registers, a handful of values spilled outside the tile loop); 6 chunks 85 us against
  // 91 us, and where no workspace allows the cut along the keys, 1 / 4 chunks 59 / 72 us against 74 / 90 us.
  // At head_dim 128 the same split is slower (whole sequences 564 us against 485 us): the staging path is
  // the limit there, and its 242 registers allow two wavefronts per SIMD at most.
  if constexpr (G <= 4 && D == 64) {
    if (shares == 1) {
      constexpr int BM4 = (4 / G) * 32;
      a.n_tiles = (a.Lq + BM4 - 1) / BM4;
      if (a.order_rows != BM4) a.order = nullptr;
      launch_main<E, D, G, 4>(a, dim3(a.Hc, a.n_tiles, 1), bounded, st);
      return;
    }
  }
  if (a.order_rows != BM) a.order = nullptr;
  launch_main<E, D, G, kWaves>(a, dim3(a.Hc, a.n_tiles, shares), bounded, st);
  if (shares > 1) {
    const int64_t items = static_cast<int64_t>(a.Lq) * a.Hq;
    hipLaunchKernelGGL((paged_prefill_merge_kernel<E, D>), dim3(static_cast<unsigned>((items + kMergeRows - 1) / kMergeRows)),
                       dim3(kMergeRows * 64), 0, st, a, shares);
  }
}

template <typename E, int D>
int launch(const PrefillArgs& a, float score_bound, void* ws, int64_t ws_bytes, hipStream_t st) {
  switch (a.Hq / a.Hc) {
    case 1: launch_group<E, D, 1>(a, score_bound, ws, ws_bytes, st); return FP_OK;
    case 2: launch_group<E, D, 2>(a, score_bound, ws, ws_bytes, st); return FP_OK;
    case 4: launch_group<E, D, 4>(a, score_bound, ws, ws_bytes, st); return FP_OK;
    case 8: launch_group<E, D, 8>(a, score_bound, ws, ws_bytes, st); return FP_OK;
    default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: Hq/Hc = %d (supported: 1, 2, 4, 8)", a.Hq / a.Hc);
  }
}

// Rows per query tile of the launch fp_paged_prefill makes for this shape with a workspace of this size (the
// same decisions as launch_group); 0 for the fp32 kernel, which takes no order.
int tile_rows_for(int Lq, int Hq, int Hc, int D, int dtype, int64_t workspace_bytes) {
  if (dtype == FP_DTYPE_F32) return 0;
  const int g = Hq / Hc;
  const int bm = (kWaves / g) * 32;
  const int n_tiles = (Lq + bm - 1) / bm;
  int shares = workspace_bytes > 0 ? key_shares_for(static_cast<int64_t>(Hc) * n_tiles, FP_DTYPE_BF16) : 1;
  while (shares > 1 && share_bytes(shares, Lq, Hq, D, 2) > workspace_bytes) --shares;
  return (g <= 4 && D == 64 && shares == 1) ? (4 / g) * 32 : bm;
}

// Query tiles of a step ordered by the key tiles they walk, longest first.  One workgroup: the largest limit of
// every tile's rows (padding rows, sequence 0, count as 0), then every tile's rank by counting the
// tiles that go before it (among equals the later tile first, as in the order the kernel uses by itself).
constexpr int kOrderThreads = 1024;
constexpr int kOrderMaxTiles = 4096;

__global__ __launch_bounds__(kOrderThreads) void prefill_tile_order_kernel(const int64_t* __restrict__ batch_idx,
                                                                           const int32_t* __restrict__ row_limit, int Lq,
                                                                           int tile_shift, int n_tiles, int* __restrict__ order) {
  __shared__ __attribute__((aligned(16))) int s_kt[kOrderMaxTiles];
  const int tid = threadIdx.x;
  for (int t = tid; t < n_tiles; t += kOrderThreads) s_kt[t] = 0;
  __syncthreads();
  // a tile is 32 rows or more and the rows run along the lanes: the lanes of half a wavefront share a tile and
  // combine their limits by lane exchanges before one of them goes to LDS
  constexpr int kBatch = 4;  // steps whose loads are requested together
  for (int r0 = 0; r0 < Lq; r0 += kBatch * kOrderThreads) {
    int64_t seq[kBatch];
    int lim[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int r = r0 + j * kOrderThreads + tid;
      seq[j] = r < Lq ? batch_idx[r] : 0;
      lim[j] = r < Lq ? row_limit[r] : 0;
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int r = r0 + j * kOrderThreads + tid;
      int m = seq[j] != 0 ? lim[j] : 0;
#pragma unroll
      for (int off = 1; off < 32; off <<= 1) m = max(m, __shfl_xor(m, off));
      if ((tid & 31) == 0 && m > 0 && r < Lq) atomicMax(&s_kt[r >> tile_shift], m);
    }
  }
  __syncthreads();
  const int padded = (n_tiles + 3) & ~3;  // the ranking reads four tiles at a time; -1 goes before nothing
  for (int t = tid; t < padded; t += kOrderThreads) s_kt[t] = t < n_tiles ? (s_kt[t] + kTileN - 1) / kTileN : -1;
  __syncthreads();
  for (int t = tid; t < n_tiles; t += kOrderThreads) {
    const int mine = s_kt[t];
    int rank = 0;
#pragma unroll 4
    for (int u = 0; u < padded; u += 4) {
      const int4 o = *reinterpret_cast<const int4*>(&s_kt[u]);
      rank += (o.x > mine || (o.x == mine && u > t)) + (o.y > mine || (o.y == mine && u + 1 > t)) +
              (o.z > mine || (o.z == mine && u + 2 > t)) + (o.w > mine || (o.w == mine && u + 3 > t));
    }
    order[rank] = t;
  }
}

}  // namespace

extern "C" int32_t fp_paged_prefill_tile_rows(int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int dtype,
                                              int64_t workspace_bytes) {
  if (Lq < 0 || Hq <= 0 || Hc <= 0 || Hq % Hc || (D != 64 && D != 128))
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill_tile_rows: bad dimension");
  const int g = Hq / Hc;
  if (g != 1 && g != 2 && g != 4 && g != 8)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill_tile_rows: Hq/Hc = %d (supported: 1, 2, 4, 8)", g);
  if (dtype != FP_DTYPE_BF16 && dtype != FP_DTYPE_F16 && dtype != FP_DTYPE_F32)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill_tile_rows: unknown dtype %d", dtype);
  return tile_rows_for(Lq, Hq, Hc, D, dtype, workspace_bytes);
}

extern "C" int fp_paged_prefill_tile_order(const int64_t* batch_idx, const int32_t* row_limit, int32_t Lq,
                                           int32_t tile_rows, int32_t* order, void* stream) {
  if (Lq < 0) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill_tile_order: negative length");
  if (tile_rows != 32 && tile_rows != 64 && tile_rows != 128 && tile_rows != 256)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill_tile_order: tile_rows = %d (32, 64, 128 or 256: ask "
                    "fp_paged_prefill_tile_rows)", tile_rows);
  if (Lq == 0) return FP_OK;
  if (!batch_idx || !row_limit || !order) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill_tile_order: null pointer");
  const int n_tiles = (Lq + tile_rows - 1) / tile_rows;
  if (n_tiles > kOrderMaxTiles)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill_tile_order: %d query tiles (at most %d)", n_tiles, kOrderMaxTiles);
  int shift = 5;
  while ((1 << shift) < tile_rows) ++shift;
  hipLaunchKernelGGL(prefill_tile_order_kernel, dim3(1), dim3(kOrderThreads), 0, static_cast<hipStream_t>(stream), batch_idx,
                     row_limit, Lq, shift, n_tiles, order);
  return fp::check_launch("fp_paged_prefill_tile_order");
}

extern "C" int fp_paged_prefill(const void* q, int64_t q_stride_row, int64_t q_stride_h, const void* pool_k,
                                const void* pool_v, const int64_t* page_table, int64_t pt_row_stride,
                                const int64_t* batch_idx, const int32_t* row_limit, void* out,
                                int64_t out_stride_row, int64_t out_stride_h, float* lse, const float* sinks,
                                int32_t Lq, int32_t Hq,
                                int32_t Hc, int32_t D, int32_t page_size, int32_t n_pages, int32_t max_batch,
                                int64_t n_slots, float scale, float score_bound, int dtype, void* workspace,
                                int64_t workspace_bytes, const int32_t* tile_order, int32_t tile_order_rows,
                                void* stream) {
  if (dtype != FP_DTYPE_BF16 && dtype != FP_DTYPE_F16 && dtype != FP_DTYPE_F32)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: unknown dtype %d", dtype);
  if (D != 64 && D != 128) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: head_dim %d (supported: 64, 128)", D);
  if (Lq < 0 || Hq <= 0 || Hc <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 || n_slots <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: bad dimension");
  if (Hq % Hc) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: Hq=%d not a multiple of Hc=%d", Hq, Hc);
  if (n_slots < page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: n_slots smaller than one page");
  if (Hc > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: Hc exceeds 65535");
  if (n_slots > INT32_MAX) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: more than 2^31-1 slots per head");
  if (Lq == 0) return FP_OK;
  if (!q || !pool_k || !pool_v || !page_table || !batch_idx || !row_limit || !out || !lse)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: null pointer");
  if (workspace && (!fp::aligned(workspace, 16) || workspace_bytes < 0))
    return fp::fail(FP_ERR_WORKSPACE, "fp_paged_prefill: the workspace must be 16-byte aligned");
  if (dtype == FP_DTYPE_F32) {
    // fp32 has a kernel of its own on the fp32 matrix instruction
    if (!fp::aligned(q, 16) || !fp::aligned(pool_k, 16) || !fp::aligned(pool_v, 16) || !fp::aligned(out, 4) ||
        (q_stride_row * 4) % 16 || (q_stride_h * 4) % 16)
      return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: q rows must be 16-byte aligned");
    const int rc32 = fp::prefill_mfma_f32(q, q_stride_row, q_stride_h, pool_k, pool_v, page_table, pt_row_stride, batch_idx,
                                          row_limit, out, out_stride_row, out_stride_h, lse, sinks, Lq, Hq, Hc, D, page_size,
                                          n_pages, max_batch, n_slots, scale, workspace, workspace_bytes,
                                          static_cast<hipStream_t>(stream));
    if (rc32 != FP_OK) return rc32;
    return fp::check_launch("fp_paged_prefill");
  }
  if (!fp::aligned(q, 16) || !fp::aligned(pool_k, 16) || !fp::aligned(pool_v, 16) || !fp::aligned(out, 8) ||
      (q_stride_row * 2) % 16 || (q_stride_h * 2) % 16 || (out_stride_row * 2) % 8 || (out_stride_h * 2) % 8)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill: q rows must be 16-byte and out rows 8-byte aligned");
  if ((static_cast<int64_t>(Lq) + 31) / 32 > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: too many query rows");
  PrefillArgs a{static_cast<const char*>(q), q_stride_row * 2, q_stride_h * 2,
                static_cast<const char*>(pool_k), static_cast<const char*>(pool_v),
                page_table, pt_row_stride, batch_idx, row_limit,
                static_cast<char*>(out), out_stride_row * 2, out_stride_h * 2, lse, sinks,
                Lq, Hq, Hc, fp::PageDiv(page_size), n_pages, max_batch, n_slots, scale * kLog2e, 0, nullptr, nullptr,
                tile_order, tile_order ? tile_order_rows : 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
  if (dtype == FP_DTYPE_BF16)
    rc = D == 64 ? launch<BF16, 64>(a, score_bound, workspace, workspace_bytes, st)
                 : launch<BF16, 128>(a, score_bound, workspace, workspace_bytes, st);
  else
    rc = D == 64 ? launch<F16, 64>(a, score_bound, workspace, workspace_bytes, st)
                 : launch<F16, 128>(a, score_bound, workspace, workspace_bytes, st);
  if (rc != FP_OK) return rc;
  return fp::check_launch("fp_paged_prefill");
}

extern "C" int64_t fp_paged_prefill_workspace_bytes(int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int dtype) {
  if (Lq < 0 || Hq <= 0 || Hc <= 0 || Hq % Hc || (D != 64 && D != 128))
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_paged_prefill_workspace_bytes: bad dimension");
  const int g = Hq / Hc;
  if (g != 1 && g != 2 && g != 4 && g != 8)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill_workspace_bytes: Hq/Hc = %d (supported: 1, 2, 4, 8)", g);
  if (Lq == 0) return 0;
  if (dtype != FP_DTYPE_BF16 && dtype != FP_DTYPE_F16 && dtype != FP_DTYPE_F32)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill_workspace_bytes: unknown dtype %d", dtype);
  const int bm = (kWaves / g) * 32;
  return share_bytes(key_shares_for(static_cast<int64_t>(Hc) * ((Lq + bm - 1) / bm), dtype), Lq, Hq, D,
                     fp::elem_bytes(dtype));
}

int fp::prefill_key_shares(int64_t wgs, int dtype) { return key_shares_for(wgs, dtype); }
int64_t fp::prefill_share_bytes(int shares, int Lq, int Hq, int D, int elem) { return share_bytes(shares, Lq, Hq, D, elem); }
