// Chunked-prefill attention over the paged cache under the hybrid mask, fp32 (the reference's
// default dtype, server/config.py:38) on the fp32 matrix instruction v_mfma_f32_32x32x2_f32.
//
// Same contract as the bf16 / f16 kernel (paged_prefill.hip; reference attention.py:18 as called
// at model.py:156-162, mask paged_attention.py:343-362): row r of the packed queries sees keys
// 0 .. row_limit[r] - 1 of sequence batch_idx[r], fetched through the page table.
//
// MFMA-bound by a wide margin (a 32-key tile costs a wavefront 128 matrix instructions of 64 cycles
// and ~100 vector instructions), so the structure is the plain one: a workgroup of 8 wavefronts owns
// one cache head and 256 / G packed query rows of each of its G query heads, a wavefront 32 rows of
// one head; K/V tiles of 32 keys are double-buffered in LDS, one barrier per tile.
//   S^T = K Q^T : a lane holds the scores of ONE query (softmax reductions stay in registers plus
//                 one exchange between the lane halves); Q is scaled when it is loaded.
//   O^T = V^T P^T : P^T is the B operand as it leaves the softmax; the A operand is read from the
//                 row-major V tile one float per lane.
#include "fp_common.h"
#include "prefill_common.h"

#include <math.h>

namespace {

using fp::load_to_lds;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kTileN = 32;         // keys per tile
constexpr float kMaxSlack = 6.f;   // the running maximum may lag a row's true maximum by this much (log2)
constexpr int kSlotTable = 4096;   // tiles of a run whose first pool slot is looked up ahead of the tile loop
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) const char* lds_ptr;  // a 32-bit LDS address

constexpr f32x16 kZero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

template <int N>
struct IntC {
  static constexpr int value = N;
};

struct Args {
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
  // key shares (grid z): unnormalised partial results for the merge pass, as in the bf16 / f16 kernel
  float* ws_acc;  // [shares, Lq, Hq, D]
  float* ws_ml;   // [shares, Lq, Hq, 2]: running maximum (log2 units), denominator
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ f32x16 mfma(float a, float b, const f32x16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// LDS layout of a tile: 32 unpadded rows of D floats, filled 16 bytes per lane.  The 16-byte chunks of
// a row are permuted on the GLOBAL side of the load so that the operand reads meet no bank conflict:
//   K: chunk c of row r sits at position c ^ (r % 16).  The S^T operand read takes one chunk of 16
//      consecutive rows at a time, which then fall into 16 different positions.
//   V: chunk c of row r sits at position c ^ 8 when (r / 4) is odd.  The O^T operand read takes 32
//      consecutive floats of row k in one lane half and of row k + 4 in the other.
__device__ __forceinline__ int kswz(int r) { return r & 15; }
__device__ __forceinline__ int vswz(int r) { return ((r >> 2) & 1) << 3; }

template <int D, int G, bool kPow2>
__global__ __launch_bounds__(kThreads, 2) void paged_prefill_f32_kernel(const Args a) {
  constexpr int RB = kWaves / G;           // 32-row blocks per workgroup
  constexpr int BM = RB * 32;              // query rows per workgroup
  constexpr int ROWB = D * 4;              // bytes of a K/V row
  constexpr int CPR = ROWB / 16;           // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;            // rows one wavefront load instruction brings in
  constexpr int NI = kTileN / (RPI * kWaves);  // load instructions per wavefront, tile and tensor
  constexpr int DC = D / 8;                // groups of 8 head_dim elements = 4 MFMA k-steps of both lane halves
  constexpr int DB = D / 32;               // 32-wide blocks of head_dim in O^T
  constexpr int TILE_BYTES = kTileN * ROWB;
  static_assert(NI >= 1 && CPR >= 16, "head_dim 64 or 128");

  __shared__ __attribute__((aligned(1024))) char s_k0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_k1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_v0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) char s_v1[TILE_BYTES];
  __shared__ int s_bidx[BM];
  __shared__ int s_red[kWaves];
  __shared__ int s_tslot[kSlotTable];

  // linear id = cache head + Hc * tile: all tiles that read one cache head run on the XCD that
  // already holds its K/V in L2
  const int hc = blockIdx.x;
  const int tile = a.n_tiles - 1 - blockIdx.y;  // later rows see more keys: longest first
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hq = hc * G + wave % G;  // query head of this wavefront
  const int rblock = wave / G;       // its block of 32 rows inside the tile
  const int lane = tid & 63;
  const int half = lane >> 5;   // which of the 2 k-values of an MFMA step this lane holds
  const int ln = lane & 31;     // query column (S^T, O^T), key row (K operand) or head_dim row (V operand)
  const int tile0 = tile * BM;

  // Everything the set-up needs from global memory is requested at once: the sequence of each row
  // of the tile, then this wavefront's row limit and Q row.  Rows outside a run keep their Q values:
  // what such a row computes is never stored.
  const int bi_row = tile0 + tid;
  const int64_t bx_raw = (tid < BM && bi_row < a.Lq) ? a.batch_idx[bi_row] : 0;
  const int row = tile0 + rblock * 32 + ln;
  const bool in_rows = row < a.Lq;
  const int lim_raw = in_rows ? a.row_limit[row] : 0;
  // Q^T operands, scaled: lane (query ln, half) holds d = 8 c + 4 half .. + 3 of group c
  f32x4 qreg[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    f32x4 w = {0, 0, 0, 0};
    if (in_rows) w = *reinterpret_cast<const f32x4*>(a.q + row * a.qs_row + hq * a.qs_h + (8 * c + 4 * half) * 4);
    qreg[c] = w * a.qscale;
  }
  if (tid < BM) {
    int64_t bx = bx_raw;
    if (bx < 0 || bx >= a.max_batch) bx = 0;
    s_bidx[tid] = static_cast<int>(bx);
  }
  __syncthreads();

  const char* kplane = a.pool_k + static_cast<int64_t>(hc) * a.n_slots * ROWB;
  const char* vplane = a.pool_v + static_cast<int64_t>(hc) * a.n_slots * ROWB;

  // ---- per-lane constants of the staging loads and of the operand reads ----
  // load instruction i of this wavefront fills LDS rows (i * kWaves + wave) * RPI .. + RPI; this lane
  // fills position lp of row lrow in that group.  kswz / vswz of the row do not depend on i.
  const int lrow = lane / CPR;
  const int lp = lane % CPR;
  const int st_row0 = wave * RPI + lrow;  // row of load instruction 0; instruction i adds i * kWaves * RPI
  const int k_src_off = (lp ^ kswz(st_row0)) * 16;
  const int v_src_off = (lp ^ vswz(st_row0)) * 16;
  // byte offset of this lane's 16 bytes from the first row of its row group
  const uint32_t lane_k = st_row0 * ROWB + k_src_off;
  const uint32_t lane_v = st_row0 * ROWB + v_src_off;
  // K operand of group c: row ln, chunk 2 c + half, at position (2 c + half) ^ kswz(ln) = (2 c) ^ ksel;
  // a row starts on a multiple of its size, so the address is that of group 0 with 32 c XORed in
  const int ksel = half ^ kswz(ln);
  const uint32_t kofs0 = ln * ROWB + ksel * 16;
  // V operand of step x (score register x of the lane: key (x / 4) * 8 + half * 4 + x % 4) and block db:
  // row = that key, float db * 32 + ln; vswz of the row is 8 * half
  uint32_t vofs[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) vofs[db] = half * 4 * ROWB + (((db * 8 + (ln >> 2)) ^ (half * 8)) * 16) + (ln & 3) * 4;

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

    const int tr = rblock * 32 + ln;  // this lane's row inside the tile
    const bool active = tr >= run0 && tr < run1 && in_rows;
    int lim = (active && sq != 0) ? lim_raw : 0;
    if (lim < 0) lim = 0;

    if (sq == 0) {
      // padding rows: out = 0, lse = -inf; each lane half clears half of the row
      if (active && gridDim.z > 1) {  // an empty share; the merge pass then writes out = 0, lse = -inf
        const int64_t p = (static_cast<int64_t>(blockIdx.z) * a.Lq + row) * a.Hq + hq;
#pragma unroll
        for (int c = 0; c < D / 8; ++c) *reinterpret_cast<f32x4*>(a.ws_acc + p * D + half * (D / 2) + c * 4) = f32x4{0, 0, 0, 0};
        if (half == 0) *reinterpret_cast<float2*>(a.ws_ml + p * 2) = float2{-INFINITY, 0.f};
      } else if (active) {
        float* o = reinterpret_cast<float*>(a.out + row * a.os_row + hq * a.os_h) + half * (D / 2);
#pragma unroll
        for (int c = 0; c < D / 2; ++c) o[c] = 0.f;
        if (half == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row] = -INFINITY;
      }
      run0 = run1;
      continue;
    }

    // key range of the run: wavefront maximum, then workgroup maximum
    int wave_max = lim;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) wave_max = max(wave_max, __shfl_xor(wave_max, off));
    wave_max = __builtin_amdgcn_readfirstlane(wave_max);
    int wave_min = active ? lim : 0x7fffffff;  // smallest limit among the active rows (tiles below it need no masking)
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) wave_min = min(wave_min, __shfl_xor(wave_min, off));
    wave_min = __builtin_amdgcn_readfirstlane(wave_min);
    __syncthreads();  // s_red, s_tslot and the LDS tiles of the previous run are free
    if (lane == 0) s_red[wave] = wave_max;
    __syncthreads();
    int kv_max = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) kv_max = max(kv_max, s_red[w]);
    kv_max = __builtin_amdgcn_readfirstlane(kv_max);
    const int n_run_tiles = (kv_max + kTileN - 1) / kTileN;
    // this workgroup's share of the run's key tiles: [kt_lo, n_kv_tiles)
    const int kt_lo = static_cast<int>(static_cast<int64_t>(n_run_tiles) * blockIdx.z / gridDim.z);
    const int n_kv_tiles = static_cast<int>(static_cast<int64_t>(n_run_tiles) * (blockIdx.z + 1) / gridDim.z);

    f32x16 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o_acc[db] = kZero16;
    float m_run = -INFINITY, l_run = 0.f;

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
    // Stages this wavefront's rows of tile kt (first slot ts, or -1) into the K and V buffers given.
    // Tiles past the run's last one are not staged.
    auto stage = [&](int kt, int ts, char* kdst, char* vdst) {
      if (kt >= n_kv_tiles) return;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int group = (i * kWaves + wave) * RPI * ROWB;  // wavefront-uniform LDS offset
        if (ts >= 0) {
          const int64_t base = (static_cast<int64_t>(ts) + i * kWaves * RPI) * ROWB;
          load_to_lds(kplane + base, lane_k, kdst + group);
          load_to_lds(vplane + base, lane_v, vdst + group);
        } else {
          const int kpos = kt * kTileN + i * kWaves * RPI + st_row0;
          int blkid, off;
          key_block(kpos, blkid, off);
          const bool in_range = kpos < kv_max && blkid < a.n_pages;
          const int64_t pg = pt_row[in_range ? blkid : 0];
          const bool ok = in_range && pg >= 0 && pg < pool_pages;
          const int64_t rowbyte = static_cast<int64_t>(ok ? static_cast<int>(pg) * a.pd.page_size + off : 0) * ROWB;
          load_to_lds(kplane + rowbyte + k_src_off, kdst + group);
          load_to_lds(vplane + rowbyte + v_src_off, vdst + group);
        }
      }
    };

    stage(kt_lo, tile_slot(kt_lo), s_k0, s_v0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's rows have landed in LDS
    __syncthreads();

    // one tile: stage tile kt + 1 into the other buffers while working on tile kt
    auto tile_step = [&](auto parity, int kt) {
      constexpr int kBuf = decltype(parity)::value;
      const lds_ptr kcur = (lds_ptr)(kBuf ? s_k1 : s_k0);
      const lds_ptr vcur = (lds_ptr)(kBuf ? s_v1 : s_v0);
      stage(kt + 1, tile_slot(kt + 1), kBuf ? s_k0 : s_k1, kBuf ? s_v0 : s_v1);

      const int key0 = kt * kTileN;
      if (key0 < wave_max) {
        // ---- S^T = K Q^T for the 32 keys of the tile: D / 2 MFMA steps, one 16-byte read per 4 ----
        f32x16 s_acc = kZero16;
        auto read_k = [&](int c) {
          return *reinterpret_cast<__attribute__((address_space(3))) const f32x4*>(kcur + (kofs0 ^ (32u * c)));
        };
        f32x4 kr[2];
        kr[0] = read_k(0);
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          if (c + 1 < DC) kr[(c + 1) & 1] = read_k(c + 1);
          const f32x4 kv = kr[c & 1];
#pragma unroll
          for (int t = 0; t < 4; ++t) s_acc = mfma(kv[t], qreg[c][t], s_acc);
        }

        // ---- online softmax, one query per lane; score x of the lane is key (x / 4) * 8 + half * 4 + x % 4 ----
        float sc[16];
#pragma unroll
        for (int x = 0; x < 16; ++x) sc[x] = s_acc[x];
        if (key0 + kTileN > wave_min) {
          asm volatile("");  // keeps this a branch: turned into selects it would run on every tile
          const int rel = lim - key0 - half * 4;
#pragma unroll
          for (int x = 0; x < 16; ++x) sc[x] = ((x >> 2) * 8 + (x & 3)) < rel ? sc[x] : -INFINITY;
        }
        float mx = sc[0];
#pragma unroll
        for (int x = 1; x < 16; ++x) mx = fmaxf(mx, sc[x]);
        mx = fp::max_across_lane_halves(mx);
        // Lazy running maximum: the reference point m_run only moves when some row's maximum has grown by
        // more than kMaxSlack (log2 units); until then exp2(s - m_run) may reach 2^kMaxSlack, harmless in
        // fp32, and the accumulators need no rescale.
        const bool moved = __any(mx > m_run + kMaxSlack);
        const float m_new = moved ? fmaxf(m_run, mx) : m_run;
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = moved ? fast_exp2(m_run - m_safe) : 1.f;
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          sc[x] = fast_exp2(sc[x] - m_safe);
          psum += sc[x];
        }
        l_run = fmaf(l_run, alpha, psum);  // alpha is 1 unless the reference point moved
        if (moved) {
          asm volatile("");  // the rescale is rare and must not run unconditionally
#pragma unroll
          for (int db = 0; db < DB; ++db) o_acc[db] *= alpha;
        }

        // ---- O^T += V^T P^T: step x pairs key (x / 4) * 8 + x % 4 (first lane half) with the key 4 rows on ----
        auto read_v = [&](int t) {
          const int x = t / DB, db = t % DB;
          return *reinterpret_cast<__attribute__((address_space(3))) const float*>(vcur + vofs[db] + ((x >> 2) * 8 + (x & 3)) * ROWB);
        };
        constexpr int kAhead = 4;
        float vr[kAhead];
#pragma unroll
        for (int t = 0; t < kAhead; ++t) vr[t] = read_v(t);
#pragma unroll
        for (int t = 0; t < 16 * DB; ++t) {
          const float va = vr[t % kAhead];
          if (t + kAhead < 16 * DB) vr[t % kAhead] = read_v(t + kAhead);
          o_acc[t % DB] = mfma(va, sc[t / DB], o_acc[t % DB]);
        }
      }

      __builtin_amdgcn_s_waitcnt(0x0F70);  // this wavefront's share of tile kt + 1 has landed
      __syncthreads();
    };

    for (int kt = kt_lo; kt < n_kv_tiles; kt += 2) {
      tile_step(IntC<0>{}, kt);
      if (kt + 1 < n_kv_tiles) tile_step(IntC<1>{}, kt + 1);
    }

    // ---- finish the run: normalise and store ----
    {
      const float l_tot = l_run + __shfl_xor(l_run, 32);
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
      if (active && gridDim.z > 1) {
        // one of several key shares: the unnormalised state goes to the merge pass
        const int64_t p = (static_cast<int64_t>(blockIdx.z) * a.Lq + row) * a.Hq + hq;
        float* po = a.ws_acc + p * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            *reinterpret_cast<f32x4*>(po + db * 32 + i4 * 8 + half * 4) =
                f32x4{o_acc[db][i4 * 4], o_acc[db][i4 * 4 + 1], o_acc[db][i4 * 4 + 2], o_acc[db][i4 * 4 + 3]};
        if (half == 0) *reinterpret_cast<float2*>(a.ws_ml + p * 2) = float2{m_run, l_tot};
      } else if (active) {
        float* o = reinterpret_cast<float*>(a.out + row * a.os_row + hq * a.os_h);
        const float lse_nat = l_tot > 0.f ? (m_run + log2f(l_tot)) * kLn2 : -INFINITY;
        // attention-sink gate of the caller's post-attention step (model.py:122-128)
        const float gate = a.sinks != nullptr ? 1.f / (1.f + __expf(a.sinks[hq] - lse_nat)) : 1.f;
        const float f = inv * gate;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            // register r holds d = db * 32 + (r / 4) * 8 + half * 4 + r % 4
            o[db * 32 + (r >> 2) * 8 + half * 4 + (r & 3)] = o_acc[db][r] * f;
          }
        }
        if (half == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row] = lse_nat;
      }
    }
    run0 = run1;
  }
}

// ---- merge of the key shares: one wavefront per (query row, query head) ----
constexpr int kMergeRows = 4;  // (row, head) pairs per workgroup

template <int D>
__global__ __launch_bounds__(kMergeRows * 64) void paged_prefill_f32_merge_kernel(const Args a, int n_shares) {
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
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc_s[s][e] = on ? a.ws_acc[p * D + lane * EPL + e] : 0.f;
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
    const float wgt = fast_exp2(m_s[s] - ms);  // 0 for a share that saw no key
    den += l_s[s] * wgt;
#pragma unroll
    for (int e = 0; e < EPL; ++e) num[e] += acc_s[s][e] * wgt;
  }
  const float lse_nat = den > 0.f ? (mn + log2f(den)) * kLn2 : -INFINITY;
  const float gate = a.sinks != nullptr ? 1.f / (1.f + __expf(a.sinks[hq] - lse_nat)) : 1.f;
  const float f = (den > 0.f ? 1.f / den : 0.f) * gate;
  float* o = reinterpret_cast<float*>(a.out + row * a.os_row + hq * a.os_h) + lane * EPL;
#pragma unroll
  for (int e = 0; e < EPL; ++e) o[e] = num[e] * f;
  if (lane == 0) a.lse[static_cast<int64_t>(hq) * a.Lq + row] = lse_nat;
}

template <int D, int G>
void launch_group(const Args& a0, void* workspace, int64_t workspace_bytes, hipStream_t st) {
  Args a = a0;
  constexpr int BM = (kWaves / G) * 32;
  a.n_tiles = (a.Lq + BM - 1) / BM;
  int shares = workspace ? fp::prefill_key_shares(static_cast<int64_t>(a.Hc) * a.n_tiles, FP_DTYPE_F32) : 1;
  while (shares > 1 && fp::prefill_share_bytes(shares, a.Lq, a.Hq, D, 4) > workspace_bytes) --shares;
  if (shares > 1) {
    a.ws_acc = static_cast<float*>(workspace);
    a.ws_ml = a.ws_acc + static_cast<int64_t>(shares) * a.Lq * a.Hq * D;
  }
  dim3 grid(a.Hc, a.n_tiles, shares);
  if (a.pd.shift >= 0)
    hipLaunchKernelGGL((paged_prefill_f32_kernel<D, G, true>), grid, dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((paged_prefill_f32_kernel<D, G, false>), grid, dim3(kThreads), 0, st, a);
  if (shares > 1) {
    const int64_t items = static_cast<int64_t>(a.Lq) * a.Hq;
    hipLaunchKernelGGL((paged_prefill_f32_merge_kernel<D>), dim3(static_cast<unsigned>((items + kMergeRows - 1) / kMergeRows)),
                       dim3(kMergeRows * 64), 0, st, a, shares);
  }
}

template <int D>
int launch(const Args& a, void* ws, int64_t ws_bytes, hipStream_t st) {
  switch (a.Hq / a.Hc) {
    case 1: launch_group<D, 1>(a, ws, ws_bytes, st); return FP_OK;
    case 2: launch_group<D, 2>(a, ws, ws_bytes, st); return FP_OK;
    case 4: launch_group<D, 4>(a, ws, ws_bytes, st); return FP_OK;
    case 8: launch_group<D, 8>(a, ws, ws_bytes, st); return FP_OK;
    default: return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: Hq/Hc = %d (supported: 1, 2, 4, 8)", a.Hq / a.Hc);
  }
}

}  // namespace

namespace fp {

int prefill_mfma_f32(const void* q, int64_t q_stride_row, int64_t q_stride_h, const void* pool_k, const void* pool_v,
                     const int64_t* page_table, int64_t pt_row_stride, const int64_t* batch_idx,
                     const int32_t* row_limit, void* out, int64_t out_stride_row, int64_t out_stride_h, float* lse,
                     const float* sinks, int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int32_t page_size,
                     int32_t n_pages, int32_t max_batch, int64_t n_slots, float scale, void* workspace,
                     int64_t workspace_bytes, hipStream_t st) {
  if ((static_cast<int64_t>(Lq) + 31) / 32 > 65535) return fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: too many query rows");
  Args a{static_cast<const char*>(q), q_stride_row * 4, q_stride_h * 4,
         static_cast<const char*>(pool_k), static_cast<const char*>(pool_v),
         page_table, pt_row_stride, batch_idx, row_limit,
         static_cast<char*>(out), out_stride_row * 4, out_stride_h * 4, lse, sinks,
         Lq, Hq, Hc, PageDiv(page_size), n_pages, max_batch, n_slots, scale * kLog2e, 0, nullptr, nullptr};
  return D == 64 ? launch<64>(a, workspace, workspace_bytes, st) : launch<128>(a, workspace, workspace_bytes, st);
}

}  // namespace fp
