// KV append: slot-mapping scatter of new K/V rows into the page pool.
//
// Semantics follow PagedKVCache.assign (reference paged_attention.py:184-232) and
// PagedKVCache.assign_prefill_no_paging (:364-393): a pure byte copy of each
// (token, head) row to pool[h, page_table[batch_idx, pos / P] * P + pos % P, :].
//
// HBM-bound.  A row is D * elem bytes (256 B at D = 128 bf16); it is moved as 16-byte
// vectors (8/4/2-byte ones when alignment asks for it), ONE vector of K and one of V per lane.
// The lanes of a launch run over the source in its memory order: for the [T, H, D] rows the
// model produces (reference model.py:116-119) over (token, head, chunk), so that consecutive
// lanes read consecutive bytes and each row is written as one 256-byte piece of its page.
// Measured at 32768 tokens x 16 heads (537 MB moved; a plain copy of that size takes 90 us):
// 98-102 us whatever the buffers' placement in memory.  More vectors per lane are slower (2: 104 us,
// 4: 107 us, 8: 117 us); a grid of (row tiles, heads) with lanes over the tokens of one head, which
// reads 256-byte pieces 4 KiB apart, takes 93 us or 115 us depending on where the allocator
// placed the buffers (the same process sees both), and dealing those workgroups so that the heads
// of a row tile run back to back on one XCD gives 98-103 us.
// The slot is computed in the kernel from the page table, there is no separate slot-mapping pass.
// Loads and stores are non-temporal: the rows are touched once and should not displace
// cache lines other kernels reuse.
#include "fp_common.h"

namespace {

// clang vector types: the non-temporal load/store builtins take these, not HIP's uint4
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

struct AppendArgs {
  char* pool_k;
  char* pool_v;
  const char* k;
  const char* v;
  int64_t ks_t, ks_h, ks_s;  // byte strides of k
  int64_t vs_t, vs_h, vs_s;  // byte strides of v
  const int64_t* page_table;
  int64_t pt_row_stride;
  const int64_t* batch_idx;
  const void* input_pos;
  int pos_i64;
  int n_tok;   // T * S
  int S;
  int chunks;  // vectors per row
  int row_bytes;
  fp::PageDiv pd;
  int n_pages;
  int max_batch;
  int64_t n_slots;
  int clamp_negative;
  int64_t item0;  // first item of this launch: a launch holds fewer than 2^32 lanes, a larger append is several
};

constexpr int kThreads = 256;

// One 16-byte vector of K and one of V per lane.  kTokenMajor: lanes run over (token, head, chunk), the
// order of a [T, H, D] source, so a load instruction reads consecutive source bytes and every row leaves
// as one 256-byte piece; otherwise grid.y = head and lanes run over (token, chunk), the order of a
// [H, T, D] source, where source and destination are both contiguous per head.  Idx = uint32_t whenever
// the item count allows (one division per lane instead of a 64-bit one).
template <typename Vec, bool kTokenMajor, typename Idx>
__global__ __launch_bounds__(kThreads) void kv_append_kernel(const AppendArgs a, int H) {
  const Idx per_tok = kTokenMajor ? static_cast<Idx>(H) * a.chunks : static_cast<Idx>(a.chunks);
  const Idx items = static_cast<Idx>(a.n_tok) * per_tok;
  const Idx i = static_cast<Idx>(a.item0) + static_cast<Idx>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= items) return;
  const int tok = static_cast<int>(i / per_tok);
  int c = static_cast<int>(i - static_cast<Idx>(tok) * per_tok);
  int h = blockIdx.y;
  if (kTokenMajor) {
    h = c / a.chunks;
    c -= h * a.chunks;
  }
  int t = tok, s = 0;
  if (a.S != 1) {
    t = tok / a.S;
    s = tok - t * a.S;
  }
  const int64_t ko = t * a.ks_t + h * a.ks_h + s * a.ks_s + static_cast<int64_t>(c) * sizeof(Vec);
  const int64_t vo = t * a.vs_t + h * a.vs_h + s * a.vs_s + static_cast<int64_t>(c) * sizeof(Vec);
  const Vec kreg = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(a.k + ko));
  const Vec vreg = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(a.v + vo));

  const int64_t b = a.batch_idx[t];
  const int64_t pos = fp::load_index(a.input_pos, tok, a.pos_i64);
  if (b < 0 || b >= a.max_batch || pos < 0) return;
  int64_t blk;
  int off;
  a.pd.split(pos, blk, off);
  if (blk >= a.n_pages) return;
  int64_t page = a.page_table[b * a.pt_row_stride + blk];
  if (a.clamp_negative && page < 0) page = 0;
  int64_t slot = page * a.pd.page_size + off;
  if (slot < 0) slot += a.n_slots;  // negative index counts from the end of the slot axis
  if (slot < 0 || slot >= a.n_slots) return;
  const int64_t dst = (static_cast<int64_t>(h) * a.n_slots + slot) * a.row_bytes + static_cast<int64_t>(c) * sizeof(Vec);
  __builtin_nontemporal_store(kreg, reinterpret_cast<Vec*>(a.pool_k + dst));
  __builtin_nontemporal_store(vreg, reinterpret_cast<Vec*>(a.pool_v + dst));
}

// A dispatch holds fewer than 2^32 lanes in each grid dimension: a larger append goes out as several launches of
// 2^31 lanes, each told where its items start.
constexpr int64_t kLaunchBlocks = (1ll << 31) / kThreads;

template <typename Vec>
int launch(const AppendArgs& a0, int H, hipStream_t stream) {
  // the source's memory order decides which index runs fastest across the lanes
  const bool token_major = a0.ks_h <= a0.ks_t && a0.vs_h <= a0.vs_t;
  const int64_t per_grid_row = static_cast<int64_t>(a0.n_tok) * a0.chunks * (token_major ? H : 1);
  const int64_t blocks = (per_grid_row + kThreads - 1) / kThreads;
  const bool narrow = per_grid_row + kThreads < (1ll << 32);
  AppendArgs a = a0;
  for (int64_t b0 = 0; b0 < blocks; b0 += kLaunchBlocks) {
    a.item0 = b0 * kThreads;
    const int64_t nb = blocks - b0 < kLaunchBlocks ? blocks - b0 : kLaunchBlocks;
    dim3 grid(static_cast<unsigned>(nb), token_major ? 1u : static_cast<unsigned>(H));
    if (token_major) {
      if (narrow)
        hipLaunchKernelGGL((kv_append_kernel<Vec, true, uint32_t>), grid, dim3(kThreads), 0, stream, a, H);
      else
        hipLaunchKernelGGL((kv_append_kernel<Vec, true, int64_t>), grid, dim3(kThreads), 0, stream, a, H);
    } else {
      if (narrow)
        hipLaunchKernelGGL((kv_append_kernel<Vec, false, uint32_t>), grid, dim3(kThreads), 0, stream, a, H);
      else
        hipLaunchKernelGGL((kv_append_kernel<Vec, false, int64_t>), grid, dim3(kThreads), 0, stream, a, H);
    }
  }
  return FP_OK;
}

}  // namespace

extern "C" int fp_kv_append(void* pool_k, void* pool_v, const void* k, const void* v,
                            int64_t k_stride_t, int64_t k_stride_h, int64_t k_stride_s,
                            int64_t v_stride_t, int64_t v_stride_h, int64_t v_stride_s,
                            const int64_t* page_table, int64_t pt_row_stride,
                            const int64_t* batch_idx, const void* input_pos, int pos_index_type,
                            int32_t T, int32_t H, int32_t S, int32_t D, int32_t page_size,
                            int32_t n_pages, int32_t max_batch, int64_t n_slots, int dtype,
                            int clamp_negative, void* stream) {
  const int eb = fp::elem_bytes(dtype);
  if (eb == 0) return fp::fail(FP_ERR_UNSUPPORTED, "fp_kv_append: unknown dtype %d", dtype);
  if (T < 0 || H <= 0 || S <= 0 || D <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 || n_slots <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_append: non-positive dimension");
  if (H > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_kv_append: H=%d exceeds 65535", H);
  if (static_cast<int64_t>(T) * S > INT32_MAX)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_kv_append: more than 2^31-1 tokens");
  if (n_slots < page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_append: n_slots smaller than one page");
  if (pos_index_type != FP_INDEX_I32 && pos_index_type != FP_INDEX_I64)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_append: bad pos_index_type");
  if (T == 0) return FP_OK;
  if (!pool_k || !pool_v || !k || !v || !page_table || !batch_idx || !input_pos)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_append: null pointer");

  AppendArgs a{static_cast<char*>(pool_k), static_cast<char*>(pool_v),
               static_cast<const char*>(k), static_cast<const char*>(v),
               k_stride_t * eb, k_stride_h * eb, k_stride_s * eb,
               v_stride_t * eb, v_stride_h * eb, v_stride_s * eb,
               page_table, pt_row_stride, batch_idx, input_pos,
               pos_index_type == FP_INDEX_I64, T * S, S, 0, D * eb, fp::PageDiv(page_size),
               n_pages, max_batch, n_slots, clamp_negative, 0};

  // widest vector every row address is a multiple of
  int vec = 16;
  auto fits = [&](int n) {
    return a.row_bytes % n == 0 && a.ks_t % n == 0 && a.ks_h % n == 0 && a.ks_s % n == 0 &&
           a.vs_t % n == 0 && a.vs_h % n == 0 && a.vs_s % n == 0 && fp::aligned(pool_k, n) &&
           fp::aligned(pool_v, n) && fp::aligned(k, n) && fp::aligned(v, n);
  };
  while (vec > eb && !fits(vec)) vec >>= 1;
  if (!fits(vec)) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_append: pointers not aligned to the element size");
  a.chunks = a.row_bytes / vec;

  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
  switch (vec) {
    case 16: rc = launch<v4u>(a, H, st); break;
    case 8: rc = launch<v2u>(a, H, st); break;
    case 4: rc = launch<uint32_t>(a, H, st); break;
    default: rc = launch<uint16_t>(a, H, st); break;
  }
  if (rc != FP_OK) return rc;
  return fp::check_launch("fp_kv_append");
}
