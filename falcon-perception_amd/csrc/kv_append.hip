// KV append: slot-mapping scatter of new K/V rows into the page pool.
//
// Semantics follow PagedKVCache.assign (reference paged_attention.py:184-232) and
// PagedKVCache.assign_prefill_no_paging (:364-393): a pure byte copy of each
// (token, head) row to pool[h, page_table[batch_idx, pos / P] * P + pos % P, :].
//
// HBM-bound.  A row is D * elem bytes (256 B at D = 128 bf16); it is moved as
// 16-byte vectors, one vector of K and one of V per lane, four such pairs in
// flight per lane.  Lanes run fastest over the bytes of a row, then over tokens
// of one head, so a wavefront writes consecutive slots of a page as one
// contiguous run and reads whole 256-byte rows of the source.  The slot is
// computed in the kernel from the page table, there is no separate slot-mapping pass.
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
};

constexpr int kThreads = 256;
constexpr int kItems = 4;  // (K, V) vector pairs per lane

template <typename Vec>
__global__ __launch_bounds__(kThreads) void kv_append_kernel(const AppendArgs a) {
  const int h = blockIdx.y;
  const int64_t items = static_cast<int64_t>(a.n_tok) * a.chunks;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kItems) + threadIdx.x;

  Vec kreg[kItems], vreg[kItems];
  int64_t dst[kItems];

#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int64_t i = base + static_cast<int64_t>(j) * kThreads;
    dst[j] = -1;
    if (i >= items) continue;
    const int tok = static_cast<int>(i / a.chunks);
    const int c = static_cast<int>(i - static_cast<int64_t>(tok) * a.chunks);
    int t = tok, s = 0;
    if (a.S != 1) {
      t = tok / a.S;
      s = tok - t * a.S;
    }
    const int64_t ko = t * a.ks_t + h * a.ks_h + s * a.ks_s + static_cast<int64_t>(c) * sizeof(Vec);
    const int64_t vo = t * a.vs_t + h * a.vs_h + s * a.vs_s + static_cast<int64_t>(c) * sizeof(Vec);
    kreg[j] = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(a.k + ko));
    vreg[j] = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(a.v + vo));

    const int64_t b = a.batch_idx[t];
    const int64_t pos = fp::load_index(a.input_pos, tok, a.pos_i64);
    if (b < 0 || b >= a.max_batch || pos < 0) continue;
    int64_t blk;
    int off;
    a.pd.split(pos, blk, off);
    if (blk >= a.n_pages) continue;
    int64_t page = a.page_table[b * a.pt_row_stride + blk];
    if (a.clamp_negative && page < 0) page = 0;
    int64_t slot = page * a.pd.page_size + off;
    if (slot < 0) slot += a.n_slots;  // negative index counts from the end of the slot axis
    if (slot < 0 || slot >= a.n_slots) continue;
    dst[j] = (static_cast<int64_t>(h) * a.n_slots + slot) * a.row_bytes + static_cast<int64_t>(c) * sizeof(Vec);
  }

#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    if (dst[j] < 0) continue;
    __builtin_nontemporal_store(kreg[j], reinterpret_cast<Vec*>(a.pool_k + dst[j]));
    __builtin_nontemporal_store(vreg[j], reinterpret_cast<Vec*>(a.pool_v + dst[j]));
  }
}

template <typename Vec>
void launch(const AppendArgs& a, int H, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(a.n_tok) * a.chunks;
  const int64_t per_block = kThreads * kItems;
  dim3 grid(static_cast<unsigned>((items + per_block - 1) / per_block), static_cast<unsigned>(H));
  hipLaunchKernelGGL(kv_append_kernel<Vec>, grid, dim3(kThreads), 0, stream, a);
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
               n_pages, max_batch, n_slots, clamp_negative};

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
  switch (vec) {
    case 16: launch<v4u>(a, H, st); break;
    case 8: launch<v2u>(a, H, st); break;
    case 4: launch<uint32_t>(a, H, st); break;
    default: launch<uint16_t>(a, H, st); break;
  }
  return fp::check_launch("fp_kv_append");
}
