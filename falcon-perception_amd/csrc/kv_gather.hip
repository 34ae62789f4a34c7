// Page gather and block-id translation: the two page-table lookups of the path.
//
// fp_kv_gather is the inverse of the append: it copies the rows of each cached
// sequence, in logical order, from the page pool into a dense [B, H, max_len, D]
// tensor.  The reference does this lookup inside its attention kernels through
// the converted block indices (paged_attention.py:279-284); it has no standalone
// gather.  HBM-bound; each row (256 B at D = 128 bf16) moves as 16-byte vectors,
// lanes fastest over the bytes of a row and then over consecutive tokens, so one
// wavefront reads and writes 1 KiB contiguous runs (whole 128-byte lines) and only
// the page base is indirect.
//
// fp_convert_block_ids is the integer lookup of convert_logical_block_mask
// (paged_attention.py:279-284): logical block ids -> physical page ids, zero tail.
#include "fp_common.h"

namespace {

typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

struct GatherArgs {
  const char* pool;
  char* out;
  int64_t os_b, os_h, os_t;  // byte strides of out
  const int64_t* page_table;
  int64_t pt_row_stride;
  const int64_t* batch_idx;
  const void* seq_lens;
  int len_i64;
  int max_len;
  int chunks;
  int row_bytes;
  fp::PageDiv pd;
  int n_pages;
  int max_batch;
  int64_t n_slots;
  int64_t item0;  // first item of this launch: a launch holds fewer than 2^32 lanes in x, a longer gather is several
};

constexpr int kThreads = 256;
// One 16-byte vector per lane: more vectors per lane measured slower (32768 tokens x 16 heads,
// 268 MB moved: 46 us with one, 47 with two, 49 with four).
template <typename Vec>
__global__ __launch_bounds__(kThreads) void kv_gather_kernel(const GatherArgs a) {
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int64_t items = static_cast<int64_t>(a.max_len) * a.chunks;
  const int64_t i = a.item0 + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= items) return;

  int64_t len = fp::load_index(a.seq_lens, b, a.len_i64);
  const int64_t row = a.batch_idx[b];
  if (row < 0 || row >= a.max_batch) len = 0;
  if (len > a.max_len) len = a.max_len;

  const int t = i < (1ll << 32) ? static_cast<int>(static_cast<uint32_t>(i) / static_cast<uint32_t>(a.chunks))
                                : static_cast<int>(i / a.chunks);
  const int c = static_cast<int>(i - static_cast<int64_t>(t) * a.chunks);
  const int64_t dst = b * a.os_b + h * a.os_h + t * a.os_t + static_cast<int64_t>(c) * sizeof(Vec);
  Vec reg = Vec(0);
  if (t < len) {
    int64_t blk;
    int off;
    a.pd.split(t, blk, off);
    if (blk < a.n_pages) {
      const int64_t page = a.page_table[row * a.pt_row_stride + blk];
      const int64_t slot = page * a.pd.page_size + off;
      if (slot >= 0 && slot < a.n_slots) {
        const int64_t src = (static_cast<int64_t>(h) * a.n_slots + slot) * a.row_bytes + static_cast<int64_t>(c) * sizeof(Vec);
        reg = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(a.pool + src));
      }
    }
  }
  __builtin_nontemporal_store(reg, reinterpret_cast<Vec*>(a.out + dst));
}

constexpr int64_t kLaunchBlocks = (1ll << 31) / kThreads;  // a dispatch holds fewer than 2^32 lanes in x

template <typename Vec>
void launch_gather(const GatherArgs& a0, int B, int H, hipStream_t stream) {
  const int64_t items = static_cast<int64_t>(a0.max_len) * a0.chunks;
  const int64_t blocks = (items + kThreads - 1) / kThreads;
  GatherArgs a = a0;
  for (int64_t b0 = 0; b0 < blocks; b0 += kLaunchBlocks) {
    a.item0 = b0 * kThreads;
    const int64_t nb = blocks - b0 < kLaunchBlocks ? blocks - b0 : kLaunchBlocks;
    dim3 grid(static_cast<unsigned>(nb), static_cast<unsigned>(H), static_cast<unsigned>(B));
    hipLaunchKernelGGL(kv_gather_kernel<Vec>, grid, dim3(kThreads), 0, stream, a);
  }
}

__global__ __launch_bounds__(kThreads) void convert_block_ids_kernel(
    const int32_t* __restrict__ kv_indices, int32_t* __restrict__ out,
    const int64_t* __restrict__ page_table, int64_t pt_row_stride,
    const int64_t* __restrict__ batch_idx, int rows_per_batch, int C, int n_pages, int max_batch) {
  const int b = blockIdx.z;
  const int r = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= n_pages) return;
  int32_t val = 0;
  if (c < C) {
    const int64_t row = batch_idx[b];
    const int32_t lb = kv_indices[(static_cast<int64_t>(b) * rows_per_batch + r) * C + c];
    if (row >= 0 && row < max_batch && lb >= 0 && lb < n_pages)
      val = static_cast<int32_t>(page_table[row * pt_row_stride + lb]);
  }
  out[(static_cast<int64_t>(b) * rows_per_batch + r) * n_pages + c] = val;
}

}  // namespace

extern "C" int fp_kv_gather(const void* pool, void* out, int64_t out_stride_b, int64_t out_stride_h,
                            int64_t out_stride_t, const int64_t* page_table, int64_t pt_row_stride,
                            const int64_t* batch_idx, const void* seq_lens, int len_index_type,
                            int32_t B, int32_t H, int32_t max_len, int32_t D, int32_t page_size,
                            int32_t n_pages, int32_t max_batch, int64_t n_slots, int dtype,
                            void* stream) {
  const int eb = fp::elem_bytes(dtype);
  if (eb == 0) return fp::fail(FP_ERR_UNSUPPORTED, "fp_kv_gather: unknown dtype %d", dtype);
  if (B < 0 || H <= 0 || max_len < 0 || D <= 0 || page_size <= 0 || n_pages <= 0 || max_batch <= 0 || n_slots <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_gather: non-positive dimension");
  if (H > 65535 || B > 65535) return fp::fail(FP_ERR_UNSUPPORTED, "fp_kv_gather: B or H exceeds 65535");
  if (n_slots < page_size)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_gather: n_slots smaller than one page");
  if (len_index_type != FP_INDEX_I32 && len_index_type != FP_INDEX_I64)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_gather: bad len_index_type");
  if (B == 0 || max_len == 0) return FP_OK;
  if (!pool || !out || !page_table || !batch_idx || !seq_lens)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_gather: null pointer");

  GatherArgs a{static_cast<const char*>(pool), static_cast<char*>(out),
               out_stride_b * eb, out_stride_h * eb, out_stride_t * eb,
               page_table, pt_row_stride, batch_idx, seq_lens, len_index_type == FP_INDEX_I64,
               max_len, 0, D * eb, fp::PageDiv(page_size), n_pages, max_batch, n_slots, 0};
  int vec = 16;
  auto fits = [&](int n) {
    return a.row_bytes % n == 0 && a.os_b % n == 0 && a.os_h % n == 0 && a.os_t % n == 0 &&
           fp::aligned(pool, n) && fp::aligned(out, n);
  };
  while (vec > eb && !fits(vec)) vec >>= 1;
  if (!fits(vec)) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_kv_gather: pointers not aligned to the element size");
  a.chunks = a.row_bytes / vec;

  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (vec) {
    case 16: launch_gather<v4u>(a, B, H, st); break;
    case 8: launch_gather<v2u>(a, B, H, st); break;
    case 4: launch_gather<uint32_t>(a, B, H, st); break;
    default: launch_gather<uint16_t>(a, B, H, st); break;
  }
  return fp::check_launch("fp_kv_gather");
}

extern "C" int fp_convert_block_ids(const int32_t* kv_indices, int32_t* out,
                                    const int64_t* page_table, int64_t pt_row_stride,
                                    const int64_t* batch_idx, int32_t B, int32_t rows_per_batch,
                                    int32_t C, int32_t n_pages, int32_t max_batch, void* stream) {
  if (B < 0 || rows_per_batch < 0 || C < 0 || n_pages <= 0 || max_batch <= 0)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_convert_block_ids: bad dimension");
  if (C > n_pages)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_convert_block_ids: mask has %d block columns, pool has %d pages", C, n_pages);
  if (B > 65535 || rows_per_batch > 65535)
    return fp::fail(FP_ERR_UNSUPPORTED, "fp_convert_block_ids: B or rows exceed 65535");
  if (B == 0 || rows_per_batch == 0) return FP_OK;
  if (!out || !page_table || !batch_idx || (C > 0 && !kv_indices))
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_convert_block_ids: null pointer");
  dim3 grid((n_pages + kThreads - 1) / kThreads, rows_per_batch, B);
  hipLaunchKernelGGL(convert_block_ids_kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     kv_indices, out, page_table, pt_row_stride, batch_idx, rows_per_batch, C, n_pages, max_batch);
  return fp::check_launch("fp_convert_block_ids");
}
