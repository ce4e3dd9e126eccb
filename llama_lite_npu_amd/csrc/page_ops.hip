// Page gather / page copy: move whole KV pages between (or within) pools.
//
// A workgroup moves one tile of 256 lanes x 16 bytes = 4 KiB; the grid is one-dimensional with
// the tile inside the page as the fastest index, so workgroups that are dispatched together walk
// a page's contiguous run of bytes. (With the move as the fastest index and tiles of 16 KiB,
// neighbouring workgroups were a whole page apart in both pools and 1 GiB of 64 KiB pages moved
// at 5.55 TB/s of read + written bytes; tile-fastest with 16 KiB tiles 5.97, with 4 KiB tiles
// 6.37 TB/s.) A page is a contiguous run of bytes, so accesses are fully coalesced. Bit exact.
// Loads and stores carry the streaming (non-temporal) hint: nothing moved here is read again soon.
#include "common.h"

namespace litekv {

constexpr int kGatherUnroll = 1;   // 16-byte items per lane

__global__ __launch_bounds__(256) void page_gather_kernel(
    const uint4_t *src_pool, uint4_t *dst_pool, const int32_t *__restrict__ src_ids,
    const int32_t *__restrict__ dst_ids, int64_t page_items, int64_t num_src_pages,
    int64_t num_dst_pages, int32_t tiles) {
  const int64_t i = blockIdx.x / (uint32_t)tiles;
  const int64_t tile = blockIdx.x - i * tiles;
  const int64_t sp = src_ids[i];
  const int64_t dp = dst_ids ? (int64_t)dst_ids[i] : i;
  if (sp < 0 || sp >= num_src_pages || dp < 0 || dp >= num_dst_pages) return;
  const uint4_t *src = src_pool + sp * page_items;
  uint4_t *dst = dst_pool + dp * page_items;
  const int64_t base = tile * (256 * kGatherUnroll) + threadIdx.x;
  uint4_t regs[kGatherUnroll];
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const int64_t c = base + u * 256;
    if (c < page_items) regs[u] = __builtin_nontemporal_load(src + c);
  }
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const int64_t c = base + u * 256;
    if (c < page_items) __builtin_nontemporal_store(regs[u], dst + c);
  }
}

static int launch_gather(const char *what, const void *src_pool, void *dst_pool,
                         const int32_t *src_ids, const int32_t *dst_ids, int32_t n,
                         int64_t page_bytes, int64_t num_src_pages, int64_t num_dst_pages,
                         void *stream) {
  LITEKV_REQUIRE(n >= 0, "%s: n %d < 0", what, n);
  if (n == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(src_pool && dst_pool && src_ids, "%s: null pointer", what);
  LITEKV_REQUIRE(page_bytes > 0 && page_bytes % 16 == 0,
                 "%s: page_bytes %lld must be a positive multiple of 16", what,
                 (long long)page_bytes);
  LITEKV_REQUIRE(aligned16(src_pool) && aligned16(dst_pool), "%s: pools must be 16-byte aligned",
                 what);
  LITEKV_REQUIRE(num_src_pages > 0 && num_dst_pages > 0, "%s: empty pool", what);
  LITEKV_REQUIRE(dst_ids != nullptr || n <= num_dst_pages,
                 "%s: %d moves do not fit a destination pool of %lld pages", what, n,
                 (long long)num_dst_pages);
  const int64_t page_items = page_bytes / 16;
  const int64_t tiles = (page_items + 256 * kGatherUnroll - 1) / (256 * kGatherUnroll);
  LITEKV_REQUIRE(tiles * n <= 0x7fffffffLL, "%s: %d pages of %lld bytes are too many for one launch",
                 what, n, (long long)page_bytes);
  hipLaunchKernelGGL(page_gather_kernel, dim3((unsigned)(tiles * n)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4_t *>(src_pool),
                     static_cast<uint4_t *>(dst_pool), src_ids, dst_ids, page_items, num_src_pages,
                     num_dst_pages, (int32_t)tiles);
  return check_launch(what);
}

}  // namespace litekv

extern "C" int litekv_page_gather(const void *src_pool, void *dst_pool, const int32_t *src_ids,
                                  const int32_t *dst_ids, int32_t n, int64_t page_bytes,
                                  int64_t num_src_pages, int64_t num_dst_pages, void *stream) {
  return litekv::launch_gather("page_gather", src_pool, dst_pool, src_ids, dst_ids, n, page_bytes,
                               num_src_pages, num_dst_pages, stream);
}

extern "C" int litekv_page_copy(void *kv_pool, const int32_t *src_ids, const int32_t *dst_ids,
                                int32_t n, int64_t page_bytes, int64_t num_pages, void *stream) {
  if (n > 0 && dst_ids == nullptr) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "page_copy: dst_ids is null");
  }
  return litekv::launch_gather("page_copy", kv_pool, kv_pool, src_ids, dst_ids, n, page_bytes,
                               num_pages, num_pages, stream);
}
