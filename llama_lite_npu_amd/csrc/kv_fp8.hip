// 8-bit KV pools (fp8 E4M3 or int8 codes, one fp32 scale per kv head): the append that quantises
// K/V rows on their way into the pages, and the page dequantiser that turns pages back into fp16
// rows.
// The pool is [slots][2 * Hkv][head_dim] bytes, K heads then V heads as in the fp16 pool, so a page is
// one contiguous run of half the size; scales[2 * Hkv] holds the K-head scales, then the V-head
// scales.
//
// One work item handles 8 elements: 16 bytes of fp16 in, 8 bytes of codes out (append), or the
// reverse (dequantise); a head row of 128 elements is 16 consecutive items (head_dim / 8 in general), so accesses are
// coalesced on both sides.
#include "kv_fp8.h"

namespace litekv {

template <int KV>
__global__ __launch_bounds__(256) void kv_append_q8_kernel(
    const half8_t *__restrict__ k, const half8_t *__restrict__ v, int64_t k_stride8,
    int64_t v_stride8, const int32_t *__restrict__ slot_mapping, uint2_t *__restrict__ pool,
    const float *__restrict__ scales, int64_t total_items, int32_t items_per_half,
    int32_t items_per_head, int64_t num_slots) {
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= total_items) return;
  const int32_t items_per_token = 2 * items_per_half;
  const int64_t token = item / items_per_token;
  const int32_t c = (int32_t)(item - token * items_per_token);
  const int64_t slot = slot_mapping[token];
  if (slot < 0 || slot >= num_slots) return;
  const half8_t x = (c < items_per_half) ? k[token * k_stride8 + c]
                                         : v[token * v_stride8 + (c - items_per_half)];
  const float inv_scale = 1.0f / scales[c / items_per_head];  // head index over K heads then V heads
  pool[slot * items_per_token + c] = half_to_codes<KV>(x, inv_scale);
}

template <int KV>
__global__ __launch_bounds__(256) void page_dequant_kernel(
    const uint2_t *__restrict__ src_pool, half8_t *__restrict__ dst_pool,
    const int32_t *__restrict__ src_ids, const int32_t *__restrict__ dst_ids,
    const float *__restrict__ scales, int32_t page_items, int32_t items_per_slot,
    int32_t items_per_head, int64_t num_src_pages, int64_t num_dst_pages) {
  const int64_t i = blockIdx.x;
  const int64_t sp = src_ids[i];
  const int64_t dp = dst_ids ? (int64_t)dst_ids[i] : i;
  if (sp < 0 || sp >= num_src_pages || dp < 0 || dp >= num_dst_pages) return;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < page_items; c += gridDim.y * 256) {
    const float scale = scales[(c % items_per_slot) / items_per_head];
    const half8_t raw = codes_to_half<KV>(__builtin_nontemporal_load(src_pool + sp * page_items + c));
    half8_t y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (half_t)((float)raw[e] * scale);
    dst_pool[dp * page_items + c] = y;
  }
}

static int check_scales_geometry(const char *what, int32_t num_kv_heads, int32_t head_dim) {
  LITEKV_REQUIRE(head_dim == kHeadDim || generic_head_dim(head_dim),
                 "%s: head_dim %d unsupported (32, 64, 128 or 256)", what, head_dim);
  LITEKV_REQUIRE(num_kv_heads > 0 && num_kv_heads <= 65535, "%s: num_kv_heads %d out of range", what,
                 num_kv_heads);
  return LITEKV_OK;
}

static int launch_kv_append_q8(const char *what, int format, const void *k, const void *v,
                               int64_t k_token_stride, int64_t v_token_stride,
                               const int32_t *slot_mapping, void *kv_pool_fp8, const float *scales,
                               int32_t num_tokens, int32_t num_kv_heads, int32_t head_dim,
                               int64_t num_slots, void *stream) {
  LITEKV_REQUIRE(num_tokens >= 0, "%s: num_tokens %d < 0", what, num_tokens);
  int rc = check_scales_geometry(what, num_kv_heads, head_dim);
  if (rc != LITEKV_OK) return rc;
  if (num_tokens == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(k && v && slot_mapping && kv_pool_fp8 && scales, "%s: null pointer", what);
  const int64_t row = (int64_t)num_kv_heads * head_dim;
  LITEKV_REQUIRE(k_token_stride >= row && v_token_stride >= row && k_token_stride % 8 == 0 &&
                     v_token_stride % 8 == 0,
                 "%s: token strides (%lld, %lld) invalid for rows of %lld elements", what,
                 (long long)k_token_stride, (long long)v_token_stride, (long long)row);
  LITEKV_REQUIRE(aligned16(k) && aligned16(v) && aligned16(kv_pool_fp8),
                 "%s: k, v and kv_pool must be 16-byte aligned", what);
  LITEKV_REQUIRE(num_slots > 0, "%s: num_slots %lld <= 0", what, (long long)num_slots);
  const int32_t items_per_half = (int32_t)(row / 8);
  const int64_t total = (int64_t)num_tokens * 2 * items_per_half;
  const int64_t blocks = (total + 255) / 256;
  LITEKV_REQUIRE(blocks <= 0x7fffffffLL, "%s: too many tokens", what);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const half8_t *>(k),
                       static_cast<const half8_t *>(v), k_token_stride / 8, v_token_stride / 8,
                       slot_mapping, static_cast<uint2_t *>(kv_pool_fp8), scales, total,
                       items_per_half, head_dim / 8, num_slots);
  };
  if (format == kKvInt8) {
    launch(kv_append_q8_kernel<kKvInt8>);
  } else {
    launch(kv_append_q8_kernel<kKvFp8>);
  }
  return check_launch(what);
}

static int launch_page_dequant(const char *what, int format, const void *kv_pool_fp8,
                               void *dst_pool, const int32_t *src_ids, const int32_t *dst_ids,
                               int32_t n, const float *scales, int32_t num_kv_heads,
                               int32_t head_dim, int32_t page_size, int64_t num_src_pages,
                               int64_t num_dst_pages, void *stream) {
  LITEKV_REQUIRE(n >= 0, "%s: n %d < 0", what, n);
  int rc = check_scales_geometry(what, num_kv_heads, head_dim);
  if (rc != LITEKV_OK) return rc;
  LITEKV_REQUIRE(page_size > 0, "%s: page_size %d <= 0", what, page_size);
  if (n == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(kv_pool_fp8 && dst_pool && src_ids && scales, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(kv_pool_fp8) && aligned16(dst_pool), "%s: pools must be 16-byte aligned",
                 what);
  LITEKV_REQUIRE(num_src_pages > 0 && num_dst_pages > 0, "%s: empty pool", what);
  LITEKV_REQUIRE(dst_ids != nullptr || n <= num_dst_pages,
                 "%s: %d pages do not fit a destination pool of %lld pages", what, n,
                 (long long)num_dst_pages);
  const int32_t items_per_slot = 2 * num_kv_heads * (head_dim / 8);
  const int64_t page_items = (int64_t)page_size * items_per_slot;
  LITEKV_REQUIRE(page_items <= 0x7fffffffLL, "%s: page too large", what);
  int64_t tiles = (page_items + 1023) / 1024;
  tiles = tiles < 1 ? 1 : (tiles > 64 ? 64 : tiles);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)n, (unsigned)tiles), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint2_t *>(kv_pool_fp8),
                       static_cast<half8_t *>(dst_pool), src_ids, dst_ids, scales,
                       (int32_t)page_items, items_per_slot, head_dim / 8, num_src_pages,
                       num_dst_pages);
  };
  if (format == kKvInt8) {
    launch(page_dequant_kernel<kKvInt8>);
  } else {
    launch(page_dequant_kernel<kKvFp8>);
  }
  return check_launch(what);
}

}  // namespace litekv

extern "C" int litekv_kv_append_fp8(const void *k, const void *v, int64_t k_token_stride,
                                    int64_t v_token_stride, const int32_t *slot_mapping,
                                    void *kv_pool_fp8, const float *scales, int32_t num_tokens,
                                    int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                                    void *stream) {
  return litekv::launch_kv_append_q8("kv_append_fp8", litekv::kKvFp8, k, v, k_token_stride,
                                     v_token_stride, slot_mapping, kv_pool_fp8, scales, num_tokens,
                                     num_kv_heads, head_dim, num_slots, stream);
}

extern "C" int litekv_kv_append_int8(const void *k, const void *v, int64_t k_token_stride,
                                     int64_t v_token_stride, const int32_t *slot_mapping,
                                     void *kv_pool_int8, const float *scales, int32_t num_tokens,
                                     int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                                     void *stream) {
  return litekv::launch_kv_append_q8("kv_append_int8", litekv::kKvInt8, k, v, k_token_stride,
                                     v_token_stride, slot_mapping, kv_pool_int8, scales, num_tokens,
                                     num_kv_heads, head_dim, num_slots, stream);
}

extern "C" int litekv_page_dequant(const void *kv_pool_fp8, void *dst_pool, const int32_t *src_ids,
                                   const int32_t *dst_ids, int32_t n, const float *scales,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_src_pages, int64_t num_dst_pages, void *stream) {
  return litekv::launch_page_dequant("page_dequant", litekv::kKvFp8, kv_pool_fp8, dst_pool, src_ids,
                                     dst_ids, n, scales, num_kv_heads, head_dim, page_size,
                                     num_src_pages, num_dst_pages, stream);
}

extern "C" int litekv_page_dequant_int8(const void *kv_pool_int8, void *dst_pool,
                                        const int32_t *src_ids, const int32_t *dst_ids, int32_t n,
                                        const float *scales, int32_t num_kv_heads, int32_t head_dim,
                                        int32_t page_size, int64_t num_src_pages,
                                        int64_t num_dst_pages, void *stream) {
  return litekv::launch_page_dequant("page_dequant_int8", litekv::kKvInt8, kv_pool_int8, dst_pool,
                                     src_ids, dst_ids, n, scales, num_kv_heads, head_dim, page_size,
                                     num_src_pages, num_dst_pages, stream);
}
