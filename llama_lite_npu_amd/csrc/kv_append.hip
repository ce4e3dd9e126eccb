// KV append: scatter the K and V rows of new tokens into their page slots.
//
// One work item moves 16 bytes (8 fp16). A token owns 2 * Hkv * D / 8 items:
// the first half comes from its K row, the second half from its V row, and
// both land contiguously in the slot row [2 * Hkv][D] of the pool, so every
// wavefront issues full 16-byte-per-lane loads and stores over 1 KiB runs.
// The path is pure data movement: bit exact by construction.
#include "common.h"

namespace litekv {

template <int UNROLL>
__global__ __launch_bounds__(256) void kv_append_kernel(
    const uint4_t *__restrict__ k, const uint4_t *__restrict__ v,
    int64_t k_stride16, int64_t v_stride16, const int32_t *__restrict__ slot_mapping,
    uint4_t *__restrict__ pool, int64_t total_items, int32_t items_per_half,
    int64_t num_slots) {
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int32_t items_per_token = 2 * items_per_half;

  uint4_t regs[UNROLL];
  int64_t dst[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t item = w + u * step;
    dst[u] = -1;
    if (item < total_items) {
      const int64_t token = item / items_per_token;
      const int32_t c = (int32_t)(item - token * items_per_token);
      const int64_t slot = slot_mapping[token];
      if (slot >= 0 && slot < num_slots) {
        dst[u] = slot * items_per_token + c;
        regs[u] = (c < items_per_half) ? k[token * k_stride16 + c]
                                       : v[token * v_stride16 + (c - items_per_half)];
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (dst[u] >= 0) pool[dst[u]] = regs[u];
  }
}

}  // namespace litekv

extern "C" int litekv_kv_append(const void *k, const void *v, int64_t k_token_stride,
                                int64_t v_token_stride, const int32_t *slot_mapping,
                                void *kv_pool, int32_t num_tokens, int32_t num_kv_heads,
                                int32_t head_dim, int64_t num_slots, void *stream) {
  using namespace litekv;
  LITEKV_REQUIRE(num_tokens >= 0, "kv_append: num_tokens %d < 0", num_tokens);
  if (num_tokens == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(k && v && slot_mapping && kv_pool, "kv_append: null pointer");
  LITEKV_REQUIRE(num_kv_heads > 0 && head_dim > 0 && head_dim % 8 == 0,
                 "kv_append: num_kv_heads %d / head_dim %d unsupported (head_dim %% 8 != 0)",
                 num_kv_heads, head_dim);
  const int64_t row = (int64_t)num_kv_heads * head_dim;
  LITEKV_REQUIRE(k_token_stride >= row && v_token_stride >= row,
                 "kv_append: token strides (%lld, %lld) smaller than a row of %lld elements",
                 (long long)k_token_stride, (long long)v_token_stride, (long long)row);
  LITEKV_REQUIRE(k_token_stride % 8 == 0 && v_token_stride % 8 == 0,
                 "kv_append: token strides must be multiples of 8 elements");
  LITEKV_REQUIRE(aligned16(k) && aligned16(v) && aligned16(kv_pool),
                 "kv_append: k, v and kv_pool must be 16-byte aligned");
  LITEKV_REQUIRE(num_slots > 0, "kv_append: num_slots %lld <= 0", (long long)num_slots);

  const int32_t items_per_half = (int32_t)(row / 8);
  const int64_t total = (int64_t)num_tokens * 2 * items_per_half;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint4_t *k16 = static_cast<const uint4_t *>(k);
  const uint4_t *v16 = static_cast<const uint4_t *>(v);
  uint4_t *pool16 = static_cast<uint4_t *>(kv_pool);
  // Small batches (decode) are launch bound: spread them over many blocks.
  if (total >= (int64_t)256 * 4 * 1024) {
    const int64_t blocks = (total + 256 * 4 - 1) / (256 * 4);
    LITEKV_REQUIRE(blocks <= 0x7fffffffLL, "kv_append: too many tokens");
    hipLaunchKernelGGL(kv_append_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s, k16, v16,
                       k_token_stride / 8, v_token_stride / 8, slot_mapping, pool16, total,
                       items_per_half, num_slots);
  } else {
    const int64_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(kv_append_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, k16, v16,
                       k_token_stride / 8, v_token_stride / 8, slot_mapping, pool16, total,
                       items_per_half, num_slots);
  }
  return check_launch("kv_append");
}
