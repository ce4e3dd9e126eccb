// Fused epilogue of the QKV projection: per-head RMSNorm of q and k, rotary position embedding
// of both, and the KV append -- the rotated k row and the v row of each token go straight into
// the token's page slot, q is updated in place. One launch instead of the reference's five
// (skip_rmsnorm x2, rope_emb_forward, torch.cat, update_kv_buffer: lite_llama/models/qwen3.py:109-130,
// 29, 62), and k/v are read once and written once.
//
// A head row (128 fp16) is held by 16 lanes, 8 elements each; a wavefront works on 4 rows. The
// sum of squares is reduced across the 16 lanes; the rotation pairs element i with i + 64, which
// lives 8 lanes away. (Head dims 32, 64 and 256: 4, 8 and 32 lanes per row, template argument L.) Rounding follows the reference where it is specified: the normalised value
// is rounded to fp16 before the weight multiply, and that product to fp16
// (`(x * rrms).to(fp16) * w`, lite_llama/kernels/skip_rmsnorm.py:137-145); the rotation
// x1*cos - x2*sin, x2*cos + x1*sin (lite_llama/kernels/rope_emb.py:79-87) is evaluated in fp32
// from fp16 inputs and rounded once.
#include <type_traits>

#include "common.h"
#include "kv_fp8.h"

namespace litekv {

template <int L>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int off = 1; off < L; off <<= 1) v += __shfl_xor(v, off, L);
  return v;
}

// KV kKvFp8 / kKvInt8: the pool holds 8-bit codes; `scales` are its per-head scales (K heads, then
// V heads) and a row is quantised on its way in, exactly as kv_append_q8_kernel would quantise
// the fp16 row.
template <int KV, int L, int TOK>
__global__ __launch_bounds__(256) void qk_norm_rope_append_kernel(
    half_t *__restrict__ q, int64_t q_stride, const half_t *__restrict__ k, int64_t k_stride,
    const half_t *__restrict__ v, int64_t v_stride, const half_t *__restrict__ q_weight,
    const half_t *__restrict__ k_weight, const half_t *__restrict__ cos_rows,
    const half_t *__restrict__ sin_rows, int64_t cs_stride, const int32_t *__restrict__ slot_mapping,
    void *__restrict__ pool_any, const float *__restrict__ scales, int64_t num_tokens,
    int32_t num_q_heads, int32_t num_kv_heads, int64_t num_slots, float eps) {
  // grid: x = group of TOK tokens, y = block of 256 / L consecutive head rows of a token (q heads,
  // k heads, v heads): no division on the way to an address, a workgroup's rows are one
  // contiguous run per token, and a lane has the loads of TOK tokens in flight. TOK is 4 for
  // prefill-sized launches (a lane with one token in flight left the launch bound by latency) and
  // 1 for decode-sized ones, which have too few tokens to fill the device in groups of four.
  constexpr int kDim = 8 * L;       // the head dim
  constexpr int kTok = TOK;
  const int l16 = threadIdx.x & (L - 1);  // lane inside the row
  const int r = (int)blockIdx.y * (256 / L) + (int)(threadIdx.x / L);
  if (r >= num_q_heads + 2 * num_kv_heads) return;  // whole L-lane groups leave together
  const bool is_v = r >= num_q_heads + num_kv_heads;
  const bool is_q = r < num_q_heads;
  const int head = is_q ? r : (is_v ? r - num_q_heads - num_kv_heads : r - num_q_heads);
  int64_t token[kTok], slot[kTok];
  bool live[kTok];
  half8_t x[kTok], c[kTok], sn[kTok];
#pragma unroll
  for (int t = 0; t < kTok; ++t) {
    token[t] = (int64_t)blockIdx.x * kTok + t;
    live[t] = token[t] < num_tokens;
    if (!live[t]) token[t] = num_tokens - 1;  // loads repeat the last token; nothing is stored
    const half_t *src = is_q   ? q + token[t] * q_stride + (int64_t)head * kDim
                        : is_v ? v + token[t] * v_stride + (int64_t)head * kDim
                               : k + token[t] * k_stride + (int64_t)head * kDim;
    x[t] = *(const half8_t *)(src + 8 * l16);
    slot[t] = slot_mapping[token[t]];
    if (cos_rows != nullptr && !is_v) {
      const int j = 8 * (l16 & (L / 2 - 1));  // index into the first dim / 2 entries of the cos / sin row
      c[t] = *(const half8_t *)(cos_rows + token[t] * cs_stride + j);
      sn[t] = *(const half8_t *)(sin_rows + token[t] * cs_stride + j);
    }
  }
  // stores 8 elements of head `kv_head` (K heads first, then V heads) of a slot
  auto store_row = [&](int64_t slot_t, int kv_head, half8_t y) {
    const int64_t at = (slot_t * (int64_t)(2 * num_kv_heads) + kv_head) * kDim + 8 * l16;
    if constexpr (KV != kKvF16) {
      *(uint2_t *)(static_cast<uint8_t *>(pool_any) + at) =
          half_to_codes<KV>(y, 1.0f / scales[kv_head]);
    } else {
      *(half8_t *)(static_cast<half_t *>(pool_any) + at) = y;
    }
  };
  const half_t *weight = is_q ? q_weight : k_weight;
  half8_t w = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  if (weight != nullptr && !is_v) w = *(const half8_t *)(weight + 8 * l16);

#pragma unroll
  for (int t = 0; t < kTok; ++t) {
    const bool slot_ok = live[t] && slot[t] >= 0 && slot[t] < num_slots;
    if (is_v) {  // a v row: plain copy into the slot
      if (slot_ok) store_row(slot[t], num_kv_heads + head, x[t]);
      continue;
    }
    half8_t y = x[t];
    if (weight != nullptr) {
      float xf[8], ss = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        xf[i] = (float)y[i];
        ss += xf[i] * xf[i];
      }
      ss = row_sum<L>(ss);
      const float rrms = 1.0f / sqrtf(ss * (1.0f / kDim) + eps);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const half_t z = (half_t)(xf[i] * rrms);
        y[i] = (half_t)((float)z * (float)w[i]);
      }
    }
    if (cos_rows != nullptr) {
      // partner: element i + dim / 2 for the first half of the row, i - dim / 2 for the second
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      u32x4 bits = __builtin_bit_cast(u32x4, y);
      u32x4 other;
#pragma unroll
      for (int i = 0; i < 4; ++i) other[i] = __shfl_xor(bits[i], L / 2, L);
      const half8_t p = __builtin_bit_cast(half8_t, other);
      const float sign = l16 < L / 2 ? -1.0f : 1.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        y[i] = (half_t)((float)y[i] * (float)c[t][i] + sign * ((float)p[i] * (float)sn[t][i]));
      }
    }
    if (is_q) {
      if (live[t]) *(half8_t *)(q + token[t] * q_stride + (int64_t)head * kDim + 8 * l16) = y;
    } else if (slot_ok) {
      store_row(slot[t], head, y);
    }
  }
}

}  // namespace litekv

namespace litekv {
static int launch_qk_epilogue(const char *what, void *q, int64_t q_token_stride, const void *k,
                              int64_t k_token_stride, const void *v, int64_t v_token_stride,
                              const void *q_norm_weight, const void *k_norm_weight,
                              const void *cos_rows, const void *sin_rows,
                              int64_t cos_sin_token_stride, const int32_t *slot_mapping,
                              void *kv_pool, const float *fp8_scales, int format, int32_t num_tokens,
                              int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                              int64_t num_slots, float rms_eps, void *stream) {
  LITEKV_REQUIRE(num_tokens >= 0, "%s: num_tokens %d < 0", what, num_tokens);
  LITEKV_REQUIRE(head_dim == kHeadDim || generic_head_dim(head_dim),
                 "%s: head_dim %d unsupported (32, 64, 128 or 256)", what, head_dim);
  LITEKV_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads <= 65535 && num_kv_heads <= 65535,
                 "%s: num_q_heads %d / num_kv_heads %d invalid", what, num_q_heads, num_kv_heads);
  if (num_tokens == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(q && k && v && slot_mapping && kv_pool, "%s: null pointer", what);
  LITEKV_REQUIRE(format == kKvF16 || fp8_scales != nullptr, "%s: scales is null", what);
  LITEKV_REQUIRE((q_norm_weight == nullptr) == (k_norm_weight == nullptr),
                 "%s: q_norm_weight and k_norm_weight go together", what);
  LITEKV_REQUIRE((cos_rows == nullptr) == (sin_rows == nullptr), "%s: cos and sin go together", what);
  LITEKV_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(kv_pool) &&
                     aligned16(q_norm_weight) && aligned16(k_norm_weight) && aligned16(cos_rows) &&
                     aligned16(sin_rows),
                 "%s: all tensors must be 16-byte aligned", what);
  LITEKV_REQUIRE(q_token_stride >= (int64_t)num_q_heads * head_dim && q_token_stride % 8 == 0 &&
                     k_token_stride >= (int64_t)num_kv_heads * head_dim && k_token_stride % 8 == 0 &&
                     v_token_stride >= (int64_t)num_kv_heads * head_dim && v_token_stride % 8 == 0,
                 "%s: token strides (%lld, %lld, %lld) invalid", what, (long long)q_token_stride,
                 (long long)k_token_stride, (long long)v_token_stride);
  if (cos_rows != nullptr) {
    LITEKV_REQUIRE(cos_sin_token_stride >= head_dim / 2 && cos_sin_token_stride % 8 == 0,
                   "%s: cos/sin token stride %lld invalid (>= %d, multiple of 8)", what,
                   (long long)cos_sin_token_stride, head_dim / 2);
  }
  LITEKV_REQUIRE(num_slots > 0, "%s: num_slots %lld <= 0", what, (long long)num_slots);
  LITEKV_REQUIRE(rms_eps >= 0.f, "%s: rms_eps %g < 0", what, (double)rms_eps);
  const int rows_per_block = 256 / (head_dim / 8);
  const int row_blocks = (num_q_heads + 2 * num_kv_heads + rows_per_block - 1) / rows_per_block;
  LITEKV_REQUIRE(row_blocks <= 65535, "%s: too many heads", what);
  // Four tokens per lane once that still leaves 16 workgroups for every compute unit (64 query /
  // 8 kv heads, one token per lane against four: 512 tokens 6.3 against 7.6 us, 2048 tokens 17.0
  // against 17.5 us, 10 366 tokens 80.7 against 71.1 us).
  const bool four = (int64_t)((num_tokens + 3) / 4) * row_blocks >= 4096;
  const int tok = four ? 4 : 1;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)((num_tokens + tok - 1) / tok), (unsigned)row_blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream),
                       static_cast<half_t *>(q), q_token_stride, static_cast<const half_t *>(k),
                       k_token_stride, static_cast<const half_t *>(v), v_token_stride,
                       static_cast<const half_t *>(q_norm_weight),
                       static_cast<const half_t *>(k_norm_weight),
                       static_cast<const half_t *>(cos_rows), static_cast<const half_t *>(sin_rows),
                       cos_sin_token_stride, slot_mapping, kv_pool, fp8_scales, (int64_t)num_tokens,
                       num_q_heads, num_kv_heads, num_slots, rms_eps);
  };
  auto by_format = [&](auto lanes) {
    constexpr int L = decltype(lanes)::value;
    if (format == kKvFp8) {
      four ? launch(qk_norm_rope_append_kernel<kKvFp8, L, 4>) : launch(qk_norm_rope_append_kernel<kKvFp8, L, 1>);
    } else if (format == kKvInt8) {
      four ? launch(qk_norm_rope_append_kernel<kKvInt8, L, 4>) : launch(qk_norm_rope_append_kernel<kKvInt8, L, 1>);
    } else {
      four ? launch(qk_norm_rope_append_kernel<kKvF16, L, 4>) : launch(qk_norm_rope_append_kernel<kKvF16, L, 1>);
    }
  };
  switch (head_dim) {
    case 32: by_format(std::integral_constant<int, 4>{}); break;
    case 64: by_format(std::integral_constant<int, 8>{}); break;
    case 256: by_format(std::integral_constant<int, 32>{}); break;
    default: by_format(std::integral_constant<int, 16>{}); break;
  }
  return check_launch(what);
}
}  // namespace litekv

extern "C" int litekv_qk_norm_rope_append(void *q, int64_t q_token_stride, const void *k,
                                          int64_t k_token_stride, const void *v,
                                          int64_t v_token_stride, const void *q_norm_weight,
                                          const void *k_norm_weight, const void *cos_rows,
                                          const void *sin_rows, int64_t cos_sin_token_stride,
                                          const int32_t *slot_mapping, void *kv_pool,
                                          int32_t num_tokens, int32_t num_q_heads,
                                          int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                                          float rms_eps, void *stream) {
  return litekv::launch_qk_epilogue("qk_norm_rope_append", q, q_token_stride, k, k_token_stride, v,
                                    v_token_stride, q_norm_weight, k_norm_weight, cos_rows, sin_rows,
                                    cos_sin_token_stride, slot_mapping, kv_pool, nullptr,
                                    litekv::kKvF16, num_tokens, num_q_heads, num_kv_heads, head_dim, num_slots,
                                    rms_eps, stream);
}

extern "C" int litekv_qk_norm_rope_append_fp8(void *q, int64_t q_token_stride, const void *k,
                                              int64_t k_token_stride, const void *v,
                                              int64_t v_token_stride, const void *q_norm_weight,
                                              const void *k_norm_weight, const void *cos_rows,
                                              const void *sin_rows, int64_t cos_sin_token_stride,
                                              const int32_t *slot_mapping, void *kv_pool_fp8,
                                              const float *scales, int32_t num_tokens,
                                              int32_t num_q_heads, int32_t num_kv_heads,
                                              int32_t head_dim, int64_t num_slots, float rms_eps,
                                              void *stream) {
  return litekv::launch_qk_epilogue("qk_norm_rope_append_fp8", q, q_token_stride, k, k_token_stride,
                                    v, v_token_stride, q_norm_weight, k_norm_weight, cos_rows,
                                    sin_rows, cos_sin_token_stride, slot_mapping, kv_pool_fp8, scales,
                                    litekv::kKvFp8, num_tokens, num_q_heads, num_kv_heads, head_dim,
                                    num_slots, rms_eps, stream);
}

extern "C" int litekv_qk_norm_rope_append_int8(void *q, int64_t q_token_stride, const void *k,
                                               int64_t k_token_stride, const void *v,
                                               int64_t v_token_stride, const void *q_norm_weight,
                                               const void *k_norm_weight, const void *cos_rows,
                                               const void *sin_rows, int64_t cos_sin_token_stride,
                                               const int32_t *slot_mapping, void *kv_pool_int8,
                                               const float *scales, int32_t num_tokens,
                                               int32_t num_q_heads, int32_t num_kv_heads,
                                               int32_t head_dim, int64_t num_slots, float rms_eps,
                                               void *stream) {
  return litekv::launch_qk_epilogue("qk_norm_rope_append_int8", q, q_token_stride, k, k_token_stride,
                                    v, v_token_stride, q_norm_weight, k_norm_weight, cos_rows,
                                    sin_rows, cos_sin_token_stride, slot_mapping, kv_pool_int8,
                                    scales, litekv::kKvInt8, num_tokens, num_q_heads, num_kv_heads,
                                    head_dim, num_slots, rms_eps, stream);
}
