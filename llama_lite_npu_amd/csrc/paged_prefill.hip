// Varlen causal FlashAttention-2 prefill for gfx950, over paged KV (block
// table) or over packed contiguous K/V.
//
// One wavefront owns 16 query rows of one head and walks the keys it may see
// in tiles of 16 tokens (one page). Per tile:
//
//   S^T[key][row]  = K_tile[16 x 128] . Q^T[128 x 16]        4 x MFMA 16x16x32
//   causal mask, online softmax per query row (fp32, exp2 domain)
//   O^T[d][row]   += V_tile^T[128 x 16] . P^T[16 x 16]       8 x MFMA 16x16x16
//
// The S^T accumulator layout equals the B-operand layout of the second
// product, so P stays in registers (cast to fp16 like the reference's
// `p.to(v.dtype)`, flashattention2_nopad.py:150). K fragments come straight
// from memory in A-operand layout; V rows are staged in LDS and read back
// transposed.
#include "common.h"

namespace litekv {

constexpr int kVPitchP = kHeadDim + 8;
constexpr float kLog2eP = 1.4426950408889634f;

// Where the keys of a sequence live.
struct PagedSource {
  const half_t *kv;             // pool [slots][2*Hkv][128]
  const int32_t *block_table;   // [B][stride]
  int32_t bt_stride;
  int32_t num_kv_heads;
  int32_t num_pages;
};
struct PackedSource {
  const half_t *k;              // [T][Hkv][128]
  const half_t *v;
  int64_t k_stride, v_stride;   // elements per token
  const int32_t *seq_starts;    // [B]
};

template <bool PAGED>
__global__ __launch_bounds__(64) void varlen_prefill_kernel(
    const half_t *__restrict__ q, int64_t q_stride, half_t *__restrict__ out, int64_t out_stride,
    PagedSource paged, PackedSource packed, const int32_t *__restrict__ q_starts_or_cu,
    const int32_t *__restrict__ q_lens_or_null, const int32_t *__restrict__ context_lens,
    int32_t num_q_heads, int32_t group, float scale_log2) {
  __shared__ __attribute__((aligned(16))) half_t vstage[kPageSize * kVPitchP];

  const int lane = threadIdx.x;
  const int n = lane & 15;  // query row inside the tile
  const int g = lane >> 4;  // lane group: keys 4g..4g+3 of a tile
  const int hq = blockIdx.y;
  const int b = blockIdx.z;
  const int h = hq / group;

  int q_start, q_len;
  if (PAGED) {
    q_start = q_starts_or_cu[b];
    q_len = q_starts_or_cu[b + 1] - q_start;
  } else {
    q_start = packed.seq_starts[b];
    q_len = q_lens_or_null[b];
  }
  const int m0 = blockIdx.x * 16;
  if (m0 >= q_len) return;
  const int ctx = (PAGED && context_lens) ? context_lens[b] : 0;
  const int kv_len = ctx + q_len;                       // keys that exist
  const int rows = (q_len - m0) < 16 ? (q_len - m0) : 16;
  const int kv_end = ctx + m0 + rows;                   // keys this tile may see
  const int row = m0 + n;                               // this lane's query row
  const bool row_ok = n < rows;
  const int q_pos = ctx + (row_ok ? row : m0 + rows - 1);

  half8_t qf[4];
  {
    const half_t *qrow = q + (int64_t)(q_start + row) * q_stride + (int64_t)hq * kHeadDim + 8 * g;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      qf[kk] = row_ok ? *(const half8_t *)(qrow + 32 * kk) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  const int64_t pool_row = (int64_t)2 * paged.num_kv_heads * kHeadDim;
  const int32_t *table = PAGED ? paged.block_table + (int64_t)b * paged.bt_stride : nullptr;

  float4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;
  float d_run = 0.f;

  const int tiles = (kv_end + kPageSize - 1) / kPageSize;
  half8_t kf[4], vf[4];

  auto load_tile = [&](int t, half8_t (&kd)[4], half8_t (&vd)[4]) {
    const half_t *kr;
    const half_t *vr[4];
    if (PAGED) {
      int pid = table[t];
      pid = pid < 0 ? 0 : (pid >= paged.num_pages ? paged.num_pages - 1 : pid);
      const int64_t slot0 = (int64_t)pid * kPageSize;
      kr = paged.kv + (slot0 + n) * pool_row + (int64_t)h * kHeadDim + 8 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vr[i] = paged.kv + (slot0 + 4 * i + g) * pool_row +
                (int64_t)(paged.num_kv_heads + h) * kHeadDim + 8 * n;
      }
    } else {
      // Rows past the sequence end may lie outside the tensors: clamp, they are masked.
      const int last = kv_len - 1;
      int tk = t * kPageSize + n;
      tk = tk > last ? last : tk;
      kr = packed.k + (int64_t)(q_start + tk) * packed.k_stride + (int64_t)h * kHeadDim + 8 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int tv = t * kPageSize + 4 * i + g;
        tv = tv > last ? last : tv;
        vr[i] = packed.v + (int64_t)(q_start + tv) * packed.v_stride + (int64_t)h * kHeadDim + 8 * n;
      }
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) kd[kk] = *(const half8_t *)(kr + 32 * kk);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half8_t x = *(const half8_t *)(vr[i]);
      vd[i] = (t * kPageSize + 4 * i + g < kv_len) ? x : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  };

  load_tile(0, kf, vf);
  for (int t = 0; t < tiles; ++t) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) *(half8_t *)(&vstage[(4 * i + g) * kVPitchP + 8 * n]) = vf[i];
    __syncthreads();

    half8_t kc[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) kc[kk] = kf[kk];
    if (t + 1 < tiles) load_tile(t + 1, kf, vf);

    float4_t st = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) st = mfma_16x16x32(kc[kk], qf[kk], st);

    float sv[4];
    const int key0 = t * kPageSize + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) sv[i] = (key0 + i <= q_pos) ? st[i] * scale_log2 : -INFINITY;
    float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
    mx = fmaxf(mx, xor_lane(mx, 16));
    mx = fmaxf(mx, xor_lane(mx, 32));
    // Key 0 is visible to every row, so m_new is finite from the first tile on; later tiles
    // that are fully masked for a row leave its state unchanged (alpha == 1, p == 0).
    const float m_new = fmaxf(m_run, mx);
    const float alpha = fast_exp2(m_run - m_new);
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) pr[i] = fast_exp2(sv[i] - m_new);
    d_run = d_run * alpha + ((pr[0] + pr[1]) + (pr[2] + pr[3]));
    m_run = m_new;
    const half4_t pt = half4_t{(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};

#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half_t *vcol = &vstage[(4 * g) * kVPitchP + 16 * j + n];
      const half4_t vt = half4_t{vcol[0], vcol[kVPitchP], vcol[2 * kVPitchP], vcol[3 * kVPitchP]};
      float4_t a = acc[j];
      a[0] *= alpha;
      a[1] *= alpha;
      a[2] *= alpha;
      a[3] *= alpha;
      acc[j] = mfma_16x16x16(vt, pt, a);
    }
  }

  float d_tot = d_run + xor_lane(d_run, 16);
  d_tot += xor_lane(d_tot, 32);
  const float inv = 1.0f / d_tot;
  if (row_ok) {
    half_t *o = out + (int64_t)(q_start + row) * out_stride + (int64_t)hq * kHeadDim + 4 * g;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      *(half4_t *)(o + 16 * j) = half4_t{(half_t)(acc[j][0] * inv), (half_t)(acc[j][1] * inv),
                                         (half_t)(acc[j][2] * inv), (half_t)(acc[j][3] * inv)};
    }
  }
}

static int validate_prefill(const char *what, const void *q, int64_t q_stride, const void *out,
                            int64_t out_stride, int32_t batch, int32_t hq, int32_t hkv,
                            int32_t head_dim, int32_t max_q_len) {
  LITEKV_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch %d out of [0, 65535]", what, batch);
  LITEKV_REQUIRE(head_dim == kHeadDim, "%s: head_dim %d unsupported (only %d)", what, head_dim,
                 kHeadDim);
  LITEKV_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0 && hq <= 65535,
                 "%s: num_q_heads %d / num_kv_heads %d invalid", what, hq, hkv);
  LITEKV_REQUIRE(max_q_len >= 0, "%s: max_q_len %d < 0", what, max_q_len);
  if (batch == 0 || max_q_len == 0) return LITEKV_OK;
  LITEKV_REQUIRE(q && out, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(q) && aligned16(out), "%s: q and out must be 16-byte aligned", what);
  const int64_t row = (int64_t)hq * head_dim;
  LITEKV_REQUIRE(q_stride >= row && q_stride % 8 == 0 && out_stride >= row && out_stride % 8 == 0,
                 "%s: token strides (%lld, %lld) invalid", what, (long long)q_stride,
                 (long long)out_stride);
  return LITEKV_OK;
}

}  // namespace litekv

extern "C" int litekv_paged_prefill(const void *q, int64_t q_token_stride, const void *kv_pool,
                                    const int32_t *block_table, int32_t block_table_stride,
                                    const int32_t *cu_q_lens, const int32_t *context_lens,
                                    void *out, int64_t out_token_stride, int32_t batch,
                                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                    int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                    float softmax_scale, void *stream) {
  using namespace litekv;
  int rc = validate_prefill("paged_prefill", q, q_token_stride, out, out_token_stride, batch,
                            num_q_heads, num_kv_heads, head_dim, max_q_len);
  if (rc != LITEKV_OK) return rc;
  LITEKV_REQUIRE(page_size == kPageSize, "paged_prefill: page_size %d unsupported (only %d)",
                 page_size, kPageSize);
  if (batch == 0 || max_q_len == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(kv_pool && block_table && cu_q_lens, "paged_prefill: null pointer");
  LITEKV_REQUIRE(aligned16(kv_pool), "paged_prefill: kv_pool must be 16-byte aligned");
  LITEKV_REQUIRE(block_table_stride >= 1, "paged_prefill: block_table_stride %d < 1",
                 block_table_stride);
  LITEKV_REQUIRE(num_pages >= 1 && num_pages <= 0x7fffffffLL / kPageSize,
                 "paged_prefill: num_pages %lld out of range", (long long)num_pages);
  PagedSource paged{static_cast<const half_t *>(kv_pool), block_table, block_table_stride,
                    num_kv_heads, (int32_t)num_pages};
  PackedSource packed{nullptr, nullptr, 0, 0, nullptr};
  const unsigned tiles = (unsigned)((max_q_len + 15) / 16);
  hipLaunchKernelGGL(varlen_prefill_kernel<true>,
                     dim3(tiles, (unsigned)num_q_heads, (unsigned)batch), dim3(64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const half_t *>(q),
                     q_token_stride, static_cast<half_t *>(out), out_token_stride, paged, packed,
                     cu_q_lens, (const int32_t *)nullptr, context_lens, num_q_heads,
                     num_q_heads / num_kv_heads, softmax_scale * kLog2eP);
  return check_launch("paged_prefill");
}

extern "C" int litekv_varlen_prefill(const void *q, int64_t q_token_stride, const void *k,
                                     int64_t k_token_stride, const void *v, int64_t v_token_stride,
                                     const int32_t *seq_starts, const int32_t *seq_lens, void *out,
                                     int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t max_seq_len,
                                     int64_t num_tokens, float softmax_scale, void *stream) {
  using namespace litekv;
  int rc = validate_prefill("varlen_prefill", q, q_token_stride, out, out_token_stride, batch,
                            num_q_heads, num_kv_heads, head_dim, max_seq_len);
  if (rc != LITEKV_OK) return rc;
  if (batch == 0 || max_seq_len == 0 || num_tokens == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(k && v && seq_starts && seq_lens, "varlen_prefill: null pointer");
  LITEKV_REQUIRE(aligned16(k) && aligned16(v), "varlen_prefill: k and v must be 16-byte aligned");
  const int64_t row = (int64_t)num_kv_heads * head_dim;
  LITEKV_REQUIRE(k_token_stride >= row && k_token_stride % 8 == 0 && v_token_stride >= row &&
                     v_token_stride % 8 == 0,
                 "varlen_prefill: k/v token strides (%lld, %lld) invalid",
                 (long long)k_token_stride, (long long)v_token_stride);
  PagedSource paged{nullptr, nullptr, 0, num_kv_heads, 1};
  PackedSource packed{static_cast<const half_t *>(k), static_cast<const half_t *>(v),
                      k_token_stride, v_token_stride, seq_starts};
  const unsigned tiles = (unsigned)((max_seq_len + 15) / 16);
  hipLaunchKernelGGL(varlen_prefill_kernel<false>,
                     dim3(tiles, (unsigned)num_q_heads, (unsigned)batch), dim3(64), 0,
                     static_cast<hipStream_t>(stream), static_cast<const half_t *>(q),
                     q_token_stride, static_cast<half_t *>(out), out_token_stride, paged, packed,
                     seq_starts, seq_lens, (const int32_t *)nullptr, num_q_heads,
                     num_q_heads / num_kv_heads, softmax_scale * kLog2eP);
  return check_launch("varlen_prefill");
}
