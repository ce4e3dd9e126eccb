// Host side of the varlen causal prefill and of the shared-prefix pass of a decode step: argument
// checks, launch shapes and the C ABI. The kernel is in prefill_tile.h.
#include "prefill_tile.h"

namespace litekv {
inline namespace LITEKV_HD_NS {
using namespace prefill_tile;

static int validate_prefill(const char *what, const void *q, int64_t q_stride, const void *out,
                            int64_t out_stride, int32_t batch, int32_t hq, int32_t hkv,
                            int32_t head_dim, int32_t max_q_len) {
  LITEKV_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch %d out of [0, 65535]", what, batch);
  LITEKV_REQUIRE(head_dim == kHD, "%s: head_dim %d unsupported (32, 64, 128 or 256)", what,
                 head_dim);
  LITEKV_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0 && hq <= 65535,
                 "%s: num_q_heads %d / num_kv_heads %d invalid", what, hq, hkv);
  LITEKV_REQUIRE(hq / hkv <= kMaxGroup, "%s: %d query heads per kv head unsupported (max %d)", what,
                 hq / hkv, kMaxGroup);
  LITEKV_REQUIRE(max_q_len >= 0, "%s: max_q_len %d < 0", what, max_q_len);
  if (batch == 0 || max_q_len == 0) return LITEKV_OK;
  LITEKV_REQUIRE(q && out, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(q) && aligned16(out), "%s: q and out must be 16-byte aligned", what);
  const int64_t row = (int64_t)hq * head_dim;
  LITEKV_REQUIRE(q_stride >= row && q_stride % 8 == 0 && out_stride >= row && out_stride % 8 == 0,
                 "%s: token strides (%lld, %lld) invalid", what, (long long)q_stride,
                 (long long)out_stride);
  // q rows are staged with 32-bit byte offsets from the block's first row
  LITEKV_REQUIRE(q_stride < (1 << 25), "%s: q token stride %lld too large", what, (long long)q_stride);
  return LITEKV_OK;
}

// How a GQA group of `group` heads is cut into workgroups of `col_tiles` column tiles (two per
// wavefront).
struct PrefillShape {
  int head_splits, heads_per_wg, row_tiles;
  unsigned row_blocks;
};
static PrefillShape prefill_shape(int group, int max_q_len, int col_tiles = kWgColTiles) {
  PrefillShape s;
  s.head_splits = (group + col_tiles - 1) / col_tiles;
  s.heads_per_wg = (group + s.head_splits - 1) / s.head_splits;
  s.row_tiles = col_tiles / s.heads_per_wg;
  s.row_blocks = (unsigned)((max_q_len + 16 * s.row_tiles - 1) / (16 * s.row_tiles));
  return s;
}

// Causal chunk attention over paged KV; `kv_scales` selects the fp8 pool.
static int launch_paged_prefill(const char *what, const void *q, int64_t q_token_stride,
                                const void *kv_pool, const float *kv_scales,
                                const int32_t *block_table, int32_t block_table_stride,
                                const int32_t *cu_q_lens, const int32_t *context_lens, void *out,
                                int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                                int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                int64_t num_pages, int32_t max_q_len, float softmax_scale,
                                void *stream, int format) {
  const bool fp8 = format != kKvF16;  // a pool of 8-bit codes
#if LITEKV_HD == 128
  if (head_dim == 64) {  // the head dim 64 build of this file
    return hd64_paged_prefill(what, q, q_token_stride, kv_pool, kv_scales, format, block_table, block_table_stride,
                              cu_q_lens, context_lens, out, out_token_stride, batch, num_q_heads,
                              num_kv_heads, page_size, num_pages, max_q_len, softmax_scale, stream);
  }
#endif
  if (head_dim != kHD && generic_head_dim(head_dim)) {  // see generic_attention.hip
    LITEKV_REQUIRE(max_q_len >= 0, "%s: max_q_len %d < 0", what, max_q_len);
    LITEKV_REQUIRE(batch == 0 || max_q_len == 0 || (kv_pool && block_table && cu_q_lens),
                   "%s: null pointer", what);
    LITEKV_REQUIRE(!fp8 || kv_scales, "%s: null pointer (kv_scales)", what);
    GenericLaunch g;
    g.q = q;
    g.q_row_stride = q_token_stride;
    g.out = out;
    g.out_row_stride = out_token_stride;
    g.kv_pool = const_cast<void *>(kv_pool);
    g.scales = kv_scales;
    g.format = format;
    g.block_table = block_table;
    g.bt_stride = block_table_stride;
    g.page_size = page_size;
    g.num_pages = num_pages;
    g.cu_q_lens = cu_q_lens;
    g.context_lens = context_lens;
    g.batch = batch;
    g.rows_per_seq = max_q_len;
    g.num_q_heads = num_q_heads;
    g.num_kv_heads = num_kv_heads;
    g.head_dim = head_dim;
    g.softmax_scale = softmax_scale;
    g.stream = stream;
    return launch_generic_attention(what, g);
  }
  int rc = validate_prefill(what, q, q_token_stride, out, out_token_stride, batch, num_q_heads,
                            num_kv_heads, head_dim, max_q_len);
  if (rc != LITEKV_OK) return rc;
  const int page_shift = page_shift_of(page_size);
  LITEKV_REQUIRE(page_shift >= 0, "%s: page_size %d unsupported (16, 32, 64, 128 or 256)", what, page_size);
  if (batch == 0 || max_q_len == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(kv_pool && block_table && cu_q_lens, "%s: null pointer", what);
  LITEKV_REQUIRE(!fp8 || kv_scales, "%s: null pointer (kv_scales)", what);
  LITEKV_REQUIRE(aligned16(kv_pool), "%s: kv_pool must be 16-byte aligned", what);
  LITEKV_REQUIRE(block_table_stride >= 1, "%s: block_table_stride %d < 1", what, block_table_stride);
  LITEKV_REQUIRE(num_pages >= 1 && num_pages <= 0x7fffffffLL / page_size,
                 "%s: num_pages %lld out of range", what, (long long)num_pages);
  LITEKV_REQUIRE(num_kv_heads <= 1024, "%s: num_kv_heads %d > 1024", what, num_kv_heads);
  PagedSource paged{static_cast<const half_t *>(kv_pool), block_table, block_table_stride,
                    num_kv_heads, (int32_t)num_pages, kv_scales, page_shift};
  PackedSource packed{nullptr, nullptr, 0, 0, nullptr};
  const int group = num_q_heads / num_kv_heads;
  const int waves = (format == kKvF16 && LITEKV_PREFILL_WAVES == kWideWaves) ? kWideWaves : kTiledWaves;
  const PrefillShape s = prefill_shape(group, max_q_len, kColTiles * waves);
  LITEKV_REQUIRE(s.row_blocks <= 65535u, "%s: max_q_len %d too large", what, max_q_len);
  const dim3 grid((unsigned)(num_kv_heads * s.head_splits), s.row_blocks, (unsigned)batch);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(waves * kWave), 0, static_cast<hipStream_t>(stream),
                       static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                       out_token_stride, paged, packed, PrefixTask{}, cu_q_lens,
                       (const int32_t *)nullptr, context_lens, group, s.head_splits, s.heads_per_wg,
                       s.row_tiles, softmax_scale * kLog2eP);
  };
  if (format == kKvInt8) {
    launch(varlen_prefill_tiled_kernel<kPagedPrefillInt8>);
  } else if (format == kKvFp8) {
    launch(varlen_prefill_tiled_kernel<kPagedPrefillFp8>);
  } else if (waves == kWideWaves) {
    launch(varlen_prefill_tiled_kernel<kPagedPrefill, kWideWaves>);
  } else {
    launch(varlen_prefill_tiled_kernel<kPagedPrefill>);
  }
  return check_launch(what);
}

// Causal attention over packed, contiguous K/V.
static int launch_varlen_prefill(const void *q, int64_t q_token_stride, const void *k,
                                 int64_t k_token_stride, const void *v, int64_t v_token_stride,
                                 const int32_t *seq_starts, const int32_t *seq_lens, void *out,
                                 int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                                 int32_t num_kv_heads, int32_t head_dim, int32_t max_seq_len,
                                 int64_t num_tokens, float softmax_scale, void *stream) {
#if LITEKV_HD == 128
  if (head_dim == 64) {  // the head dim 64 build of this file
    return hd64_varlen_prefill(q, q_token_stride, k, k_token_stride, v, v_token_stride, seq_starts,
                               seq_lens, out, out_token_stride, batch, num_q_heads, num_kv_heads,
                               max_seq_len, num_tokens, softmax_scale, stream);
  }
#endif
  if (head_dim != kHD && generic_head_dim(head_dim)) {  // see generic_attention.hip
    LITEKV_REQUIRE(max_seq_len >= 0, "varlen_prefill: max_seq_len %d < 0", max_seq_len);
    GenericLaunch g;
    g.q = q;
    g.q_row_stride = q_token_stride;
    g.out = out;
    g.out_row_stride = out_token_stride;
    g.k = k;
    g.v = v;
    g.k_stride = k_token_stride;
    g.v_stride = v_token_stride;
    g.seq_starts = seq_starts;
    g.q_lens = seq_lens;
    g.batch = num_tokens == 0 ? 0 : batch;
    g.rows_per_seq = max_seq_len;
    g.num_q_heads = num_q_heads;
    g.num_kv_heads = num_kv_heads;
    g.head_dim = head_dim;
    g.softmax_scale = softmax_scale;
    g.stream = stream;
    return launch_generic_attention("varlen_prefill", g);
  }
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
  LITEKV_REQUIRE(k_token_stride < (1 << 25) && v_token_stride < (1 << 25),
                 "varlen_prefill: k/v token strides (%lld, %lld) too large",
                 (long long)k_token_stride, (long long)v_token_stride);
  PagedSource paged{nullptr, nullptr, 0, num_kv_heads, 1, nullptr};
  PackedSource packed{static_cast<const half_t *>(k), static_cast<const half_t *>(v),
                      k_token_stride, v_token_stride, seq_starts};
  const int group = num_q_heads / num_kv_heads;
  const int waves = LITEKV_PREFILL_WAVES == kWideWaves ? kWideWaves : kTiledWaves;
  const PrefillShape s = prefill_shape(group, max_seq_len, kColTiles * waves);
  LITEKV_REQUIRE(s.row_blocks <= 65535u, "varlen_prefill: max_seq_len %d too large", max_seq_len);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel,
                       dim3((unsigned)(num_kv_heads * s.head_splits), s.row_blocks, (unsigned)batch),
                       dim3(waves * kWave), 0, static_cast<hipStream_t>(stream),
                       static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                       out_token_stride, paged, packed, PrefixTask{}, seq_starts, seq_lens,
                       (const int32_t *)nullptr, group, s.head_splits, s.heads_per_wg, s.row_tiles,
                       softmax_scale * kLog2eP);
  };
  if (waves == kWideWaves) {
    launch(varlen_prefill_tiled_kernel<kPackedPrefill, kWideWaves>);
  } else {
    launch(varlen_prefill_tiled_kernel<kPackedPrefill>);
  }
  return check_launch("varlen_prefill");
}
}  // namespace LITEKV_HD_NS

#if LITEKV_HD == 64
int hd64_paged_prefill(const char *what, const void *q, int64_t q_token_stride, const void *kv_pool,
                       const float *kv_scales, int format, const int32_t *block_table,
                       int32_t block_table_stride,
                       const int32_t *cu_q_lens, const int32_t *context_lens, void *out,
                       int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                       int32_t num_kv_heads, int32_t page_size, int64_t num_pages,
                       int32_t max_q_len, float softmax_scale, void *stream) {
  return launch_paged_prefill(what, q, q_token_stride, kv_pool, kv_scales, block_table,
                              block_table_stride, cu_q_lens, context_lens, out, out_token_stride,
                              batch, num_q_heads, num_kv_heads, 64, page_size, num_pages, max_q_len,
                              softmax_scale, stream, format);
}
int hd64_varlen_prefill(const void *q, int64_t q_token_stride, const void *k, int64_t k_token_stride,
                        const void *v, int64_t v_token_stride, const int32_t *seq_starts,
                        const int32_t *seq_lens, void *out, int64_t out_token_stride, int32_t batch,
                        int32_t num_q_heads, int32_t num_kv_heads, int32_t max_seq_len,
                        int64_t num_tokens, float softmax_scale, void *stream) {
  return launch_varlen_prefill(q, q_token_stride, k, k_token_stride, v, v_token_stride, seq_starts,
                               seq_lens, out, out_token_stride, batch, num_q_heads, num_kv_heads, 64,
                               max_seq_len, num_tokens, softmax_scale, stream);
}
#endif  // LITEKV_HD == 64
}  // namespace litekv

#if LITEKV_HD == 128  // the C ABI lives in the head dim 128 build of this file

extern "C" int litekv_paged_prefill(const void *q, int64_t q_token_stride, const void *kv_pool,
                                    const int32_t *block_table, int32_t block_table_stride,
                                    const int32_t *cu_q_lens, const int32_t *context_lens,
                                    void *out, int64_t out_token_stride, int32_t batch,
                                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                    int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                    float softmax_scale, void *stream) {
  return litekv::launch_paged_prefill("paged_prefill", q, q_token_stride, kv_pool, nullptr, block_table,
                                      block_table_stride, cu_q_lens, context_lens, out,
                                      out_token_stride, batch, num_q_heads, num_kv_heads, head_dim,
                                      page_size, num_pages, max_q_len, softmax_scale, stream,
                                      litekv::kKvF16);
}

extern "C" int litekv_paged_prefill_fp8(const void *q, int64_t q_token_stride, const void *kv_pool,
                                        const float *kv_scales, const int32_t *block_table,
                                        int32_t block_table_stride, const int32_t *cu_q_lens,
                                        const int32_t *context_lens, void *out,
                                        int64_t out_token_stride, int32_t batch,
                                        int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                        int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                        float softmax_scale, void *stream) {
  return litekv::launch_paged_prefill("paged_prefill_fp8", q, q_token_stride, kv_pool, kv_scales,
                                      block_table, block_table_stride, cu_q_lens, context_lens, out,
                                      out_token_stride, batch, num_q_heads, num_kv_heads, head_dim,
                                      page_size, num_pages, max_q_len, softmax_scale, stream,
                                      litekv::kKvFp8);
}

extern "C" int litekv_paged_prefill_int8(const void *q, int64_t q_token_stride, const void *kv_pool,
                                         const float *kv_scales, const int32_t *block_table,
                                         int32_t block_table_stride, const int32_t *cu_q_lens,
                                         const int32_t *context_lens, void *out,
                                         int64_t out_token_stride, int32_t batch,
                                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                         int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                         float softmax_scale, void *stream) {
  return litekv::launch_paged_prefill("paged_prefill_int8", q, q_token_stride, kv_pool, kv_scales,
                                      block_table, block_table_stride, cu_q_lens, context_lens, out,
                                      out_token_stride, batch, num_q_heads, num_kv_heads, head_dim,
                                      page_size, num_pages, max_q_len, softmax_scale, stream,
                                      litekv::kKvInt8);
}

extern "C" int litekv_varlen_prefill(const void *q, int64_t q_token_stride, const void *k,
                                     int64_t k_token_stride, const void *v, int64_t v_token_stride,
                                     const int32_t *seq_starts, const int32_t *seq_lens, void *out,
                                     int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t max_seq_len,
                                     int64_t num_tokens, float softmax_scale, void *stream) {
  return litekv::launch_varlen_prefill(q, q_token_stride, k, k_token_stride, v, v_token_stride,
                                       seq_starts, seq_lens, out, out_token_stride, batch,
                                       num_q_heads, num_kv_heads, head_dim, max_seq_len, num_tokens,
                                       softmax_scale, stream);
}
#endif  // LITEKV_HD == 128
