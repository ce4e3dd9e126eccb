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

// Folds the key slices of a split prefill: one wavefront per (query row, head) reads the row's
// `slices` log-sum-exps and partial rows (fp32, normalised per slice) and writes the fp16 row.
// A slice without keys has log-sum-exp -inf and weight 0; the last slice always has keys.
__global__ __launch_bounds__(4 * kWave) void prefill_split_merge_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_lse, half_t *__restrict__ out,
    int64_t out_stride, int64_t num_tokens, int32_t num_q_heads, int32_t slices) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (id >= num_tokens * num_q_heads) return;  // whole wavefronts
  const int64_t token = id / num_q_heads;
  const int head = (int)(id - token * num_q_heads);
  const int64_t piece_stride = num_tokens * num_q_heads;  // cells between the slices of a row
  const float l = lane < slices ? part_lse[lane * piece_stride + id] : -INFINITY;
  float mx = l;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, xor_lane(mx, off));
  const float w = lane < slices ? fast_exp2((l - mx) * 1.4426950408889634f) : 0.f;
  float den = w;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) den += xor_lane(den, off);
  if (2 * lane >= kHD) return;
  float o0 = 0.f, o1 = 0.f;
  for (int sidx = 0; sidx < slices; ++sidx) {  // in slice order: the sum does not depend on timing
    const float ws = __shfl(w, sidx, kWave);
    const float2 r = *(const float2 *)(part_o + (sidx * piece_stride + id) * kHD + 2 * lane);
    o0 += ws * r.x;
    o1 += ws * r.y;
  }
  const float inv = 1.0f / den;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  *(half2_t *)(out + token * out_stride + (int64_t)head * kHD + 2 * lane) =
      half2_t{(half_t)(o0 * inv), (half_t)(o1 * inv)};
}

static size_t prefill_split_workspace_bytes(int64_t num_tokens, int32_t num_q_heads, int32_t key_slices) {
  if (num_tokens <= 0 || num_q_heads <= 0 || key_slices <= 1) return 0;
  return (size_t)key_slices * (size_t)num_tokens * (size_t)num_q_heads * (kHD + 1) * sizeof(float);
}

// Key slices for a paged prefill whose row blocks alone would not fill the device, if the longest
// row sees `max_kv_len` keys: the count (at most kMaxPrefillKeySlices) with the smallest estimated
// time, 1 (do not split) unless that is at least 5 % less than unsplit. The estimate, in
// microseconds, head dim 128 (fits to one request's chunk of 64 to 512 rows over 0 to 32k cached
// tokens, 64 query / 8 kv heads): a workgroup walks max_kv_len / 64 / n key tiles at 1.0 us each
// while it has its compute unit to itself and at 1.7 us once the launch has more workgroups than
// compute units (two share one), times the rounds the launch needs on the device's resident
// slots; a cut costs the merge launch, 6 us, and a partial row (fp32) written and read back per
// query row, head and slice at 6 MB/us. (One chunk over 32k tokens, plain against sliced:
// 128 rows 527 -> 176 us, 256 rows 533 -> 298 us, 512 rows 609 -> 551 us; 128 rows over 2048 tokens
// 40 -> 30 us in four slices; 512 rows over 2048 tokens in two slices 49 -> 60 us and 128 rows of a
// fresh prompt in eight 14 -> 29 us, which the estimate rules out.)
static int32_t prefill_key_slices(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                  int32_t max_q_len, int64_t max_kv_len) {
  if (batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0 ||
      max_q_len <= 0 || max_kv_len <= 0 || num_q_heads / num_kv_heads > kMaxGroup) {
    return 1;
  }
  const PrefillShape s = prefill_shape(num_q_heads / num_kv_heads, max_q_len, kColTiles * kTiledWaves);
  const int64_t wgs = (int64_t)num_kv_heads * s.head_splits * s.row_blocks * batch;
  static thread_local int cached_device = -1, cached_cus = 0;  // compute units of the current device
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = -2;
  if (dev != cached_device) {
    int cus = 0;
    if (dev < 0 || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0) {
      cus = 256;
    }
    cached_device = dev;
    cached_cus = cus;
  }
  const int64_t cus = cached_cus;
  const int64_t slots = cus * (kHD == 64 ? 3 : 2);
  if (2 * wgs > slots) return 1;
  const double tile_us = kHD == 64 ? 0.6 : 1.0;
  const double tiles = (double)((max_kv_len + kKvTile - 1) / kKvTile);
  const double partial_us = (double)batch * max_q_len * num_q_heads * (kHD + 1) * 2.0 * sizeof(float) / 6.0e6;
  auto estimate = [&](int64_t n) {
    const int64_t resident = wgs * n;
    const double per_tile = resident <= cus ? tile_us : 1.7 * tile_us * (double)((resident + slots - 1) / slots);
    return tiles / (double)n * per_tile + (n > 1 ? 6.0 + partial_us * (double)n : 0.0);
  };
  const double unsplit = estimate(1);
  int64_t best = 1;
  double best_us = 0.95 * unsplit;
  for (int64_t n = 2; n <= kMaxPrefillKeySlices; ++n) {
    const double t = estimate(n);
    if (t < best_us) {
      best = n;
      best_us = t;
    }
  }
  return (int32_t)best;
}

// Causal chunk attention over paged KV; `kv_scales` selects the fp8 pool.
static int launch_paged_prefill(const char *what, const void *q, int64_t q_token_stride,
                                const void *kv_pool, const float *kv_scales,
                                const int32_t *block_table, int32_t block_table_stride,
                                const int32_t *cu_q_lens, const int32_t *context_lens, void *out,
                                int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                                int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                int64_t num_pages, int32_t max_q_len, float softmax_scale,
                                void *stream, int format,
                                const PrefillKeySplit &split = PrefillKeySplit{}) {
  const bool fp8 = format != kKvF16;  // a pool of 8-bit codes
  LITEKV_REQUIRE(split.key_slices >= 1 && split.key_slices <= kMaxPrefillKeySlices,
                 "%s: key_slices %d out of [1, %d]", what, split.key_slices, kMaxPrefillKeySlices);
  LITEKV_REQUIRE(split.key_slices == 1 || head_dim == 128 || head_dim == 64,
                 "%s: key slices take head_dim 64 or 128", what);
#if LITEKV_HD == 128
  if (head_dim == 64) {  // the head dim 64 build of this file
    return hd64_paged_prefill(what, q, q_token_stride, kv_pool, kv_scales, format, block_table, block_table_stride,
                              cu_q_lens, context_lens, out, out_token_stride, batch, num_q_heads,
                              num_kv_heads, page_size, num_pages, max_q_len, softmax_scale, stream, split);
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
  if (split.key_slices > 1) {
    // every block's keys in key_slices runs of tiles, one workgroup each, then the merge
    const int slices = split.key_slices;
    const int64_t rows = split.num_tokens;
    LITEKV_REQUIRE(rows >= 1 && rows * num_q_heads * slices <= 0x7fffffffLL,
                   "%s: num_tokens %lld out of range for %d key slices", what, (long long)rows, slices);
    const size_t need = prefill_split_workspace_bytes(rows, num_q_heads, slices);
    LITEKV_REQUIRE(split.workspace != nullptr && aligned16(split.workspace) && split.workspace_bytes >= need,
                   "%s: workspace of %zu bytes needed for %d key slices, got %zu", what, need, slices,
                   split.workspace_bytes);
    const PrefillShape s = prefill_shape(group, max_q_len, kColTiles * kTiledWaves);
    LITEKV_REQUIRE((uint64_t)s.row_blocks * slices <= 65535u, "%s: max_q_len %d too large for %d key slices",
                   what, max_q_len, slices);
    float *part_o = static_cast<float *>(split.workspace);
    float *part_lse = part_o + (size_t)slices * rows * num_q_heads * kHD;
    const PrefixTask task{part_o, part_lse, 0, (int32_t)rows, num_q_heads, 0, 0};
    const dim3 grid((unsigned)(num_kv_heads * s.head_splits), s.row_blocks * (unsigned)slices, (unsigned)batch);
    auto launch_slices = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, grid, dim3(kTiledWaves * kWave), 0, static_cast<hipStream_t>(stream),
                         static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                         out_token_stride, paged, packed, task, cu_q_lens, (const int32_t *)nullptr,
                         context_lens, group, s.head_splits, s.heads_per_wg, s.row_tiles,
                         softmax_scale * kLog2eP, slices);
    };
    if (format == kKvInt8) {
      launch_slices(varlen_prefill_tiled_kernel<kPagedPrefillSplitInt8>);
    } else if (format == kKvFp8) {
      launch_slices(varlen_prefill_tiled_kernel<kPagedPrefillSplitFp8>);
    } else {
      launch_slices(varlen_prefill_tiled_kernel<kPagedPrefillSplit>);
    }
    int rc2 = check_launch(what);
    if (rc2 != LITEKV_OK) return rc2;
    const int64_t merge_rows = rows * num_q_heads;
    hipLaunchKernelGGL(prefill_split_merge_kernel, dim3((unsigned)((merge_rows + 3) / 4)), dim3(4 * kWave), 0,
                       static_cast<hipStream_t>(stream), part_o, part_lse, static_cast<half_t *>(out),
                       out_token_stride, rows, num_q_heads, slices);
    return check_launch(what);
  }
  const int waves = (format == kKvF16 && LITEKV_PREFILL_WAVES == kWideWaves) ? kWideWaves : kTiledWaves;
  const PrefillShape s = prefill_shape(group, max_q_len, kColTiles * waves);
  LITEKV_REQUIRE(s.row_blocks <= 65535u, "%s: max_q_len %d too large", what, max_q_len);
  const dim3 grid((unsigned)(num_kv_heads * s.head_splits), s.row_blocks, (unsigned)batch);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(waves * kWave), 0, static_cast<hipStream_t>(stream),
                       static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                       out_token_stride, paged, packed, PrefixTask{}, cu_q_lens,
                       (const int32_t *)nullptr, context_lens, group, s.head_splits, s.heads_per_wg,
                       s.row_tiles, softmax_scale * kLog2eP, 1);
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
                       softmax_scale * kLog2eP, 1);
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
                       int32_t max_q_len, float softmax_scale, void *stream,
                       const PrefillKeySplit &split) {
  return launch_paged_prefill(what, q, q_token_stride, kv_pool, kv_scales, block_table,
                              block_table_stride, cu_q_lens, context_lens, out, out_token_stride,
                              batch, num_q_heads, num_kv_heads, 64, page_size, num_pages, max_q_len,
                              softmax_scale, stream, format, split);
}
int32_t hd64_prefill_key_slices(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                int32_t max_q_len, int64_t max_kv_len) {
  return prefill_key_slices(batch, num_q_heads, num_kv_heads, max_q_len, max_kv_len);
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

extern "C" size_t litekv_paged_prefill_split_workspace_bytes(int64_t num_tokens, int32_t num_q_heads,
                                                             int32_t head_dim, int32_t key_slices) {
  if (head_dim != 128 && head_dim != 64) return 0;
  if (num_tokens <= 0 || num_q_heads <= 0 || key_slices <= 1) return 0;
  return (size_t)key_slices * (size_t)num_tokens * (size_t)num_q_heads * (size_t)(head_dim + 1) * sizeof(float);
}

extern "C" int32_t litekv_paged_prefill_key_slices(int32_t batch, int32_t num_q_heads,
                                                   int32_t num_kv_heads, int32_t head_dim,
                                                   int32_t max_q_len, int64_t max_kv_len) {
  if (head_dim == 64) {
    return litekv::hd64_prefill_key_slices(batch, num_q_heads, num_kv_heads, max_q_len, max_kv_len);
  }
  if (head_dim != 128) return 1;
  return litekv::prefill_key_slices(batch, num_q_heads, num_kv_heads, max_q_len, max_kv_len);
}

extern "C" int litekv_paged_prefill_split(const void *q, int64_t q_token_stride, const void *kv_pool,
                                          const int32_t *block_table, int32_t block_table_stride,
                                          const int32_t *cu_q_lens, const int32_t *context_lens,
                                          void *out, int64_t out_token_stride, int32_t batch,
                                          int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                          int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                          int64_t num_tokens, int32_t key_slices, void *workspace,
                                          size_t workspace_bytes, float softmax_scale, void *stream) {
  litekv::PrefillKeySplit split;
  split.key_slices = key_slices;
  split.workspace = workspace;
  split.workspace_bytes = workspace_bytes;
  split.num_tokens = num_tokens;
  return litekv::launch_paged_prefill("paged_prefill_split", q, q_token_stride, kv_pool, nullptr,
                                      block_table, block_table_stride, cu_q_lens, context_lens, out,
                                      out_token_stride, batch, num_q_heads, num_kv_heads, head_dim,
                                      page_size, num_pages, max_q_len, softmax_scale, stream,
                                      litekv::kKvF16, split);
}

extern "C" int litekv_paged_prefill_split_q8(const void *q, int64_t q_token_stride, const void *kv_pool,
                                             const float *kv_scales, int32_t pool_is_int8,
                                             const int32_t *block_table, int32_t block_table_stride,
                                             const int32_t *cu_q_lens, const int32_t *context_lens,
                                             void *out, int64_t out_token_stride, int32_t batch,
                                             int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                             int32_t page_size, int64_t num_pages, int32_t max_q_len,
                                             int64_t num_tokens, int32_t key_slices, void *workspace,
                                             size_t workspace_bytes, float softmax_scale, void *stream) {
  litekv::PrefillKeySplit split;
  split.key_slices = key_slices;
  split.workspace = workspace;
  split.workspace_bytes = workspace_bytes;
  split.num_tokens = num_tokens;
  return litekv::launch_paged_prefill(pool_is_int8 ? "paged_prefill_split_int8" : "paged_prefill_split_fp8", q,
                                      q_token_stride, kv_pool, kv_scales, block_table, block_table_stride,
                                      cu_q_lens, context_lens, out, out_token_stride, batch, num_q_heads,
                                      num_kv_heads, head_dim, page_size, num_pages, max_q_len,
                                      softmax_scale, stream, pool_is_int8 ? litekv::kKvInt8 : litekv::kKvFp8,
                                      split);
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
