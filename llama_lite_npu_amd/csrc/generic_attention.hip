// Attention for head dims other than 128 (32, 64, 256): one kernel behind the decode and prefill
// entry points, whose tuned kernels are built around 128-wide rows. The reference kernels take
// the head dim as a compile-time block size (lite_llama/kernels/flashdecoding.py:305, 393-396;
// flashattention2_nopad.py:39-163) and serve every model config through the same call
// (lite_llama/models/model_config.py:200); this is that generality, with plain fp32 arithmetic
// instead of MFMA tiles.
//
// One wavefront per (kv head, block of query rows). It works on 16 columns, a column being one
// (query row, query head of the kv head) pair: a decode step has one query row per sequence, so
// its columns are the (up to 16) query heads of the kv head; a prefill block takes
// 16 / (query heads per kv head) neighbouring prompt rows, so that the K and V rows they share
// are read once for all of them (row i of a sequence sees its history and keys 0..i of the
// prompt: each column has its own number of keys). The wavefront walks the keys of the block's
// last row 64 at a time. Scores: lane l holds key l of the tile, reads that key's K
// row once and takes its dot product with the columns' query rows, which
// sit in LDS as fp32, already multiplied by softmax_scale * log2(e). Softmax state (running
// maximum and denominator per column) is kept by every lane alike. Values: the probabilities of
// the tile go through LDS, lane l then holds output elements l, l + 64, ... of every column and
// adds the tile's V rows, read one row per step by all lanes together.
//
// Pools of 8-bit codes are read as in the tuned kernels: codes become fp16 exactly, the K scale
// multiplies the scores, the V scale the result. The fused append of a decode step (k_new /
// v_new) writes the step's rows to the slot of token len - 1 and attends them as stored.
#include "common.h"
#include "kv_fp8.h"

namespace litekv {

constexpr int kGenericMaxDim = 256;
constexpr int kGenericMaxGroup = 16;

// What a launch works on (see generic_attention_kernel).
struct GenericTask {
  const half_t *q;
  int64_t q_row_stride;        // elements between query rows ([Hq][D] each)
  half_t *out;
  int64_t out_row_stride;
  // paged keys
  void *kv_pool;               // [slots][2*Hkv][D] fp16 or codes; null: packed keys
  const float *scales;         // 8-bit pools: K-head scales, then V-head scales
  const int32_t *block_table;  // or the plan of a balanced decode step, which lists the pages
  const int32_t *plan;
  int32_t bt_stride;
  int32_t page_size;
  int32_t num_pages;
  // packed keys
  const half_t *k, *v;         // [T][Hkv][D]
  int64_t k_stride, v_stride;
  const int32_t *seq_starts;   // [B] first packed row of each sequence
  // rows
  const int32_t *seq_lens;     // decode: [B] keys per sequence (cu_q_lens and q_lens null)
  const int32_t *cu_q_lens;    // paged prefill: [B + 1]
  const int32_t *q_lens;       // packed prefill: [B]
  const int32_t *context_lens; // paged prefill: [B] cached tokens before the chunk, or null
  // fused append of a decode step, or null
  const half_t *k_new, *v_new; // [B][Hkv][D]
  int64_t k_new_stride, v_new_stride;
  int32_t num_q_heads, num_kv_heads, group, head_dim;
  int32_t rows_per_wave;       // query rows of one sequence a wavefront takes (1 for a decode step)
  float scale_log2;
};

// Eight elements of a K or V row starting at element d8 * 8: fp16 values, or decoded codes.
template <int KV>
__device__ __forceinline__ half8_t load8(const void *row, int d8) {
  if constexpr (KV == kKvF16) {
    return *((const half8_t *)row + d8);
  } else {
    return codes_to_half<KV>(*((const uint2_t *)row + d8));
  }
}

// What the pool holds after x was appended to it (the value attention sees).
template <int KV>
__device__ __forceinline__ half8_t as_stored(half8_t x, float inv_scale) {
  if constexpr (KV == kKvF16) {
    return x;
  } else {
    return codes_to_half<KV>(half_to_codes<KV>(x, inv_scale));
  }
}

template <int KV>
__device__ __forceinline__ void store8(void *row, int d8, half8_t x, float inv_scale) {
  if constexpr (KV == kKvF16) {
    *((half8_t *)row + d8) = x;
  } else {
    *((uint2_t *)row + d8) = half_to_codes<KV>(x, inv_scale);
  }
}

// grid (head slices, blocks of rows_per_wave query rows per sequence, sequences), one wavefront
// each; a head slice is a kv head, or up to 16 of its query heads when it has more than 16 (see
// head_slice)
template <int KV>
__global__ __launch_bounds__(kWave) void generic_attention_kernel(GenericTask t) {
  __shared__ float qs[kGenericMaxGroup][kGenericMaxDim];
  __shared__ float ps[kWave][kGenericMaxGroup + 1];
  const int lane = threadIdx.x;
  const HeadSlice hs = head_slice((int)blockIdx.x, head_slices(t.group), t.group);
  const int h = hs.kv_head;
  const int row0 = blockIdx.y * t.rows_per_wave;  // first query row of the block in its sequence
  const int b = blockIdx.z;
  const int D = t.head_dim;
  const bool paged = t.kv_pool != nullptr;

  // the block's first query row, the keys that row sees, how many rows the block holds, and
  // where its sequence's packed keys start
  int64_t q_row0;
  int keys0;
  int rows_here = 1;
  int64_t packed0 = 0;
  if (t.cu_q_lens != nullptr) {
    const int q_start = t.cu_q_lens[b];
    const int q_len = t.cu_q_lens[b + 1] - q_start;
    if (row0 >= q_len) return;
    rows_here = q_len - row0 < t.rows_per_wave ? q_len - row0 : t.rows_per_wave;
    q_row0 = q_start + row0;
    keys0 = (t.context_lens ? t.context_lens[b] : 0) + row0 + 1;
  } else if (t.q_lens != nullptr) {
    if (row0 >= t.q_lens[b]) return;
    rows_here = t.q_lens[b] - row0 < t.rows_per_wave ? t.q_lens[b] - row0 : t.rows_per_wave;
    packed0 = t.seq_starts[b];
    q_row0 = packed0 + row0;
    keys0 = row0 + 1;
  } else {
    q_row0 = b;
    keys0 = t.seq_lens[b];
  }
  const int hq0 = hs.q_head0;
  if (keys0 <= 0) {  // an empty sequence of a decode step
    half_t *out_row = t.out + q_row0 * t.out_row_stride + (int64_t)hq0 * D;
    for (int i = lane; i < hs.q_heads * D; i += kWave) out_row[i] = (half_t)0.f;
    return;
  }
  const int n_keys = keys0 + rows_here - 1;  // of the block's last row: the keys the wavefront walks

  // Column g is query head g % heads_per_row of row g / heads_per_row of the block. A column
  // past the block's rows or the slice's heads repeats column 0 and is not written.
  const int heads_per_row = t.rows_per_wave > 1 ? kGenericMaxGroup / t.rows_per_wave : hs.q_heads;
  const int cols = t.rows_per_wave > 1 ? kGenericMaxGroup : hs.q_heads;
  int col_keys[kGenericMaxGroup];
  bool col_written[kGenericMaxGroup];
  int col_row[kGenericMaxGroup], col_head[kGenericMaxGroup];
#pragma unroll
  for (int g = 0; g < kGenericMaxGroup; ++g) {
    const int r = g / heads_per_row, hd = g - r * heads_per_row;
    col_written[g] = g < cols && r < rows_here && hd < hs.q_heads;
    col_row[g] = col_written[g] ? r : 0;
    col_head[g] = col_written[g] ? hd : 0;
    col_keys[g] = keys0 + col_row[g];
  }

  float k_scale = 1.0f, v_scale = 1.0f;
  if constexpr (KV != kKvF16) {
    k_scale = t.scales[h];
    v_scale = t.scales[t.num_kv_heads + h];
  }
  const float k_inv = 1.0f / k_scale, v_inv = 1.0f / v_scale;

#pragma unroll
  for (int g = 0; g < kGenericMaxGroup; ++g) {
    if (g < cols) {
      const half_t *q_col = t.q + (q_row0 + col_row[g]) * t.q_row_stride + (int64_t)(hq0 + col_head[g]) * D;
      for (int i = lane; i < D; i += kWave) qs[g][i] = (float)q_col[i] * t.scale_log2;
    }
  }
  __syncthreads();

  const int elem = KV == kKvF16 ? 2 : 1;  // bytes per stored element
  const int64_t slot_bytes = (int64_t)2 * t.num_kv_heads * D * elem;
  const int32_t *table = (paged && t.block_table) ? t.block_table + (int64_t)b * t.bt_stride : nullptr;
  // A plan lists the 16-token pages of all sequences in batch order, cut into chunk entries.
  const bool planned = paged && t.block_table == nullptr;
  const LineCut cut(planned ? t.plan[kMetaTotal] : 0, planned ? t.plan[kMetaChunks] : 1);
  const int plan_batch = planned ? t.plan[kMetaBatch] : 0;
  const int entry_stride = planned ? t.plan[kMetaEntryStride] : 0;
  const int before = planned ? t.plan[plan_seq_before_offset(plan_batch) + b] : 0;
  // the K row of key `tok` (V: + num_kv_heads * D elements in a pool)
  auto k_row_of = [&](int tok) -> const char * {
    if (planned) {
      // the plan holds at most a block-table row's worth of 16-token pages per sequence
      const int cap16 = t.bt_stride * (t.page_size >> 4);
      const int f = before + ((tok >> 4) < cap16 ? (tok >> 4) : cap16 - 1);
      const int c = cut.chunk_of(f);
      const int pid16 = t.plan[plan_entries_offset(plan_batch) + (int64_t)c * entry_stride + kEntryHeader +
                               (f - cut.chunk_start(c))];
      const int64_t slot = (int64_t)pid16 * 16 + (tok & 15);
      return (const char *)t.kv_pool + slot * slot_bytes + (int64_t)h * D * elem;
    }
    if (paged) {
      int at = tok / t.page_size;
      at = at < t.bt_stride ? at : t.bt_stride - 1;  // a length beyond the row re-reads its last entry
      int pid = table[at];
      pid = pid < 0 ? 0 : (pid >= t.num_pages ? t.num_pages - 1 : pid);
      const int64_t slot = (int64_t)pid * t.page_size + tok % t.page_size;
      return (const char *)t.kv_pool + slot * slot_bytes + (int64_t)h * D * elem;
    }
    return (const char *)(t.k + (packed0 + tok) * t.k_stride + (int64_t)h * D);
  };
  // a pool keeps a token's V heads behind its K heads
  const int64_t v_after_k = (int64_t)t.num_kv_heads * D * elem;
  auto v_row_of = [&](int tok) -> const char * {
    if (paged) return k_row_of(tok) + v_after_k;
    return (const char *)(t.v + (packed0 + tok) * t.v_stride + (int64_t)h * D);
  };

  // the step's new rows of this head, if this launch appends them (not for a length beyond what
  // the block-table row can name: the row's last page is not where that token belongs)
  const bool appends = t.k_new != nullptr &&
                       (int64_t)n_keys <= (int64_t)t.bt_stride * t.page_size;
  const half_t *k_new = appends ? t.k_new + (int64_t)b * t.k_new_stride + (int64_t)h * D : nullptr;
  const half_t *v_new = appends ? t.v_new + (int64_t)b * t.v_new_stride + (int64_t)h * D : nullptr;

  float m[kGenericMaxGroup], den[kGenericMaxGroup];
  float acc[kGenericMaxGroup][kGenericMaxDim / kWave];
#pragma unroll
  for (int g = 0; g < kGenericMaxGroup; ++g) {
    m[g] = -INFINITY;
    den[g] = 0.f;
#pragma unroll
    for (int c = 0; c < kGenericMaxDim / kWave; ++c) acc[g][c] = 0.f;
  }

  for (int t0 = 0; t0 < n_keys; t0 += kWave) {
    const int tok = t0 + lane;
    const bool live = tok < n_keys;
    const bool is_new = appends && tok == n_keys - 1;
    const char *k_row = k_row_of(live ? tok : n_keys - 1);
    float s[kGenericMaxGroup];
#pragma unroll
    for (int g = 0; g < kGenericMaxGroup; ++g) s[g] = 0.f;
    for (int d8 = 0; d8 < D / 8; ++d8) {
      half8_t kv8;
      if (is_new) {
        const half8_t fresh = *((const half8_t *)k_new + d8);
        store8<KV>(const_cast<char *>(k_row), d8, fresh, k_inv);
        kv8 = as_stored<KV>(fresh, k_inv);
        const half8_t fresh_v = *((const half8_t *)v_new + d8);
        store8<KV>(const_cast<char *>(k_row) + v_after_k, d8, fresh_v, v_inv);
      } else {
        kv8 = load8<KV>(k_row, d8);
      }
#pragma unroll
      for (int g = 0; g < kGenericMaxGroup; ++g) {
        if (g < cols) {
#pragma unroll
          for (int e = 0; e < 8; ++e) s[g] += qs[g][8 * d8 + e] * (float)kv8[e];
        }
      }
    }
    // softmax of the tile against the running state; probabilities to LDS
#pragma unroll
    for (int g = 0; g < kGenericMaxGroup; ++g) {
      if (g < cols) {
        // a key past the column's own row is masked; key 0 is in every column's first tile, so
        // the running maximum is finite from then on
        const float sv = tok < col_keys[g] ? s[g] * k_scale : -INFINITY;
        float mx = sv;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
        const float m_new = fmaxf(m[g], mx);
        const float alpha = fast_exp2(m[g] - m_new);
        const float p = fast_exp2(sv - m_new);
        float sum = p;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, kWave);
        den[g] = den[g] * alpha + sum;
        m[g] = m_new;
#pragma unroll
        for (int c = 0; c < kGenericMaxDim / kWave; ++c) acc[g][c] *= alpha;
        ps[lane][g] = p;
      }
    }
    __syncthreads();
    // values: all lanes read key j's V row together, lane l its elements l, l + 64, ...
    const int n_here = (n_keys - t0) < kWave ? (n_keys - t0) : kWave;
    for (int j = 0; j < n_here; ++j) {
      const int tok_j = t0 + j;
      const char *v_row = v_row_of(tok_j);
      const bool new_j = appends && tok_j == n_keys - 1;
#pragma unroll
      for (int c = 0; c < kGenericMaxDim / kWave; ++c) {
        const int d = lane + kWave * c;
        if (d < D) {
          float val;
          if (new_j) {
            val = (float)as_stored<KV>(*((const half8_t *)v_new + d / 8), v_inv)[d % 8];
          } else {
            val = (float)load8<KV>(v_row, d / 8)[d % 8];
          }
#pragma unroll
          for (int g = 0; g < kGenericMaxGroup; ++g) {
            if (g < cols) acc[g][c] += ps[j][g] * val;
          }
        }
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int g = 0; g < kGenericMaxGroup; ++g) {
    if (col_written[g]) {
      const float inv = v_scale / den[g];
      half_t *out_col = t.out + (q_row0 + col_row[g]) * t.out_row_stride + (int64_t)(hq0 + col_head[g]) * D;
#pragma unroll
      for (int c = 0; c < kGenericMaxDim / kWave; ++c) {
        const int d = lane + kWave * c;
        if (d < D) out_col[d] = (half_t)(acc[g][c] * inv);
      }
    }
  }
}

bool generic_head_dim(int32_t head_dim) { return head_dim == 32 || head_dim == 64 || head_dim == 256; }

int launch_generic_attention(const char *what, const GenericLaunch &a) {
  LITEKV_REQUIRE(generic_head_dim(a.head_dim), "%s: head_dim %d unsupported (32, 64, 128 or 256)",
                 what, a.head_dim);
  LITEKV_REQUIRE(a.batch >= 0 && a.batch <= 65535, "%s: batch %d out of [0, 65535]", what, a.batch);
  LITEKV_REQUIRE(a.num_q_heads > 0 && a.num_kv_heads > 0 && a.num_q_heads % a.num_kv_heads == 0 &&
                     a.num_q_heads <= 65535,
                 "%s: num_q_heads %d / num_kv_heads %d invalid", what, a.num_q_heads, a.num_kv_heads);
  const int group = a.num_q_heads / a.num_kv_heads;
  LITEKV_REQUIRE(group <= kMaxGroup, "%s: %d query heads per kv head unsupported (max %d)", what,
                 group, kMaxGroup);
  LITEKV_REQUIRE(a.rows_per_seq >= 0 && a.rows_per_seq <= 65535, "%s: %d query rows per sequence",
                 what, a.rows_per_seq);
  if (a.batch == 0 || a.rows_per_seq == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(a.q && a.out, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(a.q) && aligned16(a.out), "%s: q and out must be 16-byte aligned", what);
  const int64_t row = (int64_t)a.num_q_heads * a.head_dim;
  LITEKV_REQUIRE(a.q_row_stride >= row && a.q_row_stride % 8 == 0 && a.out_row_stride >= row,
                 "%s: row strides (%lld, %lld) invalid", what, (long long)a.q_row_stride,
                 (long long)a.out_row_stride);
  LITEKV_REQUIRE(a.seq_lens || a.cu_q_lens || a.q_lens, "%s: null pointer (lengths)", what);
  if (a.kv_pool != nullptr) {
    LITEKV_REQUIRE((a.block_table != nullptr && a.bt_stride >= 1) || a.plan != nullptr,
                   "%s: block table missing", what);
    LITEKV_REQUIRE(page_shift_of(a.page_size) >= 0,
                   "%s: page_size %d unsupported (16, 32, 64, 128 or 256)", what, a.page_size);
    LITEKV_REQUIRE(a.num_pages >= 1 && a.num_pages <= 0x7fffffffLL / a.page_size,
                   "%s: num_pages %lld out of range", what, (long long)a.num_pages);
    LITEKV_REQUIRE(aligned16(a.kv_pool), "%s: kv_pool must be 16-byte aligned", what);
    LITEKV_REQUIRE(a.format == kKvF16 || a.scales != nullptr, "%s: scales is null", what);
  } else {
    LITEKV_REQUIRE(a.k && a.v && a.seq_starts && a.q_lens, "%s: null pointer (packed keys)", what);
    LITEKV_REQUIRE(aligned16(a.k) && aligned16(a.v), "%s: k and v must be 16-byte aligned", what);
    const int64_t kv_row = (int64_t)a.num_kv_heads * a.head_dim;
    LITEKV_REQUIRE(a.k_stride >= kv_row && a.v_stride >= kv_row && a.k_stride % 8 == 0 &&
                       a.v_stride % 8 == 0,
                   "%s: k / v strides (%lld, %lld) invalid", what, (long long)a.k_stride,
                   (long long)a.v_stride);
  }
  LITEKV_REQUIRE((a.k_new == nullptr) == (a.v_new == nullptr), "%s: k_new and v_new go together", what);
  if (a.k_new != nullptr) {
    const int64_t kv_row = (int64_t)a.num_kv_heads * a.head_dim;
    LITEKV_REQUIRE(a.seq_lens != nullptr && a.kv_pool != nullptr, "%s: the fused append is a decode step's",
                   what);
    LITEKV_REQUIRE(aligned16(a.k_new) && aligned16(a.v_new) && a.k_new_stride >= kv_row &&
                       a.v_new_stride >= kv_row && a.k_new_stride % 8 == 0 && a.v_new_stride % 8 == 0,
                   "%s: k_new / v_new invalid", what);
  }
  GenericTask t{};
  t.q = static_cast<const half_t *>(a.q);
  t.q_row_stride = a.q_row_stride;
  t.out = static_cast<half_t *>(a.out);
  t.out_row_stride = a.out_row_stride;
  t.kv_pool = a.kv_pool;
  t.scales = a.scales;
  t.block_table = a.block_table;
  t.plan = a.plan;
  t.bt_stride = a.bt_stride;
  t.page_size = a.page_size;
  t.num_pages = (int32_t)a.num_pages;
  t.k = static_cast<const half_t *>(a.k);
  t.v = static_cast<const half_t *>(a.v);
  t.k_stride = a.k_stride;
  t.v_stride = a.v_stride;
  t.seq_starts = a.seq_starts;
  t.seq_lens = a.seq_lens;
  t.cu_q_lens = a.cu_q_lens;
  t.q_lens = a.q_lens;
  t.context_lens = a.context_lens;
  t.k_new = static_cast<const half_t *>(a.k_new);
  t.v_new = static_cast<const half_t *>(a.v_new);
  t.k_new_stride = a.k_new_stride;
  t.v_new_stride = a.v_new_stride;
  t.num_q_heads = a.num_q_heads;
  t.num_kv_heads = a.num_kv_heads;
  t.group = group;
  t.head_dim = a.head_dim;
  // a decode step has one query row per sequence; a prefill block takes as many rows as fit the
  // 16 columns beside the (at most 16) query heads of a slice
  const int slices = head_slices(group);
  const int heads_per_slice = (group + slices - 1) / slices;
  int rows_per_wave = 1;
  if (a.cu_q_lens != nullptr || a.q_lens != nullptr) {
    while (rows_per_wave * 2 * heads_per_slice <= kGenericMaxGroup) rows_per_wave *= 2;
  }
  t.rows_per_wave = rows_per_wave;
  t.scale_log2 = a.softmax_scale * 1.4426950408889634f;
  const int slice_heads = a.num_kv_heads * head_slices(group);
  LITEKV_REQUIRE(slice_heads <= 65535, "%s: num_q_heads %d too large", what, a.num_q_heads);
  const dim3 grid((unsigned)slice_heads, (unsigned)((a.rows_per_seq + rows_per_wave - 1) / rows_per_wave),
                  (unsigned)a.batch);
  const hipStream_t stream = static_cast<hipStream_t>(a.stream);
  const int format = a.kv_pool != nullptr ? a.format : kKvF16;
  if (format == kKvInt8) {
    hipLaunchKernelGGL(generic_attention_kernel<kKvInt8>, grid, dim3(kWave), 0, stream, t);
  } else if (format == kKvFp8) {
    hipLaunchKernelGGL(generic_attention_kernel<kKvFp8>, grid, dim3(kWave), 0, stream, t);
  } else {
    hipLaunchKernelGGL(generic_attention_kernel<kKvF16>, grid, dim3(kWave), 0, stream, t);
  }
  return check_launch(what);
}

}  // namespace litekv
