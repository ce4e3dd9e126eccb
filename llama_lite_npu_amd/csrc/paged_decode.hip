// Paged flash-decoding for gfx950: split kernel + deterministic merge.
//
// Split kernel, one wavefront per (kv head, split, sequence). A wavefront
// walks its pages; for each 16-token page it computes, with all Hq/Hkv query
// heads of the kv head at once (so K/V bytes are read from HBM exactly once):
//
//   S^T[token][head]  = K_page[16 x 128] . Q^T[128 x 16]      4 x MFMA 16x16x32
//   online softmax over tokens, per head column (fp32, exp2 domain)
//   O^T[d][head]     += V_page^T[128 x 16] . P^T[16 x 16]      8 x MFMA 16x16x16
//
// The S^T accumulator layout (lane l: head l%16, tokens 4*(l/16)..+3) is also
// the B-operand layout of the second product, so probabilities never leave
// their lane. K fragments are loaded straight from the page in A-operand
// layout (64 contiguous bytes per token per instruction); V rows are loaded
// as full 256-byte rows, staged in LDS and read back transposed. Softmax row
// reductions run over the 4 lane groups with wavefront shuffles.
//
// Split boundaries are a pure function of the sequence length, so the result
// does not depend on scheduling; the merge kernel combines the fp32 partials
// in split order with the usual log-sum-exp weights.
#include "common.h"

namespace litekv {

constexpr int kVPitch = kHeadDim + 8;  // fp16 elements per staged V row (272 bytes)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__host__ __device__ __forceinline__ int splits_for_pages(int pages, int max_splits,
                                                         int min_pages_per_split) {
  int n = (pages + min_pages_per_split - 1) / min_pages_per_split;
  n = n < 1 ? 1 : n;
  return n < max_splits ? n : max_splits;
}

__global__ __launch_bounds__(64) void paged_decode_split_kernel(
    const half_t *__restrict__ q, int64_t q_batch_stride, const half_t *__restrict__ kv,
    const int32_t *__restrict__ block_table, int32_t bt_stride,
    const int32_t *__restrict__ seq_lens, half_t *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_lse, int32_t num_q_heads, int32_t num_kv_heads, int32_t group,
    int32_t max_splits, int32_t min_pages_per_split, int32_t num_pages, float scale_log2) {
  __shared__ __attribute__((aligned(16))) half_t vstage[kPageSize * kVPitch];

  const int lane = threadIdx.x;
  const int n = lane & 15;   // query head inside the group (column of S^T)
  const int g = lane >> 4;   // lane group: owns tokens 4g..4g+3 of a page
  const int h = blockIdx.x;  // kv head
  const int split = blockIdx.y;
  const int b = blockIdx.z;

  const int len = seq_lens[b];
  const int hq = h * group + n;
  if (len <= 0) {
    if (split == 0 && n < group) {
      half_t *o = out + ((int64_t)b * num_q_heads + hq) * kHeadDim;
#pragma unroll
      for (int j = 0; j < 8; ++j) *(half4_t *)(o + 16 * j + 4 * g) = half4_t{0, 0, 0, 0};
    }
    return;
  }
  const int pages = (len + kPageSize - 1) / kPageSize;
  const int n_splits = splits_for_pages(pages, max_splits, min_pages_per_split);
  if (split >= n_splits) return;
  const int p0 = (int)(((int64_t)split * pages) / n_splits);
  const int p1 = (int)(((int64_t)(split + 1) * pages) / n_splits);

  // Q^T as B operand: lane (n, g) holds q[head n][32*kk + 8*g .. +7].
  half8_t qf[4];
  {
    const half_t *qrow = q + (int64_t)b * q_batch_stride + (int64_t)hq * kHeadDim + 8 * g;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      qf[kk] = (n < group) ? *(const half8_t *)(qrow + 32 * kk) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  const int64_t row_stride = (int64_t)2 * num_kv_heads * kHeadDim;  // elements per slot
  const half_t *k_base = kv + (int64_t)h * kHeadDim + 8 * g;                     // + slot row n
  const half_t *v_base = kv + (int64_t)(num_kv_heads + h) * kHeadDim + 8 * n;    // + slot row 4i+g
  const int32_t *table = block_table + (int64_t)b * bt_stride;

  float4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;  // running max (log2 domain), identical in the 4 lanes of a head
  float d_run = 0.f;        // this lane's share of the running denominator

  int table_regs = 0;  // page ids p0 + 64*c + lane of the current 64-page chunk
  half8_t kf[4], vf[4];

  auto load_page = [&](int p, half8_t (&kd)[4], half8_t (&vd)[4]) {
    int pid = __builtin_amdgcn_readlane(table_regs, (p - p0) & 63);
    pid = pid < 0 ? 0 : (pid >= num_pages ? num_pages - 1 : pid);
    const int64_t slot0 = (int64_t)pid * kPageSize;
    const half_t *kr = k_base + (slot0 + n) * row_stride;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) kd[kk] = *(const half8_t *)(kr + 32 * kk);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = 4 * i + g;
      half8_t x = *(const half8_t *)(v_base + (slot0 + t) * row_stride);
      // Slots past the sequence end hold arbitrary bits: keep them out of the MFMA.
      vd[i] = (p * kPageSize + t < len) ? x : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  };

  {
    const int idx = p0 + lane;
    table_regs = (idx < p1) ? table[idx] : 0;
  }
  load_page(p0, kf, vf);

  for (int p = p0; p < p1; ++p) {
    // Stage V of page p (rows 4i+g, 16-byte column n).
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) *(half8_t *)(&vstage[(4 * i + g) * kVPitch + 8 * n]) = vf[i];
    __syncthreads();

    half8_t kc[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) kc[kk] = kf[kk];

    // Prefetch page p+1 while page p is being reduced.
    if (p + 1 < p1) {
      if (((p + 1 - p0) & 63) == 0) {
        const int idx = p + 1 + lane;
        table_regs = (idx < p1) ? table[idx] : 0;
      }
      load_page(p + 1, kf, vf);
    }

    float4_t st = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) st = mfma_16x16x32(kc[kk], qf[kk], st);

    float sv[4];
    const int tok0 = p * kPageSize + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) sv[i] = (tok0 + i < len) ? st[i] * scale_log2 : -INFINITY;
    float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
    mx = fmaxf(mx, xor_lane(mx, 16));
    mx = fmaxf(mx, xor_lane(mx, 32));
    const float m_new = fmaxf(m_run, mx);  // finite: every page of the range has a valid token
    const float alpha = fast_exp2(m_run - m_new);
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) pr[i] = fast_exp2(sv[i] - m_new);
    d_run = d_run * alpha + ((pr[0] + pr[1]) + (pr[2] + pr[3]));
    m_run = m_new;
    const half4_t pt = half4_t{(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};

#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half_t *vcol = &vstage[(4 * g) * kVPitch + 16 * j + n];
      const half4_t vt = half4_t{vcol[0], vcol[kVPitch], vcol[2 * kVPitch], vcol[3 * kVPitch]};
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
  if (n < group) {
    if (n_splits == 1) {
      half_t *o = out + ((int64_t)b * num_q_heads + hq) * kHeadDim + 4 * g;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        *(half4_t *)(o + 16 * j) = half4_t{(half_t)(acc[j][0] * inv), (half_t)(acc[j][1] * inv),
                                           (half_t)(acc[j][2] * inv), (half_t)(acc[j][3] * inv)};
      }
    } else {
      const int64_t cell = ((int64_t)b * num_q_heads + hq) * max_splits + split;
      float *po = part_o + cell * kHeadDim + 4 * g;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        *(float4_t *)(po + 16 * j) =
            float4_t{acc[j][0] * inv, acc[j][1] * inv, acc[j][2] * inv, acc[j][3] * inv};
      }
      if (g == 0) part_lse[cell] = (m_run + fast_log2(d_tot)) * kLn2;
    }
  }
}

// One block per (query head, sequence), one lane per output element.
__global__ __launch_bounds__(kHeadDim) void paged_decode_merge_kernel(
    const int32_t *__restrict__ seq_lens, half_t *__restrict__ out,
    const float *__restrict__ part_o, const float *__restrict__ part_lse, int32_t num_q_heads,
    int32_t max_splits, int32_t min_pages_per_split) {
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int d = threadIdx.x;
  const int len = seq_lens[b];
  if (len <= 0) return;
  const int pages = (len + kPageSize - 1) / kPageSize;
  const int n_splits = splits_for_pages(pages, max_splits, min_pages_per_split);
  if (n_splits == 1) return;  // the split kernel already wrote the final row
  const int64_t cell0 = ((int64_t)b * num_q_heads + hq) * max_splits;
  const float *lse = part_lse + cell0;
  const float *po = part_o + cell0 * kHeadDim + d;
  float mx = -INFINITY;
  for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, lse[s]);
  float num = 0.f, den = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float w = fast_exp2((lse[s] - mx) * kLog2e);
    num += w * po[(int64_t)s * kHeadDim];
    den += w;
  }
  out[((int64_t)b * num_q_heads + hq) * kHeadDim + d] = (half_t)(num / den);
}

struct DecodeArgs {
  const void *q;
  int64_t q_batch_stride;
  const void *kv_pool;
  const int32_t *block_table;
  int32_t block_table_stride;
  const int32_t *seq_lens;
  void *out;
  void *workspace;
  size_t workspace_bytes;
  int32_t batch, num_q_heads, num_kv_heads, head_dim, page_size;
  int64_t num_pages;
  int32_t max_splits, min_pages_per_split;
  float softmax_scale;
  void *stream;
};

static size_t workspace_bytes_for(int64_t batch, int64_t hq, int64_t d, int64_t s) {
  if (batch <= 0 || hq <= 0 || d <= 0 || s <= 1) return 0;
  return (size_t)(batch * hq * s * (d + 1)) * sizeof(float);
}

static int validate_common(const char *what, const DecodeArgs &a, bool need_inputs) {
  LITEKV_REQUIRE(a.batch >= 0, "%s: batch %d < 0", what, a.batch);
  LITEKV_REQUIRE(a.head_dim == kHeadDim, "%s: head_dim %d unsupported (only %d)", what, a.head_dim,
                 kHeadDim);
  LITEKV_REQUIRE(a.page_size == kPageSize, "%s: page_size %d unsupported (only %d)", what,
                 a.page_size, kPageSize);
  LITEKV_REQUIRE(a.num_q_heads > 0, "%s: num_q_heads %d <= 0", what, a.num_q_heads);
  LITEKV_REQUIRE(a.max_splits >= 1 && a.max_splits <= 65535, "%s: max_splits %d out of [1, 65535]",
                 what, a.max_splits);
  LITEKV_REQUIRE(a.min_pages_per_split >= 1, "%s: min_pages_per_split %d < 1", what,
                 a.min_pages_per_split);
  LITEKV_REQUIRE(a.batch <= 65535, "%s: batch %d > 65535", what, a.batch);
  if (a.batch == 0) return LITEKV_OK;
  LITEKV_REQUIRE(a.seq_lens && a.out, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(a.out), "%s: out must be 16-byte aligned", what);
  if (a.max_splits > 1) {
    const size_t need = workspace_bytes_for(a.batch, a.num_q_heads, a.head_dim, a.max_splits);
    LITEKV_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= need,
                   "%s: workspace of %zu bytes needed for %d splits, got %zu", what, need,
                   a.max_splits, a.workspace ? a.workspace_bytes : (size_t)0);
    LITEKV_REQUIRE(aligned16(a.workspace), "%s: workspace must be 16-byte aligned", what);
  }
  if (need_inputs) {
    LITEKV_REQUIRE(a.q && a.kv_pool && a.block_table, "%s: null pointer", what);
    LITEKV_REQUIRE(a.num_kv_heads > 0 && a.num_q_heads % a.num_kv_heads == 0,
                   "%s: num_q_heads %d not a multiple of num_kv_heads %d", what, a.num_q_heads,
                   a.num_kv_heads);
    LITEKV_REQUIRE(a.num_q_heads / a.num_kv_heads <= 16,
                   "%s: %d query heads per kv head unsupported (max 16)", what,
                   a.num_q_heads / a.num_kv_heads);
    LITEKV_REQUIRE(a.q_batch_stride >= (int64_t)a.num_q_heads * a.head_dim &&
                       a.q_batch_stride % 8 == 0,
                   "%s: q_batch_stride %lld invalid", what, (long long)a.q_batch_stride);
    LITEKV_REQUIRE(aligned16(a.q) && aligned16(a.kv_pool), "%s: q and kv_pool must be 16-byte aligned",
                   what);
    LITEKV_REQUIRE(a.block_table_stride >= 1, "%s: block_table_stride %d < 1", what,
                   a.block_table_stride);
    LITEKV_REQUIRE(a.num_pages >= 1 && a.num_pages <= 0x7fffffffLL / kPageSize,
                   "%s: num_pages %lld out of range", what, (long long)a.num_pages);
  }
  return LITEKV_OK;
}

static float *lse_of(const DecodeArgs &a) {
  return static_cast<float *>(a.workspace) +
         (size_t)a.batch * a.num_q_heads * a.max_splits * a.head_dim;
}

static int launch_split(const DecodeArgs &a) {
  int rc = validate_common("paged_decode_split", a, true);
  if (rc != LITEKV_OK || a.batch == 0) return rc;
  const int group = a.num_q_heads / a.num_kv_heads;
  float *part_o = a.max_splits > 1 ? static_cast<float *>(a.workspace) : nullptr;
  float *part_lse = a.max_splits > 1 ? lse_of(a) : nullptr;
  hipLaunchKernelGGL(paged_decode_split_kernel,
                     dim3((unsigned)a.num_kv_heads, (unsigned)a.max_splits, (unsigned)a.batch),
                     dim3(64), 0, static_cast<hipStream_t>(a.stream),
                     static_cast<const half_t *>(a.q), a.q_batch_stride,
                     static_cast<const half_t *>(a.kv_pool), a.block_table, a.block_table_stride,
                     a.seq_lens, static_cast<half_t *>(a.out), part_o, part_lse, a.num_q_heads,
                     a.num_kv_heads, group, a.max_splits, a.min_pages_per_split,
                     (int32_t)a.num_pages, a.softmax_scale * kLog2e);
  return check_launch("paged_decode_split");
}

static int launch_merge(const DecodeArgs &a) {
  int rc = validate_common("paged_decode_merge", a, false);
  if (rc != LITEKV_OK || a.batch == 0 || a.max_splits == 1) return rc;
  hipLaunchKernelGGL(paged_decode_merge_kernel, dim3((unsigned)a.num_q_heads, (unsigned)a.batch),
                     dim3(kHeadDim), 0, static_cast<hipStream_t>(a.stream), a.seq_lens,
                     static_cast<half_t *>(a.out), static_cast<const float *>(a.workspace),
                     lse_of(a), a.num_q_heads, a.max_splits, a.min_pages_per_split);
  return check_launch("paged_decode_merge");
}

}  // namespace litekv

extern "C" size_t litekv_paged_decode_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                      int32_t head_dim, int32_t max_splits) {
  return litekv::workspace_bytes_for(batch, num_q_heads, head_dim, max_splits);
}

extern "C" int litekv_paged_decode_split(const void *q, int64_t q_batch_stride, const void *kv_pool,
                                         const int32_t *block_table, int32_t block_table_stride,
                                         const int32_t *seq_lens, void *out, void *workspace,
                                         size_t workspace_bytes, int32_t batch,
                                         int32_t num_q_heads, int32_t num_kv_heads,
                                         int32_t head_dim, int32_t page_size, int64_t num_pages,
                                         int32_t max_splits, int32_t min_pages_per_split,
                                         float softmax_scale, void *stream) {
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, max_splits, min_pages_per_split, softmax_scale, stream};
  return litekv::launch_split(a);
}

extern "C" int litekv_paged_decode_merge(const int32_t *seq_lens, void *out, const void *workspace,
                                         size_t workspace_bytes, int32_t batch,
                                         int32_t num_q_heads, int32_t head_dim, int32_t page_size,
                                         int32_t max_splits, int32_t min_pages_per_split,
                                         void *stream) {
  litekv::DecodeArgs a{nullptr, 0, nullptr, nullptr, 1, seq_lens, out,
                       const_cast<void *>(workspace), workspace_bytes, batch, num_q_heads, 1,
                       head_dim, page_size, 1, max_splits, min_pages_per_split, 0.f, stream};
  return litekv::launch_merge(a);
}

extern "C" int litekv_paged_decode(const void *q, int64_t q_batch_stride, const void *kv_pool,
                                   const int32_t *block_table, int32_t block_table_stride,
                                   const int32_t *seq_lens, void *out, void *workspace,
                                   size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_pages, int32_t max_splits,
                                   int32_t min_pages_per_split, float softmax_scale, void *stream) {
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, max_splits, min_pages_per_split, softmax_scale, stream};
  int rc = litekv::launch_split(a);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a);
}
