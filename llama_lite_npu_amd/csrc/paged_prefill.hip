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
#include <type_traits>

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

// ---------------------------------------------------------------------------------------------
// Tiled kernel. One workgroup of 8 wavefronts owns, for one sequence and one KV head, a block of
// BM = 16 * row_tiles query rows of ALL group heads: 16 * (group * row_tiles) <= 256 columns in
// the N dimension of the MFMA tiles, 2 N-tiles (32 columns) per wavefront. Keys are walked in
// tiles of 64 tokens (4 pages) staged in LDS once per workgroup, so a K/V byte fetched from
// L2/HBM serves every head of the GQA group and every row of the block. Per tile and wavefront:
//
//   S^T[64 keys][32 cols] = K_tile . Q^T        4 M-tiles x 2 N-tiles x 4 k-steps  (16x16x32)
//   softmax per column (lazy max, scale folded into the exponent)
//   O^T[128 d][32 cols]  += V_tile^T . P^T      8 M-tiles x 2 N-tiles x 2 k-steps  (16x16x32)
//
// In the second product the k index of one MFMA runs over 32 keys in the order (keys 4g..4g+3
// of one 16-key tile, then the same of the next tile) for lane group g: exactly what two S^T
// accumulator tiles hold, and what two transposing LDS reads of V deliver, so P never leaves
// its lane. 32 columns per wavefront keep it under 256 registers, so two wavefronts share each
// SIMD and one's softmax (vector ALU) overlaps the other's MFMAs. The next K/V tile is
// prefetched into registers while the current one is consumed.
// ---------------------------------------------------------------------------------------------
constexpr int kKvTile = 64;
constexpr int kTilePitch = kHeadDim + 8;  // fp16 elements per staged row (272 bytes)
constexpr int kColTiles = 2;              // N-tiles per wavefront
constexpr int kTiledWaves = 8;

template <bool PAGED>
__global__ __launch_bounds__(kTiledWaves * kWave) void varlen_prefill_tiled_kernel(
    const half_t *__restrict__ q, int64_t q_stride, half_t *__restrict__ out, int64_t out_stride,
    PagedSource paged, PackedSource packed, const int32_t *__restrict__ q_starts_or_cu,
    const int32_t *__restrict__ q_lens_or_null, const int32_t *__restrict__ context_lens,
    int32_t num_q_heads, int32_t group, int32_t row_tiles, float scale_log2) {
  __shared__ __attribute__((aligned(16))) half_t ktile[kKvTile * kTilePitch];
  __shared__ __attribute__((aligned(16))) half_t vtile[kKvTile * kTilePitch];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int n = lane & 15;
  const int g = lane >> 4;
  const int h = blockIdx.y;  // kv head
  const int b = blockIdx.z;

  int q_start, q_len;
  if (PAGED) {
    q_start = q_starts_or_cu[b];
    q_len = q_starts_or_cu[b + 1] - q_start;
  } else {
    q_start = packed.seq_starts[b];
    q_len = q_lens_or_null[b];
  }
  const int block_rows = 16 * row_tiles;
  const int m0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * block_rows;  // long blocks first
  if (m0 >= q_len) return;
  const int ctx = (PAGED && context_lens) ? context_lens[b] : 0;
  const int kv_len = ctx + q_len;
  const int rows = (q_len - m0) < block_rows ? (q_len - m0) : block_rows;
  const int kv_end = ctx + m0 + rows;  // keys the block may see
  const int n_col_tiles = group * row_tiles;

  // This wavefront's column tiles: tile t = head (t / row_tiles), rows 16 * (t % row_tiles) ..
  half8_t qf[kColTiles][4];
  int q_pos[kColTiles];
  int out_row[kColTiles];   // packed row index, or -1
  int out_head[kColTiles];
#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    const int t = wave * kColTiles + u;
    const int head = t / row_tiles;
    const int row = m0 + (t - head * row_tiles) * 16 + n;
    const bool ok = t < n_col_tiles && row < q_len;
    const int hq = h * group + (head < group ? head : 0);
    const int last = q_len - 1;
    q_pos[u] = ctx + (row < last ? row : last);
    out_row[u] = ok ? q_start + row : -1;
    out_head[u] = hq;
    const half_t *qrow =
        q + (int64_t)(q_start + (ok ? row : 0)) * q_stride + (int64_t)hq * kHeadDim + 8 * g;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      qf[u][kk] = ok ? *(const half8_t *)(qrow + 32 * kk) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  float4_t acc[8][kColTiles];
  float m_run[kColTiles], d_run[kColTiles];
#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    m_run[u] = -INFINITY;
    d_run[u] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j][u] = float4_t{0.f, 0.f, 0.f, 0.f};
  }

  // Staging: thread (r = tid / 16, c = tid % 16) moves 16-byte column c of rows r and 32 + r of the
  // tile; the 4 rows of one wavefront lie in one page.
  const int srow = tid >> 4;   // 0..31
  const int scol = tid & 15;
  const int64_t pool_row = (int64_t)2 * paged.num_kv_heads * kHeadDim;
  const int32_t *table = PAGED ? paged.block_table + (int64_t)b * paged.bt_stride : nullptr;
  const int last_key = kv_len - 1;
  half8_t kreg[2], vreg[2];

  auto fetch_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int tok = kt * kKvTile + 32 * i + srow;
      tok = tok < last_key ? tok : last_key;  // rows past the end are masked; keep the address valid
      const half_t *kp, *vp;
      if (PAGED) {
        int pidx = __builtin_amdgcn_readfirstlane(kt * 4 + 2 * i + (srow >> 4));
        const int last_page = last_key >> 4;
        pidx = pidx < last_page ? pidx : last_page;
        int pid = table[pidx];
        pid = pid < 0 ? 0 : (pid >= paged.num_pages ? paged.num_pages - 1 : pid);
        const int64_t slot = (int64_t)pid * kPageSize + (tok - pidx * kPageSize);
        kp = paged.kv + slot * pool_row + (int64_t)h * kHeadDim + 8 * scol;
        vp = kp + (int64_t)paged.num_kv_heads * kHeadDim;
      } else {
        kp = packed.k + (int64_t)(q_start + tok) * packed.k_stride + (int64_t)h * kHeadDim + 8 * scol;
        vp = packed.v + (int64_t)(q_start + tok) * packed.v_stride + (int64_t)h * kHeadDim + 8 * scol;
      }
      kreg[i] = *(const half8_t *)kp;
      vreg[i] = *(const half8_t *)vp;
    }
  };

  float4_t st[4][kColTiles];
  half8_t pk[kColTiles][2];

  // Softmax of the raw scores in `st` (tile kt) into `pk`: p = 2^(s * scale - m) with m kept in
  // scaled units. MASKED tiles reach past the block's first row; the others skip the compares.
  auto softmax_tile = [&](int kt, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int key0 = kt * kKvTile;
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
      if (MASKED) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (key0 + 16 * m + 4 * g + i > q_pos[u]) st[m][u][i] = -INFINITY;
          }
        }
      }
      float mx = fmaxf(fmaxf(st[0][u][0], st[0][u][1]), fmaxf(st[0][u][2], st[0][u][3]));
#pragma unroll
      for (int m = 1; m < 4; ++m) {
        mx = fmaxf(mx, fmaxf(fmaxf(st[m][u][0], st[m][u][1]), fmaxf(st[m][u][2], st[m][u][3])));
      }
      mx = fmaxf(mx, xor_lane(mx, 16));
      mx = fmaxf(mx, xor_lane(mx, 32));
      mx *= scale_log2;  // scale > 0: max and scaling commute; -inf stays -inf
      if (__builtin_amdgcn_ballot_w64(mx > m_run[u] + 8.0f) != 0) {
        const float m_new = fmaxf(m_run[u], mx);
        const float alpha = fast_exp2(m_run[u] - m_new);
        d_run[u] *= alpha;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          acc[j][u][0] *= alpha;
          acc[j][u][1] *= alpha;
          acc[j][u][2] *= alpha;
          acc[j][u][3] *= alpha;
        }
        m_run[u] = m_new;
      }
      const float neg_m = -m_run[u];
      float sum = 0.f;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p0 = fast_exp2(__builtin_fmaf(st[2 * s2][u][i], scale_log2, neg_m));
          const float p1 = fast_exp2(__builtin_fmaf(st[2 * s2 + 1][u][i], scale_log2, neg_m));
          sum += p0 + p1;
          pk[u][s2][i] = (half_t)p0;
          pk[u][s2][4 + i] = (half_t)p1;
        }
      }
      d_run[u] += sum;
    }
  };

  const int n_tiles = (kv_end + kKvTile - 1) / kKvTile;
  fetch_tile(0);
  for (int kt = 0; kt < n_tiles; ++kt) {
    __syncthreads();  // every wavefront is done reading the previous tile
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = 32 * i + srow;
      half8_t x = vreg[i];
      // Slots past the sequence end hold arbitrary bits: keep them out of the MFMA.
      if (kt * kKvTile + r >= kv_len) x = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      *(half8_t *)(&ktile[r * kTilePitch + 8 * scol]) = kreg[i];
      *(half8_t *)(&vtile[r * kTilePitch + 8 * scol]) = x;
    }
    __syncthreads();
    if (kt + 1 < n_tiles) fetch_tile(kt + 1);

    // S^T = K . Q^T
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) st[m][u] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const half8_t a = *(const half8_t *)(&ktile[(16 * m + n) * kTilePitch + 32 * kk + 8 * g]);
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) st[m][u] = mfma_16x16x32(a, qf[u][kk], st[m][u]);
      }
    }

    if (kt * kKvTile + kKvTile - 1 > ctx + m0) softmax_tile(kt, std::true_type{});
    else softmax_tile(kt, std::false_type{});

    // O^T += V^T . P^T
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const half_t *vlo = &vtile[(32 * s2 + 4 * g + (n >> 2)) * kTilePitch + 16 * j + 4 * (n & 3)];
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) short4_t *)vlo);
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) short4_t *)(vlo + 16 * kTilePitch));
        typedef short short8_t __attribute__((ext_vector_type(8)));
        const short8_t both = short8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const half8_t a = __builtin_bit_cast(half8_t, both);
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) acc[j][u] = mfma_16x16x32(a, pk[u][s2], acc[j][u]);
      }
    }
  }

#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    float d_tot = d_run[u] + xor_lane(d_run[u], 16);
    d_tot += xor_lane(d_tot, 32);
    const float inv = 1.0f / d_tot;
    if (out_row[u] >= 0) {
      half_t *o = out + (int64_t)out_row[u] * out_stride + (int64_t)out_head[u] * kHeadDim + 4 * g;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        *(half4_t *)(o + 16 * j) =
            half4_t{(half_t)(acc[j][u][0] * inv), (half_t)(acc[j][u][1] * inv),
                    (half_t)(acc[j][u][2] * inv), (half_t)(acc[j][u][3] * inv)};
      }
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
  const int group = num_q_heads / num_kv_heads;
  LITEKV_REQUIRE(group <= 16, "paged_prefill: %d query heads per kv head unsupported (max 16)",
                 group);
  const int row_tiles = 16 / group;  // 16 * group * row_tiles <= 256 columns per workgroup
  const unsigned blocks = (unsigned)((max_q_len + 16 * row_tiles - 1) / (16 * row_tiles));
  hipLaunchKernelGGL(varlen_prefill_tiled_kernel<true>,
                     dim3(blocks, (unsigned)num_kv_heads, (unsigned)batch),
                     dim3(kTiledWaves * kWave), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                     out_token_stride, paged, packed, cu_q_lens, (const int32_t *)nullptr,
                     context_lens, num_q_heads, group, row_tiles, softmax_scale * kLog2eP);
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
  const int group = num_q_heads / num_kv_heads;
  LITEKV_REQUIRE(group <= 16, "varlen_prefill: %d query heads per kv head unsupported (max 16)",
                 group);
  const int row_tiles = 16 / group;
  const unsigned blocks = (unsigned)((max_seq_len + 16 * row_tiles - 1) / (16 * row_tiles));
  hipLaunchKernelGGL(varlen_prefill_tiled_kernel<false>,
                     dim3(blocks, (unsigned)num_kv_heads, (unsigned)batch),
                     dim3(kTiledWaves * kWave), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half_t *>(q), q_token_stride, static_cast<half_t *>(out),
                     out_token_stride, paged, packed, seq_starts, seq_lens,
                     (const int32_t *)nullptr, num_q_heads, group, row_tiles,
                     softmax_scale * kLog2eP);
  return check_launch("varlen_prefill");
}
