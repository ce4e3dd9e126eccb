// Paged flash-decoding for gfx950: two schedules over one page kernel, and
// the deterministic log-sum-exp merge.
//
// Page step (shared by both schedules). A wavefront owns one kv head and walks
// 16-token pages; all Hq/Hkv query heads of that kv head ride in the 16-wide N
// dimension of the MFMA tiles, so K/V bytes are read from HBM exactly once:
//
//   S^T[token][head]  = K_page[16 x 128] . Q^T[128 x 16]      4 x MFMA 16x16x32
//   online softmax over tokens, per head column (fp32, exp2 domain)
//   O^T[d][head]     += V_page^T[128 x 16] . P^T[16 x 16]      8 x MFMA 16x16x16
//
// The S^T accumulator layout (lane l: head l%16, tokens 4*(l/16)..+3) is also
// the B-operand layout of the second product, so probabilities never leave
// their lane. K fragments are loaded straight from the page in A-operand
// layout (64 contiguous bytes per token per instruction); V rows are loaded
// as full 256-byte rows, staged in LDS and read back with the transposing LDS
// read. Softmax reductions over the 4 lane groups use wavefront shuffles.
// DEPTH pages per wavefront are kept in flight in registers.
//
// Schedule "splits" (litekv_paged_decode): grid (kv head, split, sequence),
// one wavefront each; sequence b is cut into n_b splits at page boundaries
// floor(s * pages_b / n_b).
//
// Schedule "balanced" (litekv_paged_decode_balanced): the pages of all
// sequences, concatenated, are cut into equal chunks; one workgroup of up to
// 8 wavefronts (one per kv head) streams one chunk, crossing sequence
// boundaries as needed, so every CU gets the same number of bytes whatever the
// length distribution, and the kv heads of a page are fetched together.
//
// In both schedules the cuts are a pure function of seq_lens and of host
// scalars, and the merge adds the fp32 partials in index order: results do not
// depend on timing.
#include <atomic>
#include <type_traits>

#include "common.h"
#include "kv_fp8.h"
#include "prefill_tile.h"

// This file is compiled once per head dim its kernels are tuned for: as itself for 128, and
// through paged_decode_hd64.hip (which defines LITEKV_HD and includes it) for 64. Everything
// below lives in an inline namespace named after the head dim, so the two sets of kernels and
// launchers are distinct symbols; the extern "C" entry points exist in the 128 build only and hand
// head dim 64 to the launchers of the other build (litekv::hd64_*, declared in common.h).
// At 64 the lane maps are those of 128 with half the MFMA k-steps and half the output column
// tiles; lanes whose 16-byte column of a V row would lie past the row re-read the column of
// their twin (n % 8) and stage it in a part of the LDS row nobody reads.
namespace litekv {
inline namespace LITEKV_HD_NS {

constexpr int kHD = LITEKV_HD;       // head dim of this build of the file
constexpr int kKSteps = kHD / 32;    // MFMA k-steps of a score product (fp16 fragments of 8)
constexpr int kJTiles = kHD / 16;    // 16-column tiles of an output row
constexpr int kVCols = kHD / 8;      // 16-byte columns of an fp16 row
constexpr int kVPitch = 128 + 8;     // fp16 elements per staged V row (272 bytes), whatever kHD
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Pages a wavefront keeps in flight in registers (K fragments and V rows of DEPTH pages are
// requested before the oldest one is consumed).
#ifndef LITEKV_DECODE_DEPTH
#define LITEKV_DECODE_DEPTH 2
#endif
// The running max of a head is only raised when the new page exceeds it by more than this many
// powers of two; until then probabilities are formed against the older, smaller max (they stay
// below 2^kMaxSlack, far inside fp16 range) and the accumulator rescale is skipped. The final
// division by the denominator cancels the choice of max exactly.
constexpr float kMaxSlack = 8.0f;

__host__ __device__ __forceinline__ int pages_of(int len) {
  return len > 0 ? (len + kPageSize - 1) / kPageSize : 0;
}

__host__ __device__ __forceinline__ int splits_for_pages(int pages, int max_splits,
                                                         int min_pages_per_split) {
  int n = (pages + min_pages_per_split - 1) / min_pages_per_split;
  n = n < 1 ? 1 : n;
  return n < max_splits ? n : max_splits;
}

// One page of an fp16 pool as this lane requested it.
struct PageRegs {
  half8_t k[4];  // A-operand fragments of K: token n, d = 32*kk + 8*g .. +7
  half8_t v[4];  // V rows 4*i + g, 16-byte column n
};

// One page of a pool of 8-bit codes (fp8 or int8): the same bytes per lane in half as many loads. The sum over d of a
// dot product may run in any order as long as K and q agree, so a lane takes 16 consecutive
// codes per load and MFMA step kk uses its lower or upper 8:
//   k[j]: token n, d = 16*(g + 4*j) .. +15      step kk = 2*j + (0: lower, 1: upper 8 codes)
//   v[i]: V row 8*i + 2*g + n%2, d = 16*(n/2) .. +15
// Neighbouring lanes hold the same column of two neighbouring rows: the 32 bytes a lane stages per
// row (16 codes as fp16) then fall on different LDS banks for the eight lanes a 16-byte store
// serves per cycle. (With eight neighbouring lanes on one row, 32 bytes apart, every such store
// took two cycles: half of the kernel's LDS cycles were bank conflicts.)
template <int KV>
struct PageRegsQ8 {
  uint4_t k[2];
  uint4_t v[2];
};

// Storage of the pool a kernel reads: fp16, or the codes of format KV (kKvFp8, kKvInt8).
__device__ __forceinline__ int q8_v_row(int n, int g) { return 2 * g + (n & 1); }  // inside its block of 8 rows
__device__ __forceinline__ int q8_v_col(int n) { return n >> 1; }                 // in units of 16 codes
template <int KV> struct KvStore { typedef uint8_t elem; typedef PageRegsQ8<KV> page; };
template <> struct KvStore<kKvF16> { typedef half_t elem; typedef PageRegs page; };

// Softmax state and output accumulator of the (up to 16) query heads of one kv head.
// acc[j][i] is O^T[d = 16j + 4g + i][head n]; m is shared by the 4 lanes of a head, d is this
// lane's share of the denominator.
struct HeadState {
  float4_t acc[8];
  float m;
  float d;
  __device__ __forceinline__ void reset() {
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
    m = -INFINITY;
    d = 0.f;
  }
};

// Orders this wavefront's LDS writes before its later LDS reads (and the reverse) for the
// compiler; the LDS unit itself executes one wavefront's accesses in issue order.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Q^T as B operand: lane (n, g) holds q[head n][32*kk + 8*g .. +7]; lanes past the group get 0.
__device__ __forceinline__ void load_q(half8_t (&qf)[4], const half_t *q_row0, int n, int g,
                                       int group) {
  const half_t *qrow = q_row0 + (int64_t)n * kHD + 8 * g;
#pragma unroll
  for (int kk = 0; kk < kKSteps; ++kk) {
    qf[kk] = (n < group) ? *(const half8_t *)(qrow + 32 * kk) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
}

// The same for an fp8 pool, in the d order of PageRegsFp8::k.
__device__ __forceinline__ void load_q_fp8_order(half8_t (&qf)[4], const half_t *q_row0, int n, int g,
                                                 int group) {
  const half_t *qrow = q_row0 + (int64_t)n * kHD + 16 * g;
#pragma unroll
  for (int kk = 0; kk < kKSteps; ++kk) {
    qf[kk] = (n < group) ? *(const half8_t *)(qrow + 64 * (kk >> 1) + 8 * (kk & 1))
                         : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
}

// Requests one page: k_lane / v_lane already point at this lane's row and column of page 0.
// K/V bytes are used once per launch: the loads carry the streaming (non-temporal) hint, which
// keeps the step metadata and q rows in L2 and measured 2 % (C2) to 7 % (C5) faster.
// `dummy` (wavefront-uniform) marks a request past the end of the chunk, issued only to keep the
// number of loads in flight constant: every lane then reads the same 16 bytes of the page
// (streaming loads do not stay in L2, so re-reading the whole last page would cost HBM traffic).
__device__ __forceinline__ void request_page(PageRegs &r, const half_t *k_lane,
                                             const half_t *v_lane, int64_t page_off,
                                             int64_t row_stride, bool dummy = false,
                                             const half_t *pool = nullptr) {
  const half_t *kr = dummy ? pool + page_off : k_lane + page_off;
  const int64_t k_step = dummy ? 0 : 32;
#pragma unroll
  for (int kk = 0; kk < kKSteps; ++kk) r.k[kk] = __builtin_nontemporal_load((const half8_t *)(kr + kk * k_step));
  const half_t *vr = dummy ? pool + page_off : v_lane + page_off;
  const int64_t v_step = dummy ? 0 : 4 * row_stride;
#pragma unroll
  for (int i = 0; i < 4; ++i) r.v[i] = __builtin_nontemporal_load((const half8_t *)(vr + i * v_step));
}

// 8-bit pool: k_lane points at token n, code 16*g; v_lane at row q8_v_row, code 16*q8_v_col.
template <int KV>
__device__ __forceinline__ void request_page(PageRegsQ8<KV> &r, const uint8_t *k_lane,
                                             const uint8_t *v_lane, int64_t page_off,
                                             int64_t row_stride, bool dummy = false,
                                             const uint8_t *pool = nullptr) {
  const uint8_t *kr = dummy ? pool + page_off : k_lane + page_off;
  const int64_t k_step = dummy ? 0 : 64;
#pragma unroll
  for (int j = 0; j < kHD / 64; ++j) r.k[j] = __builtin_nontemporal_load((const uint4_t *)(kr + j * k_step));
  const uint8_t *vr = dummy ? pool + page_off : v_lane + page_off;
  const int64_t v_step = dummy ? 0 : 8 * row_stride;
#pragma unroll
  for (int i = 0; i < 2; ++i) r.v[i] = __builtin_nontemporal_load((const uint4_t *)(vr + i * v_step));
}

// Folds page `p` (tokens 16p .. 16p+15 of a sequence of `len` tokens) into the state. `kf` are
// the page's K fragments, `stage_v(tail)` writes its V rows [16][128] into vstage (zeros for rows
// past the sequence end when `tail`).
template <typename StageV>
__device__ __forceinline__ void attend_core(HeadState &st, const half8_t (&kf)[4],
                                            const half8_t (&qf)[4], const half_t *vt_lane, int p,
                                            int len, int n, int g, float scale_log2,
                                            StageV stage_v) {
  const bool tail = (p + 1) * kPageSize > len;  // wavefront-uniform: last, partly filled page
  wave_lds_fence();
  stage_v(tail);
  wave_lds_fence();

  // two accumulators: the dependent MFMA chain is two deep instead of four
  float4_t s = mfma_16x16x32(kf[0], qf[0], float4_t{0.f, 0.f, 0.f, 0.f});
  float4_t s1 = mfma_16x16x32(kf[kKSteps / 2], qf[kKSteps / 2], float4_t{0.f, 0.f, 0.f, 0.f});
  if constexpr (kKSteps == 4) {
    s = mfma_16x16x32(kf[1], qf[1], s);
    s1 = mfma_16x16x32(kf[3], qf[3], s1);
  }

  float sv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) sv[i] = (s[i] + s1[i]) * scale_log2;
  if (tail) {
    const int tok0 = p * kPageSize + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) sv[i] = (tok0 + i < len) ? sv[i] : -INFINITY;
  }
  float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
  mx = max_over_lane_groups(mx);
  // mx is finite (the page holds at least one valid token). Raise the reference max only when
  // some head needs it; the branch is wavefront-uniform.
  if (__builtin_amdgcn_ballot_w64(mx > st.m + kMaxSlack) != 0) {
    const float m_new = fmaxf(st.m, mx);
    const float alpha = fast_exp2(st.m - m_new);
    st.d *= alpha;
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) {
      st.acc[j][0] *= alpha;
      st.acc[j][1] *= alpha;
      st.acc[j][2] *= alpha;
      st.acc[j][3] *= alpha;
    }
    st.m = m_new;
  }
  float pr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) pr[i] = fast_exp2(sv[i] - st.m);
  st.d += (pr[0] + pr[1]) + (pr[2] + pr[3]);
  const half4_t pt = half4_t{(half_t)pr[0], (half_t)pr[1], (half_t)pr[2], (half_t)pr[3]};

#pragma unroll
  for (int j = 0; j < kJTiles; ++j) {
    // V^T fragment: lane (n, g) receives V[4g .. 4g+3][16j + n] from the transposing LDS read
    // (lane i of a 16-lane group passes the address of row i/4, columns 4*(i%4) .. +3).
    const half4_t vt = __builtin_bit_cast(
        half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                     (__attribute__((address_space(3))) short4_t *)(vt_lane + 16 * j)));
    st.acc[j] = mfma_16x16x16(vt, pt, st.acc[j]);
  }
}


__device__ __forceinline__ void attend_page(HeadState &st, const PageRegs &r,
                                            const half8_t (&qf)[4], half_t *vstage,
                                            const half_t *vt_lane, int p, int len, int n, int g,
                                            float scale_log2) {
  attend_core(st, r.k, qf, vt_lane, p, len, n, g, scale_log2, [&](bool tail) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half8_t x = r.v[i];
      // Slots past the sequence end hold arbitrary bits: keep them out of the MFMA.
      if (tail && p * kPageSize + 4 * i + g >= len) x = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      *(half8_t *)(&vstage[(4 * i + g) * kVPitch + 8 * n]) = x;
    }
  });
}

// A page of codes: they become fp16 exactly (the head's scales are applied by the caller).
template <int KV>
__device__ __forceinline__ void attend_page(HeadState &st, const PageRegsQ8<KV> &r,
                                            const half8_t (&qf)[4], half_t *vstage,
                                            const half_t *vt_lane, int p, int len, int n, int g,
                                            float scale_log2) {
  const half8_t kf[4] = {codes_to_half<KV>(uint2_t{r.k[0][0], r.k[0][1]}),
                         codes_to_half<KV>(uint2_t{r.k[0][2], r.k[0][3]}),
                         codes_to_half<KV>(uint2_t{r.k[1][0], r.k[1][1]}),
                         codes_to_half<KV>(uint2_t{r.k[1][2], r.k[1][3]})};
  attend_core(st, kf, qf, vt_lane, p, len, n, g, scale_log2, [&](bool tail) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 8 * i + q8_v_row(n, g);
      half8_t lo = codes_to_half<KV>(uint2_t{r.v[i][0], r.v[i][1]});
      half8_t hi = codes_to_half<KV>(uint2_t{r.v[i][2], r.v[i][3]});
      if (tail && p * kPageSize + row >= len) {
        lo = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        hi = lo;
      }
      half_t *dst = &vstage[row * kVPitch + 16 * q8_v_col(n)];
      *(half8_t *)dst = lo;
      *(half8_t *)(dst + 8) = hi;
    }
  });
}

// Writes the normalised state either as the final fp16 row or as an fp32 partial + log-sum-exp.
// Head n of the group writes out_row + n*D, or part_row + n*part_head_stride and
// part_lse_cell + n*lse_head_stride.
__device__ __forceinline__ void store_state(const HeadState &st, bool final_row, half_t *out_row,
                                            float *part_row, int64_t part_head_stride,
                                            float *part_lse_cell, int64_t lse_head_stride, int n,
                                            int g, int group, float out_scale = 1.0f) {
  float d_tot = st.d + xor_lane(st.d, 16);
  d_tot += xor_lane(d_tot, 32);
  const float inv = out_scale / d_tot;  // out_scale: the V scale of an fp8 pool
  if (n >= group) return;
  if (final_row) {
    half_t *o = out_row + (int64_t)n * kHD + 4 * g;
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) {
      *(half4_t *)(o + 16 * j) =
          half4_t{(half_t)(st.acc[j][0] * inv), (half_t)(st.acc[j][1] * inv),
                  (half_t)(st.acc[j][2] * inv), (half_t)(st.acc[j][3] * inv)};
    }
  } else {
    float *po = part_row + (int64_t)n * part_head_stride + 4 * g;
    const float lse = (st.m + fast_log2(d_tot)) * kLn2;
    {
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
        // Partials are read once, by the merge launch: streaming stores leave for memory as they
        // are issued instead of waiting in L2 for the write-back at the end of the kernel
        // (C2: 0.6 us per layer).
        __builtin_nontemporal_store(float4_t{st.acc[j][0] * inv, st.acc[j][1] * inv,
                                             st.acc[j][2] * inv, st.acc[j][3] * inv},
                                    (float4_t *)(po + 16 * j));
      }
      if (g == 0) __builtin_nontemporal_store(lse, part_lse_cell + (int64_t)n * lse_head_stride);
    }
  }
}

// A finished state parked in LDS instead of being stored: stores count in the same hardware
// counter as loads on this architecture, so a store issued in the middle of a chunk makes every
// later counted wait of the page loop also wait for the store's acknowledgement (2.65 us per
// sequence crossing on C2). The parked values are the ones store_state would have written
// (normalised fp32 and the log-sum-exp); unpark_state writes them out at the end of the chunk,
// each lane reading back what it wrote itself.
constexpr int kParkHeads = 8;                                  // query heads per kv head that fit
constexpr int kParkFloats = kParkHeads * kHD + 16;        // rows, then one log-sum-exp per head

__device__ __forceinline__ void park_state(const HeadState &st, float *park, int n, int g,
                                           int group, float out_scale) {
  float d_tot = st.d + xor_lane(st.d, 16);
  d_tot += xor_lane(d_tot, 32);
  const float inv = out_scale / d_tot;
  if (n >= group) return;
  float *row = park + n * kHD + 4 * g;
#pragma unroll
  for (int j = 0; j < kJTiles; ++j) {
    *(float4_t *)(row + 16 * j) = float4_t{st.acc[j][0] * inv, st.acc[j][1] * inv,
                                           st.acc[j][2] * inv, st.acc[j][3] * inv};
  }
  if (g == 0) park[kParkHeads * kHD + n] = (st.m + fast_log2(d_tot)) * kLn2;
}

__device__ __forceinline__ void unpark_state(const float *park, bool final_row, half_t *out_row,
                                             float *part_row, float *part_lse_cell, int n, int g,
                                             int group) {
  if (final_row) {
    if (n >= group) return;
    const float *row = park + n * kHD + 4 * g;
    half_t *o = out_row + (int64_t)n * kHD + 4 * g;
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) {
      const float4_t x = *(const float4_t *)(row + 16 * j);
      *(half4_t *)(o + 16 * j) = half4_t{(half_t)x[0], (half_t)x[1], (half_t)x[2], (half_t)x[3]};
    }
  } else {
    // The partial rows of the group's heads are one contiguous run in the workspace and in the
    // parking area alike: the whole wavefront copies it 1 KiB per instruction.
    wave_lds_fence();
    const int lane = 16 * g + n;
#pragma unroll
    for (int i = 0; i < kParkHeads * kHD / 256; ++i) {
      const int at = 4 * (64 * i + lane);
      if (at < group * kHD) {
        __builtin_nontemporal_store(*(const float4_t *)(park + at), (float4_t *)(part_row + at));
      }
    }
    if (lane < group) __builtin_nontemporal_store(park[kParkHeads * kHD + lane], part_lse_cell + lane);
  }
}

// Waits for every vector memory load this wavefront has in flight (s_waitcnt vmcnt(0), other
// counters untouched). Used at the end of rarely taken branches that load into registers the
// main loop reads: without it the compiler must assume those loads are still pending after the
// branch joins the main path, and would drain the whole prefetch queue on every iteration.
__device__ __forceinline__ void wait_vector_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

__device__ __forceinline__ int clamp_page(int pid, int num_pages) {
  return pid < 0 ? 0 : (pid >= num_pages ? num_pages - 1 : pid);
}

// Pools whose pages hold 16 << shift tokens: the kernels keep working on 16-token pages, and the
// 16-token page j of a sequence is part j % (1 << shift) of the sequence's page j >> shift, whose
// tokens are contiguous in the pool. `entry` is the block-table entry of that page.
__device__ __forceinline__ int sub_page_id(int entry, int j, int shift, int num_pages) {
  return (clamp_page(entry, num_pages) << shift) + (j & ((1 << shift) - 1));
}

// This lane's parts of the step's new K and V rows (fp16, head h of one sequence): the pieces
// that sit where the lane's page registers hold the token's row (see PageRegs / PageRegsFp8).
template <bool FP8>
__device__ __forceinline__ void load_new_rows(uint4_t (&kr)[4], uint4_t (&vr)[2], const half_t *kn,
                                              const half_t *vn, int n, int g) {
  if constexpr (FP8) {
#pragma unroll
    for (int j = 0; j < kHD / 64; ++j) {
      kr[2 * j] = *(const uint4_t *)(kn + 64 * j + 16 * g);
      kr[2 * j + 1] = *(const uint4_t *)(kn + 64 * j + 16 * g + 8);
    }
    vr[0] = *(const uint4_t *)(vn + 16 * (q8_v_col(n) & (kHD / 16 - 1)));
    vr[1] = *(const uint4_t *)(vn + 16 * (q8_v_col(n) & (kHD / 16 - 1)) + 8);
  } else {
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) kr[kk] = *(const uint4_t *)(kn + 32 * kk + 8 * g);
    vr[0] = *(const uint4_t *)(vn + 8 * (n & (kVCols - 1)));
    vr[1] = uint4_t{0, 0, 0, 0};  // fp8 only
  }
}

// Step metadata that no launch of the decode kernel modifies (plan entries, sequence lengths) is
// read through the constant address space: with a wavefront-uniform address such a load is
// always a scalar load, whatever fences and atomics surround it, so it never joins the in-order
// queue of the vector loads that stream K/V.
typedef const __attribute__((address_space(4))) int32_t *uniform_i32_ptr;
__device__ __forceinline__ uniform_i32_ptr as_uniform(const int32_t *p) {
  return (uniform_i32_ptr)(uintptr_t)p;
}

// ---------------------------------------------------------------------------------------------
// Schedule "splits": one wavefront per (kv head, split, sequence).
// Partials: part_o[b][hq][split][D], part_lse[b][hq][split].
// The wavefronts are independent (no barrier). A workgroup holds 1, 2 or 4 of them (blockDim.x /
// 64; neighbouring kv heads of one sequence and split), chosen by the host: few wavefronts want
// one per workgroup so that they spread over all compute units, many short ones want four,
// because the dispatcher places workgroups at a fixed rate whatever their size (512 sequences of
// 32 tokens, 8 kv heads: 30.5 us as 4096 workgroups). Not eight: at three wavefronts per SIMD a
// compute unit would hold one such workgroup and leave a third of its slots empty.
// ---------------------------------------------------------------------------------------------
constexpr int kSplitWaves = 4;

// The sequence whose length is the r-th largest of the batch (ties by index). A grid whose
// workgroups outnumber the device's slots is dispatched in index order; with the sequence as the
// slowest index and ragged lengths, the launch then ends with the long pieces of whichever
// sequences come last while most compute units idle (128 sequences of 8192 to 32768 tokens in 16
// splits each on 512 slots: list scheduling in batch order ends at 1.25 times the mean load of a
// slot, longest sequences first at 1.04 times). So blockIdx.z counts sequences from the longest
// down. Every wavefront finds its sequence for itself (no barrier, no workspace): lane l holds
// the lengths of sequences l, l + 64, ...; the r-th largest length is found bit by bit from the
// top (31 rounds of one comparison and one population count per 64 sequences), then the tie is
// resolved by index. A few hundred instructions for a batch of 256.
constexpr int kMaxOrderedBatch = 256;
// `capacity`: the most tokens a block-table row can name; lengths count up to it (the kernel reads
// no page beyond the row either). *length_out: the sequence's length as it was ranked, at least 0.
__device__ __forceinline__ int sequence_of_rank(const int32_t *seq_lens, int batch, int r, int lane,
                                                int capacity, int *length_out) {
  constexpr int kRegs = kMaxOrderedBatch / kWave;
  const int regs = (batch + kWave - 1) / kWave;  // wavefront-uniform
  int len[kRegs];
#pragma unroll
  for (int p = 0; p < kRegs; ++p) {
    const int i = kWave * p + lane;
    int v = (p < regs && i < batch) ? seq_lens[i] : -1;
    v = v < capacity ? v : capacity;
    len[p] = i < batch ? (v > 0 ? v : 0) : -1;  // lanes past the batch never count
  }
  auto at_least = [&](int t) {  // sequences whose length is >= t
    int c = 0;
#pragma unroll
    for (int p = 0; p < kRegs; ++p) {
      if (p < regs) c += __builtin_popcountll(__builtin_amdgcn_ballot_w64(len[p] >= t));
    }
    return c;
  };
  int v = 0;  // the largest t with more than r sequences of length >= t: the length of rank r
  for (int bit = 31 - __builtin_clz(capacity | 1); bit >= 0; --bit) {
    const int t = v | (1 << bit);
    if (at_least(t) > r) v = t;
  }
  *length_out = v;
  int k = r - at_least(v + 1);  // its place among the sequences of exactly that length
#pragma unroll
  for (int p = 0; p < kRegs; ++p) {
    if (p < regs) {
      uint64_t same = __builtin_amdgcn_ballot_w64(len[p] == v);
      const int n = __builtin_popcountll(same);
      if (k >= 0 && k < n) {
        for (int skip = 0; skip < k; ++skip) same &= same - 1;  // drop the k lowest lanes
        return kWave * p + (int)__builtin_ctzll(same);
      }
      k -= n;
    }
  }
  return r;  // not reached for r < batch
}

extern __shared__ __attribute__((aligned(16))) half_t split_vstage[];  // [waves][kPageSize * kVPitch]
// ORDERED: blockIdx.z is a rank by length instead of the sequence (see sequence_of_rank); an
// instantiation of its own, so that launches bound by the dispatch of many short workgroups keep
// the short prologue.
template <int DEPTH, int KV, bool APPEND, bool ORDERED = false>
__global__ __launch_bounds__(kSplitWaves *kWave) void paged_decode_split_kernel(
    const half_t *__restrict__ q, int64_t q_batch_stride,
    typename KvStore<KV>::elem *__restrict__ kv, const float *__restrict__ scales,
    const int32_t *__restrict__ block_table, int32_t bt_stride,
    const int32_t *__restrict__ seq_lens, const half_t *__restrict__ k_new,
    const half_t *__restrict__ v_new, int64_t k_new_stride, int64_t v_new_stride,
    half_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_lse,
    int32_t num_q_heads, int32_t num_kv_heads, int32_t group_all, int32_t slices, int32_t max_splits,
    int32_t min_pages_per_split, int32_t num_pages, int32_t page_shift, float scale_log2) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int n = lane & 15;   // query head inside the slice (column of S^T)
  const int g = lane >> 4;   // lane group: owns tokens 4g..4g+3 of a page
  // a kv head with more than 16 query heads is served in slices of up to 16 (see head_slice)
  const HeadSlice hs = head_slice(blockIdx.x * (blockDim.x >> 6) + wave, slices, group_all);
  const int h = hs.kv_head;
  const int group = hs.q_heads;
  const int split = blockIdx.y;
  half_t *vstage = split_vstage + wave * (kPageSize * kVPitch);
  int b = blockIdx.z, len;
  if constexpr (ORDERED) {
    const int64_t capacity = (int64_t)bt_stride << (page_shift + 4);
    b = sequence_of_rank(seq_lens, (int)gridDim.z, (int)blockIdx.z, lane,
                         capacity < 0x40000000 ? (int)capacity : 0x40000000, &len);
    b = __builtin_amdgcn_readfirstlane(b);
    len = __builtin_amdgcn_readfirstlane(len);
    // a length beyond the row keeps its own value for the masks below
    if (len >= capacity) len = seq_lens[b];
  } else {
    len = seq_lens[b];
  }
  const int hq0 = hs.q_head0;
  half_t *out_row = out + ((int64_t)b * num_q_heads + hq0) * kHD;
  if (len <= 0) {
    if (split == 0 && n < group) {
      half_t *o = out_row + (int64_t)n * kHD;
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) *(half4_t *)(o + 16 * j + 4 * g) = half4_t{0, 0, 0, 0};
    }
    return;
  }
  const int pages = pages_of(len);
  const int n_splits = splits_for_pages(pages, max_splits, min_pages_per_split);
  if (split >= n_splits) return;
  const int p0 = (int)(((int64_t)split * pages) / n_splits);
  const int p1 = (int)(((int64_t)(split + 1) * pages) / n_splits);

  constexpr bool FP8 = KV != kKvF16;  // 8-bit codes (either format): the layout they share
  typedef typename KvStore<KV>::elem Elem;
  typedef typename KvStore<KV>::page Page;
  half8_t qf[4];
  float v_scale = 1.0f, k_inv = 1.0f, v_inv = 1.0f;
  if constexpr (FP8) {  // the K scale joins the softmax scale, the V scale the normalisation
    load_q_fp8_order(qf, q + (int64_t)b * q_batch_stride + (int64_t)hq0 * kHD, n, g, group);
    const float ks = scales[h];
    scale_log2 *= ks;
    v_scale = scales[num_kv_heads + h];
    k_inv = 1.0f / ks;  // the step's new rows are quantised with the reciprocals
    v_inv = 1.0f / v_scale;
  } else {
    load_q(qf, q + (int64_t)b * q_batch_stride + (int64_t)hq0 * kHD, n, g, group);
  }
  // Fused append: the wavefront that attends the sequence's last page writes the step's token
  // into it. Its rows are requested here, before the pages.
  uint4_t k_row[4] = {}, v_row[2] = {};
  if constexpr (APPEND) {
    load_new_rows<FP8>(k_row, v_row, k_new + (int64_t)b * k_new_stride + (int64_t)h * kHD,
                       v_new + (int64_t)b * v_new_stride + (int64_t)h * kHD, n, g);
  }

  const int64_t row_stride = (int64_t)2 * num_kv_heads * kHD;  // elements per slot
  // this lane's row and column inside page 0 (see PageRegs / PageRegsFp8)
  Elem *k_lane = kv + (int64_t)h * kHD + (FP8 ? 16 : 8) * g + n * row_stride;
  Elem *v_lane = FP8 ? kv + (int64_t)(num_kv_heads + h) * kHD + 16 * (q8_v_col(n) & (kHD / 16 - 1)) +
                           q8_v_row(n, g) * row_stride
                     : kv + (int64_t)(num_kv_heads + h) * kHD + 8 * (n & (kVCols - 1)) + g * row_stride;
  const half_t *vt_lane = &vstage[(4 * g + (n >> 2)) * kVPitch + 4 * (n & 3)];
  const int32_t *table = block_table + (int64_t)b * bt_stride;

  HeadState st;
  st.reset();
  Page buf[DEPTH];

  // Page ids are wavefront-uniform: they travel through scalar loads one step ahead of their
  // use. Requests past the range still issue their loads (16 bytes of its last page), which keeps
  // the number of vector loads in flight a compile-time constant, so each wait names exactly the
  // page it needs and never drains the younger prefetches.
  // A length beyond what a block-table row can name (the host cannot check lengths that live on
  // the device) re-reads the row's last entry instead of reading past it, and appends nothing.
  const bool fits_table = pages <= (bt_stride << page_shift);
  auto page_id = [&](int p) {
    const int pp = p < p1 ? p : p1 - 1;
    int at = pp >> page_shift;
    at = at < bt_stride ? at : bt_stride - 1;
    return sub_page_id(table[at], pp, page_shift, num_pages);
  };
  int pid_next = page_id(p0);
  auto request = [&](int p, Page &r) {
    const int64_t page_off = (int64_t)pid_next * kPageSize * row_stride;
    pid_next = page_id(p + 1);
    request_page(r, k_lane, v_lane, page_off, row_stride, p >= p1, kv);
  };

#pragma unroll
  for (int dd = 0; dd < DEPTH; ++dd) request(p0 + dd, buf[dd]);
  for (int p = p0; p < p1; p += DEPTH) {
#pragma unroll
    for (int dd = 0; dd < DEPTH; ++dd) {
      if (p + dd < p1) {
        if (APPEND && fits_table && (p + dd + 1) * kPageSize >= len) {
          // The sequence's last page: the step's new token (logical position len - 1) goes to
          // the pool and replaces the stale values this wavefront loaded before the write; an
          // fp8 pool gets the codes the append kernel would store and is attended as stored.
          // (Written out here: behind a function taking the page by reference the page
          // registers of both pages in flight end up in scratch memory.)
          const int t_new = (len - 1) & (kPageSize - 1);
          const int64_t slot_off = ((int64_t)page_id(p + dd) * kPageSize + t_new) * row_stride;
          Page &r = buf[dd];
          if constexpr (FP8) {
            if (n == t_new) {
              uint8_t *dst = kv + slot_off + (int64_t)h * kHD + 16 * g;
#pragma unroll
              for (int j = 0; j < kHD / 64; ++j) {
                const uint2_t lo = half_to_codes<KV>(__builtin_bit_cast(half8_t, k_row[2 * j]), k_inv);
                const uint2_t hi = half_to_codes<KV>(__builtin_bit_cast(half8_t, k_row[2 * j + 1]), k_inv);
                const uint4_t x = uint4_t{lo[0], lo[1], hi[0], hi[1]};
                r.k[j] = x;
                *(uint4_t *)(dst + 64 * j) = x;
              }
            }
            if (q8_v_row(n, g) == (t_new & 7)) {
              const uint2_t lo = half_to_codes<KV>(__builtin_bit_cast(half8_t, v_row[0]), v_inv);
              const uint2_t hi = half_to_codes<KV>(__builtin_bit_cast(half8_t, v_row[1]), v_inv);
              const uint4_t x = uint4_t{lo[0], lo[1], hi[0], hi[1]};
              *(uint4_t *)(kv + slot_off + (int64_t)(num_kv_heads + h) * kHD + 16 * (q8_v_col(n) & (kHD / 16 - 1))) = x;
#pragma unroll
              for (int i = 0; i < 2; ++i) {
                if (i == (t_new >> 3)) r.v[i] = x;
              }
            }
          } else {
            if (n == t_new) {
              half_t *dst = kv + slot_off + (int64_t)h * kHD + 8 * g;
#pragma unroll
              for (int kk = 0; kk < kKSteps; ++kk) {
                const half8_t x = __builtin_bit_cast(half8_t, k_row[kk]);
                r.k[kk] = x;
                *(half8_t *)(dst + 32 * kk) = x;
              }
            }
            if (g == (t_new & 3)) {
              const half8_t x = __builtin_bit_cast(half8_t, v_row[0]);
              *(half8_t *)(kv + slot_off + (int64_t)(num_kv_heads + h) * kHD + 8 * (n & (kVCols - 1))) = x;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                if (i == (t_new >> 2)) r.v[i] = x;
              }
            }
          }
        }
        attend_page(st, buf[dd], qf, vstage, vt_lane, p + dd, len, n, g, scale_log2);
      }
      request(p + dd + DEPTH, buf[dd]);
    }
  }

  const int64_t cell = ((int64_t)b * num_q_heads + hq0) * max_splits + split;
  store_state(st, n_splits == 1, out_row, part_o + cell * kHD, (int64_t)max_splits * kHD,
              part_lse + cell, max_splits, n, g, group, v_scale);
}

// Merges partial rows of one query head into its final fp16 row; run by one whole wavefront.
// The partials come in two runs: n1 of them at lse1[s * lse1_stride], po1[s * po1_stride .. +D),
// then n2 more at lse2 / po2 (n2 may be 0). Lane s holds the weight of partial s (blocks of 64
// partials); each lane accumulates two output elements over the partials in index order, with
// independent row loads kept in flight.
template <bool TWO_RUNS>
__device__ __forceinline__ void merge_row(const float *__restrict__ lse1, int64_t lse1_stride,
                                          const float *__restrict__ po1, int64_t po1_stride, int n1,
                                          const float *__restrict__ lse2, int64_t lse2_stride,
                                          const float *__restrict__ po2, int64_t po2_stride, int n2,
                                          half_t *out_row, int lane) {
  const int n_parts = TWO_RUNS ? n1 + n2 : n1;
  // lane l holds elements 2l, 2l + 1 of the row; with a row of 64 the upper lanes re-read
  // element 0 and store nothing
  const bool live_col = 2 * lane < kHD;
  const int mcol = live_col ? 2 * lane : 0;
  auto lse_of = [&](int s) {
    if (!TWO_RUNS || s < n1) return lse1[(int64_t)s * lse1_stride];
    return lse2[(int64_t)(s - n1) * lse2_stride];
  };
  auto row_of = [&](int s) {
    if (!TWO_RUNS || s < n1) return po1 + (int64_t)s * po1_stride;
    return po2 + (int64_t)(s - n1) * po2_stride;
  };
  if (n_parts <= 16) {
    // The usual case (a sequence spans a few chunks, with or without the slices of a shared
    // prefix): every row and the log-sum-exps are requested at once, so the launch waits for one
    // round trip to memory instead of one per group of rows. Same weights and the same order of
    // additions as the general path below.
    float2 r[16];
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      r[s] = float2{0.f, 0.f};
      if (s < n_parts) r[s] = *(const float2 *)(row_of(s) + mcol);
    }
    const float l = lane < n_parts ? lse_of(lane) : -INFINITY;
    float mx = l;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, xor_lane(mx, off));
    const float w = fast_exp2((l - mx) * kLog2e);
    float den = w;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) den += xor_lane(den, off);
    float num0 = 0.f, num1 = 0.f;
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      if (s < n_parts) {
        const float ws = __shfl(w, s, kWave);
        num0 += ws * r[s].x;
        num1 += ws * r[s].y;
      }
    }
    const float inv = 1.0f / den;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    if (live_col) *(half2_t *)(out_row + mcol) = half2_t{(half_t)(num0 * inv), (half_t)(num1 * inv)};
    return;
  }
  float mx = -INFINITY;
  for (int s0 = 0; s0 < n_parts; s0 += kWave) {
    const float l = (s0 + lane < n_parts) ? lse_of(s0 + lane) : -INFINITY;
    mx = fmaxf(mx, l);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, xor_lane(mx, off));
  float den = 0.f, num0 = 0.f, num1 = 0.f;
  for (int s0 = 0; s0 < n_parts; s0 += kWave) {
    const float l = (s0 + lane < n_parts) ? lse_of(s0 + lane) : -INFINITY;
    const float w = fast_exp2((l - mx) * kLog2e);
    den += w;
    const int cnt = (n_parts - s0) < kWave ? (n_parts - s0) : kWave;
    int s = 0;
    for (; s + 4 <= cnt; s += 4) {
      float2 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) r[u] = *(const float2 *)(row_of(s0 + s + u) + mcol);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float wu = __shfl(w, s + u, kWave);
        num0 += wu * r[u].x;
        num1 += wu * r[u].y;
      }
    }
    for (; s < cnt; ++s) {
      const float2 r = *(const float2 *)(row_of(s0 + s) + mcol);
      const float wu = __shfl(w, s, kWave);
      num0 += wu * r.x;
      num1 += wu * r.y;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) den += xor_lane(den, off);
  const float inv = 1.0f / den;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  if (live_col) *(half2_t *)(out_row + mcol) = half2_t{(half_t)(num0 * inv), (half_t)(num1 * inv)};
}

// Schedule "splits" merge: one wavefront per (query head, sequence).
__global__ __launch_bounds__(kWave) void paged_decode_merge_kernel(
    const int32_t *__restrict__ seq_lens, half_t *__restrict__ out,
    const float *__restrict__ part_o, const float *__restrict__ part_lse, int32_t num_q_heads,
    int32_t max_splits, int32_t min_pages_per_split) {
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int len = seq_lens[b];
  if (len <= 0) return;
  const int n_splits = splits_for_pages(pages_of(len), max_splits, min_pages_per_split);
  if (n_splits == 1) return;  // the split kernel already wrote the final row
  const int64_t cell0 = ((int64_t)b * num_q_heads + hq) * max_splits;
  merge_row<false>(part_lse + cell0, 1, part_o + cell0 * kHD, kHD, n_splits, nullptr, 0,
                   nullptr, 0, 0, out + ((int64_t)b * num_q_heads + hq) * kHD, threadIdx.x);
}

// ---------------------------------------------------------------------------------------------
// Schedule "balanced": the pages of all sequences, concatenated in batch order, form one line
// of `total` pages per kv head; it is cut into `chunks` pieces of floor(total / chunks) or one
// more pages. Wavefront (head h, chunk c) streams the pages of its piece, finishing one sequence
// and starting the next where the line crosses a sequence boundary. A workgroup holds
// `heads_per_wg` heads of `replicas` consecutive chunks.
//
// The cuts are made once per decode step by the plan kernel (block tables and lengths are the
// same for every layer of a step) and stored as one entry per chunk:
//   entry[0] first page on the line   entry[1] one past its last page
//   entry[2] sequence of the first page (low half) and the next sequence with pages (high half)
//   entry[3], entry[4] the first sequence's [first, last) page, entry[7] its length
//   entry[5], entry[6] for the merge by chunk boundary (see decode_plan_kernel)
//   entry[8 ..] the chunk's physical page ids, in line order
// so a wavefront needs one dependent hop (its entry) before it can request q, K and V.
//
// The piece of sequence b inside chunk c is partial slot c + b (strictly increasing along the
// line, so slots never collide): part_o[slot][hq][D], part_lse[slot][hq]. A sequence lying
// inside one chunk is written to `out` directly; the others are merged, in chunk order, by a
// second small launch (one wavefront per sequence and kv head).
//
// Shared prefix: when every sequence of the step starts with the same `skip` physical pages
// (a cached system prompt), the line holds only the pages after them, and those `skip` pages are
// attended once for all sequences by the MFMA-tiled kernel of paged_prefill.hip, whose columns
// are the (sequence, query head) pairs. Its per-key-slice partials join the merge as a second
// run of pieces; no sequence is then written directly. Merging inside the decode
// kernel was measured and rejected: pieces written by other XCDs only become visible through
// device-scope cache write-back / invalidate or write-through accesses, and either costs far
// more than the 3 us of a launch boundary.
// ---------------------------------------------------------------------------------------------
constexpr int kMaxWavesPerWg = 8;
// (the layout of a plan buffer -- kPlanMeta, kEntryHeader, the meta words, plan_entries_offset,
// LineCut -- is in common.h: the kernel for other head dims reads page ids from a plan too)

// Entry stride (int32 words) that holds the largest possible chunk: no sequence has more than
// `bt_stride` pages, so total <= batch * bt_stride.
__host__ __device__ __forceinline__ int plan_entry_stride(int batch, int bt_stride, int chunks) {
  const int64_t max_total = (int64_t)batch * bt_stride;
  const int max_chunk_pages = (int)((max_total + chunks - 1) / chunks);
  return round_up(kEntryHeader + max_chunk_pages, 4);
}

// One block per sequence: places the sequence's pages on the line, fills the entries they fall
// into and records which chunks the sequence spans; block 0 also writes the meta words and
// marks the chunks past the end of the line as empty.
__global__ __launch_bounds__(256) void decode_plan_kernel(
    const int32_t *__restrict__ block_table, int32_t table_stride, int32_t bt_stride,
    const int32_t *__restrict__ seq_lens, int32_t batch, int32_t num_kv_heads, int32_t chunks,
    int32_t entry_stride, int32_t num_pages, int32_t page_shift, int32_t skip,
    int32_t *__restrict__ plan) {
  // table_stride: entries per block-table row; bt_stride, skip: the same row and the shared
  // prefix counted in 16-token pages (entries << page_shift)
  __shared__ int red[4][3];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  int before = 0, total = 0;
  int next_b = batch;  // the next sequence after b that has pages on the line, or batch
  for (int i = tid; i < batch; i += 256) {
    int pg = pages_of(seq_lens[i]);
    pg = (pg < bt_stride ? pg : bt_stride) - skip;
    pg = pg > 0 ? pg : 0;
    total += pg;
    before += (i < b) ? pg : 0;
    next_b = (i > b && pg > 0 && i < next_b) ? i : next_b;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    total += __shfl_xor(total, off, kWave);
    before += __shfl_xor(before, off, kWave);
    const int other = __shfl_xor(next_b, off, kWave);
    next_b = other < next_b ? other : next_b;
  }
  if ((tid & 63) == 0) {
    red[tid >> 6][0] = total;
    red[tid >> 6][1] = before;
    red[tid >> 6][2] = next_b;
  }
  __syncthreads();
  total = red[0][0] + red[1][0] + red[2][0] + red[3][0];
  before = red[0][1] + red[1][1] + red[2][1] + red[3][1];
  next_b = min(min(red[0][2], red[1][2]), min(red[2][2], red[3][2]));
  // The line of `total` pages is cut into `chunks` pieces whose sizes differ by at most one page:
  // the first `rem` chunks hold quot + 1 pages, the others quot (none when quot == 0). With a
  // fixed ceil(total / chunks) pages per chunk the last chunks would stay empty whenever total is
  // just above a multiple of chunks (5 % of the compute units idle at 18.004 pages per chunk).
  const LineCut cut(total, chunks);
  const int quot = cut.quot, rem = cut.rem;
  auto chunk_start = [&](int c) { return cut.chunk_start(c); };
  auto chunk_of = [&](int f) { return cut.chunk_of(f); };
  int32_t *entries = plan + plan_entries_offset(batch);

  if (b == 0) {
    if (tid == 0) {
      plan[kMetaTotal] = total;
      plan[kMetaChunkPages] = quot + (rem > 0 ? 1 : 0);
      plan[kMetaChunks] = chunks;
      plan[kMetaBatch] = batch;
      plan[kMetaEntryStride] = entry_stride;
      plan[kMetaKvHeads] = num_kv_heads;
      plan[kMetaSkip] = skip;
    }
    for (int c = tid; c < chunks; c += 256) {
      if (quot == 0 && c >= rem) {  // a chunk without pages
        entries[(int64_t)c * entry_stride + 0] = 0;
        entries[(int64_t)c * entry_stride + 1] = 0;
        entries[(int64_t)c * entry_stride + 5] = -1;
      }
    }
  }
  int my_pages = pages_of(seq_lens[b]);
  my_pages = (my_pages < bt_stride ? my_pages : bt_stride) - skip;
  my_pages = my_pages > 0 ? my_pages : 0;
  if (tid == 0) {
    const int c_first = chunk_of(before);
    plan[plan_seq_before_offset(batch) + b] = before;
    plan[plan_seq_info_offset() + 2 * b] = c_first;
    plan[plan_seq_info_offset() + 2 * b + 1] =
        my_pages > 0 ? chunk_of(before + my_pages - 1) - c_first + 1 : 0;
  }
  const int32_t *row = block_table + (int64_t)b * table_stride;
  for (int p = tid; p < my_pages; p += 256) {
    const int f = before + p;
    const int c = chunk_of(f);
    const int first = chunk_start(c);
    int32_t *e = entries + (int64_t)c * entry_stride;
    e[kEntryHeader + (f - first)] =
        sub_page_id(row[(p + skip) >> page_shift], p + skip, page_shift, num_pages);
    if (f == first) {
      e[0] = f;
      e[1] = chunk_start(c + 1);
      e[2] = b | (next_b << 16);  // both at most 65535
      e[3] = before;
      e[4] = before + my_pages;
      e[7] = seq_lens[b];
      // for a merge by chunk boundary: the sequence whose pieces start in the chunk before this
      // one and continue here, and how many chunks it spans (-1: none starts there)
      const bool continues = before < f && chunk_of(before) == c - 1;
      e[5] = continues ? b : -1;
      e[6] = continues ? chunk_of(before + my_pages - 1) - (c - 1) + 1 : 0;
    }
  }
}

// Merge of many partial rows by a whole workgroup of kMergeWaves wavefronts (a single long
// sequence spans every chunk of the step: one wavefront adding 256 rows one round trip after the
// other took 23 us). Every wavefront merges a contiguous quarter of the pieces against the common
// maximum, in index order and with 16 row loads in flight; wavefront 0 then adds the four partial
// sums in wavefront order, so the result does not depend on timing.
constexpr int kMergeWaves = 4;

__device__ __forceinline__ void merge_row_wide(const float *__restrict__ lse, int64_t lse_stride,
                                               const float *__restrict__ po, int64_t po_stride,
                                               int n_parts, half_t *out_row, int tid, float *red) {
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const bool live_col = 2 * lane < kHD;  // see merge_row
  const int mcol = live_col ? 2 * lane : 0;
  float mx = -INFINITY;
  for (int s = tid; s < n_parts; s += kMergeWaves * kWave) mx = fmaxf(mx, lse[(int64_t)s * lse_stride]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, xor_lane(mx, off));
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

  const int per = (n_parts + kMergeWaves - 1) / kMergeWaves;
  const int s_begin = wave * per;
  const int s_end = s_begin + per < n_parts ? s_begin + per : n_parts;
  float den = 0.f, num0 = 0.f, num1 = 0.f;
  for (int base = s_begin; base < s_end; base += kWave) {
    const float l = (base + lane < s_end) ? lse[(int64_t)(base + lane) * lse_stride] : -INFINITY;
    const float w = fast_exp2((l - mx) * kLog2e);
    den += w;
    const int cnt = (s_end - base) < kWave ? (s_end - base) : kWave;
    int s = 0;
    for (; s + 16 <= cnt; s += 16) {
      float2 r[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) r[u] = *(const float2 *)(po + (int64_t)(base + s + u) * po_stride + mcol);
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const float wu = __shfl(w, s + u, kWave);
        num0 += wu * r[u].x;
        num1 += wu * r[u].y;
      }
    }
    for (; s < cnt; ++s) {
      const float2 r = *(const float2 *)(po + (int64_t)(base + s) * po_stride + mcol);
      const float wu = __shfl(w, s, kWave);
      num0 += wu * r.x;
      num1 += wu * r.y;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) den += xor_lane(den, off);
  float *sums = red + 8;  // [kMergeWaves][kHD], then the denominators
  if (live_col) {
    sums[wave * kHD + mcol] = num0;
    sums[wave * kHD + mcol + 1] = num1;
  }
  if (lane == 0) sums[kMergeWaves * kHD + wave] = den;
  __syncthreads();
  if (wave != 0) return;
  float d = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
  for (int w2 = 0; w2 < kMergeWaves; ++w2) {
    o0 += sums[w2 * kHD + mcol];
    o1 += sums[w2 * kHD + mcol + 1];
    d += sums[kMergeWaves * kHD + w2];
  }
  const float inv = 1.0f / d;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  if (live_col) *(half2_t *)(out_row + mcol) = half2_t{(half_t)(o0 * inv), (half_t)(o1 * inv)};
}

// The same merge with the row's elements shared out among kMergeDimSlices workgroups of 32
// elements each, for steps of a few long sequences: their rows are few (one per query head and
// sequence) and one workgroup per row reads its 256 pieces through a single compute unit's memory
// path (a 16k-token sequence alone: 6.7 us of a 22 us layer, on 64 of 256 compute units). Sixteen
// lanes read the slice's 128 bytes of a piece, so the 256 threads take 16 pieces per load and each
// thread every sixteenth piece, all its loads in flight at once for up to 256 pieces; the sixteen
// partial sums are added in index order by the first sixteen lanes.
constexpr int kMergeSliceDims = 32;
constexpr int kMergeDimSlices = kHD / kMergeSliceDims;
constexpr int kMergeRedFloats = 8 + 16 * kMergeSliceDims + 16 > 8 + kMergeWaves * kHD + kMergeWaves
                                    ? 8 + 16 * kMergeSliceDims + 16
                                    : 8 + kMergeWaves * kHD + kMergeWaves;

__device__ __forceinline__ void merge_row_sliced(const float *__restrict__ lse, int64_t lse_stride,
                                                 const float *__restrict__ po, int64_t po_stride,
                                                 int n_parts, half_t *out_row, int tid, int slice,
                                                 float *red) {
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = tid & 15;
  const int r = tid >> 4;  // 0..15: which of 16 pieces per sweep
  const int col = slice * kMergeSliceDims + 2 * l16;
  float den = 0.f, num0 = 0.f, num1 = 0.f;
  auto block_max = [&](float mx) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, xor_lane(mx, off));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  };
  // the thread's pieces base, base + 16, ...: their log-sum-exps and its two elements of their rows
  auto request = [&](int base, float (&l)[16], float2 (&row)[16]) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int s = base + 16 * u;
      const bool live = s < n_parts;
      const int at = live ? s : base;
      l[u] = live ? lse[(int64_t)at * lse_stride] : -INFINITY;
      row[u] = *(const float2 *)(po + (int64_t)at * po_stride + col);
    }
  };
  auto add = [&](const float (&l)[16], const float2 (&row)[16], float mx) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const float w = fast_exp2((l[u] - mx) * kLog2e);  // 0 for a piece past the end
      den += w;
      num0 += w * row[u].x;
      num1 += w * row[u].y;
    }
  };
  if (n_parts <= 256) {
    // one sweep: rows and log-sum-exps are requested together, the maximum comes from the
    // log-sum-exps the threads hold (every piece is held by sixteen of them): one round trip
    float l[16];
    float2 row[16];
    request(r < n_parts ? r : 0, l, row);
    float mine = -INFINITY;
    if (r < n_parts) {
#pragma unroll
      for (int u = 0; u < 16; ++u) mine = fmaxf(mine, l[u]);
    }
    const float mx = block_max(mine);
    if (r < n_parts) add(l, row, mx);
  } else {
    float mine = -INFINITY;
    for (int s = tid; s < n_parts; s += kMergeWaves * kWave) mine = fmaxf(mine, lse[(int64_t)s * lse_stride]);
    const float mx = block_max(mine);
    for (int base = r; base < n_parts; base += 256) {
      float l[16];
      float2 row[16];
      request(base, l, row);
      add(l, row, mx);
    }
  }
  float *sums = red + 8;  // [16][kMergeSliceDims], then the sixteen denominators
  sums[r * kMergeSliceDims + 2 * l16] = num0;
  sums[r * kMergeSliceDims + 2 * l16 + 1] = num1;
  if (l16 == 0) sums[16 * kMergeSliceDims + r] = den;
  __syncthreads();
  if (tid >= 16) return;
  float d = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
  for (int r2 = 0; r2 < 16; ++r2) {
    o0 += sums[r2 * kMergeSliceDims + 2 * l16];
    o1 += sums[r2 * kMergeSliceDims + 2 * l16 + 1];
    d += sums[16 * kMergeSliceDims + r2];
  }
  const float inv = 1.0f / d;
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  *(half2_t *)(out_row + col) = half2_t{(half_t)(o0 * inv), (half_t)(o1 * inv)};
}

// Balanced-schedule merge, one workgroup per (query head, sequence) -- or, without a shared
// prefix and with more sequences than chunk boundaries, per (query head, boundary): only a
// sequence that crosses a boundary has pieces to merge -- : combines the sequence's
// pieces (partial slots c_first + b, c_first + b + 1, ...) if it spans several chunks, and the
// `pre_splits` partials of the shared prefix if there is one. Up to 16 pieces (and any number
// with a shared prefix) are merged by the first wavefront alone.
__global__ __launch_bounds__(kMergeWaves *kWave) void paged_decode_balanced_merge_kernel(
    const int32_t *__restrict__ plan, const int32_t *__restrict__ seq_lens,
    half_t *__restrict__ out, const float *__restrict__ part_o,
    const float *__restrict__ part_lse, const float *__restrict__ pre_o,
    const float *__restrict__ pre_lse, int32_t pre_splits, int32_t batch, int32_t num_q_heads,
    int32_t by_boundary, int32_t bt_stride, int32_t chunks, int32_t heads_per_wg) {
  __shared__ float red[kMergeRedFloats];
  // heads_per_wg 1: the workgroup has one row (query head); 4: each wavefront has its own
  const int hq = blockIdx.x * heads_per_wg + (heads_per_wg > 1 ? (int)(threadIdx.x >> 6) : 0);
  int b = blockIdx.y;
  int c_first, n_parts;
  if (by_boundary) {
    // blockIdx.y names the boundary between chunks y and y + 1; the header of chunk y + 1 says
    // which sequence, if any, has its first piece in chunk y and goes on (decode_plan_kernel).
    const int32_t *e = plan + plan_entries_offset(batch) +
                       (int64_t)(blockIdx.y + 1) * plan_entry_stride(batch, bt_stride, chunks);
    b = e[5];
    if (b < 0) return;
    c_first = blockIdx.y;
    n_parts = e[6];
  } else {
    c_first = plan[plan_seq_info_offset() + 2 * b];
    n_parts = plan[plan_seq_info_offset() + 2 * b + 1];
  }
  if (pre_splits == 0 && n_parts <= 1) return;  // empty, or written directly by the decode kernel
  if (pre_splits != 0 && seq_lens[b] <= 0) return;  // the decode kernel zeroed the row
  const int64_t cell0 = (int64_t)(c_first + b) * num_q_heads + hq;
  const int64_t pre0 = (int64_t)b * num_q_heads + hq;
  const int64_t pre_step = (int64_t)batch * num_q_heads;
  half_t *out_row = out + ((int64_t)b * num_q_heads + hq) * kHD;
  if (gridDim.z > 1) {
    // the launch shares a long row's elements out among the workgroups z (heads_per_wg is 1);
    // any other row is the first one's alone
    if (pre_splits == 0 && n_parts > 16) {
      merge_row_sliced(part_lse + cell0, num_q_heads, part_o + cell0 * kHD, (int64_t)num_q_heads * kHD,
                       n_parts, out_row, threadIdx.x, (int)blockIdx.z, red);
      return;
    }
    if (blockIdx.z != 0) return;
  }
  if (pre_splits == 0 && n_parts > 16 && blockDim.x == kMergeWaves * kWave) {  // uniform in the workgroup
    // a long row takes the whole workgroup; with a row per wavefront the rows take turns
    for (int r = 0; r < heads_per_wg; ++r) {
      const int shift = heads_per_wg > 1 ? r - (int)(threadIdx.x >> 6) : 0;  // from this wavefront's row to row r
      merge_row_wide(part_lse + cell0 + shift, num_q_heads, part_o + (cell0 + shift) * kHD,
                     (int64_t)num_q_heads * kHD, n_parts, out_row + (int64_t)shift * kHD,
                     threadIdx.x, red);
      __syncthreads();
    }
    return;
  }
  if (heads_per_wg == 1 && threadIdx.x >= kWave) return;
  const int lane = threadIdx.x & (kWave - 1);
  if (pre_splits == 0) {
    merge_row<false>(part_lse + cell0, num_q_heads, part_o + cell0 * kHD,
                     (int64_t)num_q_heads * kHD, n_parts, nullptr, 0, nullptr, 0, 0, out_row,
                     lane);
  } else {
    merge_row<true>(part_lse + cell0, num_q_heads, part_o + cell0 * kHD,
                    (int64_t)num_q_heads * kHD, n_parts, pre_lse + pre0, pre_step,
                    pre_o + pre0 * kHD, pre_step * kHD, pre_splits, out_row, lane);
  }
}

// LDS of a workgroup of the balanced kernel: the V staging rows of its wavefronts, then their
// parking areas.
constexpr int kBalancedVstageBytes = kMaxWavesPerWg * kPageSize * kVPitch * (int)sizeof(half_t);
constexpr int kBalancedLdsBytes = kBalancedVstageBytes + kMaxWavesPerWg * kParkFloats * (int)sizeof(float);

// What a workgroup of the balanced kernel does is in balanced_body.inc. It is compiled into the
// kernel below and into this function, which the kernel of a step behind a shared prefix
// (prefix_step_kernel) runs as one of its two roles, on the workgroup standing at (block_x,
// block_y) of the balanced grid and with its two LDS areas.
template <int DEPTH, int KV>
__device__ __forceinline__ void balanced_body(
    half_t (*vstage_all)[kPageSize * kVPitch], float (*park_all)[kParkFloats], const int block_x,
    const int block_y,
    const half_t *__restrict__ q, int64_t q_batch_stride,
    typename KvStore<KV>::elem *__restrict__ kv, const float *__restrict__ scales,
    const int32_t *__restrict__ seq_lens, const int32_t *__restrict__ plan,
    const half_t *__restrict__ k_new, const half_t *__restrict__ v_new, int64_t k_new_stride,
    int64_t v_new_stride, half_t *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_lse, int32_t bt_stride, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t group_all, int32_t slices, int32_t heads_per_wg,
    int32_t replicas, int32_t chunks, int32_t skip, float scale_log2) {
#include "balanced_body.inc"
}

template <int DEPTH, int KV>
__global__ __launch_bounds__(kMaxWavesPerWg * kWave) void paged_decode_balanced_kernel(
    const half_t *__restrict__ q, int64_t q_batch_stride,
    typename KvStore<KV>::elem *__restrict__ kv, const float *__restrict__ scales,
    const int32_t *__restrict__ seq_lens, const int32_t *__restrict__ plan,
    const half_t *__restrict__ k_new, const half_t *__restrict__ v_new, int64_t k_new_stride,
    int64_t v_new_stride, half_t *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_lse, int32_t bt_stride, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t group_all, int32_t slices, int32_t heads_per_wg,
    int32_t replicas, int32_t chunks, int32_t skip, float scale_log2) {
  __shared__ __attribute__((aligned(16))) half_t vstage_all[kMaxWavesPerWg][kPageSize * kVPitch];
  __shared__ __attribute__((aligned(16))) float park_all[kMaxWavesPerWg][kParkFloats];
  const int block_x = (int)blockIdx.x, block_y = (int)blockIdx.y;
#include "balanced_body.inc"
}

// ---------------------------------------------------------------------------------------------
// A decode step behind a shared prefix as ONE launch with two roles. The first `prefix_wgs`
// workgroups attend the shared pages for the whole batch (prefill_tile.h in its shared-prefix
// mode: columns = (sequence, query head) pairs, one key slice per workgroup, normalised fp32
// partials out); the others are the workgroups of the balanced kernel over the pages behind the
// prefix. The prefix role is bound by the matrix pipes of the few compute units it occupies, the
// other by memory: as two launches they ran one after the other (17 + 20 us on 64 sequences
// sharing 2048 tokens), each leaving half the device idle; two streams cost more in forks and
// joins between hardware queues than they overlapped. Prefix workgroups come first in the grid:
// they are the long ones, and x = kv head keeps a head's slices on one XCD. Registers are those
// of the prefix role (two wavefronts per SIMD), so a compute unit holds one workgroup of either
// role.
// ---------------------------------------------------------------------------------------------
template <int KV> struct PrefixMode { static constexpr int value = prefill_tile::kSharedPrefix; };
template <> struct PrefixMode<kKvFp8> { static constexpr int value = prefill_tile::kSharedPrefixFp8; };
template <> struct PrefixMode<kKvInt8> { static constexpr int value = prefill_tile::kSharedPrefixInt8; };

template <int PW>
constexpr int prefix_step_lds_bytes() {
  return prefill_tile::tile_lds_bytes<PW>() > kBalancedLdsBytes ? prefill_tile::tile_lds_bytes<PW>()
                                                                 : kBalancedLdsBytes;
}

template <int DEPTH, int KV, int PW>
__global__ __launch_bounds__(kMaxWavesPerWg * kWave) void prefix_step_kernel(
    prefill_tile::PagedSource shared, prefill_tile::PrefixTask task, int32_t prefix_wgs,
    int32_t prefix_col_blocks, int32_t decode_wgs_x,
    const half_t *__restrict__ q, int64_t q_batch_stride,
    typename KvStore<KV>::elem *__restrict__ kv, const float *__restrict__ scales,
    const int32_t *__restrict__ seq_lens, const int32_t *__restrict__ plan,
    const half_t *__restrict__ k_new, const half_t *__restrict__ v_new, int64_t k_new_stride,
    int64_t v_new_stride, half_t *__restrict__ out, float *__restrict__ part_o,
    float *__restrict__ part_lse, int32_t bt_stride, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t group_all, int32_t slices, int32_t heads_per_wg,
    int32_t replicas, int32_t chunks, int32_t skip, float scale_log2) {
  __shared__ __attribute__((aligned(1024))) char lds[prefix_step_lds_bytes<PW>()];
  const int id = (int)blockIdx.x;
  if (id < prefix_wgs) {
    if ((int)threadIdx.x >= PW * kWave) return;  // the role has PW wavefronts; no barrier counts the others
    const int h = id % num_kv_heads;
    const int rest = id / num_kv_heads;
    const int col_block = rest % prefix_col_blocks;
    const int key_slice = rest / prefix_col_blocks;
    prefill_tile::prefill_tile_body<PrefixMode<KV>::value, PW>(
        (uint32_t)(uintptr_t)(prefill_tile::lds_half_t *)lds, h, col_block, key_slice, 1, q, (int64_t)0,
        (half_t *)nullptr, (int64_t)0, shared, prefill_tile::PackedSource{nullptr, nullptr, 0, 0, nullptr},
        task, (const int32_t *)nullptr, (const int32_t *)nullptr, (const int32_t *)nullptr, group_all, 1,
        group_all, 1, scale_log2);
    return;
  }
  const int d = id - prefix_wgs;
  balanced_body<DEPTH, KV>(reinterpret_cast<half_t(*)[kPageSize * kVPitch]>(lds),
                           reinterpret_cast<float(*)[kParkFloats]>(lds + kBalancedVstageBytes),
                           d % decode_wgs_x, d / decode_wgs_x, q, q_batch_stride, kv, scales, seq_lens,
                           plan, k_new, v_new, k_new_stride, v_new_stride, out, part_o, part_lse,
                           bt_stride, batch, num_q_heads, num_kv_heads, group_all, slices, heads_per_wg,
                           replicas, chunks, skip, scale_log2);
}

}  // namespace LITEKV_HD_NS
}  // namespace litekv

// ---------------------------------------------------------------------------------------------
// Host side: argument checks and launches.
// ---------------------------------------------------------------------------------------------
namespace litekv {
inline namespace LITEKV_HD_NS {



// Checks shared by every decode entry point; `need_inputs` is false for the merge-only calls.
static int validate_decode(const char *what, const DecodeArgs &a, size_t workspace_needed,
                           bool need_inputs) {
  LITEKV_REQUIRE(a.batch >= 0 && a.batch <= 65535, "%s: batch %d out of [0, 65535]", what, a.batch);
  LITEKV_REQUIRE(a.head_dim == kHD, "%s: head_dim %d unsupported (32, 64, 128 or 256)", what,
                 a.head_dim);
  LITEKV_REQUIRE(page_shift_of(a.page_size) >= 0, "%s: page_size %d unsupported (16, 32, 64, 128 or 256)",
                 what, a.page_size);
  LITEKV_REQUIRE(a.num_q_heads > 0 && a.num_q_heads <= 65535, "%s: num_q_heads %d out of range",
                 what, a.num_q_heads);
  if (a.batch == 0) return LITEKV_OK;
  LITEKV_REQUIRE(a.seq_lens && a.out, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(a.out), "%s: out must be 16-byte aligned", what);
  if (workspace_needed > 0) {
    LITEKV_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= workspace_needed,
                   "%s: workspace of %zu bytes needed, got %zu", what, workspace_needed,
                   a.workspace ? a.workspace_bytes : (size_t)0);
    LITEKV_REQUIRE(aligned16(a.workspace), "%s: workspace must be 16-byte aligned", what);
  }
  if (need_inputs) {
    LITEKV_REQUIRE(a.q && a.kv_pool && a.block_table, "%s: null pointer", what);
    LITEKV_REQUIRE(a.num_kv_heads > 0 && a.num_q_heads % a.num_kv_heads == 0,
                   "%s: num_q_heads %d not a multiple of num_kv_heads %d", what, a.num_q_heads,
                   a.num_kv_heads);
    LITEKV_REQUIRE(a.num_q_heads / a.num_kv_heads <= kMaxGroup,
                   "%s: %d query heads per kv head unsupported (max %d)", what,
                   a.num_q_heads / a.num_kv_heads, kMaxGroup);
    LITEKV_REQUIRE(a.q_batch_stride >= (int64_t)a.num_q_heads * a.head_dim &&
                       a.q_batch_stride % 8 == 0,
                   "%s: q_batch_stride %lld invalid", what, (long long)a.q_batch_stride);
    LITEKV_REQUIRE(aligned16(a.q) && aligned16(a.kv_pool),
                   "%s: q and kv_pool must be 16-byte aligned", what);
    LITEKV_REQUIRE(a.block_table_stride >= 1, "%s: block_table_stride %d < 1", what,
                   a.block_table_stride);
    LITEKV_REQUIRE(a.num_pages >= 1 && a.num_pages <= 0x7fffffffLL / a.page_size,
                   "%s: num_pages %lld out of range", what, (long long)a.num_pages);
    LITEKV_REQUIRE((int64_t)a.block_table_stride * (a.page_size / kPageSize) <= 0x7fffffffLL / 4,
                   "%s: block_table_stride %d too large", what, a.block_table_stride);
  }
  return LITEKV_OK;
}

// A decode step at a head dim the tuned kernels do not take (32, 64, 256): one launch of the
// kernel of generic_attention.hip writes the final rows, whatever the schedule asked for; no
// workspace is used. `plan` replaces the block table for the balanced entry points, which are
// not given one.
static int launch_generic_decode(const char *what, const DecodeArgs &a, const float *scales,
                                 int format, const int32_t *plan = nullptr) {
  LITEKV_REQUIRE(a.batch == 0 || a.seq_lens != nullptr, "%s: null pointer", what);
  GenericLaunch g;
  g.q = a.q;
  g.q_row_stride = a.q_batch_stride;
  g.out = a.out;
  g.out_row_stride = (int64_t)a.num_q_heads * a.head_dim;
  g.kv_pool = const_cast<void *>(a.kv_pool);
  g.scales = scales;
  g.format = scales != nullptr ? format : kKvF16;
  g.block_table = plan != nullptr ? nullptr : a.block_table;
  g.plan = plan;
  g.bt_stride = a.block_table_stride;
  g.page_size = a.page_size;
  g.num_pages = a.num_pages;
  g.seq_lens = a.seq_lens;
  g.k_new = a.k_new;
  g.v_new = a.v_new;
  g.k_new_stride = a.k_new_stride;
  g.v_new_stride = a.v_new_stride;
  g.batch = a.batch;
  g.rows_per_seq = 1;
  g.num_q_heads = a.num_q_heads;
  g.num_kv_heads = a.num_kv_heads;
  g.head_dim = a.head_dim;
  g.softmax_scale = a.softmax_scale;
  g.stream = a.stream;
  LITEKV_REQUIRE(a.kv_pool != nullptr || a.batch == 0, "%s: null pointer", what);
  return launch_generic_attention(what, g);
}

// ---- schedule "splits" ----

static size_t splits_workspace_bytes(int64_t batch, int64_t hq, int64_t d, int64_t s) {
  if (batch <= 0 || hq <= 0 || d <= 0 || s <= 1) return 0;
  return (size_t)(batch * hq * s * (d + 1)) * sizeof(float);
}

// The kernels count in 16-token pages: the caller's lower bound on a split, given in pages of the
// pool, in those (saturating).
static int32_t min_16_token_pages(int32_t min_pages_per_split, int32_t page_size) {
  const int64_t m = (int64_t)min_pages_per_split * (page_size / kPageSize);
  return (int32_t)(m < 0x7fffffffLL ? m : 0x7fffffffLL);
}

static int check_split_plan(const char *what, int32_t max_splits, int32_t min_pages_per_split) {
  LITEKV_REQUIRE(max_splits >= 1 && max_splits <= 65535, "%s: max_splits %d out of [1, 65535]", what,
                 max_splits);
  LITEKV_REQUIRE(min_pages_per_split >= 1, "%s: min_pages_per_split %d < 1", what,
                 min_pages_per_split);
  return LITEKV_OK;
}

// Compute units of the current device.
static int device_cus() {
  static thread_local int cached_device = -1;
  static thread_local int cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != cached_device) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0) {
      cus = 256;
    }
    cached_device = dev;
    cached_cus = cus;
  }
  return cached_cus;
}

// fp8_scales: the scales of a pool of 8-bit codes of format `format` (kKvFp8, kKvInt8), or null.
// Optional HIP events bracketing the next decode launch of this thread (the balanced kernel or the
// per-sequence split kernel, not their merge launches): profiling.
static thread_local hipEvent_t g_profile_start = nullptr;
static thread_local hipEvent_t g_profile_stop = nullptr;

static int launch_split(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split,
                        const float *fp8_scales = nullptr, int format = kKvFp8) {
  const char *what = !fp8_scales          ? "paged_decode_split"
                     : format == kKvInt8 ? "paged_decode_split_int8"
                                         : "paged_decode_split_fp8";
  int rc = check_split_plan(what, max_splits, min_pages_per_split);
  if (rc != LITEKV_OK) return rc;
#if LITEKV_HD == 128
  if (a.head_dim == 64) return hd64_split(a, max_splits, min_pages_per_split, fp8_scales, format);
#endif
  if (a.head_dim != kHD) return launch_generic_decode(what, a, fp8_scales, format);
  rc = validate_decode(what, a,
                       splits_workspace_bytes(a.batch, a.num_q_heads, a.head_dim, max_splits), true);
  if (rc != LITEKV_OK) return rc;
  if (a.batch == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(a.num_kv_heads <= 65535, "%s: num_kv_heads %d > 65535", what, a.num_kv_heads);
  const int group = a.num_q_heads / a.num_kv_heads;
  const int slices = head_slices(group);           // wavefronts per kv head
  const int slice_heads = a.num_kv_heads * slices;
  LITEKV_REQUIRE(slice_heads <= 65535, "%s: num_q_heads %d too large", what, a.num_q_heads);
  float *part_o = max_splits > 1 ? static_cast<float *>(a.workspace) : nullptr;
  float *part_lse =
      max_splits > 1 ? part_o + (size_t)a.batch * a.num_q_heads * max_splits * a.head_dim : nullptr;
  // Wavefronts per workgroup: as many kv heads of one (sequence, split) -- they have the same
  // pages and the same trip count, and a token's K and V rows are contiguous over the heads -- as
  // leave at least two workgroups per compute unit (C5, 16 splits: 1011 us per layer with one
  // wavefront per workgroup, 930 with its four kv heads together).
  const int64_t units = (int64_t)a.batch * slice_heads * max_splits;
  int waves = kSplitWaves;
  while (waves > 1 && (units / waves < 512 || slice_heads % waves != 0)) waves >>= 1;
  const dim3 grid((unsigned)(slice_heads / waves), (unsigned)max_splits, (unsigned)a.batch);
  const dim3 block((unsigned)(waves * kWave));
  const size_t lds = (size_t)waves * kPageSize * kVPitch * sizeof(half_t);
  // Sequences from the longest down once the launch has more workgroups than the device holds at
  // a time (see sequence_of_rank; a launch that is resident at once ends with its longest piece
  // in any order), for block tables wide enough that a split can be 16 pages long: finding its
  // sequence costs a wavefront about a microsecond, which pieces of a page or two would not
  // return (200 sequences of 64 to 256 tokens in 16 splits: 82 us in batch order, 120 us ranked;
  // 256 sequences of 128 to 1024 tokens in 4 splits: 150 against 134 us).
  const int64_t row_pages = (int64_t)a.block_table_stride << page_shift_of(a.page_size);
  const bool longest_first = max_splits > 1 && a.k_new == nullptr && a.batch <= kMaxOrderedBatch &&
                             units / waves > 3 * (int64_t)device_cus() &&
                             row_pages >= 16 * (int64_t)max_splits;
  LITEKV_REQUIRE((a.k_new == nullptr) == (a.v_new == nullptr), "%s: k_new and v_new go together", what);
  if (a.k_new != nullptr) {
    const int64_t row = (int64_t)a.num_kv_heads * a.head_dim;
    LITEKV_REQUIRE(aligned16(a.k_new) && aligned16(a.v_new), "%s: k_new, v_new must be 16-byte aligned",
                   what);
    LITEKV_REQUIRE(a.k_new_stride >= row && a.v_new_stride >= row && a.k_new_stride % 8 == 0 &&
                       a.v_new_stride % 8 == 0,
                   "%s: k_new/v_new strides (%lld, %lld) invalid", what, (long long)a.k_new_stride,
                   (long long)a.v_new_stride);
  }
  // The pool is written only by the instantiations with the fused append.
  void *pool = const_cast<void *>(a.kv_pool);
  hipEvent_t ev0 = g_profile_start, ev1 = g_profile_stop;
  g_profile_start = g_profile_stop = nullptr;
  auto launch = [&](auto kernel, auto *kv) {
    hipExtLaunchKernelGGL(kernel, grid, block, lds, static_cast<hipStream_t>(a.stream), ev0, ev1, 0,
                       static_cast<const half_t *>(a.q), a.q_batch_stride, kv, fp8_scales,
                       a.block_table, a.block_table_stride, a.seq_lens,
                       static_cast<const half_t *>(a.k_new), static_cast<const half_t *>(a.v_new),
                       a.k_new_stride, a.v_new_stride, static_cast<half_t *>(a.out), part_o, part_lse,
                       a.num_q_heads, a.num_kv_heads, group, slices, max_splits,
                       min_16_token_pages(min_pages_per_split, a.page_size), (int32_t)a.num_pages,
                       page_shift_of(a.page_size), a.softmax_scale * kLog2e);
  };
  auto by_append = [&](auto kv_tag, auto *kv) {
    constexpr int KV = decltype(kv_tag)::value;
    if (a.k_new != nullptr) {
      launch(paged_decode_split_kernel<LITEKV_DECODE_DEPTH, KV, true>, kv);
    } else if (longest_first) {
      launch(paged_decode_split_kernel<LITEKV_DECODE_DEPTH, KV, false, true>, kv);
    } else {
      launch(paged_decode_split_kernel<LITEKV_DECODE_DEPTH, KV, false>, kv);
    }
  };
  if (fp8_scales != nullptr && format == kKvInt8) {
    by_append(std::integral_constant<int, kKvInt8>{}, static_cast<uint8_t *>(pool));
  } else if (fp8_scales != nullptr) {
    by_append(std::integral_constant<int, kKvFp8>{}, static_cast<uint8_t *>(pool));
  } else {
    by_append(std::integral_constant<int, kKvF16>{}, static_cast<half_t *>(pool));
  }
  return check_launch(what);
}

static int launch_merge(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split) {
  const char *what = "paged_decode_merge";
  int rc = check_split_plan(what, max_splits, min_pages_per_split);
  if (rc != LITEKV_OK) return rc;
#if LITEKV_HD == 128
  if (a.head_dim == 64) return hd64_merge(a, max_splits, min_pages_per_split);
#endif
  if (a.head_dim != kHD && generic_head_dim(a.head_dim)) {  // launch_generic_decode wrote the rows
    clear_error();
    return LITEKV_OK;
  }
  rc = validate_decode(what, a,
                       splits_workspace_bytes(a.batch, a.num_q_heads, a.head_dim, max_splits),
                       false);
  if (rc != LITEKV_OK) return rc;
  if (a.batch == 0 || max_splits == 1) {
    clear_error();
    return LITEKV_OK;
  }
  const float *part_o = static_cast<const float *>(a.workspace);
  const float *part_lse = part_o + (size_t)a.batch * a.num_q_heads * max_splits * a.head_dim;
  hipLaunchKernelGGL(paged_decode_merge_kernel, dim3((unsigned)a.num_q_heads, (unsigned)a.batch),
                     dim3(kWave), 0, static_cast<hipStream_t>(a.stream), a.seq_lens,
                     static_cast<half_t *>(a.out), part_o, part_lse, a.num_q_heads, max_splits,
                     min_16_token_pages(min_pages_per_split, a.page_size));
  return check_launch(what);
}

// ---- schedule "balanced" ----

struct BalancedShape {
  int heads_per_wg;  // kv heads served by one workgroup (one wavefront each)
  int replicas;      // consecutive chunks served by one workgroup
  int head_groups;   // grid.y
};

static BalancedShape balanced_shape(int num_kv_heads) {
  BalancedShape s;
  s.heads_per_wg = num_kv_heads < kMaxWavesPerWg ? num_kv_heads : kMaxWavesPerWg;
  s.replicas = kMaxWavesPerWg / s.heads_per_wg;
  s.head_groups = (num_kv_heads + s.heads_per_wg - 1) / s.heads_per_wg;
  return s;
}

static size_t balanced_workspace_bytes(int64_t batch, int64_t hq, int64_t d, int64_t chunks) {
  if (batch <= 0 || hq <= 0 || d <= 0 || chunks <= 0) return 0;
  return (size_t)((chunks + batch) * hq * (d + 1)) * sizeof(float);
}
// With a shared prefix: the pieces of the private pages, then the prefix partials of up to
// kMaxPrefixSplits key slices.
static size_t prefix_workspace_bytes(int64_t batch, int64_t hq, int64_t d, int64_t chunks) {
  if (batch <= 0 || hq <= 0 || d <= 0 || chunks <= 0) return 0;
  return balanced_workspace_bytes(batch, hq, d, chunks) +
         (size_t)(kMaxPrefixSplits * batch * hq * (d + 1)) * sizeof(float);
}

// bt_stride: block-table entries per row times page_size / 16
static size_t plan_bytes_for(int64_t batch, int64_t bt_stride, int64_t hkv, int64_t chunks) {
  if (batch <= 0 || bt_stride <= 0 || hkv <= 0 || chunks <= 0) return 0;
  const int64_t words = plan_entries_offset((int)batch) +
                        chunks * plan_entry_stride((int)batch, (int)bt_stride, (int)chunks);
  return (size_t)words * sizeof(int32_t);
}

// Chunks per kv head that give every CU of the current device one workgroup.
static int auto_chunks(int num_kv_heads) {
  const BalancedShape s = balanced_shape(num_kv_heads);
  const int wgs = (device_cus() + s.head_groups - 1) / s.head_groups;
  return wgs * s.replicas;
}

static int check_chunks(const char *what, int32_t batch, int32_t bt_stride, int32_t hkv,
                        int32_t chunks) {
  LITEKV_REQUIRE(chunks >= 1 && chunks <= (1 << 20), "%s: chunks %d out of [1, 2^20]", what, chunks);
  LITEKV_REQUIRE(bt_stride >= 1, "%s: block_table_stride %d < 1", what, bt_stride);
  LITEKV_REQUIRE(hkv >= 1 && hkv <= 65535, "%s: num_kv_heads %d out of range", what, hkv);
  LITEKV_REQUIRE((int64_t)batch * bt_stride <= 0x7fffffffLL / 4,
                 "%s: batch * block_table_stride too large", what);
  return LITEKV_OK;
}

// How the shared pages of a step are cut for the prefix role of prefix_step_kernel: `wide` says
// that its workgroups have 8 wavefronts (256 columns) instead of 4 (128), `col_blocks` how many
// of them cover the batch's (sequence, query head) pairs of one kv head, `splits` the key slices.
struct PrefixShape {
  bool wide;
  int col_blocks, splits, keys_per_split, prefix_keys, wgs;
};
static PrefixShape prefix_shape(int batch, int group, int num_kv_heads, int shared_pages16,
                                bool fp16_pool, int block_waves) {
  // (fp16_pool: false for 8-bit codes, which eight wavefronts stage at head dim 128 only)
  PrefixShape s;
  s.prefix_keys = shared_pages16 * kPageSize;
  const int cols = batch * group;
  // Eight wavefronts share every staged K/V tile among twice the columns and leave twice the
  // compute units to the other role; they take fp16 K/V and a batch that fills them.
  s.wide = (fp16_pool || kHD == 128) && block_waves == prefill_tile::kWideWaves &&
           cols > 16 * prefill_tile::kWgColTiles;
  const int wg_cols = 16 * prefill_tile::kColTiles * (s.wide ? prefill_tile::kWideWaves : prefill_tile::kTiledWaves);
  s.col_blocks = (cols + wg_cols - 1) / wg_cols;
  // Enough key slices for 512 wavefronts of this role (a quarter of the device's slots), at
  // least 128 keys each: every slice is one more partial row per (sequence, head) to write here
  // and to read in the merge (64 sequences sharing 2048 tokens, per layer, as separate launches:
  // 8 slices 47.1 us, 4 slices 44.3 us, 2 slices 49.3 us).
  const int target_wgs = s.wide ? 64 : 128;
  int splits = target_wgs / (num_kv_heads * s.col_blocks);
  splits = splits < 1 ? 1 : (splits > kMaxPrefixSplits ? kMaxPrefixSplits : splits);
  const int max_by_keys = (s.prefix_keys + 127) / 128;
  splits = splits < max_by_keys ? splits : max_by_keys;
  int keys_per_split = (s.prefix_keys + splits - 1) / splits;
  keys_per_split = (keys_per_split + prefill_tile::kKvTile - 1) / prefill_tile::kKvTile * prefill_tile::kKvTile;
  s.keys_per_split = keys_per_split;
  s.splits = (s.prefix_keys + keys_per_split - 1) / keys_per_split;
  s.wgs = num_kv_heads * s.col_blocks * s.splits;
  return s;
}

// Chunks per kv head for a step behind a shared prefix: the workgroups of both roles of
// prefix_step_kernel should be resident at once (a compute unit holds one of either), so the
// private pages get the compute units the prefix role leaves, less a sixteenth of the device
// (64 sequences sharing 2048 tokens, 64 prefix workgroups, per layer: 256 chunks 39.7 us, 192
// 33.6 us, 176 33.1 us).
static int auto_prefix_chunks(int batch, int num_q_heads, int num_kv_heads, int shared_pages16,
                              bool fp16_pool) {
  const int group = num_q_heads / num_kv_heads;
  const BalancedShape s = balanced_shape(num_kv_heads * head_slices(group));
  const PrefixShape ps = prefix_shape(batch, group, num_kv_heads, shared_pages16, fp16_pool,
                                      s.heads_per_wg * s.replicas);
  const int cus = device_cus();
  int wgs = cus - ps.wgs - cus / 16;
  wgs = wgs > cus / 4 ? wgs : cus / 4;
  wgs = (wgs + s.head_groups - 1) / s.head_groups;
  return wgs * s.replicas;
}

}  // namespace LITEKV_HD_NS
}  // namespace litekv

#if LITEKV_HD == 128  // the C ABI lives in the head dim 128 build of this file
extern "C" int32_t litekv_paged_decode_balanced_chunks(int32_t num_kv_heads) {
  return num_kv_heads > 0 ? litekv::auto_chunks(num_kv_heads) : 0;
}

extern "C" int32_t litekv_paged_decode_prefix_chunks(int32_t batch, int32_t num_q_heads,
                                                     int32_t num_kv_heads, int32_t head_dim,
                                                     int32_t page_size, int32_t shared_pages,
                                                     int32_t pool_is_fp16) {
  const int shift = litekv::page_shift_of(page_size);
  if (batch <= 0 || num_kv_heads <= 0 || num_q_heads <= 0 || num_q_heads % num_kv_heads != 0 ||
      num_q_heads / num_kv_heads > litekv::kMaxGroup || shift < 0 || shared_pages <= 0 ||
      shared_pages > (1 << 20)) {
    return num_kv_heads > 0 ? litekv::auto_chunks(num_kv_heads) : 0;
  }
  (void)head_dim;  // both tuned builds cut the prefix alike; other head dims ignore the chunk count
  return litekv::auto_prefix_chunks(batch, num_q_heads, num_kv_heads, shared_pages << shift,
                                    pool_is_fp16 != 0);
}

extern "C" size_t litekv_paged_decode_balanced_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                               int32_t head_dim, int32_t chunks) {
  return litekv::balanced_workspace_bytes(batch, num_q_heads, head_dim, chunks);
}

extern "C" size_t litekv_decode_plan_bytes(int32_t batch, int32_t block_table_stride,
                                           int32_t num_kv_heads, int32_t chunks) {
  return litekv::plan_bytes_for(batch, block_table_stride, num_kv_heads, chunks);
}

extern "C" size_t litekv_decode_plan_bytes_paged(int32_t batch, int32_t block_table_stride,
                                                 int32_t num_kv_heads, int32_t chunks,
                                                 int32_t page_size) {
  const int shift = litekv::page_shift_of(page_size);
  if (shift < 0) return 0;
  return litekv::plan_bytes_for(batch, (int64_t)block_table_stride << shift, num_kv_heads, chunks);
}

#endif  // LITEKV_HD == 128
namespace litekv {
inline namespace LITEKV_HD_NS {
static int launch_plan(const char *what, const int32_t *block_table, int32_t block_table_stride,
                       const int32_t *seq_lens, int32_t batch, int32_t num_kv_heads,
                       int32_t page_size, int64_t num_pages, int32_t chunks, int32_t shared_pages,
                       void *plan, size_t plan_bytes, void *stream) {
  LITEKV_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch %d out of [0, 65535]", what, batch);
  const int shift = page_shift_of(page_size);
  LITEKV_REQUIRE(shift >= 0, "%s: page_size %d unsupported (16, 32, 64, 128 or 256)", what, page_size);
  LITEKV_REQUIRE(block_table_stride >= 1 && block_table_stride <= (0x7fffffff >> 4),
                 "%s: block_table_stride %d out of range", what, block_table_stride);
  const int32_t sub_stride = block_table_stride << shift;  // a row in 16-token pages
  int rc = check_chunks(what, batch, sub_stride, num_kv_heads, chunks);
  if (rc != LITEKV_OK) return rc;
  LITEKV_REQUIRE(shared_pages >= 0 && shared_pages <= block_table_stride,
                 "%s: shared_pages %d out of [0, block_table_stride %d]", what, shared_pages,
                 block_table_stride);
  if (batch == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(block_table && seq_lens && plan, "%s: null pointer", what);
  LITEKV_REQUIRE(aligned16(plan), "%s: plan must be 16-byte aligned", what);
  LITEKV_REQUIRE(num_pages >= 1 && num_pages <= 0x7fffffffLL / page_size,
                 "%s: num_pages %lld out of range", what, (long long)num_pages);
  const size_t need = plan_bytes_for(batch, sub_stride, num_kv_heads, chunks);
  LITEKV_REQUIRE(plan_bytes >= need, "%s: plan buffer of %zu bytes needed, got %zu", what, need,
                 plan_bytes);
  hipLaunchKernelGGL(decode_plan_kernel, dim3((unsigned)batch), dim3(256), 0,
                     static_cast<hipStream_t>(stream), block_table, block_table_stride, sub_stride,
                     seq_lens, batch, num_kv_heads, chunks,
                     plan_entry_stride(batch, sub_stride, chunks), (int32_t)num_pages, shift,
                     shared_pages << shift, static_cast<int32_t *>(plan));
  return check_launch(what);
}
}  // namespace LITEKV_HD_NS
}  // namespace litekv

#if LITEKV_HD == 128  // the C ABI lives in the head dim 128 build of this file
extern "C" int litekv_decode_plan(const int32_t *block_table, int32_t block_table_stride,
                                  const int32_t *seq_lens, int32_t batch, int32_t num_kv_heads,
                                  int32_t page_size, int64_t num_pages, int32_t chunks, void *plan,
                                  size_t plan_bytes, void *stream) {
  return litekv::launch_plan("decode_plan", block_table, block_table_stride, seq_lens, batch,
                             num_kv_heads, page_size, num_pages, chunks, 0, plan, plan_bytes,
                             stream);
}

extern "C" int litekv_decode_plan_prefix(const int32_t *block_table, int32_t block_table_stride,
                                         const int32_t *seq_lens, int32_t batch,
                                         int32_t num_kv_heads, int32_t page_size, int64_t num_pages,
                                         int32_t chunks, int32_t shared_pages, void *plan,
                                         size_t plan_bytes, void *stream) {
  return litekv::launch_plan("decode_plan_prefix", block_table, block_table_stride, seq_lens, batch,
                             num_kv_heads, page_size, num_pages, chunks, shared_pages, plan,
                             plan_bytes, stream);
}

extern "C" int litekv_profile_next_decode(void *start_event, void *stop_event) {
  litekv::g_profile_start = static_cast<hipEvent_t>(start_event);
  litekv::g_profile_stop = static_cast<hipEvent_t>(stop_event);
  return LITEKV_OK;
}

#endif  // LITEKV_HD == 128
namespace litekv {
inline namespace LITEKV_HD_NS {
// The balanced decode step; with shared_pages > 0 preceded by the shared-prefix launch.
static int launch_balanced(const char *what, const void *q, int64_t q_batch_stride, void *kv_pool,
                           const float *fp8_scales, const int32_t *block_table,
                           const int32_t *seq_lens, void *plan,
                           size_t plan_bytes, const void *k_new, const void *v_new,
                           int64_t k_new_stride, int64_t v_new_stride, void *out, void *workspace,
                           size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                           int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                           int64_t num_pages, int32_t block_table_stride, int32_t chunks,
                           int32_t shared_pages, float softmax_scale, void *stream,
                           int format = kKvFp8) {
  const int shift = page_shift_of(page_size);
  LITEKV_REQUIRE(shift >= 0, "%s: page_size %d unsupported (16, 32, 64, 128 or 256)", what, page_size);
  LITEKV_REQUIRE(block_table_stride >= 1 && block_table_stride <= (0x7fffffff >> 4),
                 "%s: block_table_stride %d out of range", what, block_table_stride);
  const int32_t sub_stride = block_table_stride << shift;  // a block-table row in 16-token pages
  int rc = check_chunks(what, batch, sub_stride, num_kv_heads, chunks);
  if (rc != LITEKV_OK) return rc;
  static const int32_t dummy_table = 0;  // the decode kernel reads page ids from the plan
  DecodeArgs a{q, q_batch_stride, kv_pool, block_table ? block_table : &dummy_table,
               block_table_stride, seq_lens, out, workspace, workspace_bytes, batch, num_q_heads,
               num_kv_heads, head_dim, page_size, num_pages, softmax_scale, stream};
#if LITEKV_HD == 128
  if (head_dim == 64) {
    return hd64_balanced(what, q, q_batch_stride, kv_pool, fp8_scales, block_table, shared_pages,
                         seq_lens, plan, plan_bytes,
                         k_new, v_new, k_new_stride, v_new_stride, out, workspace, workspace_bytes,
                         batch, num_q_heads, num_kv_heads, page_size, num_pages, block_table_stride,
                         chunks, softmax_scale, stream, format);
  }
#endif
  if (head_dim != kHD) {
    // other head dims: the generic kernel, which takes its page ids from the block table where
    // the caller gave one (then shared pages are attended like any others), else from the plan
    a.k_new = k_new;
    a.v_new = v_new;
    a.k_new_stride = k_new_stride;
    a.v_new_stride = v_new_stride;
    if (block_table == nullptr && batch > 0) {
      LITEKV_REQUIRE(plan != nullptr && aligned16(plan), "%s: plan must be a 16-byte aligned buffer",
                     what);
      const size_t need_plan = plan_bytes_for(batch, sub_stride, num_kv_heads, chunks);
      LITEKV_REQUIRE(plan_bytes >= need_plan, "%s: plan buffer of %zu bytes needed, got %zu", what,
                     need_plan, plan_bytes);
    }
    return launch_generic_decode(what, a, fp8_scales, format,
                                 block_table == nullptr ? static_cast<const int32_t *>(plan) : nullptr);
  }
  const size_t ws_need = shared_pages > 0
                             ? prefix_workspace_bytes(batch, num_q_heads, head_dim, chunks)
                             : balanced_workspace_bytes(batch, num_q_heads, head_dim, chunks);
  rc = validate_decode(what, a, ws_need, true);
  if (rc != LITEKV_OK) return rc;
  LITEKV_REQUIRE(shared_pages >= 0 && shared_pages <= block_table_stride,
                 "%s: shared_pages %d out of [0, block_table_stride %d]", what, shared_pages,
                 block_table_stride);
  if (batch == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(plan != nullptr && aligned16(plan), "%s: plan must be a 16-byte aligned buffer",
                 what);
  const size_t need = plan_bytes_for(batch, sub_stride, num_kv_heads, chunks);
  LITEKV_REQUIRE(plan_bytes >= need, "%s: plan buffer of %zu bytes needed, got %zu", what, need,
                 plan_bytes);
  LITEKV_REQUIRE((k_new == nullptr) == (v_new == nullptr), "%s: k_new and v_new go together", what);
  if (k_new != nullptr) {
    const int64_t row = (int64_t)num_kv_heads * head_dim;
    LITEKV_REQUIRE(aligned16(k_new) && aligned16(v_new), "%s: k_new, v_new must be 16-byte aligned",
                   what);
    LITEKV_REQUIRE(k_new_stride >= row && v_new_stride >= row && k_new_stride % 8 == 0 &&
                       v_new_stride % 8 == 0,
                   "%s: k_new/v_new strides (%lld, %lld) invalid", what, (long long)k_new_stride,
                   (long long)v_new_stride);
  }
  const int slices = head_slices(num_q_heads / num_kv_heads);  // wavefronts per kv head and chunk
  const BalancedShape s = balanced_shape(num_kv_heads * slices);
  LITEKV_REQUIRE(s.head_groups <= 65535, "%s: num_kv_heads %d too large", what, num_kv_heads);
  float *part_o = static_cast<float *>(workspace);
  float *part_lse = part_o + (size_t)(chunks + batch) * num_q_heads * head_dim;
  float *pre_o = part_lse + (size_t)(chunks + batch) * num_q_heads;
  float *pre_lse = pre_o + (size_t)kMaxPrefixSplits * batch * num_q_heads * head_dim;
  int pre_splits = 0;
  const unsigned wgs = (unsigned)((chunks + s.replicas - 1) / s.replicas);
  hipEvent_t ev0 = g_profile_start, ev1 = g_profile_stop;
  g_profile_start = g_profile_stop = nullptr;
  const dim3 block((unsigned)(kWave * s.heads_per_wg * s.replicas));
  const int group = num_q_heads / num_kv_heads;
  if (shared_pages > 0) {
    // one launch, two roles (see prefix_step_kernel)
    LITEKV_REQUIRE(block_table != nullptr, "%s: block_table is null", what);
    LITEKV_REQUIRE(num_kv_heads <= 1024, "%s: num_kv_heads %d > 1024", what, num_kv_heads);
    LITEKV_REQUIRE(shared_pages <= (1 << 20), "%s: shared_pages %d out of range", what, shared_pages);
    // the prefix role numbers its partial rows (slice, sequence, head) in 32 bits
    LITEKV_REQUIRE((int64_t)kMaxPrefixSplits * batch * num_q_heads < 0x7fffffffLL,
                   "%s: batch %d x %d query heads too large for a shared prefix", what, batch, num_q_heads);
    const PrefixShape ps = prefix_shape(batch, group, num_kv_heads, shared_pages << shift,
                                        fp8_scales == nullptr, (int)(block.x / kWave));
    const int64_t total_wgs = (int64_t)ps.wgs + (int64_t)wgs * s.head_groups;
    LITEKV_REQUIRE(total_wgs <= 0x7fffffffLL, "%s: batch %d too large", what, batch);
    pre_splits = ps.splits;
    // only the first shared_pages entries of block-table row 0 are read
    prefill_tile::PagedSource shared{static_cast<const half_t *>(kv_pool), block_table, shared_pages,
                                     num_kv_heads, (int32_t)num_pages, fp8_scales, shift};
    prefill_tile::PrefixTask task{pre_o, pre_lse, q_batch_stride, batch, num_q_heads, ps.prefix_keys,
                                  ps.keys_per_split};
    auto launch = [&](auto kernel, auto *kv) {
      hipExtLaunchKernelGGL(kernel, dim3((unsigned)total_wgs), block, 0, static_cast<hipStream_t>(stream),
                            ev0, ev1, 0, shared, task, ps.wgs, ps.col_blocks, (int32_t)wgs,
                            static_cast<const half_t *>(q), q_batch_stride, kv, fp8_scales, seq_lens,
                            static_cast<const int32_t *>(plan), static_cast<const half_t *>(k_new),
                            static_cast<const half_t *>(v_new), k_new_stride, v_new_stride,
                            static_cast<half_t *>(out), part_o, part_lse, sub_stride, batch,
                            num_q_heads, num_kv_heads, group, slices, s.heads_per_wg, s.replicas, chunks,
                            shared_pages << shift, softmax_scale * kLog2e);
    };
    constexpr int kWide8 = kHD == 128 ? prefill_tile::kWideWaves : prefill_tile::kTiledWaves;
    if (fp8_scales != nullptr && format == kKvInt8) {
      if (ps.wide) {
        launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvInt8, kWide8>, static_cast<uint8_t *>(kv_pool));
      } else {
        launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvInt8, prefill_tile::kTiledWaves>,
               static_cast<uint8_t *>(kv_pool));
      }
    } else if (fp8_scales != nullptr) {
      if (ps.wide) {
        launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvFp8, kWide8>, static_cast<uint8_t *>(kv_pool));
      } else {
        launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvFp8, prefill_tile::kTiledWaves>,
               static_cast<uint8_t *>(kv_pool));
      }
    } else if (ps.wide) {
      launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvF16, prefill_tile::kWideWaves>,
             static_cast<half_t *>(kv_pool));
    } else {
      launch(prefix_step_kernel<LITEKV_DECODE_DEPTH, kKvF16, prefill_tile::kTiledWaves>,
             static_cast<half_t *>(kv_pool));
    }
  } else {
    const dim3 grid(wgs, (unsigned)s.head_groups);
    auto launch = [&](auto kernel, auto *kv) {
      hipExtLaunchKernelGGL(kernel, grid, block, 0, static_cast<hipStream_t>(stream), ev0, ev1, 0,
                            static_cast<const half_t *>(q), q_batch_stride, kv, fp8_scales, seq_lens,
                            static_cast<const int32_t *>(plan), static_cast<const half_t *>(k_new),
                            static_cast<const half_t *>(v_new), k_new_stride, v_new_stride,
                            static_cast<half_t *>(out), part_o, part_lse, sub_stride, batch,
                            num_q_heads, num_kv_heads, group, slices, s.heads_per_wg, s.replicas,
                            chunks, 0, softmax_scale * kLog2e);
    };
    if (fp8_scales != nullptr && format == kKvInt8) {
      launch(paged_decode_balanced_kernel<LITEKV_DECODE_DEPTH, kKvInt8>, static_cast<uint8_t *>(kv_pool));
    } else if (fp8_scales != nullptr) {
      launch(paged_decode_balanced_kernel<LITEKV_DECODE_DEPTH, kKvFp8>, static_cast<uint8_t *>(kv_pool));
    } else {
      launch(paged_decode_balanced_kernel<LITEKV_DECODE_DEPTH, kKvF16>, static_cast<half_t *>(kv_pool));
    }
  }
  rc = check_launch(what);
  if (rc != LITEKV_OK) return rc;
  // A sequence has at most block_table_stride pages, so it spans at most that many chunks: the
  // four-wavefront merge of long rows (more than 16 pieces, never with a shared prefix) is only
  // launched where such a row can exist; the other wavefronts of a workgroup would leave at once
  // and only cost their dispatch (C4: 9.9 -> 7 us).
  const int max_pieces = chunks < sub_stride ? chunks : sub_stride;
  const int merge_waves = (pre_splits == 0 && max_pieces > 16) ? kMergeWaves : 1;
  // Sequences inside one chunk were written by the decode kernel; at most chunks - 1 sequences
  // cross a chunk boundary. A batch of twice as many is merged by boundary (B 1024 of up to 40
  // tokens: layer 58.7 -> 50.0 us; at B 256..300 one workgroup per sequence is still faster).
  const bool by_boundary = pre_splits == 0 && batch >= 2 * chunks;
  const int merge_rows = by_boundary ? chunks - 1 : batch;
  if (merge_rows == 0) {
    clear_error();
    return LITEKV_OK;
  }
  // Many short rows are bound by the dispatch of their workgroups: four rows per workgroup then,
  // one per wavefront (B 256 of up to 256 tokens: layer 53.5 -> 47.2 us).
  const int merge_heads = (merge_waves == kMergeWaves && num_q_heads % kMergeWaves == 0 &&
                           (int64_t)merge_rows * num_q_heads >= 8192)
                              ? kMergeWaves
                              : 1;
  // Few rows that may be long (a handful of long sequences): a row's elements go to
  // kMergeDimSlices workgroups, so that its pieces are read through as many compute units
  // (see merge_row_sliced); with more rows than that the workgroups already cover the device.
  const int dim_slices = (merge_waves == kMergeWaves && merge_heads == 1 &&
                          (int64_t)merge_rows * num_q_heads * kMergeDimSlices <= 4 * (int64_t)device_cus())
                             ? kMergeDimSlices
                             : 1;
  hipLaunchKernelGGL(paged_decode_balanced_merge_kernel,
                     dim3((unsigned)(num_q_heads / merge_heads), (unsigned)merge_rows, (unsigned)dim_slices),
                     dim3(merge_waves * kWave), 0,
                     static_cast<hipStream_t>(stream), static_cast<const int32_t *>(plan), seq_lens,
                     static_cast<half_t *>(out), part_o, part_lse, pre_o, pre_lse, pre_splits,
                     batch, num_q_heads, by_boundary ? 1 : 0, sub_stride, chunks, merge_heads);
  return check_launch("paged_decode_balanced_merge");
}
}  // namespace LITEKV_HD_NS
}  // namespace litekv

#if LITEKV_HD == 128  // the C ABI lives in the head dim 128 build of this file
extern "C" int litekv_paged_decode_balanced(
    const void *q, int64_t q_batch_stride, void *kv_pool, const int32_t *seq_lens, void *plan,
    size_t plan_bytes, const void *k_new, const void *v_new, int64_t k_new_stride,
    int64_t v_new_stride, void *out, void *workspace, size_t workspace_bytes, int32_t batch,
    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
    int64_t num_pages, int32_t block_table_stride, int32_t chunks, float softmax_scale,
    void *stream) {
  return litekv::launch_balanced("paged_decode_balanced", q, q_batch_stride, kv_pool, nullptr, nullptr,
                                 seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, 0, softmax_scale, stream);
}

extern "C" int litekv_paged_decode_balanced_fp8(
    const void *q, int64_t q_batch_stride, void *kv_pool_fp8, const float *scales,
    const int32_t *seq_lens, void *plan, size_t plan_bytes, const void *k_new, const void *v_new,
    int64_t k_new_stride, int64_t v_new_stride, void *out, void *workspace, size_t workspace_bytes,
    int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
    int64_t num_pages, int32_t block_table_stride, int32_t chunks, float softmax_scale,
    void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_balanced_fp8: scales is null");
  }
  return litekv::launch_balanced("paged_decode_balanced_fp8", q, q_batch_stride, kv_pool_fp8, scales,
                                 nullptr, seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, 0, softmax_scale, stream);
}

extern "C" int litekv_paged_decode_balanced_int8(
    const void *q, int64_t q_batch_stride, void *kv_pool_int8, const float *scales,
    const int32_t *seq_lens, void *plan, size_t plan_bytes, const void *k_new, const void *v_new,
    int64_t k_new_stride, int64_t v_new_stride, void *out, void *workspace, size_t workspace_bytes,
    int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
    int64_t num_pages, int32_t block_table_stride, int32_t chunks, float softmax_scale,
    void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_balanced_int8: scales is null");
  }
  return litekv::launch_balanced("paged_decode_balanced_int8", q, q_batch_stride, kv_pool_int8, scales,
                                 nullptr, seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, 0, softmax_scale, stream, litekv::kKvInt8);
}

extern "C" size_t litekv_paged_decode_prefix_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                             int32_t head_dim, int32_t chunks) {
  return litekv::prefix_workspace_bytes(batch, num_q_heads, head_dim, chunks);
}

extern "C" int litekv_paged_decode_prefix(
    const void *q, int64_t q_batch_stride, void *kv_pool, const int32_t *block_table,
    const int32_t *seq_lens, void *plan, size_t plan_bytes, const void *k_new, const void *v_new,
    int64_t k_new_stride, int64_t v_new_stride, void *out, void *workspace, size_t workspace_bytes,
    int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
    int64_t num_pages, int32_t block_table_stride, int32_t chunks, int32_t shared_pages,
    float softmax_scale, void *stream) {
  return litekv::launch_balanced("paged_decode_prefix", q, q_batch_stride, kv_pool, nullptr, block_table,
                                 seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, shared_pages, softmax_scale, stream);
}

extern "C" int litekv_paged_decode_prefix_fp8(
    const void *q, int64_t q_batch_stride, void *kv_pool_fp8, const float *scales,
    const int32_t *block_table, const int32_t *seq_lens, void *plan, size_t plan_bytes,
    const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride, void *out,
    void *workspace, size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t num_pages,
    int32_t block_table_stride, int32_t chunks, int32_t shared_pages, float softmax_scale,
    void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_prefix_fp8: scales is null");
  }
  return litekv::launch_balanced("paged_decode_prefix_fp8", q, q_batch_stride, kv_pool_fp8, scales,
                                 block_table, seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, shared_pages, softmax_scale, stream);
}

extern "C" int litekv_paged_decode_prefix_int8(
    const void *q, int64_t q_batch_stride, void *kv_pool_int8, const float *scales,
    const int32_t *block_table, const int32_t *seq_lens, void *plan, size_t plan_bytes,
    const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride, void *out,
    void *workspace, size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t num_pages,
    int32_t block_table_stride, int32_t chunks, int32_t shared_pages, float softmax_scale,
    void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_prefix_int8: scales is null");
  }
  return litekv::launch_balanced("paged_decode_prefix_int8", q, q_batch_stride, kv_pool_int8, scales,
                                 block_table, seq_lens, plan, plan_bytes, k_new, v_new, k_new_stride,
                                 v_new_stride, out, workspace, workspace_bytes, batch, num_q_heads,
                                 num_kv_heads, head_dim, page_size, num_pages, block_table_stride,
                                 chunks, shared_pages, softmax_scale, stream, litekv::kKvInt8);
}

extern "C" size_t litekv_paged_decode_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                      int32_t head_dim, int32_t max_splits) {
  return litekv::splits_workspace_bytes(batch, num_q_heads, head_dim, max_splits);
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
                       page_size, num_pages, softmax_scale, stream};
  return litekv::launch_split(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_merge(const int32_t *seq_lens, void *out, const void *workspace,
                                         size_t workspace_bytes, int32_t batch,
                                         int32_t num_q_heads, int32_t head_dim, int32_t page_size,
                                         int32_t max_splits, int32_t min_pages_per_split,
                                         void *stream) {
  litekv::DecodeArgs a{nullptr, 0, nullptr, nullptr, 1, seq_lens, out,
                       const_cast<void *>(workspace), workspace_bytes, batch, num_q_heads, 1,
                       head_dim, page_size, 1, 0.f, stream};
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_fp8(const void *q, int64_t q_batch_stride,
                                       const void *kv_pool_fp8, const float *scales,
                                       const int32_t *block_table, int32_t block_table_stride,
                                       const int32_t *seq_lens, void *out, void *workspace,
                                       size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                       int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                       int64_t num_pages, int32_t max_splits,
                                       int32_t min_pages_per_split, float softmax_scale,
                                       void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_fp8: scales is null");
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool_fp8, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split, batch > 0 ? scales : nullptr);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_int8(const void *q, int64_t q_batch_stride,
                                       const void *kv_pool_int8, const float *scales,
                                       const int32_t *block_table, int32_t block_table_stride,
                                       const int32_t *seq_lens, void *out, void *workspace,
                                       size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                       int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                       int64_t num_pages, int32_t max_splits,
                                       int32_t min_pages_per_split, float softmax_scale,
                                       void *stream) {
  if (scales == nullptr && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_int8: scales is null");
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool_int8, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split, batch > 0 ? scales : nullptr,
                                litekv::kKvInt8);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
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
                       page_size, num_pages, softmax_scale, stream};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_append(const void *q, int64_t q_batch_stride, void *kv_pool,
                                          const int32_t *block_table, int32_t block_table_stride,
                                          const int32_t *seq_lens, const void *k_new,
                                          const void *v_new, int64_t k_new_stride,
                                          int64_t v_new_stride, void *out, void *workspace,
                                          size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                          int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                          int64_t num_pages, int32_t max_splits,
                                          int32_t min_pages_per_split, float softmax_scale,
                                          void *stream) {
  if ((k_new == nullptr || v_new == nullptr) && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, "paged_decode_append: k_new / v_new is null");
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream, k_new, v_new, k_new_stride,
                       v_new_stride};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_append_fp8(
    const void *q, int64_t q_batch_stride, void *kv_pool_fp8, const float *scales,
    const int32_t *block_table, int32_t block_table_stride, const int32_t *seq_lens,
    const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride, void *out,
    void *workspace, size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t num_pages,
    int32_t max_splits, int32_t min_pages_per_split, float softmax_scale, void *stream) {
  if ((scales == nullptr || k_new == nullptr || v_new == nullptr) && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT,
                        "paged_decode_append_fp8: scales / k_new / v_new is null");
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool_fp8, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream, k_new, v_new, k_new_stride,
                       v_new_stride};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split, batch > 0 ? scales : nullptr);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

extern "C" int litekv_paged_decode_append_int8(
    const void *q, int64_t q_batch_stride, void *kv_pool_int8, const float *scales,
    const int32_t *block_table, int32_t block_table_stride, const int32_t *seq_lens,
    const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride, void *out,
    void *workspace, size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
    int32_t num_kv_heads, int32_t head_dim, int32_t page_size, int64_t num_pages,
    int32_t max_splits, int32_t min_pages_per_split, float softmax_scale, void *stream) {
  if ((scales == nullptr || k_new == nullptr || v_new == nullptr) && batch > 0) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT,
                        "paged_decode_append_int8: scales / k_new / v_new is null");
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool_int8, block_table, block_table_stride, seq_lens, out,
                       workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream, k_new, v_new, k_new_stride,
                       v_new_stride};
  int rc = litekv::launch_split(a, max_splits, min_pages_per_split, batch > 0 ? scales : nullptr,
                                litekv::kKvInt8);
  if (rc != LITEKV_OK) return rc;
  return litekv::launch_merge(a, max_splits, min_pages_per_split);
}

// ---------------------------------------------------------------------------------------------
// litekv_paged_decode_static: litekv_paged_decode for callers that cannot allocate. The partial
// rows and log-sum-exps of the split kernel live in a file-scope device array instead of a
// caller's workspace. Every device the library runs on holds its own copy of the array until
// the process ends; its address on a device is looked up once, with that device current.
// ---------------------------------------------------------------------------------------------
#endif  // LITEKV_HD == 128
#if LITEKV_HD == 128
namespace litekv {
inline namespace LITEKV_HD_NS {

static __device__ __align__(256) unsigned char scratch[LITEKV_STATIC_SCRATCH_BYTES];

constexpr int kMaxStaticDevices = 64;
// Device address of `scratch` per device ordinal (null until looked up). Written once per
// device; a race between two first calls stores the same address twice.
static std::atomic<void *> g_scratch_ptr[kMaxStaticDevices];

// Set while a call is enqueueing its two launches on a device: a second host thread that enters
// meanwhile would interleave its launches with them on the shared array and is turned away.
static std::atomic<bool> g_scratch_busy[kMaxStaticDevices];

static int static_scratch(const char *what, hipStream_t stream, void **ptr_out, int *dev_out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) {
    return fail(LITEKV_ERR_LAUNCH, "%s: hipGetDevice failed: %s", what, hipGetErrorString(err));
  }
  LITEKV_REQUIRE(dev >= 0 && dev < kMaxStaticDevices, "%s: device ordinal %d out of [0, %d)", what,
                 dev, kMaxStaticDevices);
  *dev_out = dev;
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    // The lookup is not a stream operation: under a capture it would either fail or end the
    // capture with an error that the next, unrelated call reports.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
        capturing != hipStreamCaptureStatusNone) {
      return fail(LITEKV_ERR_INVALID_ARGUMENT,
                  "%s: first call on device %d is inside a stream capture; call once with batch 0 "
                  "before capturing",
                  what, dev);
    }
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      return fail(LITEKV_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", what,
                  dev, hipGetErrorString(err));
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *ptr_out = ptr;
  return LITEKV_OK;
}

}  // namespace LITEKV_HD_NS
}  // namespace litekv
#endif  // LITEKV_HD == 128

#if LITEKV_HD == 128  // the C ABI lives in the head dim 128 build of this file
extern "C" int litekv_paged_decode_static(const void *q, int64_t q_batch_stride, const void *kv_pool,
                                          const int32_t *block_table, int32_t block_table_stride,
                                          const int32_t *seq_lens, void *out, int32_t batch,
                                          int32_t num_q_heads, int32_t num_kv_heads,
                                          int32_t head_dim, int32_t page_size, int64_t num_pages,
                                          int32_t max_splits, int32_t min_pages_per_split,
                                          float softmax_scale, void *stream) {
  const char *what = "paged_decode_static";
  LITEKV_REQUIRE(batch >= 0 && num_q_heads > 0 && head_dim > 0 && max_splits >= 1 &&
                     max_splits <= 65535,
                 "%s: batch %d, num_q_heads %d, head_dim %d or max_splits %d out of range", what,
                 batch, num_q_heads, head_dim, max_splits);
  // the product is formed in 64 bits from values below 2^16 (batch, heads, splits are checked
  // again by the shared validation) or small (head_dim)
  LITEKV_REQUIRE(batch <= 65535 && num_q_heads <= 65535 && head_dim <= 1024,
                 "%s: batch %d, num_q_heads %d or head_dim %d out of range", what, batch,
                 num_q_heads, head_dim);
  const size_t need = litekv::splits_workspace_bytes(batch, num_q_heads, head_dim, max_splits);
  LITEKV_REQUIRE(need <= (size_t)LITEKV_STATIC_SCRATCH_BYTES,
                 "%s: batch %d x %d query heads x %d splits needs %zu bytes of partial results, the "
                 "built-in scratch holds %zu; use litekv_paged_decode with a workspace",
                 what, batch, num_q_heads, max_splits, need, (size_t)LITEKV_STATIC_SCRATCH_BYTES);
  // Every call resolves the array's address on its device, also one with batch 0: that is the
  // warm-up a caller makes before it starts capturing.
  void *ws = nullptr;
  int dev = 0;
  int rc = litekv::static_scratch(what, static_cast<hipStream_t>(stream), &ws, &dev);
  if (rc != LITEKV_OK) return rc;
  if (litekv::g_scratch_busy[dev].exchange(true, std::memory_order_acquire)) {
    return litekv::fail(LITEKV_ERR_INVALID_ARGUMENT,
                        "%s: another thread is inside this call on device %d; calls that share the "
                        "built-in scratch must not overlap",
                        what, dev);
  }
  litekv::DecodeArgs a{q, q_batch_stride, kv_pool, block_table, block_table_stride, seq_lens, out,
                       need > 0 ? ws : nullptr, need, batch, num_q_heads, num_kv_heads, head_dim,
                       page_size, num_pages, softmax_scale, stream};
  rc = litekv::launch_split(a, max_splits, min_pages_per_split);
  if (rc == LITEKV_OK) rc = litekv::launch_merge(a, max_splits, min_pages_per_split);
  litekv::g_scratch_busy[dev].store(false, std::memory_order_release);
  return rc;
}

#endif  // LITEKV_HD == 128

#if LITEKV_HD == 64
// What the head dim 128 build, which owns the C ABI, calls for head_dim == 64 (see common.h).
namespace litekv {
int hd64_split(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split,
               const float *scales, int format) {
  return launch_split(a, max_splits, min_pages_per_split, scales, format);
}
int hd64_merge(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split) {
  return launch_merge(a, max_splits, min_pages_per_split);
}
int hd64_balanced(const char *what, const void *q, int64_t q_batch_stride, void *kv_pool,
                  const float *scales, const int32_t *block_table, int32_t shared_pages,
                  const int32_t *seq_lens, void *plan, size_t plan_bytes,
                  const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride,
                  void *out, void *workspace, size_t workspace_bytes, int32_t batch,
                  int32_t num_q_heads, int32_t num_kv_heads, int32_t page_size, int64_t num_pages,
                  int32_t block_table_stride, int32_t chunks, float softmax_scale, void *stream,
                  int format) {
  return launch_balanced(what, q, q_batch_stride, kv_pool, scales, block_table, seq_lens, plan,
                         plan_bytes, k_new, v_new, k_new_stride, v_new_stride, out, workspace,
                         workspace_bytes, batch, num_q_heads, num_kv_heads, kHD, page_size, num_pages,
                         block_table_stride, chunks, shared_pages, softmax_scale, stream, format);
}
}  // namespace litekv
#endif  // LITEKV_HD == 64
