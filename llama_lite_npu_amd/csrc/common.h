// Shared declarations of liblitekv: vector types, MFMA fragment helpers,
// host-side argument checks and the thread-local error string.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/litekv.h"
#include "../../include/litekv_profile.h"

namespace litekv {

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));

constexpr int kHeadDim = 128;   // elements per head row (256 bytes of fp16)
constexpr int kPageSize = 16;   // tokens per page
constexpr int kWave = 64;       // lanes per wavefront on CDNA

// ---- host side -----------------------------------------------------------

// Records `msg` as this thread's last error and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// log2(page_size / 16) for the page sizes the kernels take (16, 32, 64, 128, 256 tokens: the
// reference documents "typically 16-256", lite_llama/executor/paged_attention.py:27), or -1. The
// attention kernels keep their 16-token page step and walk a larger page as 2 .. 16 consecutive
// 16-token pieces.
inline int page_shift_of(int32_t page_size) {
  for (int shift = 0; shift <= 4; ++shift) {
    if (page_size == (16 << shift)) return shift;
  }
  return -1;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Turns the status of the launch just issued into an ABI status.
int check_launch(const char *what);

#define LITEKV_REQUIRE(cond, ...)                                         \
  do {                                                                    \
    if (!(cond)) return ::litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

// Query heads per kv head the kernels take. The decode kernels hold the query heads of a kv head
// in the 16 columns of an MFMA tile; a larger group is served as `head_slices(group)` slices of
// the kv head, each a wavefront of its own with up to 16 of the group's query heads (the
// reference's grid is per query head with no bound, lite_llama/kernels/flashdecoding.py:44,
// 170-175). K/V of such a head is then read once per slice.
constexpr int kMaxGroup = 64;
__host__ __device__ __forceinline__ int head_slices(int group) { return (group + 15) / 16; }
struct HeadSlice {
  int kv_head;   // whose K/V rows and scales the slice reads
  int q_head0;   // first query head of the slice
  int q_heads;   // query heads in the slice (columns in use)
};
// Slice `hv` of the launch's kv_heads * slices slices (slices of one kv head are neighbours).
__host__ __device__ __forceinline__ HeadSlice head_slice(int hv, int slices, int group) {
  if (slices == 1) return HeadSlice{hv, hv * group, group};  // the usual case, without the divisions
  const int kv = hv / slices, sub = hv - kv * slices;
  const int per = (group + slices - 1) / slices;
  const int left = group - sub * per;
  return HeadSlice{kv, kv * group + sub * per, left < per ? left : per};
}

// Most key slices the shared-prefix kernel may cut the prefix into (bounds its workspace).
constexpr int kMaxPrefixSplits = 8;

// ---- the plan of a balanced decode step (made by decode_plan_kernel in paged_decode.hip) -------
// Plan buffer (int32 words): meta[kPlanMeta]; per sequence (first chunk, number of chunks it
// spans); per sequence the position of its first 16-token page on the line; the chunk entries.
constexpr int kPlanMeta = 16;      // int32 words of plan meta data
constexpr int kEntryHeader = 8;    // int32 words of an entry before its page ids
// plan meta words
constexpr int kMetaTotal = 0, kMetaChunkPages = 1, kMetaChunks = 2, kMetaBatch = 3,
              kMetaEntryStride = 4, kMetaKvHeads = 5, kMetaSkip = 6;

__host__ __device__ __forceinline__ int round_up(int x, int m) { return (x + m - 1) / m * m; }
__host__ __device__ __forceinline__ int plan_seq_info_offset() { return kPlanMeta; }
__host__ __device__ __forceinline__ int plan_seq_before_offset(int batch) {
  return kPlanMeta + round_up(2 * batch, 4);
}
__host__ __device__ __forceinline__ int plan_entries_offset(int batch) {
  return plan_seq_before_offset(batch) + round_up(batch, 4);
}

// The cut of a line of `total` pages into `chunks` pieces whose sizes differ by at most one page:
// the first `rem` chunks hold quot + 1 pages, the others quot (none when quot == 0).
struct LineCut {
  int quot, rem, big_end;  // big_end: pages covered by the larger chunks
  __host__ __device__ LineCut(int total, int chunks)
      : quot(total / chunks), rem(total - (total / chunks) * chunks), big_end(0) {
    big_end = rem * (quot + 1);
  }
  __host__ __device__ int chunk_start(int c) const { return c * quot + (c < rem ? c : rem); }
  __host__ __device__ int chunk_of(int f) const {
    if (f < big_end) return f / (quot + 1);
    return quot > 0 ? rem + (f - big_end) / quot : rem;
  }
};

// One decode call, as the launchers of paged_decode.hip take it.
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
  float softmax_scale;
  void *stream;
  // the step's new rows [B][Hkv][D] for the append fused into the splits schedule (or null)
  const void *k_new = nullptr;
  const void *v_new = nullptr;
  int64_t k_new_stride = 0, v_new_stride = 0;
};

// A paged prefill whose blocks are cut into key slices (see kPagedPrefillSplit in prefill_tile.h):
// how many, the workspace for the slices' partial rows, and the query rows of the launch.
struct PrefillKeySplit {
  int32_t key_slices = 1;   // 1: no split, nothing else is read
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  int64_t num_tokens = 0;   // query rows of the launch (cu_q_lens[batch])
};
constexpr int kMaxPrefillKeySlices = 8;

// The launchers of the head dim 64 build of paged_prefill.hip (paged_prefill_hd64.hip).
int hd64_paged_prefill(const char *what, const void *q, int64_t q_token_stride, const void *kv_pool,
                       const float *kv_scales, int format, const int32_t *block_table,
                       int32_t block_table_stride,
                       const int32_t *cu_q_lens, const int32_t *context_lens, void *out,
                       int64_t out_token_stride, int32_t batch, int32_t num_q_heads,
                       int32_t num_kv_heads, int32_t page_size, int64_t num_pages,
                       int32_t max_q_len, float softmax_scale, void *stream,
                       const PrefillKeySplit &split);
int32_t hd64_prefill_key_slices(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                int32_t max_q_len, int64_t max_kv_len);
int hd64_varlen_prefill(const void *q, int64_t q_token_stride, const void *k, int64_t k_token_stride,
                        const void *v, int64_t v_token_stride, const int32_t *seq_starts,
                        const int32_t *seq_lens, void *out, int64_t out_token_stride, int32_t batch,
                        int32_t num_q_heads, int32_t num_kv_heads, int32_t max_seq_len,
                        int64_t num_tokens, float softmax_scale, void *stream);

// The launchers of the head dim 64 build of paged_decode.hip (paged_decode_hd64.hip), to which the
// head dim 128 build, which owns the C ABI, hands calls with head_dim == 64. `scales` marks a pool
// of 8-bit codes of format `format` (kv_fp8.h).
int hd64_split(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split,
               const float *scales, int format);
int hd64_merge(const DecodeArgs &a, int32_t max_splits, int32_t min_pages_per_split);
int hd64_balanced(const char *what, const void *q, int64_t q_batch_stride, void *kv_pool,
                  const float *scales, const int32_t *block_table, int32_t shared_pages,
                  const int32_t *seq_lens, void *plan, size_t plan_bytes,
                  const void *k_new, const void *v_new, int64_t k_new_stride, int64_t v_new_stride,
                  void *out, void *workspace, size_t workspace_bytes, int32_t batch,
                  int32_t num_q_heads, int32_t num_kv_heads, int32_t page_size, int64_t num_pages,
                  int32_t block_table_stride, int32_t chunks, float softmax_scale, void *stream,
                  int format);

// Attention for the head dims the tuned kernels (128) do not take: 32, 64 and 256
// (generic_attention.hip). A launch is a decode step (seq_lens), a paged prefill (cu_q_lens,
// context_lens) or a packed prefill (kv_pool null; k, v, seq_starts, q_lens); `rows_per_seq` is
// 1 for decode and the longest prompt or chunk otherwise. `format` is the pool's storage format
// (kv_fp8.h); k_new / v_new fuse a decode step's append.
struct GenericLaunch {
  const void *q = nullptr;
  int64_t q_row_stride = 0;
  void *out = nullptr;
  int64_t out_row_stride = 0;
  void *kv_pool = nullptr;
  const float *scales = nullptr;
  int format = 0;
  const int32_t *block_table = nullptr;  // or, for a balanced decode step, its plan:
  const int32_t *plan = nullptr;
  int32_t bt_stride = 0;
  int32_t page_size = 16;
  int64_t num_pages = 0;
  const void *k = nullptr, *v = nullptr;
  int64_t k_stride = 0, v_stride = 0;
  const int32_t *seq_starts = nullptr;
  const int32_t *seq_lens = nullptr;
  const int32_t *cu_q_lens = nullptr;
  const int32_t *q_lens = nullptr;
  const int32_t *context_lens = nullptr;
  const void *k_new = nullptr, *v_new = nullptr;
  int64_t k_new_stride = 0, v_new_stride = 0;
  int32_t batch = 0, rows_per_seq = 1;
  int32_t num_q_heads = 0, num_kv_heads = 0, head_dim = 0;
  float softmax_scale = 1.0f;
  void *stream = nullptr;
};
bool generic_head_dim(int32_t head_dim);
int launch_generic_attention(const char *what, const GenericLaunch &a);

// ---- device side ---------------------------------------------------------

// 2^x on the transcendental unit (v_exp_f32); exp2(-inf) == 0.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Value held by lane (lane ^ mask) of the same wavefront.
__device__ __forceinline__ float xor_lane(float v, int mask) { return __shfl_xor(v, mask, kWave); }

// Maximum over the four lanes l, l^16, l^32, l^48 (the lane groups that share a column of an
// MFMA accumulator). v_permlane16_swap exchanges the odd 16-lane rows of its first operand with
// the even rows of its second, v_permlane32_swap the upper half of the first with the lower half
// of the second; fed the same value twice, the two results hold each lane's own value and its
// partner's, so their maximum is the pairwise maximum: two vector ALU instructions per step
// instead of a round trip through the LDS crossbar. Written as asm: the compiler's builtin for
// these instructions hands back the first result in both elements of its return value, which
// turns the maximum into a broadcast of lane group 0. The s_nop covers the wait states between a
// vector ALU write and a permlane read of the same register, which nobody inserts around asm.
__device__ __forceinline__ float max_over_lane_groups(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  a = __builtin_fmaxf(a, b);
  b = a;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return __builtin_fmaxf(a, b);
}

// D(16x16) += A(16x32) * B(32x16), fp16 inputs, fp32 accumulate.
// Lane l supplies A[l % 16][8*(l/16) .. +7] and B[8*(l/16) .. +7][l % 16];
// it receives D[4*(l/16) + i][l % 16] in element i.
__device__ __forceinline__ float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// D(16x16) += A(16x16) * B(16x16): lane l supplies A[l % 16][4*(l/16) .. +3] and
// B[4*(l/16) .. +3][l % 16]; D as above.
__device__ __forceinline__ float4_t mfma_16x16x16(half4_t a, half4_t b, float4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
}

}  // namespace litekv
