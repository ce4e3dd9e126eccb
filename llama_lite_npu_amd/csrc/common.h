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

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Turns the status of the launch just issued into an ABI status.
int check_launch(const char *what);

#define LITEKV_REQUIRE(cond, ...)                                         \
  do {                                                                    \
    if (!(cond)) return ::litekv::fail(LITEKV_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

// Most key slices the shared-prefix kernel may cut the prefix into (bounds its workspace).
constexpr int kMaxPrefixSplits = 8;

// Attention of every (sequence, query head) of a decode step over the first `shared_pages`
// pages of block-table row 0 (which all sequences share), as normalised fp32 partial rows
// part_o[split][batch][Hq][128] and log-sum-exps part_lse[split][batch][Hq]; *splits_out
// receives the number of key slices written. `fp8_scales` (K heads, then V heads) marks an fp8 pool.
// Defined beside the prefill kernel it reuses.
int launch_shared_prefix(const void *q, int64_t q_batch_stride, const void *kv_pool,
                         const float *fp8_scales,
                         const int32_t *block_table, int32_t batch, int32_t num_q_heads,
                         int32_t num_kv_heads, int64_t num_pages, int32_t shared_pages,
                         int32_t page_shift, float *part_o, float *part_lse, float softmax_scale,
                         hipStream_t stream, int *splits_out, int format);

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
