// Varlen causal FlashAttention-2 prefill for gfx950, over paged KV (block table) or over packed
// contiguous K/V (reference: lite_llama/kernels/flashattention2_nopad.py:9-166 and
// paged_chunk_flashattention.py:12-222).
//
// A workgroup of 4 wavefronts owns 128 score columns: up to 8 query heads of one KV head (the
// GQA group) times 16 * row_tiles query rows, 32 columns per wavefront. It walks the keys the
// block may see in tiles of 64 (two halves of 32 for the softmax). Per tile and wavefront:
//
//   S^T[key][col]  = K_tile[64 x 128] . Q^T[128 x 32]         32 x MFMA 16x16x32
//   causal mask, online softmax per column (fp32, exp2 domain, lazy rescale)
//   O^T[d][col]   += V_tile^T[128 x 64] . P^T[64 x 32]         32 x MFMA 16x16x32
//   l[col]        += 1^T . P^T                                   4 x MFMA 16x16x32
//
// Both products are computed transposed so that the accumulator layout of S^T (lane = column,
// 4 consecutive keys per lane group) is the B-operand layout of the second product: P stays in
// its lane, cast to fp16 like the reference's `p.to(v.dtype)` (flashattention2_nopad.py:150).
// The k index of one second-product MFMA runs over (keys 4g..4g+3 of a 16-key tile, then the
// same of the next tile) for lane group g, which is what two S^T accumulator tiles hold and what
// two transposing LDS reads of V deliver. The softmax denominator is one more MFMA against a
// tile of ones, which also reduces it across lane groups.
//
// K/V tiles go from HBM straight into LDS (global_load_lds_dwordx4, no registers in between),
// double buffered: the loads of tile t+1 are in flight while tile t is consumed, and one
// barrier per tile orders them. The direct load writes 64 lanes x 16 bytes contiguously, so
// rows are unpadded (256 bytes) and the 16-byte chunks of a row are XOR-swizzled instead: the
// lane that fills slot p of row r fetches chunk p ^ f(r) from memory. f differs for K (read
// back as 16-byte rows by 16 lanes of different rows) and V (read back transposed, 8 rows x
// 32 bytes at a time); both reads are then free of bank conflicts.
//
// In the fast tiles the score accumulators start from -m / c (m the running maximum of their
// column, c the softmax scale times log2 e) instead of zero, so the MFMA result times c is the
// exponent: a probability costs one multiply, one v_exp_f32 and half a packed conversion. q is not
// pre-multiplied by c: rounding q * c to fp16 would cost the scores 2^-12 of every channel's
// share. Whether the running maximum still holds is checked on the packed fp16
// probabilities (any above 2^8, or not finite, sends the sub-tile to general_tile), not by a
// column maximum over the fp32 scores.
//
// The accumulators are only ever rescaled in straight-line code (general_tile): a conditional
// rescale inside the key loop makes the compiler copy all 72 accumulator registers at the join
// on every tile. Tiles below the diagonal run in a loop of three straight-line blocks, each laid
// out as a pipeline with scheduling fences and group barriers: the eight K fragments of a
// half-tile are requested at once and each register is refilled with the other half's fragment as
// soon as its MFMA pair has issued; V fragments are requested a block ahead of their use; the
// exponentials of one half run beside the MFMAs of the other; the next tile's HBM -> LDS loads
// leave a quarter at a time between MFMA pairs instead of in one burst behind the barrier.
//
// q and the output move as whole 256-byte rows: q comes in through the direct HBM -> LDS load
// (into the half that tile 1 takes later) and is read back as fragments; the accumulators, which
// hold O^T (4 consecutive d of one row per lane), are transposed through LDS after the last tile
// and leave 4 rows per store instruction. Straight from registers, every q load and output store
// touched 16 rows with 64 / 32 bytes each.
//
// About 235 registers per lane leave two wavefronts per SIMD: two workgroups share a compute
// unit and drift apart, so one's softmax (vector ALU) overlaps the other's MFMAs and a
// finishing block's prologue/epilogue hides behind its neighbour. Grid: x = kv head (times the
// head split), y = row block (long blocks first), z = sequence; with 8 kv heads a head's blocks
// all land on one XCD and share its L2.
#pragma once

#include <type_traits>

#include "common.h"
#include "head_dim.h"
#include "kv_fp8.h"

// Wavefronts per workgroup of the fp16 prefill launches: 4, or 8 (twice the query rows on every
// staged K/V tile, one workgroup per compute unit instead of two; measured 2 to 5 % slower on
// ragged prompts of 128 to 2048 tokens, 1 % faster on 8192-token ones).
#ifndef LITEKV_PREFILL_WAVES
#define LITEKV_PREFILL_WAVES 4
#endif

namespace litekv {
inline namespace LITEKV_HD_NS {
namespace prefill_tile {

constexpr int kHD = LITEKV_HD;              // head dim of this build of the file
constexpr int kKSteps = kHD / 32;           // MFMA k steps of the first product
constexpr int kJTiles = kHD / 16;           // 16-row tiles of O^T; also K fragments per 32-key half
constexpr int kChunks = kHD / 8;            // 16-byte chunks of a staged row
constexpr int kRowsPerLoad = 64 / kChunks;  // rows one direct-load instruction (64 x 16 bytes) fills
constexpr int kLoadsPerWave = 16 / kRowsPerLoad;  // such instructions per wavefront, tile and operand

// XOR applied to the 16-byte chunk index of staged row r, for K (and q) and for V. A row of 256
// bytes covers all 64 banks, so consecutive rows must differ in the chunk; rows of 128 bytes
// alternate between the bank halves, so it is every second row that must.
__device__ __forceinline__ int k_swz(int r) { return kHD == 128 ? (r & 15) : ((r >> 1) & 7); }
__device__ __forceinline__ int v_swz(int r) { return kHD == 128 ? 2 * (r & 7) : 2 * ((r >> 1) & 3); }

constexpr float kLog2eP = 1.4426950408889634f;

// Where the keys of a sequence live.
struct PagedSource {
  const half_t *kv;             // pool [slots][2*Hkv][128], fp16 (or E4M3 codes, one byte each)
  const int32_t *block_table;   // [B][stride]
  int32_t bt_stride;
  int32_t num_kv_heads;
  int32_t num_pages;
  const float *scales;          // fp8 pool: value = code * scale, K heads then V heads
  int32_t page_shift;           // pages of 16 << page_shift tokens
};
// Shared-prefix decode (mode kSharedPrefix): the columns are (sequence, query head) pairs of one
// decode step, the keys are a slice of the pages every sequence starts with, and the result is
// a normalised fp32 partial row + log-sum-exp per column, for the decode merge.
// Prefill over key slices (mode kPagedPrefillSplit) writes the same kind of partial rows, one
// per (key slice, query row, head): `batch` then counts the query rows of the launch.
struct PrefixTask {
  float *part_o;            // [splits][batch][Hq][128]
  float *part_lse;          // [splits][batch][Hq]
  int64_t q_batch_stride;   // elements between the q rows of consecutive sequences
  int32_t batch;
  int32_t num_q_heads;
  int32_t prefix_keys;      // shared pages * 16
  int32_t keys_per_split;   // multiple of the key tile
};
struct PackedSource {
  const half_t *k;              // [T][Hkv][128]
  const half_t *v;
  int64_t k_stride, v_stride;   // elements per token
  const int32_t *seq_starts;    // [B]
};

constexpr int kKvTile = 64;
constexpr int kColTiles = 2;      // 16-column tiles per wavefront
constexpr int kTiledWaves = 4;    // wavefronts of a workgroup, unless the kernel is built for kWideWaves
constexpr int kWideWaves = 8;     // fp16 prefill only: twice the columns on every staged K/V tile
constexpr int kWgColTiles = kColTiles * kTiledWaves;
constexpr int kTileHalfs = kKvTile * kHD;  // one staged tile: 64 rows of 2 * kHD bytes

typedef __attribute__((address_space(3))) half_t lds_half_t;
typedef __attribute__((address_space(3))) half8_t lds_half8_t;
typedef __attribute__((address_space(3))) short4_t lds_short4_t;
typedef short short8_t __attribute__((ext_vector_type(8)));

// Plain maxima. This file is compiled with -fno-honor-nans, so the compiler does not wrap every
// operand in a NaN-quieting self-max and fuses pairs into v_max3_f32. (They must stay compiler
// instructions: an asm v_max3 reading an MFMA result gets none of the wait states that the
// compiler inserts between an MFMA and the first use of its result.)
__device__ __forceinline__ float vmax3(float a, float b, float c) {
  return __builtin_fmaxf(__builtin_fmaxf(a, b), c);
}
__device__ __forceinline__ float vmax2(float a, float b) { return __builtin_fmaxf(a, b); }
constexpr int kPagedPrefill = 0, kPackedPrefill = 1, kSharedPrefix = 2, kPagedPrefillFp8 = 3,
              kSharedPrefixFp8 = 4, kPagedPrefillInt8 = 5, kSharedPrefixInt8 = 6,
              kPagedPrefillSplit = 7, kPagedPrefillSplitFp8 = 8, kPagedPrefillSplitInt8 = 9;
// kPagedPrefillSplit: a launch with too few row blocks to fill the device (one request's chunk
// over a long history) cuts every block's keys into `key_slices` runs of tiles, one workgroup
// each; a slice leaves a normalised fp32 partial row + log-sum-exp per (query row, head), and a
// merge launch folds the slices of a row (prefill_split_merge_kernel in paged_prefill.hip).

// The body of the kernel, run by a workgroup of W wavefronts that stands at (block_x, block_y,
// block_z) of a grid block_y runs over grid_y values of; k_lds is the LDS byte address of its
// staging area (tile_lds_bytes<W>() bytes, 1 KiB aligned). A function, so that the decode step
// with a shared prefix can run it as one role of its launch (paged_decode.hip).
template <int W>
constexpr int tile_lds_bytes() { return (W == kWideWaves ? 6 : 4) * kTileHalfs * 2; }

template <int MODE, int W>
__device__ __forceinline__ void prefill_tile_body(
    const uint32_t k_lds, const int block_x, const int block_y, const int block_z, const int grid_y,
    const half_t *__restrict__ q, int64_t q_stride, half_t *__restrict__ out, int64_t out_stride,
    const PagedSource &paged, const PackedSource &packed, const PrefixTask &prefix,
    const int32_t *__restrict__ q_starts_or_cu, const int32_t *__restrict__ q_lens_or_null,
    const int32_t *__restrict__ context_lens, int32_t group, int32_t head_splits,
    int32_t heads_per_wg, int32_t row_tiles, float scale_log2, const int key_slice = 0,
    const int key_slices = 1) {
  constexpr bool PAGED = MODE != kPackedPrefill;
  // causal prefill over one slice of the block's keys
  constexpr bool KSPLIT = MODE == kPagedPrefillSplit || MODE == kPagedPrefillSplitFp8 ||
                          MODE == kPagedPrefillSplitInt8;
  // An fp8 pool cannot take the direct HBM -> LDS load: its codes go through registers, are
  // converted to fp16 (exactly) and written to LDS in the same swizzled layout, so everything
  // after the staging is shared. The K scale joins the softmax scale, the V scale the final
  // normalisation, as in the decode kernel.
  constexpr bool FP8 = MODE == kPagedPrefillFp8 || MODE == kSharedPrefixFp8 ||
                       MODE == kPagedPrefillInt8 || MODE == kSharedPrefixInt8 ||
                       MODE == kPagedPrefillSplitFp8 || MODE == kPagedPrefillSplitInt8;  // 8-bit codes
  constexpr int KV = (MODE == kPagedPrefillInt8 || MODE == kSharedPrefixInt8 ||
                      MODE == kPagedPrefillSplitInt8) ? kKvInt8 : kKvFp8;
  constexpr bool SHARED = MODE == kSharedPrefix || MODE == kSharedPrefixFp8 || MODE == kSharedPrefixInt8;
  // (rows of 64 codes staged by 8 wavefronts would leave a lane 8 codes, half a 16-byte load)
  static_assert(W == kTiledWaves || (W == kWideWaves && (!FP8 || kHD == 128)),
                "eight wavefronts: fp16 K/V, or 8-bit codes at head dim 128");
  // Rows of a 64-key tile one wavefront stages (a page, or half of one), and the direct-load
  // instructions that takes per operand.
  constexpr int kRowsPerWave = kKvTile / W;
  constexpr int kLoads = kRowsPerWave / kRowsPerLoad;
  // Two tiles of K, then two of V: tile t sits in half t % 2. Eight wavefronts have a third
  // region of the same size behind them: q of wavefronts 4..7, and room for the output rows.
  const uint32_t v_lds = k_lds + 4u * kTileHalfs;  // LDS byte addresses
  const uint32_t x_lds = v_lds + 4u * kTileHalfs;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int n = lane & 15;
  const int g = lane >> 4;
  const int h = block_x / head_splits;  // kv head
  const int head0 = (block_x - h * head_splits) * heads_per_wg;
  const int heads_here = (group - head0) < heads_per_wg ? (group - head0) : heads_per_wg;
  const int b = block_z;
  // q reaches the MFMA as the caller gave it: the products of fp16 q and K elements are exact and
  // summed in fp32, and the softmax scale (times log2 e, times the K scale of a pool of 8-bit
  // codes) multiplies the finished score in fp32 (k_mul). Folded into q instead, the product
  // would be rounded to fp16 once more: an error of 2^-12 of every channel's share of a score,
  // which rows with a few large channels of q and K (scores tens of log2 units apart) turn into
  // percent-level errors of their probabilities.
  float v_scale = 1.0f, k_mul = scale_log2;
  if constexpr (FP8) {
    k_mul *= paged.scales[h];
    v_scale = paged.scales[paged.num_kv_heads + h];
  }
  const float k_mul_inv = 1.0f / k_mul;

  // What the block works on: query rows m0.. of sequence b (prefill), or the column block
  // block_y of all (sequence, head) pairs against key slice block_z (shared prefix).
  //   kv_end  one past the last key the block may see      diag  last key every column sees
  //   tile0   first key tile (tiles are counted from it)   last_key  last key that exists
  int q_start = 0, q_len = 0, m0 = 0, ctx = 0, kv_end, diag, last_key;
  int tile0 = 0;
  if constexpr (SHARED) {
    const int key_begin = block_z * prefix.keys_per_split;
    if (key_begin >= prefix.prefix_keys) return;
    kv_end = key_begin + prefix.keys_per_split;
    kv_end = kv_end < prefix.prefix_keys ? kv_end : prefix.prefix_keys;
    diag = kv_end - 1;
    last_key = prefix.prefix_keys - 1;
    tile0 = key_begin / kKvTile;
  } else {
    if (PAGED) {
      q_start = q_starts_or_cu[b];
      q_len = q_starts_or_cu[b + 1] - q_start;
    } else {
      q_start = packed.seq_starts[b];
      q_len = q_lens_or_null[b];
    }
    const int block_rows = 16 * row_tiles;
    // Long blocks first, all heads of a row block next to each other.
    m0 = (grid_y - 1 - block_y) * block_rows;
    if (m0 >= q_len) return;
    ctx = (PAGED && context_lens) ? context_lens[b] : 0;
    const int rows = (q_len - m0) < block_rows ? (q_len - m0) : block_rows;
    kv_end = ctx + m0 + rows;
    diag = ctx + m0;
    last_key = ctx + q_len - 1;
    if constexpr (KSPLIT) {
      // The tiles every row of the block sees in full (`plain` of them) are shared out among the
      // slices; the last slice also takes the tiles at the diagonal, and starts no later than
      // the last plain tile, so that each of its rows sees at least one key.
      const int total = (kv_end + kKvTile - 1) / kKvTile;
      const int plain = (diag + 1) / kKvTile;
      const int last_start = plain > 0 ? plain - 1 : 0;
      const int per = (plain + key_slices - 1) / key_slices;
      int t_begin = key_slice * per;
      t_begin = t_begin < last_start ? t_begin : last_start;
      int t_end = (key_slice + 1) * per;
      t_end = key_slice == key_slices - 1 ? total : (t_end < last_start ? t_end : last_start);
      if (t_end <= t_begin) {
        // Nothing for this slice: its partial rows say so (log-sum-exp -inf, a row of zeros).
        for (int t = wave * kColTiles; t < wave * kColTiles + kColTiles; ++t) {
          const int head = t / row_tiles;
          const int row = m0 + (t - head * row_tiles) * 16 + n;
          if (head < heads_here && row < q_len) {
            const int64_t cell = ((int64_t)key_slice * prefix.batch + q_start + row) * prefix.num_q_heads +
                                 h * group + head0 + head;
            if (g == 0) prefix.part_lse[cell] = -INFINITY;
            float4_t *dst = (float4_t *)(prefix.part_o + cell * kHD) + g * (kHD / 16);
#pragma unroll
            for (int i = 0; i < kHD / 16; ++i) dst[i] = float4_t{0.f, 0.f, 0.f, 0.f};
          }
        }
        return;
      }
      tile0 = t_begin;
      kv_end = kv_end < t_end * kKvTile ? kv_end : t_end * kKvTile;
    }
  }
  const int n_tiles = (kv_end + kKvTile - 1) / kKvTile - tile0;

  // ---- staging addresses -------------------------------------------------------------------
  // Direct-load instruction i of wavefront w fills tile rows kRowsPerWave * w + 4i .. +3 (one
  // page per wavefront, or half of one): lane l writes slot l % 16 of row 4i + l / 16.
  const int r_loc = lane / kChunks;
  const int slot = lane % kChunks;
  const int sub = (kRowsPerWave * wave) & 15;   // first row of this wavefront's rows inside their page
  const uint32_t k_pitch = PAGED ? 2u * paged.num_kv_heads * kHD * (FP8 ? 1u : 2u)
                                 : (uint32_t)packed.k_stride * 2u;
  const uint32_t v_pitch = PAGED ? k_pitch : (uint32_t)packed.v_stride * 2u;
  // byte offsets from the page (paged) or from the wavefront's first row (packed)
  uint32_t koff[kLoadsPerWave], voff[kLoadsPerWave];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int rip = kRowsPerLoad * i + r_loc;   // row among this wavefront's rows
    const int ck = slot ^ k_swz(sub + rip);      // the swizzle goes by the row of the tile
    const int cv = slot ^ v_swz(sub + rip);
    const int src_row = (PAGED ? sub : 0) + rip;
    koff[i] = src_row * k_pitch + (uint32_t)(h * kHD + 8 * ck) * 2u;
    voff[i] = src_row * v_pitch +
              (uint32_t)(((PAGED ? paged.num_kv_heads : 0) + h) * kHD + 8 * cv) * 2u;
  }
  const int32_t *table =
      PAGED ? paged.block_table + (SHARED ? 0 : (int64_t)b * paged.bt_stride) : nullptr;
  const int last_page = last_key >> 4;
  // The kernel works on 16-token pages: page j of them is part j % (1 << page_shift) of the
  // sequence's page j >> page_shift, whose tokens are contiguous in the pool.
  auto page_of = [&](int pidx) {
    int at = pidx >> paged.page_shift;
    at = at < paged.bt_stride ? at : paged.bt_stride - 1;  // a length beyond the row re-reads its last entry
    int pid = table[at];
    pid = pid < 0 ? 0 : (pid >= paged.num_pages ? paged.num_pages - 1 : pid);
    return (pid << paged.page_shift) + (pidx & ((1 << paged.page_shift) - 1));
  };

  // Starts the loads of tile kt into its LDS half. The instruction is written as asm so that the
  // compiler does not make later LDS reads of the *other* half wait for it; the wait is the
  // explicit vmcnt(0) before the barrier that publishes the tile.
  // 8-bit pools: a row's codes are shared out among kLanesPerRow lanes, kRawVecs 16-byte vectors
  // of codes per lane and operand
  constexpr int kLanesPerRow = kWave / kRowsPerWave;
  constexpr int kCodesPerLane = kHD / kLanesPerRow;
  constexpr int kRawVecs = FP8 ? kCodesPerLane / 16 : 1;
  uint4_t raw_k[kRawVecs], raw_v[kRawVecs];  // this lane's codes of K and of V of the tile requested last
  auto issue_tile = [&](int kt) {
    const int row0 = (tile0 + kt) * kKvTile + kRowsPerWave * wave;  // first key of this wavefront's rows
    if constexpr (FP8) {
      // lane l: row l / kLanesPerRow of the wavefront's rows, kCodesPerLane codes of the head's row
      int pidx = (tile0 + kt) * 4 + (kRowsPerWave * wave) / 16;
      pidx = pidx < last_page ? pidx : last_page;
      const int pid = page_of(pidx);
      int tok = row0 + lane / kLanesPerRow;
      tok = tok < last_key ? tok : last_key;  // rows past the last key re-read it
      const int src_row = tok - pidx * kPageSize;
      const uint8_t *base = (const uint8_t *)paged.kv +
                            ((int64_t)pid * kPageSize + src_row) * (int64_t)k_pitch +
                            kCodesPerLane * (lane % kLanesPerRow);
      const uint8_t *kp = base + h * kHD;
      const uint8_t *vp = base + (paged.num_kv_heads + h) * kHD;
#pragma unroll
      for (int i = 0; i < kRawVecs; ++i) {
        raw_k[i] = *(const uint4_t *)(kp + 16 * i);
        raw_v[i] = *(const uint4_t *)(vp + 16 * i);
      }
      return;
    }
    const char *kbase, *vbase;
    int src0;  // key index the bases point at
    if (PAGED) {
      int pidx = (tile0 + kt) * 4 + (kRowsPerWave * wave) / 16;
      pidx = pidx < last_page ? pidx : last_page;
      const int pid = page_of(pidx);
      kbase = (const char *)paged.kv + (int64_t)pid * ((int64_t)kPageSize * k_pitch);
      vbase = kbase;
      src0 = pidx * kPageSize;
    } else {
      const int first = row0 < last_key ? row0 : last_key;
      kbase = (const char *)packed.k + (int64_t)(q_start + first) * k_pitch;
      vbase = (const char *)packed.v + (int64_t)(q_start + first) * v_pitch;
      src0 = first;
    }
    const uint32_t dst = (uint32_t)((kt & 1) * kTileHalfs + kRowsPerWave * wave * kHD) * 2u;
    auto load_rows = [&](uint32_t i, uint32_t ko, uint32_t vo) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(k_lds + dst + 1024u * i), "v"(ko), "s"(kbase)
                   : "memory", "m0");
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(v_lds + dst + 1024u * i), "v"(vo), "s"(vbase)
                   : "memory", "m0");
    };
    if (row0 + kRowsPerWave - 1 <= last_key) {
#pragma unroll
      for (int i = 0; i < kLoads; ++i) load_rows(i, koff[i], voff[i]);
    } else {
      // Only in the last tile of a sequence. Rows past the last key re-read it: finite values
      // that zero probabilities multiply.
      const int off0 = PAGED ? row0 - sub : row0;  // the key the offsets count from
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        const int rip = kRowsPerLoad * i + r_loc;
        int tok = row0 + rip;
        tok = tok < last_key ? tok : last_key;
        const uint32_t back = (uint32_t)(row0 + rip - tok) - (uint32_t)(off0 - src0);
        // source row = offset row - back: inside the page / at the clamped packed row
        load_rows(i, koff[i] - back * k_pitch, voff[i] - back * v_pitch);
      }
    }
  };

  // q rows come in as whole 256-byte rows, 4 per direct-load instruction, into a region of the
  // LDS half that tile 1 will take (8 KiB per wavefront, private to it), swizzled like a K tile;
  // the fragments are read back from there. Requested before tile 0: vmcnt counts in order.
  uint32_t q_lds = 0;
  if constexpr (!SHARED) {
    q_lds = wave < 4 ? ((wave & 2) ? v_lds : k_lds) + (uint32_t)(kTileHalfs * 2 + (wave & 1) * (64 * kHD))
                     : x_lds + (uint32_t)((wave - 4) * (64 * kHD));
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
      const int t = wave * kColTiles + u;
      const int head = t / row_tiles;
      const int row0 = m0 + (t - head * row_tiles) * 16;
      const int hq = h * group + head0 + (head < heads_here ? head : 0);
      const int first = row0 < q_len ? row0 : q_len - 1;
      const char *base = (const char *)(q + (int64_t)(q_start + first) * q_stride + (int64_t)hq * kHD);
#pragma unroll
      for (int i = 0; i < kLoadsPerWave; ++i) {
        int rip = kRowsPerLoad * i + r_loc;
        const int chunk = slot ^ k_swz(rip);
        rip = first + rip < q_len ? rip : q_len - 1 - first;  // rows past the end re-read the last one
        const uint32_t off = (uint32_t)rip * (uint32_t)q_stride * 2u + 16u * (uint32_t)chunk;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(q_lds + (uint32_t)(32 * kHD) * u + 1024u * i), "v"(off), "s"(base)
                     : "memory", "m0");
      }
    }
  }
  issue_tile(0);

  // ---- this wavefront's columns: tile t = head (t / row_tiles), rows 16 * (t % row_tiles) ..
  half8_t qf[kColTiles][kKSteps];
  int q_pos[kColTiles];
  int out_row[kColTiles];   // packed row index, or -1
  int out_head[kColTiles];
#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    const int t = wave * kColTiles + u;
    bool ok;
    int hq;
    const half_t *qrow;
    if constexpr (SHARED) {
      const int col = block_y * (16 * kColTiles * W) + 16 * t + n;  // (sequence, head) pair
      ok = col < prefix.batch * group;
      const int seq = ok ? col / group : 0;
      hq = h * group + (ok ? col - seq * group : 0);
      q_pos[u] = kv_end - 1;
      out_row[u] = ok ? seq : -1;
      qrow = q + (int64_t)seq * prefix.q_batch_stride + (int64_t)hq * kHD + 8 * g;
    } else {
      const int head = t / row_tiles;
      const int row = m0 + (t - head * row_tiles) * 16 + n;
      ok = head < heads_here && row < q_len;
      hq = h * group + head0 + (head < heads_here ? head : 0);
      const int last = q_len - 1;
      q_pos[u] = ctx + (row < last ? row : last);
      out_row[u] = ok ? q_start + row : -1;
      qrow = q + (int64_t)(q_start + (ok ? row : 0)) * q_stride + (int64_t)hq * kHD + 8 * g;
    }
    out_head[u] = hq;
    if constexpr (!SHARED) continue;
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) {
      qf[u][kk] = ok ? *(const half8_t *)(qrow + 32 * kk) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  if constexpr (!SHARED) {
    // the loads of tile 0 (K and V) were requested after q's
    if constexpr (FP8) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kRawVecs));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kLoads));
    }
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) {
        qf[u][kk] = *(const lds_half8_t *)(uintptr_t)(
            q_lds + (uint32_t)(32 * kHD) * u + (uint32_t)(n * 2 * kHD + 16 * ((4 * kk + g) ^ k_swz(n))));
      }
    }
  }

  float4_t acc[kJTiles][kColTiles];
  float4_t dsum[kColTiles];
  float m_run[kColTiles];
  // Seed of the score accumulators in the fast tiles: -m_run (divided by k_mul), in all four
  // elements, so that the MFMA result is already the exponent.
  float4_t seed[kColTiles];
#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    m_run[u] = -INFINITY;
    seed[u] = float4_t{0.f, 0.f, 0.f, 0.f};
    dsum[u] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) acc[j][u] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  const half8_t ones = half8_t{1, 1, 1, 1, 1, 1, 1, 1};

  // Swizzled read addresses (LDS bytes) for the tile half in use; they flip between the halves
  // once per tile.
  // K, A operand of S^T: row 16m + n, chunk (4kk + g) ^ n.
  uint32_t k_addr[kKSteps];
#pragma unroll
  for (int kk = 0; kk < kKSteps; ++kk) {
    k_addr[kk] = k_lds + 2u * (uint32_t)(n * kHD + 8 * ((4 * kk + g) ^ k_swz(n)));
  }
  // V^T, A operand of O^T: row 32 s2 + 4g + n/4 (+16), halfs 16j + 4(n%4); chunk pair j ^ (r%8).
  const int v_row = 4 * g + (n >> 2);
  uint32_t v_addr[kJTiles];
#pragma unroll
  for (int j = 0; j < kJTiles; ++j) {
    v_addr[j] = v_lds + 2u * (uint32_t)(v_row * kHD + 8 * ((2 * j) ^ v_swz(v_row)) + 4 * (n & 3));
  }
  int flip = kTileHalfs * 2;  // bytes to the other half
  auto flip_halves = [&]() {
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) k_addr[kk] += flip;
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) v_addr[j] += flip;
    flip = -flip;
  };

  float4_t st[2][kColTiles];
  half8_t pk[kColTiles];

  // S^T of 32 keys (rows 32 s2 .. +31 of the staged K tile) against this wavefront's columns.
  auto scores_into = [&](float4_t (&st)[2][kColTiles], int s2, auto seeded_tag) {
    constexpr bool SEEDED = decltype(seeded_tag)::value;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) st[m][u] = SEEDED ? seed[u] : float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) {
        const half8_t a =
            *(const lds_half8_t *)(uintptr_t)(k_addr[kk] + 2u * (32 * s2 + 16 * m) * kHD);
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) st[m][u] = mfma_16x16x32(a, qf[u][kk], st[m][u]);
      }
    }
  };
  // -inf on the keys column u may not see; key0 = first key of the sub-tile.
  auto mask_sub = [&](int u, int key0) {
    const int lim = q_pos[u] - key0 - 4 * g;  // key offset 16m + i is visible iff <= lim
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (16 * m + i > lim) st[m][u][i] = -INFINITY;
      }
    }
  };
  // Column maxima of `st`, in scaled (log2) units.
  auto column_max_of = [&](const float4_t (&st)[2][kColTiles], int u) {
    float mx = vmax3(st[0][u][0], st[0][u][1], st[0][u][2]);
    mx = vmax3(mx, st[0][u][3], st[1][u][0]);
    mx = vmax3(mx, st[1][u][1], st[1][u][2]);
    mx = vmax2(mx, st[1][u][3]);
    return max_over_lane_groups(mx) * k_mul;  // k_mul > 0: max and scaling commute
  };
  // p = 2^(s * scale - m), cast to fp16, in B-operand order.
  typedef float float2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  // General path: p = 2^(s * k_mul - m) from unseeded scores.
  auto exponentials_of = [&](const float4_t (&st)[2][kColTiles], half8_t (&pk)[kColTiles], int u) {
    const float neg_m = -m_run[u];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int i = 0; i < 4; i += 2) {
        const float2_t p = float2_t{fast_exp2(__builtin_fmaf(st[m][u][i], k_mul, neg_m)),
                                    fast_exp2(__builtin_fmaf(st[m][u][i + 1], k_mul, neg_m))};
        const half2_t ph = __builtin_convertvector(p, half2_t);
        pk[u][4 * m + i] = ph[0];
        pk[u][4 * m + i + 1] = ph[1];
      }
    }
  };
  // Fast path: the scores were seeded with -m / k_mul, so they are the exponents up to that factor.
  auto exponentials_seeded = [&](const float4_t (&st)[2][kColTiles], half8_t (&pk)[kColTiles], int u) {
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int i = 0; i < 4; i += 2) {
        const float2_t p = float2_t{fast_exp2(st[m][u][i] * k_mul), fast_exp2(st[m][u][i + 1] * k_mul)};
        const half2_t ph = __builtin_convertvector(p, half2_t);
        pk[u][4 * m + i] = ph[0];
        pk[u][4 * m + i + 1] = ph[1];
      }
    }
  };
  // True if any probability of the sub-tile exceeds 2^8 (or is not finite): the running maximum
  // is then too low for these keys and the sub-tile has to be redone with a rescale. Probabilities
  // are non-negative, so their fp16 bit patterns order like their values.
  auto overflowed = [&](const half8_t (&pk)[kColTiles]) -> bool {
    typedef _Float16 half8v __attribute__((ext_vector_type(8)));
    const half8v mx8 = __builtin_elementwise_max(pk[0], pk[1]);
    typedef _Float16 half4v __attribute__((ext_vector_type(4)));
    const half4v lo4 = __builtin_shufflevector(mx8, mx8, 0, 1, 2, 3);
    const half4v hi4 = __builtin_shufflevector(mx8, mx8, 4, 5, 6, 7);
    const half4v mx4 = __builtin_elementwise_max(lo4, hi4);
    const half2_t mx2 = __builtin_elementwise_max(__builtin_shufflevector(mx4, mx4, 0, 1),
                                                  __builtin_shufflevector(mx4, mx4, 2, 3));
    const uint32_t bits = __builtin_bit_cast(uint32_t, mx2);
    const uint32_t top = (bits & 0xffffu) > (bits >> 16) ? (bits & 0xffffu) : (bits >> 16);
    return __builtin_amdgcn_ballot_w64(top > 0x5C00u) != 0;  // 0x5C00 = 256.0
  };
  // O^T += V^T . P^T,  l += 1^T . P^T for keys 32 s2 .. +31 of the staged V tile.
  auto accumulate_with = [&](const half8_t (&pk)[kColTiles], int s2) {
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) dsum[u] = mfma_16x16x32(ones, pk[u], dsum[u]);
#pragma unroll
    for (int j = 0; j < kJTiles; ++j) {
      const uint32_t at = v_addr[j] + 2u * 32 * s2 * kHD;
      const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t *)(uintptr_t)at);
      const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_short4_t *)(uintptr_t)(at + 2u * 16 * kHD));
      const short8_t both = short8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      const half8_t a = __builtin_bit_cast(half8_t, both);
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) acc[j][u] = mfma_16x16x32(a, pk[u], acc[j][u]);
    }
  };
  // V^T fragment j (A operand: d rows 16j.., keys 32 s2 + {4g..4g+3, 16+4g..}) of the staged tile.
  auto load_vfrag = [&](int j, int s2) -> half8_t {
    const uint32_t at = v_addr[j] + 2u * 32 * s2 * kHD;
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t *)(uintptr_t)at);
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (lds_short4_t *)(uintptr_t)(at + 2u * 16 * kHD));
    const short8_t both = short8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(half8_t, both);
  };
  auto scores_sub = [&](int s2) { scores_into(st, s2, std::false_type{}); };
  auto column_max = [&](int u) { return column_max_of(st, u); };
  auto exponentials = [&](int u) { exponentials_of(st, pk, u); };
  auto accumulate_sub = [&](int s2) { accumulate_with(pk, s2); };
  float4_t st1[2][kColTiles];  // scores of the second half of a fast tile
  half8_t pk1[kColTiles];

  // Publishes tile kt (already requested) and requests tile kt + 1 into the other half.
  auto sync_and_prefetch = [&](int kt, bool issue_next = true) {
    if constexpr (FP8) {
      // The codes of tile kt (requested a tile ago) become fp16 rows in its LDS half: 16-byte
      // chunk c of row r goes where the direct load of the fp16 path would have put it.
      const int r = sub + lane / kLanesPerRow;   // row inside the page: what the swizzle goes by
      const uint32_t row_at =
          (uint32_t)((kt & 1) * kTileHalfs + (kRowsPerWave * wave + lane / kLanesPerRow) * kHD) * 2u;
#pragma unroll
      for (int j = 0; j < kCodesPerLane / 8; ++j) {
        const int chunk = (kCodesPerLane / 8) * (lane % kLanesPerRow) + j;
        const uint4_t ck = raw_k[j >> 1], cv = raw_v[j >> 1];
        const half8_t kh = codes_to_half<KV>((j & 1) ? uint2_t{ck[2], ck[3]} : uint2_t{ck[0], ck[1]});
        const half8_t vh = codes_to_half<KV>((j & 1) ? uint2_t{cv[2], cv[3]} : uint2_t{cv[0], cv[1]});
        *(lds_half8_t *)(uintptr_t)(k_lds + row_at + 16u * (uint32_t)(chunk ^ k_swz(r))) = kh;
        *(lds_half8_t *)(uintptr_t)(v_lds + row_at + 16u * (uint32_t)(chunk ^ v_swz(r))) = vh;
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's part of tile kt is in LDS
    __syncthreads();                     // ... and everyone's; everyone is done with tile kt-1
    if (issue_next && kt + 1 < n_tiles) issue_tile(kt + 1);
  };
  // The same loads for a tile that lies wholly inside the sequence's keys, split in two steps so
  // that they can ride between MFMAs instead of leaving in one burst behind the barrier:
  // tile_bases() reads the page id (scalar), issue_rows(i) requests row group i of K and of V.
  const char *next_kbase = nullptr, *next_vbase = nullptr;
  uint32_t next_dst = 0;
  // The page ids of a tile's four pages, one per lane (lane l: page l % 4 of the tile), requested a
  // whole tile before tile_bases() needs them: as a scalar value read on the spot the id cost
  // every tile a round trip to memory in front of its first MFMA.
  auto page_ids_of_tile = [&](int kt) -> int {
    if constexpr (!PAGED) return 0;
    int pidx = (tile0 + kt) * 4 + (lane & 3);
    pidx = pidx < last_page ? pidx : last_page;
    return page_of(pidx);
  };
  int ids_ahead = 0;  // of the tile after the one being staged
  auto tile_bases = [&](int kt) {
    const int row0 = (tile0 + kt) * kKvTile + kRowsPerWave * wave;
    if (PAGED) {
      const int pid = __builtin_amdgcn_readlane(ids_ahead, (kRowsPerWave * wave) / 16);
      next_kbase = (const char *)paged.kv + (int64_t)pid * ((int64_t)kPageSize * k_pitch);
      next_vbase = next_kbase;
    } else {
      next_kbase = (const char *)packed.k + (int64_t)(q_start + row0) * k_pitch;
      next_vbase = (const char *)packed.v + (int64_t)(q_start + row0) * v_pitch;
    }
    next_dst = (uint32_t)((kt & 1) * kTileHalfs + kRowsPerWave * wave * kHD) * 2u;
  };
  auto issue_rows = [&](int i) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(k_lds + next_dst + 1024u * i), "v"(koff[i]), "s"(next_kbase)
                 : "memory", "m0");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(v_lds + next_dst + 1024u * i), "v"(voff[i]), "s"(next_vbase)
                 : "memory", "m0");
  };

  // General sub-tiles of tile kt from `first` on: causal mask, and the accumulators are rescaled
  // to the new running maximum unconditionally (straight-line code: a branch around the
  // rescale makes the compiler copy every accumulator at the join, on every tile). Used for the
  // first tile and wherever the fast loop saw a maximum grow.
  auto general_tile = [&](int kt, int first) {
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const int key0 = (tile0 + kt) * kKvTile + 32 * s2;
      if (s2 < first) continue;
      if (key0 >= kv_end) break;  // nothing visible in the second half
      scores_sub(s2);
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) {
        mask_sub(u, key0);
        const float m_new = vmax2(m_run[u], column_max(u));
        const float alpha = fast_exp2(m_run[u] - m_new);
        m_run[u] = m_new;
        const float sd = -m_new * k_mul_inv;
        seed[u] = float4_t{sd, sd, sd, sd};
        dsum[u] *= alpha;
#pragma unroll
        for (int j = 0; j < kJTiles; ++j) acc[j][u] *= alpha;
        exponentials(u);
      }
      accumulate_sub(s2);
    }
  };

  // Fast tiles kt .. kt_end-1: they proceed only while no column maximum exceeds the running one
  // by more than 8 (p stays below 2^8: far inside fp16 and fp32 range), so the accumulators are
  // touched by nothing but MFMAs. Returns 0 at kt_end, else 1 + the sub-tile of tile kt that
  // has to be redone with a rescale.
  int kt = 1;
  auto fast_tiles = [&](int kt_end, auto masked_tag) -> int {
    constexpr bool MASKED = decltype(masked_tag)::value;
    for (; kt < kt_end; ++kt) {
      sync_and_prefetch(kt);
      flip_halves();
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int key0 = (tile0 + kt) * kKvTile + 32 * s2;
        if (MASKED && key0 >= kv_end) break;
        scores_into(st, s2, std::true_type{});
        if (MASKED) {
          mask_sub(0, key0);
          mask_sub(1, key0);
        }
        exponentials_seeded(st, pk, 0);
        exponentials_seeded(st, pk, 1);
        if (overflowed(pk)) return 1 + s2;
        accumulate_sub(s2);
      }
    }
    return 0;
  };

  // Fast tiles below the diagonal: both halves' scores first, one growth check, then the halves'
  // exponentials and second products, so that in each basic block MFMAs of one half can run
  // beside the vector ALU work of the other. Returns like fast_tiles (a grown tile is redone
  // from its first half).
  constexpr int kIssueEvery = kJTiles / kLoads;  // MFMA pairs between two row groups of the next tile
  auto fast_plain_tiles = [&](int kt_end) -> int {
    if constexpr (!FP8) {
      if (kt < kt_end) ids_ahead = page_ids_of_tile(kt + 1);
    }
    for (; kt < kt_end; ++kt) {
      sync_and_prefetch(kt, FP8);
      flip_halves();
      if constexpr (!FP8) {
        tile_bases(kt + 1);
        ids_ahead = page_ids_of_tile(kt + 2);
      }
      // Block 1: scores of both halves, the first half's exponentials beside the second half's
      // MFMAs, and the first half's V fragments requested before the block ends.
      // Region 1: all eight K fragments of the first half are requested at once.
      auto load_kfrag = [&](int s2, int i) -> half8_t {   // fragment i = (kk = i / 2, m = i % 2)
        return *(const lds_half8_t *)(uintptr_t)(k_addr[i >> 1] + 2u * (32 * s2 + 16 * (i & 1)) * kHD);
      };
      half8_t kf[kJTiles];
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) kf[i] = load_kfrag(0, i);
#pragma unroll
      for (int m = 0; m < 2; ++m) {
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) st[m][u] = st1[m][u] = seed[u];
      }
      __builtin_amdgcn_sched_barrier(0);
      // Region 2: the first half's MFMAs; each fragment register takes the second half's
      // fragment once its pair is issued. Four accumulators in rotation: no MFMA waits for
      // the one before it.
      half8_t kf1[kJTiles];
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) {
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) st[i & 1][u] = mfma_16x16x32(kf[i], qf[u][i >> 1], st[i & 1][u]);
        kf1[i] = load_kfrag(1, i);
        if constexpr (!FP8) {
          if (i % kIssueEvery == kIssueEvery - 1) issue_rows(i / kIssueEvery);
        }
      }
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (!FP8 && i % kIssueEvery == kIssueEvery - 1) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // Region 3: the second half's MFMAs beside the first half's exponentials; the first
      // half's V fragments are requested on the way.
      half8_t vf[kJTiles];
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) {
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) st1[i & 1][u] = mfma_16x16x32(kf1[i], qf[u][i >> 1], st1[i & 1][u]);
        vf[i] = load_vfrag(i, 0);
      }
      exponentials_seeded(st, pk, 0);
      exponentials_seeded(st, pk, 1);
      const bool over_a = overflowed(pk);
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
      }
      if (over_a) return 1;
      // Block 2: second product of the first half beside the second half's exponentials; each
      // fragment register takes the second half's fragment as soon as its MFMAs are issued.
      half8_t vf2[kJTiles];
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) dsum[u] = mfma_16x16x32(ones, pk[u], dsum[u]);
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) acc[j][u] = mfma_16x16x32(vf[j], pk[u], acc[j][u]);
        vf2[j] = load_vfrag(j, 1);
      }
      exponentials_seeded(st1, pk1, 0);
      exponentials_seeded(st1, pk1, 1);
      const bool over_b = overflowed(pk1);
#pragma unroll
      for (int i = 0; i < kJTiles; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
      if (over_b) return 2;
      // Block 3: second product of the second half.
#pragma unroll
      for (int u = 0; u < kColTiles; ++u) dsum[u] = mfma_16x16x32(ones, pk1[u], dsum[u]);
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
#pragma unroll
        for (int u = 0; u < kColTiles; ++u) acc[j][u] = mfma_16x16x32(vf2[j], pk1[u], acc[j][u]);
      }
    }
    return 0;
  };

  {
    // Tiles whose last key is at or below the block's first row need no mask.
    int n_plain = (diag + 1) / kKvTile - tile0;
    n_plain = n_plain < n_tiles ? n_plain : n_tiles;
    sync_and_prefetch(0);
    general_tile(0, 0);
    while (kt < n_tiles) {
      int n_spread = (last_key + 1) / kKvTile - 1 - tile0;   // tiles kt < n_spread: tile kt + 1 is full
      n_spread = n_spread < n_tiles - 1 ? n_spread : n_tiles - 1;
      n_spread = n_spread < n_plain ? n_spread : n_plain;
      int grew = fast_plain_tiles(n_spread);
      if (grew == 0) grew = fast_tiles(n_tiles, std::true_type{});
      if (grew != 0) {
        general_tile(kt, grew - 1);
        ++kt;
      }
    }
  }

  if constexpr (!SHARED && !KSPLIT) {
    // The accumulators hold O^T: a lane has 4 consecutive d of one row, so stored directly every
    // store instruction would touch 16 rows with 32 bytes each. The rows go through LDS instead
    // (the K/V tiles are done with) and leave as whole 256-byte rows, 4 rows per instruction.
    constexpr int kOutPitch = 2 * kHD + 16;  // bytes; at 128: 68 dwords, a half-wave's 8-byte writes hit 64 banks
    __syncthreads();                              // every wavefront is done reading the last tile
    const uint32_t mine = W == kWideWaves
                              ? k_lds + (uint32_t)(wave * kColTiles * 16 * kOutPitch)
                              : ((wave & 2) ? v_lds : k_lds) + (uint32_t)((wave & 1) * kColTiles * 16 * kOutPitch);
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
      const float inv = v_scale / dsum[u][0];
      const uint32_t at = mine + (uint32_t)((u * 16 + n) * kOutPitch + 8 * g);
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
        *(__attribute__((address_space(3))) half4_t *)(uintptr_t)(at + 32u * j) =
            half4_t{(half_t)(acc[j][u][0] * inv), (half_t)(acc[j][u][1] * inv),
                    (half_t)(acc[j][u][2] * inv), (half_t)(acc[j][u][3] * inv)};
      }
    }
    // lane l carries chunk l % kChunks of row l / kChunks + kRowsPerLoad * step
    const int chunk = slot, r4 = r_loc;
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
#pragma unroll
      for (int step = 0; step < kLoadsPerWave; ++step) {
        const int r = kRowsPerLoad * step + r4;
        const half8_t row = *(const lds_half8_t *)(uintptr_t)(mine + (uint32_t)((u * 16 + r) * kOutPitch + 16 * chunk));
        const int t = wave * kColTiles + u;
        const int head = t / row_tiles;
        const int qrow_idx = m0 + (t - head * row_tiles) * 16 + r;
        if (head < heads_here && qrow_idx < q_len) {
          *(half8_t *)(out + (int64_t)(q_start + qrow_idx) * out_stride + (int64_t)out_head[u] * kHD +
                       8 * chunk) = row;
        }
      }
    }
    return;
  }
  if constexpr (SHARED || KSPLIT) {
    // The partial rows (fp32, normalised) leave as whole rows like the output of a prefill block:
    // a lane holds 4 consecutive elements of each of its column's 16-element groups, so stored
    // straight from registers one instruction would touch 16 rows with 64 bytes each. One column
    // tile at a time goes through this wavefront's part of the K/V staging area (the tiles are
    // done with) and leaves 1 KiB per instruction.
    constexpr int kPartPitch = 4 * kHD + 16;           // bytes; rows 4 banks apart: a 16-lane group's writes hit 64 banks
    constexpr int kRowLanes = kHD / 4;                 // lanes that carry one row (16 bytes each)
    constexpr int kRowsPerStore = kWave / kRowLanes;   // rows one store instruction writes
    __syncthreads();                                   // every wavefront is done reading the last tile
    const uint32_t mine = k_lds + (uint32_t)(wave * 16 * kPartPitch);
    typedef __attribute__((address_space(3))) float4_t lds_float4_t;
#pragma unroll
    for (int u = 0; u < kColTiles; ++u) {
      const float inv = v_scale / dsum[u][0];
      // the partial row of this lane's column (the same in its four lane groups), or -1
      const int piece = SHARED ? block_z : key_slice;  // which partial of the row this block writes
      const int cell = out_row[u] >= 0
                           ? (piece * prefix.batch + out_row[u]) * prefix.num_q_heads + out_head[u]
                           : -1;
      if (g == 0 && cell >= 0) {
        // read once, by the merge launch: streaming stores (see store_state in paged_decode.hip)
        __builtin_nontemporal_store((m_run[u] + fast_log2(dsum[u][0])) * 0.6931471805599453f,
                                    prefix.part_lse + cell);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the reads of the tile before are done
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
        *(lds_float4_t *)(uintptr_t)(mine + (uint32_t)(n * kPartPitch + 4 * (16 * j + 4 * g))) =
            float4_t{acc[j][u][0] * inv, acc[j][u][1] * inv, acc[j][u][2] * inv, acc[j][u][3] * inv};
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int step = 0; step < 16 / kRowsPerStore; ++step) {
        const int r = kRowsPerStore * step + lane / kRowLanes;      // column of the tile = row staged
        const int c = lane % kRowLanes;
        const int row_cell = __shfl(cell, r, kWave);
        const float4_t x = *(const lds_float4_t *)(uintptr_t)(mine + (uint32_t)(r * kPartPitch + 16 * c));
        if (row_cell >= 0) {
          __builtin_nontemporal_store(x, (float4_t *)(prefix.part_o + (int64_t)row_cell * kHD + 4 * c));
        }
      }
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < kColTiles; ++u) {
    const float inv = v_scale / dsum[u][0];
    if (out_row[u] >= 0) {
      half_t *o = out + (int64_t)out_row[u] * out_stride + (int64_t)out_head[u] * kHD + 4 * g;
#pragma unroll
      for (int j = 0; j < kJTiles; ++j) {
        *(half4_t *)(o + 16 * j) =
            half4_t{(half_t)(acc[j][u][0] * inv), (half_t)(acc[j][u][1] * inv),
                    (half_t)(acc[j][u][2] * inv), (half_t)(acc[j][u][3] * inv)};
      }
    }
  }
}

template <int MODE, int W = kTiledWaves>
__global__ __launch_bounds__(W *kWave, W == kWideWaves ? 1 : (kHD == 64 ? 3 : 2)) void varlen_prefill_tiled_kernel(
    const half_t *__restrict__ q, int64_t q_stride, half_t *__restrict__ out, int64_t out_stride,
    PagedSource paged, PackedSource packed, PrefixTask prefix,
    const int32_t *__restrict__ q_starts_or_cu, const int32_t *__restrict__ q_lens_or_null,
    const int32_t *__restrict__ context_lens, int32_t group, int32_t head_splits,
    int32_t heads_per_wg, int32_t row_tiles, float scale_log2, int32_t key_slices) {
  __shared__ __attribute__((aligned(1024))) half_t lds_all[tile_lds_bytes<W>() / 2];
  if constexpr (MODE == kPagedPrefillSplit || MODE == kPagedPrefillSplitFp8 ||
                MODE == kPagedPrefillSplitInt8) {
    // blockIdx.y = row block * key_slices + slice: the slices of a block are neighbours
    const int by = (int)blockIdx.y / key_slices;
    prefill_tile_body<MODE, W>((uint32_t)(uintptr_t)(lds_half_t *)lds_all, (int)blockIdx.x, by,
                               (int)blockIdx.z, (int)gridDim.y / key_slices, q, q_stride, out, out_stride,
                               paged, packed, prefix, q_starts_or_cu, q_lens_or_null, context_lens, group,
                               head_splits, heads_per_wg, row_tiles, scale_log2,
                               (int)blockIdx.y - by * key_slices, key_slices);
  } else {
    prefill_tile_body<MODE, W>((uint32_t)(uintptr_t)(lds_half_t *)lds_all, (int)blockIdx.x, (int)blockIdx.y,
                               (int)blockIdx.z, (int)gridDim.y, q, q_stride, out, out_stride, paged, packed,
                               prefix, q_starts_or_cu, q_lens_or_null, context_lens, group, head_splits,
                               heads_per_wg, row_tiles, scale_log2);
  }
}

}  // namespace prefill_tile
}  // namespace LITEKV_HD_NS
}  // namespace litekv
