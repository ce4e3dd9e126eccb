// Per-step metadata of a decode batch, advanced on the device: every sequence grows by one
// token, the slot that token's K/V goes to is looked up in the request's page list, and the
// batch's block-table rows are gathered into batch order. The reference does this on the host
// every step (PagedReqTokensManager.extend_req + batch_metadata,
// lite_llama/executor/paged_attention.py:287-359, then update_kv_index,
// lite_llama/kernels/update_kv_index.py:41-74, and three host-to-device copies in
// NpuGraphRunner.replay, lite_llama/executor/npu_graph.py:183-197); here it is one small launch
// that a captured graph can hold, so a replayed decode step needs nothing from the host as long
// as the pages were reserved ahead.
//
// One workgroup per sequence: lane 0 advances the length and writes slot / position, all lanes
// copy the page list.
#include "common.h"

namespace litekv {

__global__ __launch_bounds__(256) void decode_advance_kernel(
    const int32_t *__restrict__ request_tables, int64_t request_table_stride, int32_t max_requests,
    const int32_t *__restrict__ request_ids, const int32_t *__restrict__ capacity,
    int32_t *__restrict__ seq_lens, int64_t *__restrict__ seq_lens_i64,
    int32_t *__restrict__ slot_mapping, int64_t *__restrict__ position_ids,
    int32_t *__restrict__ block_table, int64_t block_table_stride, int32_t width,
    int32_t *__restrict__ overflow, int32_t page_size, int32_t num_pages, int32_t increment) {
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int32_t r = request_ids[b];
  const bool r_ok = r >= 0 && r < max_requests;
  const int32_t *row = request_tables + (int64_t)(r_ok ? r : 0) * request_table_stride;

  for (int p = tid; p < width; p += 256) {
    block_table[(int64_t)b * block_table_stride + p] = r_ok ? row[p] : 0;
  }
  if (tid != 0) return;

  const int32_t len = seq_lens[b];
  const int64_t room = (int64_t)width * page_size;
  int64_t cap = capacity != nullptr ? (int64_t)capacity[b] : room;
  cap = cap < room ? cap : room;
  const int64_t want = (int64_t)len + increment;
  const bool ok = r_ok && len >= 0 && want <= cap;
  // A refused row becomes empty for good: length -1 (every kernel of the path treats a length
  // <= 0 as "no tokens": zero output, nothing appended), slot -1 (the append kernels skip it),
  // and it stays refused on later steps. Keeping its old length would let the step's append,
  // which writes at logical position length - 1, overwrite the last cached token.
  const int32_t next = ok ? (int32_t)want : -1;
  int32_t slot = -1;  // the append kernels skip a negative slot
  if (ok && next >= 1) {
    const int32_t page = row[(next - 1) / page_size];
    if (page >= 0 && page < num_pages) slot = page * page_size + (next - 1) % page_size;
  }
  seq_lens[b] = next;
  if (seq_lens_i64 != nullptr) seq_lens_i64[b] = next;
  slot_mapping[b] = slot;
  if (position_ids != nullptr) position_ids[b] = next >= 1 ? next - 1 : 0;
  if (!ok && overflow != nullptr) overflow[0] = 1;
}

}  // namespace litekv

extern "C" int litekv_decode_advance(const int32_t *request_tables, int64_t request_table_stride,
                                     int32_t max_requests, const int32_t *request_ids,
                                     const int32_t *capacity, int32_t *seq_lens,
                                     int64_t *seq_lens_i64, int32_t *slot_mapping,
                                     int64_t *position_ids, int32_t *block_table,
                                     int64_t block_table_stride, int32_t width, int32_t *overflow,
                                     int32_t batch, int32_t page_size, int64_t num_pages,
                                     int32_t increment, void *stream) {
  using namespace litekv;
  const char *what = "decode_advance";
  LITEKV_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch %d out of [0, 65535]", what, batch);
  LITEKV_REQUIRE(page_size > 0, "%s: page_size %d <= 0", what, page_size);
  LITEKV_REQUIRE(num_pages > 0 && num_pages * page_size <= 0x7fffffffLL,
                 "%s: num_pages %lld out of range (slots must fit int32)", what, (long long)num_pages);
  LITEKV_REQUIRE(max_requests > 0, "%s: max_requests %d <= 0", what, max_requests);
  LITEKV_REQUIRE(width > 0 && (int64_t)width <= request_table_stride &&
                     (int64_t)width <= block_table_stride,
                 "%s: width %d must be in (0, min(request_table_stride %lld, block_table_stride %lld)]",
                 what, width, (long long)request_table_stride, (long long)block_table_stride);
  LITEKV_REQUIRE((int64_t)width * page_size <= 0x7fffffffLL, "%s: width %d too large", what, width);
  LITEKV_REQUIRE(increment == 0 || increment == 1, "%s: increment %d must be 0 or 1", what,
                 increment);
  if (batch == 0) {
    clear_error();
    return LITEKV_OK;
  }
  LITEKV_REQUIRE(request_tables && request_ids && seq_lens && slot_mapping && block_table,
                 "%s: null pointer", what);
  hipLaunchKernelGGL(decode_advance_kernel, dim3((unsigned)batch), dim3(256), 0,
                     static_cast<hipStream_t>(stream), request_tables, request_table_stride,
                     max_requests, request_ids, capacity, seq_lens, seq_lens_i64, slot_mapping,
                     position_ids, block_table, block_table_stride, width, overflow, page_size,
                     (int32_t)num_pages, increment);
  return check_launch(what);
}
