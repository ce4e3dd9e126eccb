/*
 * litekv_profile.h -- measurement aid of liblitekv.so, kept apart from the
 * product ABI (litekv.h): every entry point declared there is stateless and
 * re-entrant, this one keeps state between calls.
 */
#ifndef LITEKV_PROFILE_H
#define LITEKV_PROFILE_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * No counterpart in the reference. The next decode launch of head dim 128 made
 * by the calling thread -- litekv_paged_decode_balanced / _prefix, or the split
 * launch of litekv_paged_decode / _split / _append, any pool format -- carries
 * the two hipEvent_t handles as the start and stop events of its decode
 * kernel's own dispatch (not the merge launch that may follow), so its
 * device-side duration can be read with hipEventElapsedTime without extra
 * packets in the stream. The request is held per thread until that launch
 * consumes it; pass NULLs to cancel.
 */
int litekv_profile_next_decode(void *start_event, void *stop_event);

#ifdef __cplusplus
}
#endif
#endif /* LITEKV_PROFILE_H */
