// The tuned attention kernels are written for one head dim per build: their sources are compiled
// as they stand for 128 and once more with LITEKV_HD 64 (paged_decode_hd64.hip,
// paged_prefill_hd64.hip). Everything of such a build sits in an inline namespace named after the
// head dim, so the two builds link side by side; the C ABI is in the 128 build, which hands
// 64-wide calls to the hd64_* launchers of the other.
#pragma once

#ifndef LITEKV_HD
#define LITEKV_HD 128
#endif
#if LITEKV_HD == 128
#define LITEKV_HD_NS hd128
#elif LITEKV_HD == 64
#define LITEKV_HD_NS hd64
#else
#error "LITEKV_HD must be 128 or 64"
#endif
