// The head dim 64 build of paged_prefill.hip (paged in every pool format, or packed): see the note at the top
// of that file.
#define LITEKV_HD 64
#include "paged_prefill.hip"
