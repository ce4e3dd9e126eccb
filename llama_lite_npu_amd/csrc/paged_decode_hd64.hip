// The head dim 64 build of the decode kernels and their launchers: paged_decode.hip with its
// lane maps cut to 64-wide rows (see the note at the top of that file). The C ABI stays in the
// head dim 128 build, which calls litekv::hd64_split / hd64_merge / hd64_balanced defined here.
#define LITEKV_HD 64
#include "paged_decode.hip"
