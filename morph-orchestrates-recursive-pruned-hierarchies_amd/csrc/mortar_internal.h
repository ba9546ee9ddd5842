// Shared declarations of libmortar_hip.so (host side).
#ifndef MORTAR_INTERNAL_H
#define MORTAR_INTERNAL_H

#include "../../include/mortar_hip.h"

// Records the calling thread's error message and returns `code`.
int mortar_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

int mortar_check_bcsr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb);

// Plain product on the +-1 / 0 codes alone, unrounded: y32[m, :] = sum over the kept blocks of codes . x[m, :] in fp32
// (the one-scale kernels with the scale left out).  Returns MORTAR_NO_KERNEL when the pack has no such kernel for M rows.
#define MORTAR_NO_KERNEL (-100)
__attribute__((visibility("hidden"))) int mortar_spmm_codes_f32(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x,
                                                                 int64_t M, int64_t ldx, float *y32, int64_t ldy, void *stream);

#endif
