// Shared declarations of libmortar_hip.so (host side).
#ifndef MORTAR_INTERNAL_H
#define MORTAR_INTERNAL_H

#include "../../include/mortar_hip.h"

// Records the calling thread's error message and returns `code`.
int mortar_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

int mortar_check_bcsr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb);

#endif
