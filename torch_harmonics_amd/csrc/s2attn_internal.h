// Shared by the translation units of libs2attn.so; not installed.
#pragma once

#include "../../include/s2attn.h"

// Records a printf-style message for s2attn_last_error() and returns `code`.
int s2attn_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Shared by the plan builder and the hybrid kernels: runs at least S2_LMIN long go through the matrix cores, shorter ones
// through vector chunks of S2_VC neighbors; two adjacent short-run latitudes are paired when every merged band fits one chunk.
#define S2_LMIN 32
#define S2_VC 9
#define S2_PAIR_MAX_RUNS 32 /* merged runs a pair may have (the kernels keep them in LDS) */
