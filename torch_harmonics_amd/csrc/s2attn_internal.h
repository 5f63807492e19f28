// Shared by the translation units of libs2attn.so; not installed.
#pragma once

#include "../../include/s2attn.h"

// Records a printf-style message for s2attn_last_error() and returns `code`.
int s2attn_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
