// Small arithmetic helpers shared by the layers (utility/common.cpp:15-54 of
// the reference keeps the same names).  Host allocations of the layers are
// plain malloc; device memory comes from the arena in device.h.
#pragma once

#include <stddef.h>

inline int min(int a, int b) { return (a < b) ? a : b; }

// round num up to a multiple of align
inline int align_ceil(int num, int align) { return num + (align - (num % align)) % align; }
