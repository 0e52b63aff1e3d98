// Host-side error plumbing shared by the API translation units.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../../include/tritium_mi355x.h"

// Records a thread-local message and returns `code`.
int tk_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// BackendError::ShapeMismatch{expected, got}
int tk_fail_mismatch(size_t expected, size_t got);
// BackendError::OutOfMemory{requested}
int tk_fail_oom(size_t requested);
