// Per-thread error text behind smat_last_error().
#pragma once

namespace smat {
// Stores a printf-style message for the calling thread and returns `code`.
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
} // namespace smat
