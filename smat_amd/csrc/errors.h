// Per-thread error text behind smat_last_error().
#pragma once
#include <exception>
#include <new>

namespace smat {
// Stores a printf-style message for the calling thread and returns `code`.
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Runs the body of an extern "C" entry point; no C++ exception leaves the library (a garbled size in a file
// or an absurd dimension ends in an error code, not in std::terminate of the host program).
template <class F> int guarded(const char *what, F &&body) noexcept
{
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return set_error(-3 /* SMAT_ERR_NOMEM */, "%s: out of host memory", what);
    } catch (const std::exception &e) {
        return set_error(-3 /* SMAT_ERR_NOMEM */, "%s: %s", what, e.what());
    }
}
} // namespace smat
