// Every device allocation of the library goes through these two, so that one pair of counters says how many
// there were: the test of the entry point that allocates nothing reads them (smat_internal_alloc_counts).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

namespace smat {
extern std::atomic<long long> g_dev_mallocs, g_dev_frees;

template <class T> inline hipError_t dev_malloc(T **p, size_t bytes)
{
    g_dev_mallocs.fetch_add(1, std::memory_order_relaxed);
    return hipMalloc(reinterpret_cast<void **>(p), bytes);
}
inline hipError_t dev_free(void *p)
{
    g_dev_frees.fetch_add(1, std::memory_order_relaxed);
    return hipFree(p);
}
} // namespace smat
