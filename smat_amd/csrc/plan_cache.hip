// The drop-in entry point smat_spmm_bcsr_f16 and the small plan cache behind it.
//
// The reference's launcher (src/cuda_hgemm/src/mma/mmaCBT.cu:83-88) gets nothing but device pointers, and its
// harness calls it again and again with the same arguments (common/tester.h:177-182,342-357).  The fast kernels
// of this library want a plan (a work list made on the host from row_ptr / col_idx).  So the first call with a
// given (device, row_ptr, col_idx, M, K, nnzb, N) copies the two index arrays to the host, makes a plan and keeps
// it; later calls with the same key reuse it.  The warm-up launch of a benchmark absorbs the one-off cost, as
// it absorbs the reference's first launch.
//
// Staleness.  The key is made of pointers and sizes: a caller that writes ANOTHER block pattern into the same
// arrays is caught by a checksum of row_ptr / col_idx taken on the device on the first call and on every
// CHECK_EVERY-th call after it (synchronous: a small kernel and an 8-byte copy), or tells the library with
// smat_plan_cache_clear().  Block VALUES are read live by the kernels a cached plan may choose (row-wise, sweep),
// so values may change freely between calls; plans that keep a copy of the values (compact, mixed) are only
// made when SMAT_PLAN_CACHE=values promises that values do not change without smat_plan_cache_clear().
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/smat.h"
#include "devmem.h"
#include "errors.h"

using namespace smat;

namespace {

constexpr int CACHE_ENTRIES = 8;
constexpr uint64_t CHECK_EVERY_DEFAULT = 64;

__host__ __device__ inline unsigned long long mix64(unsigned long long x)
{
    x ^= x >> 30; x *= 0xbf58476d1ce4e5b9ull;
    x ^= x >> 27; x *= 0x94d049bb133111ebull;
    x ^= x >> 31;
    return x;
}
// Order-independent checksum of two int32 arrays: sum of mix64(position, value) over both.
__global__ __launch_bounds__(256) void pattern_checksum_kernel(const int32_t *__restrict__ row_ptr, long n_rp,
                                                               const int32_t *__restrict__ col_idx, long n_ci,
                                                               unsigned long long *__restrict__ out)
{
    unsigned long long sum = 0;
    const long total = n_rp + n_ci;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const unsigned v = (unsigned)(i < n_rp ? row_ptr[i] : col_idx[i - n_rp]);
        sum += mix64(((unsigned long long)i << 32) | v);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d);
    if ((threadIdx.x & 63) == 0) atomicAdd(out, sum);
}
unsigned long long host_checksum(const int32_t *rp, long n_rp, const int32_t *ci, long n_ci)
{
    unsigned long long sum = 0;
    for (long i = 0; i < n_rp; i++) sum += mix64(((unsigned long long)i << 32) | (unsigned)rp[i]);
    for (long i = 0; i < n_ci; i++) sum += mix64(((unsigned long long)(i + n_rp) << 32) | (unsigned)ci[i]);
    return sum;
}

struct Entry {
    int device = -1;
    const void *row_ptr = nullptr, *col_idx = nullptr, *vals = nullptr; // vals is part of the key only for plans that copy values
    size_t M = 0, K = 0, nnzb = 0, N = 0;
    smat_plan *plan = nullptr; // nullptr: no plan could be made for this key, the launch goes without
    unsigned long long checksum = 0;
    uint64_t calls = 0, last_use = 0;
};

struct Cache {
    std::mutex mutex;
    std::vector<Entry> entries;
    uint64_t clock = 0;
    uint64_t check_every = CHECK_EVERY_DEFAULT;
    int64_t built = 0, hits = 0, rebuilt = 0; // for smat_internal_plan_cache_stats
    unsigned long long *d_sum[64] = {nullptr}; // one 8-byte word per device for the checksum kernel
} g_cache;

enum Mode { MODE_OFF, MODE_PATTERN, MODE_VALUES };
Mode cache_mode()
{
    const char *e = getenv("SMAT_PLAN_CACHE");
    if (!e || !*e) return MODE_PATTERN;
    if (!strcmp(e, "0") || !strcmp(e, "off") || !strcmp(e, "false")) return MODE_OFF;
    if (!strcmp(e, "values")) return MODE_VALUES;
    return MODE_PATTERN;
}

hipError_t device_checksum(int dev, const int32_t *row_ptr, size_t mb, const int32_t *col_idx, size_t nnzb, unsigned long long *out)
{
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    hipError_t e = hipSuccess;
    if (!g_cache.d_sum[dev]) e = dev_malloc(&g_cache.d_sum[dev], sizeof(unsigned long long));
    if (e != hipSuccess) return e;
    unsigned long long *d = g_cache.d_sum[dev];
    // the null stream: ordered behind whatever wrote the arrays there, and before the launch that follows
    e = hipMemsetAsync(d, 0, sizeof *d, nullptr);
    if (e != hipSuccess) return e;
    const long total = (long)mb + 1 + (long)nnzb;
    const unsigned blocks = (unsigned)std::min<long>((total + 255) / 256, 256L * 8);
    hipLaunchKernelGGL(pattern_checksum_kernel, dim3(blocks), dim3(256), 0, nullptr, row_ptr, (long)mb + 1, col_idx, (long)nnzb, d);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return hipMemcpy(out, d, sizeof *out, hipMemcpyDeviceToHost);
}

// Makes the plan of an entry from the device arrays (synchronous).  Leaves plan == nullptr when none can be made.
void build_entry(Entry &en, const uint16_t *vals, Mode mode)
{
    en.plan = nullptr;
    const size_t mb = en.M / 16;
    std::vector<int32_t> rp(mb + 1), ci(en.nnzb);
    if (hipMemcpy(rp.data(), en.row_ptr, rp.size() * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) return;
    if (en.nnzb && hipMemcpy(ci.data(), en.col_idx, ci.size() * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) return;
    en.checksum = host_checksum(rp.data(), (long)rp.size(), ci.data(), (long)ci.size());
    smat_spmm_opts o = {SMAT_B_COL_MAJOR, SMAT_C_F16, SMAT_KERNEL_AUTO, 0, nullptr};
    smat_plan *p = nullptr;
    if (smat_plan_create(&p, rp.data(), en.nnzb ? ci.data() : nullptr, en.M, en.K, en.nnzb, en.N, &o) != SMAT_OK) return; // e.g. a row_ptr that is none
    if (mode == MODE_VALUES && en.nnzb &&
        smat_plan_attach_values(p, vals, static_cast<const int32_t *>(en.row_ptr), static_cast<const int32_t *>(en.col_idx), rp.data()) != SMAT_OK) {
        smat_plan_destroy(p);
        return;
    }
    en.plan = p;
    g_cache.built++;
}

} // namespace

extern "C" int smat_plan_cache_clear(void)
{
    std::lock_guard<std::mutex> lock(g_cache.mutex);
    for (Entry &en : g_cache.entries)
        if (en.plan) smat_plan_destroy(en.plan);
    g_cache.entries.clear();
    return SMAT_OK;
}

// Test hooks (not part of smat.h): {plans built, launches that found their plan, plans rebuilt after a checksum
// mismatch, entries held}; and how often the checksum is taken (0 = the default).
extern "C" void smat_internal_plan_cache_stats(int64_t *out)
{
    std::lock_guard<std::mutex> lock(g_cache.mutex);
    out[0] = g_cache.built; out[1] = g_cache.hits; out[2] = g_cache.rebuilt; out[3] = (int64_t)g_cache.entries.size();
}
extern "C" void smat_internal_plan_cache_check_every(uint64_t n)
{
    std::lock_guard<std::mutex> lock(g_cache.mutex);
    g_cache.check_every = n ? n : CHECK_EVERY_DEFAULT;
}

extern "C" int smat_spmm_bcsr_f16(const uint16_t *vals, const int32_t *row_ptr, const int32_t *col_idx,
                                   const uint16_t *B, uint16_t *C, size_t M, size_t N, size_t K, size_t nnzb,
                                   const int32_t *block_info, const int32_t *rel_map)
{
    (void)block_info;
    (void)rel_map;
    const Mode mode = cache_mode();
    // arguments that no plan can be made for go straight to the launch, which reports them
    if (mode == MODE_OFF || !row_ptr || !B || !C || M == 0 || N == 0 || K == 0 || M % 16 || K % 16 || N % 8 ||
        (nnzb && (!vals || !col_idx)) || M / 16 > 0x7ffffff0u || nnzb > 0x7ffffff0u)
        return smat_spmm_bcsr_f16_ex(vals, row_ptr, col_idx, B, C, M, N, K, nnzb, nullptr, nullptr);
    return smat::guarded("smat_spmm_bcsr_f16", [&]() -> int {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return set_error(SMAT_ERR_HIP, "hipGetDevice failed");
        std::lock_guard<std::mutex> lock(g_cache.mutex);
        Entry *en = nullptr;
        for (Entry &c : g_cache.entries)
            if (c.device == dev && c.row_ptr == row_ptr && c.col_idx == col_idx && c.M == M && c.K == K && c.nnzb == nnzb &&
                c.N == N && (mode != MODE_VALUES || c.vals == vals)) {
                en = &c;
                break;
            }
        if (!en) {
            if ((int)g_cache.entries.size() >= CACHE_ENTRIES) { // the entry used longest ago makes room
                size_t old = 0;
                for (size_t i = 1; i < g_cache.entries.size(); i++)
                    if (g_cache.entries[i].last_use < g_cache.entries[old].last_use) old = i;
                if (g_cache.entries[old].plan) smat_plan_destroy(g_cache.entries[old].plan);
                g_cache.entries.erase(g_cache.entries.begin() + (long)old);
            }
            Entry fresh;
            fresh.device = dev; fresh.row_ptr = row_ptr; fresh.col_idx = col_idx; fresh.vals = mode == MODE_VALUES ? vals : nullptr;
            fresh.M = M; fresh.K = K; fresh.nnzb = nnzb; fresh.N = N;
            build_entry(fresh, vals, mode);
            g_cache.entries.push_back(fresh);
            en = &g_cache.entries.back();
        } else {
            g_cache.hits++;
            if (en->plan && en->calls % g_cache.check_every == 0) { // the arrays behind the pointers: still the plan's pattern?
                unsigned long long now = 0;
                if (device_checksum(dev, row_ptr, M / 16, col_idx, nnzb, &now) != hipSuccess || now != en->checksum) {
                    smat_plan_destroy(en->plan);
                    build_entry(*en, vals, mode);
                    g_cache.rebuilt++;
                }
            }
        }
        en->calls++;
        en->last_use = ++g_cache.clock;
        return smat_spmm_bcsr_f16_ex(vals, row_ptr, col_idx, B, C, M, N, K, nnzb, nullptr, en->plan);
    });
}
