// Host-side IEEE binary16 conversions (no device code here).
#pragma once
#include <cstdint>
#include <cstring>

namespace smat {

// double -> half, round-to-nearest-even in one step (no intermediate float, so
// no double rounding).  Matches assigning a double to a `half`, which is what the
// reference loader does (src/cuda_hgemm/src/common/mmio_highlevel.h:708).
inline uint16_t half_from_double(double d)
{
    uint64_t x;
    std::memcpy(&x, &d, sizeof x);
    const uint16_t sign = static_cast<uint16_t>((x >> 48) & 0x8000u);
    const int64_t e = static_cast<int64_t>((x >> 52) & 0x7ff);
    const uint64_t frac = x & 0xfffffffffffffULL;
    if (e == 0x7ff) return static_cast<uint16_t>(sign | 0x7c00u | (frac ? 0x200u : 0u));
    if (e == 0) return sign;
    const int64_t eh = e - 1023 + 15; // biased half exponent
    if (eh >= 31) return static_cast<uint16_t>(sign | 0x7c00u);
    const uint64_t sig = frac | (1ULL << 52);
    const int drop = eh > 0 ? 42 : static_cast<int>(43 - eh); // low bits that do not fit
    if (drop >= 54) return sign;
    uint64_t q = sig >> drop;
    const uint64_t rem = sig & ((1ULL << drop) - 1), tie = 1ULL << (drop - 1);
    if (rem > tie || (rem == tie && (q & 1))) ++q;
    if (eh <= 0) return static_cast<uint16_t>(sign | q); // subnormal (q == 1024 is the smallest normal)
    return static_cast<uint16_t>(sign | ((static_cast<uint64_t>(eh - 1) << 10) + q));
}

inline float half_to_float(uint16_t h)
{
    const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff, bits;
    if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e != 0) {
        bits = sign | ((e + 112) << 23) | (m << 13);
    } else if (m == 0) {
        bits = sign;
    } else {
        e = 113;
        while (!(m & 0x400)) { m <<= 1; --e; }
        bits = sign | (e << 23) | ((m & 0x3ff) << 13);
    }
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return f;
}

} // namespace smat
