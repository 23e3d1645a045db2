// Division of a 32-bit unsigned number by a divisor fixed at launch time: one multiply-high and a few shifts
// (Granlund & Montgomery, "Division by invariant integers using multiplication", figure 4.1, N = 32); exact for
// every n < 2^32 and d >= 1.  Plain C++ on the host (also compiled by the host-side tests), __umulhi on the device.
#pragma once

#if defined(__HIPCC__)
#define SIMNETS_HOST_DEVICE __host__ __device__ __forceinline__
#else
#define SIMNETS_HOST_DEVICE inline
#endif

namespace simnets {

struct FastDiv {
    unsigned mul, sh1, sh2, d;
};

inline FastDiv make_fast_div(unsigned d)
{
    FastDiv f;
    unsigned l = 0;
    while (l < 32 && (1ull << l) < d)
        ++l;  // ceil(log2 d)
    f.mul = (unsigned)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    f.sh1 = l < 1 ? l : 1;
    f.sh2 = l > 0 ? l - 1 : 0;
    f.d = d;
    return f;
}

SIMNETS_HOST_DEVICE unsigned fast_div(unsigned n, const FastDiv &f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const unsigned t = __umulhi(f.mul, n);
#else
    const unsigned t = (unsigned)(((unsigned long long)f.mul * n) >> 32);
#endif
    return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

}  // namespace simnets
