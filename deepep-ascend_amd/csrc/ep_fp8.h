// fp32 -> OCP FP8 e4m3fn in integer arithmetic: round to nearest even, no saturation, every
// magnitude above 464 (and NaN/Inf) encodes as NaN 0x7F.  This is the conversion
// `tensor.to(torch.float8_e4m3fn)` performs, which the reference quantiser
// (deep_ep/utils/math.py:36-38) relies on.  Shared by host and device code.
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define EP_HD __host__ __device__ inline
#else
#define EP_HD static inline
#endif

EP_HD uint32_t ep_f32_bits_to_e4m3fn(uint32_t bits) {
    const uint32_t sign = (bits >> 24) & 0x80u;
    uint32_t a = bits & 0x7fffffffu;
    uint32_t r;
    if (a > 0x43e80000u) {                    // |x| > 464  (incl. Inf, NaN)
        r = 0x7fu;
    } else if (a < 0x3c800000u) {             // |x| < 2^-6: result is a multiple of 2^-9
        float f;
        memcpy(&f, &a, 4);
        f += 16384.0f;                        // ulp(2^14) == 2^-9, so the add rounds to nearest even there
        uint32_t t;
        memcpy(&t, &f, 4);
        r = t - 0x46800000u;
    } else {                                  // normal: keep 3 mantissa bits
        const uint32_t odd = (a >> 20) & 1u;
        a += 0xc4000000u + 0x7ffffu + odd;    // rebias exponent by (7 - 127) and round half to even
        r = a >> 20;
    }
    return r | sign;
}
