// Split-fp16 arithmetic shared by the kernels that run fp32 GEMMs on the fp16 matrix cores:
// a value v scaled by a power of two s is carried as hi + lo with hi = fp16(v s), lo = fp16(v s - hi),
// and a product takes three MFMAs (lo hi, hi lo, hi hi) accumulated in fp32.
#pragma once
#include <hip/hip_runtime.h>

namespace mg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));


// power of two s with amax * s in [2^14, 2^15); *inv = 1/s.  amax >= 0; zero, tiny, inf and nan give
// a finite in-range scale (the products then follow fp16/fp32 arithmetic on their own)
__device__ __forceinline__ float pow2_scale(float amax, float* inv) {
    int e = (int)(__float_as_uint(amax) >> 23) & 0xff;
    int se = 268 - e;                   // 127 + 14 - (e - 127)
    if (e == 255) se = 127;
    se = se < 1 ? 1 : (se > 253 ? 253 : se);
    *inv = __uint_as_float((unsigned)(254 - se) << 23);
    return __uint_as_float((unsigned)se << 23);
}

struct HalfSplit4 {
    halfx4 hi, lo;
};

__device__ __forceinline__ HalfSplit4 split(float4 v, float s) {
    HalfSplit4 r;
    const float in[4] = {v.x * s, v.y * s, v.z * s, v.w * s};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const _Float16 h = (_Float16)in[k];
        r.hi[k] = h;
        r.lo[k] = (_Float16)(in[k] - (float)h);
    }
    return r;
}

constexpr int kCK = 32;                     // k per chunk (two MFMA steps)
constexpr int kRowW = 80;                   // bytes per LDS row of one W plane (64 + 16 pad)

}  // namespace mg
