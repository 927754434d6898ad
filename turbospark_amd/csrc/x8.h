// Block-scaled fp8 activations (struct X8): the quantiser shared by the kernels that produce them.
#pragma once
#include "tsv_internal.h"

namespace tsv {

// E8M0 byte of a block whose largest magnitude is amax: amax * 2^-(byte - 127) lies in [128, 256),
// inside e4m3's range (largest finite value 448).  A block of zeros (or of values below 2^-120)
// gets byte 0.  An infinite or NaN amax gives a finite scale, and the conversion then writes NaN.
__device__ __forceinline__ int x8_scale_byte(float amax) {
    const int e = (int)((__float_as_uint(amax) >> 23) & 0xFFu);
    return max(e - 7, 0);
}

// One term of four values: the packed e4m3 word of r[0..3] / 2^(byte - 127), bytes in argument
// order, rounded to nearest even; r is left holding what the term did not capture (exactly: the
// scale is a power of two and the difference of two nearby floats is a float).
__device__ __forceinline__ uint32_t x8_term4(float (&r)[4], int byte) {
    typedef float float2v __attribute__((ext_vector_type(2)));
    const float inv = __uint_as_float((uint32_t)(254 - byte) << 23), sc = __uint_as_float((uint32_t)byte << 23);
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(r[0] * inv, r[1] * inv, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(r[2] * inv, r[3] * inv, w, true);
    const float2v d0 = __builtin_amdgcn_cvt_pk_f32_fp8(w, false), d1 = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    r[0] = __builtin_fmaf(-d0[0], sc, r[0]);
    r[1] = __builtin_fmaf(-d0[1], sc, r[1]);
    r[2] = __builtin_fmaf(-d1[0], sc, r[2]);
    r[3] = __builtin_fmaf(-d1[1], sc, r[3]);
    return (uint32_t)w;
}

__device__ __forceinline__ float x8_amax4(const float (&r)[4]) {
    return fmaxf(fmaxf(fabsf(r[0]), fabsf(r[1])), fmaxf(fabsf(r[2]), fabsf(r[3])));
}

}  // namespace tsv
