// Device helpers of the A8 activation quantiser, shared by the kernels that quantise activations
// (kernels/cuda/operators/op30_activation_quantization.py:14-18, 49-65).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace orx {

// fp16 scale of a group from its largest magnitude: max(amax / 127, 2^-24), or 1 for an all-zero group.
__device__ __forceinline__ __half a8_scale(float amax) {
    const float raw_scale = fmaxf(__fdiv_rn(amax, 127.0f), 5.9604644775390625e-08f);
    return amax > 0.f ? __float2half_rn(raw_scale) : __float2half_rn(1.0f);
}

// rint(value / scale), clamped: the product with the reciprocal decides, except within 2^-14 of a
// tie, where the correctly rounded quotient does.  The product is within 4 units in the last place
// of the quotient (|quotient| < 128.5, so 2^-15 at most), so the two round alike everywhere else;
// the reference's kernel takes the same shortcut (kernels/cuda/model/rotation_a8.py:153-164).
__device__ __forceinline__ int8_t quantise(float value, float scale, float inverse) {
    const float guess = value * inverse;
    float r = rintf(guess);
    if (fabsf(fabsf(guess - r) - 0.5f) < 6.103515625e-05f) r = rintf(__fdiv_rn(value, scale));
    return (int8_t)fmaxf(-127.f, fminf(127.f, r));
}

// Four codes packed into one word; one test (and, rarely, four exact quotients) for the four.
// A product's distance from its rounded value is at most 0.5, so "within 2^-14 of a tie" is
// "farther than 0.5 - 2^-14 from the rounded value".  The clamped integer plus 1.5 * 2^23 has the
// integer in its low mantissa bits in two's complement: the low byte of that word is the int8 code.
__device__ __forceinline__ uint32_t quantise4(const float (&value)[4], float scale, float inverse) {
    float r[4];
    float farthest = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float guess = value[j] * inverse;
        r[j] = rintf(guess);
        farthest = fmaxf(farthest, fabsf(guess - r[j]));
    }
    if (farthest > 0.49993896484375f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = rintf(__fdiv_rn(value[j], scale));
    }
    uint32_t word[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) word[j] = __float_as_uint(__builtin_amdgcn_fmed3f(r[j], -127.f, 127.f) + 12582912.0f);
    // byte 0 of the first operand's partner (second argument), then byte 0 of the first argument
    const uint32_t low = __builtin_amdgcn_perm(word[1], word[0], 0x0C0C0400u);
    const uint32_t high = __builtin_amdgcn_perm(word[3], word[2], 0x0C0C0400u);
    return low | (high << 16);
}

// fp16(silu(gate) * up) in fp32 with a stable sigmoid (kernels/cuda/operators/op04_swiglu.py:6-17).
__device__ __forceinline__ float swiglu_value(__half gate, __half up) {
    const float g = __half2float(gate), u = __half2float(up);
    const float e = expf(-fabsf(g));
    const float sigmoid = __fdiv_rn(g >= 0.f ? 1.0f : e, 1.0f + e);  // one division serves both signs of the gate
    // one fp16 rounding here: the value a downstream quantiser sees is the materialised fp16
    return __half2float(__float2half_rn((g * sigmoid) * u));
}

}  // namespace orx
