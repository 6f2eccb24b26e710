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
__device__ __forceinline__ uint32_t quantise4(const float (&value)[4], float scale, float inverse) {
    float r[4];
    float nearest = 1.0f;  // smallest distance of a product from a tie
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float guess = value[j] * inverse;
        r[j] = rintf(guess);
        nearest = fminf(nearest, fabsf(fabsf(guess - r[j]) - 0.5f));
    }
    if (nearest < 6.103515625e-05f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = rintf(__fdiv_rn(value[j], scale));
    }
    uint32_t packed = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) packed |= ((uint32_t)(uint8_t)(int8_t)fmaxf(-127.f, fminf(127.f, r[j]))) << (8 * j);
    return packed;
}

}  // namespace orx
