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

// ---- nibble planes ------------------------------------------------------------------------------
// The reference's INT4 expert kernels take A8 codes as two planes of u32 words: nibble i of a word holds the low
// (unsigned) or high (signed) nibble of code {0,2,1,3,4,6,5,7}[i] of its group of eight
// (kernels/cuda/model/e8p_core.py:63-78, rotation_a8.py:489-491).  x = codes 0..3, y = codes 4..7, one byte each.
__device__ __forceinline__ uint32_t low_word_first(uint32_t x) { return (x & 0x00000F0Fu) | ((x >> 12) & 0x0000F0F0u); }
__device__ __forceinline__ uint32_t low_word_second(uint32_t y) { return ((y << 16) & 0x0F0F0000u) | ((y << 4) & 0xF0F00000u); }
__device__ __forceinline__ uint32_t high_word_first(uint32_t x) { return ((x >> 4) & 0x00000F0Fu) | ((x >> 16) & 0x0000F0F0u); }
__device__ __forceinline__ uint32_t high_word_second(uint32_t y) { return ((y << 12) & 0x0F0F0000u) | (y & 0xF0F00000u); }
__device__ __forceinline__ uint32_t low_word(uint32_t x, uint32_t y) { return low_word_first(x) | low_word_second(y); }
__device__ __forceinline__ uint32_t high_word(uint32_t x, uint32_t y) { return high_word_first(x) | high_word_second(y); }

// Word j of plane row `row`: row-major (rows, K/8), or K64-major (K/64, rows, 8) (kernels/cuda/model/e8p_prefill.py:79-80)
__device__ __forceinline__ int64_t plane_index(int group_major, int plane_rows, int words, int64_t row, int j) {
    return group_major ? ((int64_t)(j >> 3) * plane_rows + row) * 8 + (j & 7) : row * words + j;
}

}  // namespace orx
