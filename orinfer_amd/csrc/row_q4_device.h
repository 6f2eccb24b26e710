// Device-side decode of row-scaled scalar Q4 weights (kernels/cuda/model/q4_projection.py:1-30,
// python/orinfer_build/quantization/row_q4.py:45-51): a nibble holds three magnitude bits and a sign bit,
// weight = +-magnitudes[nibble & 7], negative when bit 3 is set; nibble i of a u16 word is weight i of its four.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace orx {

// Four nibbles (bits 0-15 of `word`) -> four int8 weights, one per byte.  `low` and `high` hold magnitudes 0-3 and
// 4-7 as bytes.  The negation is bytewise ~m + 1, which cannot carry: magnitudes are at least 1.
__device__ __forceinline__ uint32_t decode_row_q4(uint32_t word, uint32_t low, uint32_t high) {
    uint32_t x = word & 0xFFFFu;
    x = (x | (x << 8)) & 0x00FF00FFu;
    x = (x | (x << 4)) & 0x0F0F0F0Fu;  // one nibble per byte
    const uint32_t magnitude = __builtin_amdgcn_perm(high, low, x & 0x07070707u);
    const uint32_t negative = ((x >> 3) & 0x01010101u) * 0xFFu;
    return (magnitude ^ negative) + (negative & 0x01010101u);
}

// Four nibbles already spread one per byte (bits 0-3 of every byte) -> four int8 weights.
__device__ __forceinline__ uint32_t decode_row_q4_bytes(uint32_t x, uint32_t low, uint32_t high) {
    const uint32_t magnitude = __builtin_amdgcn_perm(high, low, x & 0x07070707u);
    const uint32_t sign = (x >> 3) & 0x01010101u;
    return (magnitude ^ (sign * 0xFFu)) + sign;
}

}  // namespace orx
