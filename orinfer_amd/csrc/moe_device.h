// Device helpers of the MoE router shared by the kernels that select routes
// (kernels/cuda/model/moe.py:413-494): the routing launch itself and the single-token expert
// projection that selects its token's routes in its own set-up.
#pragma once
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

namespace orx {

// Total order on finite fp32 with -0 == +0 (moe.py:449-465): larger key = larger score.
__device__ __forceinline__ uint32_t ordered_key(float value) {
    const uint32_t bits = __float_as_uint(value);
    if (value == 0.f) return 0x80000000u;
    return (bits & 0x80000000u) ? ~bits : bits ^ 0x80000000u;
}
__device__ __forceinline__ float key_value(uint32_t ordered) {
    return __uint_as_float((ordered & 0x80000000u) ? ordered ^ 0x80000000u : ~ordered);
}

// Maximum of a 64-bit key over the wave with data-parallel-primitive moves only (no LDS round
// trips: the selection loop below is a chain of top_k dependent reductions).  Quad swaps, half-row
// and row mirrors give every lane its row's maximum; two broadcasts carry it across rows into
// lane 63, which is then read back as a scalar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void dpp_max_step(uint32_t& hi, uint32_t& lo) {
    // lanes outside ROW_MASK receive their own value back
    const uint32_t other_hi = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)hi, CTRL, ROW_MASK, 0xF, false);
    const uint32_t other_lo = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)lo, CTRL, ROW_MASK, 0xF, false);
    const bool take = other_hi > hi || (other_hi == hi && other_lo > lo);
    hi = take ? other_hi : hi;
    lo = take ? other_lo : lo;
}
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
    uint32_t hi = (uint32_t)(v >> 32), lo = (uint32_t)v;
    dpp_max_step<0xB1, 0xF>(hi, lo);   // quad_perm [1,0,3,2]
    dpp_max_step<0x4E, 0xF>(hi, lo);   // quad_perm [2,3,0,1]
    dpp_max_step<0x141, 0xF>(hi, lo);  // row_half_mirror
    dpp_max_step<0x140, 0xF>(hi, lo);  // row_mirror
    dpp_max_step<0x142, 0xA>(hi, lo);  // row_bcast:15 into rows 1 and 3
    dpp_max_step<0x143, 0xC>(hi, lo);  // row_bcast:31 into rows 2 and 3
    const uint32_t top_hi = (uint32_t)__builtin_amdgcn_readlane((int)hi, 63);
    const uint32_t top_lo = (uint32_t)__builtin_amdgcn_readlane((int)lo, 63);
    return ((unsigned long long)top_hi << 32) | top_lo;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    return v;
}

// The routes of one row, by one wave: each lane keeps LOCAL = ceil(E/64) keys (rounded up to a power
// of two) in registers.  Key = ordered score in the high word, (E - id) in the low word, so one max
// picks the score and the lowest id on ties.  Lane `rank` writes ids[row, rank] and prob[row, rank].
template <int LOCAL>
__device__ __forceinline__ void select_routes(const float* __restrict__ logits, int* ids, float* prob, int row, int e,
                                              int top_k, int renormalize, int lane) {
    unsigned long long keys[LOCAL];
    float all_exp = 0.f;
    float local_max = -INFINITY;
#pragma unroll
    for (int j = 0; j < LOCAL; ++j) {
        const int id = j * 64 + lane;
        keys[j] = 0ull;
        if (id < e) {
            const float v = logits[(int64_t)row * e + id];
            keys[j] = ((unsigned long long)ordered_key(v) << 32) | (unsigned long long)(uint32_t)(e - id);
            local_max = fmaxf(local_max, v);
        }
    }
    float global_max = local_max;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) global_max = fmaxf(global_max, __shfl_xor(global_max, offset, 64));
    if (!renormalize) {
#pragma unroll
        for (int j = 0; j < LOCAL; ++j) {
            const int id = j * 64 + lane;
            if (id < e) all_exp += expf(logits[(int64_t)row * e + id] - global_max);
        }
        all_exp = wave_sum(all_exp);
    }
    float mine = 0.f;  // numerator of rank == lane
    for (int rank = 0; rank < top_k; ++rank) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int j = 0; j < LOCAL; ++j) best = keys[j] > best ? keys[j] : best;
        best = wave_max_u64(best);
        const int id = e - (int)(uint32_t)(best & 0xFFFFFFFFull);
        const float score = key_value((uint32_t)(best >> 32));
#pragma unroll
        for (int j = 0; j < LOCAL; ++j)
            if (j * 64 + lane == id) keys[j] = 0ull;
        if (lane == rank) {
            ids[(int64_t)row * top_k + rank] = id;
            mine = expf(score - global_max);
        }
    }
    const float selected_sum = wave_sum(lane < top_k ? mine : 0.f);
    if (lane < top_k) prob[(int64_t)row * top_k + lane] = __fdiv_rn(mine, renormalize ? selected_sum : all_exp);
}

}  // namespace orx
