// Activation A8 quantiser and the fp16 SwiGLU boundary in front of it.
//
// activation_quantization follows kernels/cuda/operators/op30_activation_quantization.py:
// per (row, group): amax -> scale = fp16(max(amax/127, 2^-24)) (1 when amax == 0) ->
// code = clamp(rint(x / fp32(scale)), -127, 127) with a correctly rounded divide and
// ties-to-even (:14-18, :49-65, contract text :71-78).  `fused` quantises
// fp16(silu(gate)*up) read from X[rows, 2K] (:43-46, op04_swiglu.py:6-17).
// The kernel is memory-bound: one fp16 read (twice, second pass from L2) and one int8 write.
//
// rotate_activation_a8 follows kernels/cuda/model/rotation_a8.py:188-224,369-383: x * sign, seven
// butterfly stages inside every block of 128 channels in fp32, one multiply by fp32(128^-1/2), an
// fp16 materialisation, then the same row-wise A8 rule.  Every stage is one fp32 add or subtract
// in the order of the numpy oracle (quantization/vq.py:20-31), so codes and scales are bit-exact.
//
// e8p_q4_embedding follows kernels/cuda/model/e8p_q4.py:83-140: gather rows of a K-major two-stage
// bank by token id, decode to int8, undo the rotation (unsigned butterflies, * fp32(128^-1/2),
// * row scale, * sign), one fp16 cast; ids outside the vocabulary give zero rows.
#include <hip/hip_fp16.h>

#include <cstring>

#include "a8_device.h"
#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

template <bool FUSED, bool MASKED>
__device__ __forceinline__ float load_value(const __half* __restrict__ x, const uint8_t* __restrict__ mask,
                                            int64_t row_base, int k, int col) {
    float v;
    if (FUSED)
        v = swiglu_value(x[row_base + col], x[row_base + k + col]);
    else
        v = __half2float(x[row_base + col]);
    if (MASKED && mask[col] != 0) v = 0.f;
    return v;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    const int waves = (blockDim.x + 63) >> 6;
    float r = scratch[0];
    for (int i = 1; i < waves; ++i) r = fmaxf(r, scratch[i]);
    return r;
}

// grid (rows, groups), 256 threads.  STAGED (dynamic LDS of one group of fp16 values): a thread keeps
// the 16-byte pieces it read for the maximum in LDS and quantises them from there.  With many rows
// of long groups in flight the second read no longer hits the L2 cache (8192 rows of 17408: every
// CU holds 8 rows of 34 KB), so it would cost HBM traffic a second time.
template <bool FUSED, bool MASKED, int THREADS = 256, bool STAGED = false>
__global__ __launch_bounds__(THREADS) void a8_kernel(const __half* __restrict__ x, const uint8_t* __restrict__ mask,
                                                     int8_t* __restrict__ q, __half* __restrict__ s, int k, int group,
                                                     int groups) {
    extern __shared__ __align__(16) uint4 staged[];
    __shared__ float scratch[THREADS / 64];
    const int row = blockIdx.x, g = blockIdx.y;
    const int first = g * group;
    const int width = min(group, k - first);
    const int64_t in_base = (int64_t)row * (FUSED ? 2 * k : k);
    const int64_t out_base = (int64_t)row * k;
    // 8 halves per thread per step when everything is 16-byte aligned and unmasked/unfused
    const bool vector = !FUSED && !MASKED && (k % 8 == 0) && (group % 8 == 0) &&
                        ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((reinterpret_cast<uintptr_t>(q) & 7) == 0);
    float amax = 0.f;
    typedef _Float16 half_pair __attribute__((ext_vector_type(2)));
    half_pair amax2 = {(_Float16)0.f, (_Float16)0.f};  // largest magnitudes so far as two fp16 lanes: comparing needs no conversion
    // a group of at most one 16-byte piece per thread stays in registers between the two passes
    // (only in the 16-wave form: carrying the piece through the loops costs the 4-wave form its
    // overlap of loads, 28 -> 48 us at 8192 x 5120)
    const bool held = THREADS == 1024 && vector && width / 8 <= THREADS;
    uint4 kept = make_uint4(0u, 0u, 0u, 0u);
    if (STAGED && vector) {
        // four pieces per thread leave together (clamped, so unconditional): a long group would
        // otherwise cost one load latency per piece
        const uint4* src = reinterpret_cast<const uint4*>(x + in_base + first);
        const int pieces = width / 8;
        for (int base = threadIdx.x; base < pieces; base += 4 * THREADS) {
            uint4 raw[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) raw[u] = src[min(base + u * THREADS, pieces - 1)];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = base + u * THREADS;
                if (i < pieces) staged[i] = raw[u];  // read back below by this thread only
                const uint32_t words[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    amax2 = __builtin_elementwise_max(amax2, __builtin_bit_cast(half_pair, words[j] & 0x7FFF7FFFu));
            }
        }
        amax = fmaxf((float)amax2[0], (float)amax2[1]);
    } else if (vector) {
        const uint4* src = reinterpret_cast<const uint4*>(x + in_base + first);
        for (int i = threadIdx.x; i < width / 8; i += blockDim.x) {
            const uint4 raw = src[i];
            if (THREADS == 1024) kept = raw;
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                amax2 = __builtin_elementwise_max(amax2, __builtin_bit_cast(half_pair, words[j] & 0x7FFF7FFFu));
        }
        amax = fmaxf((float)amax2[0], (float)amax2[1]);
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x)
            amax = fmaxf(amax, fabsf(load_value<FUSED, MASKED>(x, mask, in_base, k, first + i)));
    }
    amax = block_max(amax, scratch);
    const float raw_scale = fmaxf(__fdiv_rn(amax, 127.0f), 5.9604644775390625e-08f);
    const __half stored = amax > 0.f ? __float2half_rn(raw_scale) : __float2half_rn(1.0f);
    if (threadIdx.x == 0) s[(int64_t)row * groups + g] = stored;
    const float scale = __half2float(stored);
    const float inverse = __frcp_rn(scale);
    if (vector) {
        const uint4* src = reinterpret_cast<const uint4*>(x + in_base + first);
        uint2* dst = reinterpret_cast<uint2*>(q + out_base + first);
        for (int i = threadIdx.x; i < width / 8; i += blockDim.x) {
            const uint4 raw = held ? kept : STAGED ? staged[i] : src[i];
            const __half* h = reinterpret_cast<const __half*>(&raw);
            const float low[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
            const float high[4] = {__half2float(h[4]), __half2float(h[5]), __half2float(h[6]), __half2float(h[7])};
            dst[i] = make_uint2(quantise4(low, scale, inverse), quantise4(high, scale, inverse));
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x)
            q[out_base + first + i] = quantise(load_value<FUSED, MASKED>(x, mask, in_base, k, first + i), scale, inverse);
    }
}

// Seven butterfly stages over one block of 128 channels held by a half wave (lane l32 holds channels
// 4*l32 .. 4*l32+3), the multiply by fp32(128^-1/2) and the fp16 materialisation; returns the largest
// magnitude of the four fp16 results.
__device__ __forceinline__ float rotate_block(float (&v)[4], int l32, __half (&out)[4]) {
    // distance 1 and 2: inside the lane
    {
        const float a = v[0] + v[1], b = v[0] - v[1], c = v[2] + v[3], d = v[2] - v[3];
        v[0] = a + c, v[2] = a - c, v[1] = b + d, v[3] = b - d;
    }
    // distance 4 .. 64: lanes at distance 1 .. 16.  The upper lane of a pair keeps left - right, the
    // lower one left + right: both are partner + (own with the sign flipped in the upper lane), one
    // fp32 add.  The partner comes through the data-parallel lane controls where they can express
    // the exchange (quad permutes, row rotate by 8, two masked row shifts by 4), else a shuffle.
#pragma unroll
    for (int bit = 0; bit < 5; ++bit) {
        const uint32_t flip = ((uint32_t)(l32 >> bit) & 1u) << 31;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int own = __float_as_int(v[j]);
            int partner;
            if (bit == 0)
                partner = __builtin_amdgcn_update_dpp(0, own, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
            else if (bit == 1)
                partner = __builtin_amdgcn_update_dpp(0, own, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
            else if (bit == 2) {
                partner = __builtin_amdgcn_update_dpp(own, own, 0x104, 0xF, 0x5, false);      // row_shl:4 into banks 0, 2
                partner = __builtin_amdgcn_update_dpp(partner, own, 0x114, 0xF, 0xA, false);  // row_shr:4 into banks 1, 3
            } else if (bit == 3)
                partner = __builtin_amdgcn_update_dpp(0, own, 0x128, 0xF, 0xF, true);  // row_ror:8
            else
                partner = __float_as_int(__shfl_xor(v[j], 16, 64));
            v[j] = __int_as_float(partner) + __int_as_float(own ^ (int)flip);
        }
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float scaled = v[j] * 0.08838834764831845f;
        // opaque: the fp16 cast below must round the fp32 product, not a fused multiply-convert
        asm volatile("" : "+v"(scaled));
        out[j] = __float2half_rn(scaled);
        amax = fmaxf(amax, fabsf(__half2float(out[j])));
    }
    return amax;
}

// Row scale from the largest magnitude, stored once, and the int8 codes of the fp16 row in LDS.
__device__ __forceinline__ void quantise_row(const __half* rotated, float amax, int8_t* __restrict__ q,
                                             __half* __restrict__ s, int row, int k) {
    const int tid = threadIdx.x;
    const float raw_scale = fmaxf(__fdiv_rn(amax, 127.0f), 5.9604644775390625e-08f);
    const __half stored = amax > 0.f ? __float2half_rn(raw_scale) : __float2half_rn(1.0f);
    if (tid == 0) s[row] = stored;
    const float scale = __half2float(stored);
    const float inverse = __frcp_rn(scale);
    for (int i = tid; i < k / 4; i += blockDim.x) {
        const uint2 raw = *reinterpret_cast<const uint2*>(rotated + 4 * i);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const float values[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
        *reinterpret_cast<uint32_t*>(q + (int64_t)row * k + 4 * i) = quantise4(values, scale, inverse);
    }
}

// Short groups (at most 512 values): one wave per (row, group), four per workgroup, a lane holds one
// 16-byte piece; the maximum is a wave reduction, so there is no barrier and no second read.
template <bool FUSED>
__global__ __launch_bounds__(256) void a8_wave_kernel(const __half* __restrict__ x, int8_t* __restrict__ q,
                                                      __half* __restrict__ s, int k, int group, int groups, int rows) {
    const int lane = threadIdx.x & 63;
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);  // wave-uniform
    if (unit >= rows * groups) return;
    const int row = unit / groups, g = unit % groups;
    const int first = g * group;
    const int width = min(group, k - first);
    const int64_t in_base = (int64_t)row * (FUSED ? 2 * k : k);
    const int64_t out_base = (int64_t)row * k;
    const bool vector = (k % 8 == 0) && (group % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                        ((reinterpret_cast<uintptr_t>(q) & 7) == 0);
    float value[8];
    float amax = 0.f;
    if (vector) {
        const bool live = lane < width / 8;
        const int piece = live ? lane : 0;
        const uint4 raw = *reinterpret_cast<const uint4*>(x + in_base + first + 8 * piece);
        uint4 raw_up = make_uint4(0u, 0u, 0u, 0u);
        if (FUSED) raw_up = *reinterpret_cast<const uint4*>(x + in_base + k + first + 8 * piece);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const __half* up = reinterpret_cast<const __half*>(&raw_up);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            value[j] = FUSED ? swiglu_value(h[j], up[j]) : __half2float(h[j]);
            if (live) amax = fmaxf(amax, fabsf(value[j]));
        }
    } else {
        for (int i = lane; i < width; i += 64) amax = fmaxf(amax, fabsf(load_value<FUSED, false>(x, nullptr, in_base, k, first + i)));
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
    const float raw_scale = fmaxf(__fdiv_rn(amax, 127.0f), 5.9604644775390625e-08f);
    const __half stored = amax > 0.f ? __float2half_rn(raw_scale) : __float2half_rn(1.0f);
    if (lane == 0) s[(int64_t)row * groups + g] = stored;
    const float scale = __half2float(stored);
    const float inverse = __frcp_rn(scale);
    if (vector) {
        if (lane < width / 8) {
            const float low[4] = {value[0], value[1], value[2], value[3]}, high[4] = {value[4], value[5], value[6], value[7]};
            *reinterpret_cast<uint2*>(q + out_base + first + 8 * lane) =
                make_uint2(quantise4(low, scale, inverse), quantise4(high, scale, inverse));
        }
    } else {
        for (int i = lane; i < width; i += 64)
            q[out_base + first + i] = quantise(load_value<FUSED, false>(x, nullptr, in_base, k, first + i), scale, inverse);
    }
}

constexpr int kRotateBatch = 5;
constexpr int kRotateWideRows = 256;  // up to one row per CU

// One workgroup per row, 4 waves (16 when rows are few: the latency of one row is what counts then);
// a wave takes two blocks of 128 channels per step (one per half
// wave), a lane holds 4 consecutive channels: stages 1 and 2 are local, stages 4..64 are lane
// exchanges at distance 1..16.  The rotated fp16 row is kept in LDS for the second pass.
// The rotation pass of one row: the rotated fp16 values go to `rotated` (LDS), the return value is the
// largest magnitude this thread has seen.
template <bool SWIGLU, int THREADS>
__device__ __forceinline__ float rotate_row_to_lds(const __half* __restrict__ x, const int8_t* __restrict__ signs,
                                                   __half* rotated, int row, int k) {
    constexpr int kWaves = THREADS / 64;
    constexpr int kBatch = THREADS == 256 ? kRotateBatch : 2;  // steps whose loads leave together
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half_wave = lane >> 5, l32 = lane & 31;
    const int blocks = k / 128;
    const int64_t in_base = (int64_t)row * (SWIGLU ? 2 * k : k);
    float amax = 0.f;
    // kRotateBatch steps at a time, all their loads first: a row is only a few KiB, and one step's
    // load-to-use latency per step would leave the memory system idle
    for (int base = wave; 2 * base < blocks; base += kWaves * kBatch) {  // wave-uniform trip counts
        uint2 raw[kBatch], raw_up[kBatch];
        uint32_t sign_word[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int block = 2 * (base + kWaves * u) + half_wave;
            const int first = (block < blocks ? block : 0) * 128 + 4 * l32;  // clamped, so unconditional
            raw[u] = *reinterpret_cast<const uint2*>(x + in_base + first);
            sign_word[u] = *reinterpret_cast<const uint32_t*>(signs + first);
            raw_up[u] = make_uint2(0u, 0u);
            if (SWIGLU) raw_up[u] = *reinterpret_cast<const uint2*>(x + in_base + k + first);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (2 * (base + kWaves * u) >= blocks) break;
            const int block = 2 * (base + kWaves * u) + half_wave;
            const bool live = block < blocks;
            const int first = (live ? block : 0) * 128 + 4 * l32;
            const __half* h = reinterpret_cast<const __half*>(&raw[u]);
            const __half* up = reinterpret_cast<const __half*>(&raw_up[u]);
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float value = SWIGLU ? swiglu_value(h[j], up[j]) : __half2float(h[j]);
                const float sign = (float)(int8_t)(sign_word[u] >> (8 * j));
                v[j] = live ? value * sign : 0.f;
            }
            __half out[4];
            amax = fmaxf(amax, rotate_block(v, l32, out));
            if (live) *reinterpret_cast<uint2*>(rotated + first) = *reinterpret_cast<const uint2*>(out);
        }
    }
    return amax;
}

template <bool SWIGLU, int THREADS = 256>
__global__ __launch_bounds__(THREADS) void rotate_a8_kernel(const __half* __restrict__ x, const int8_t* __restrict__ signs,
                                                            int8_t* __restrict__ q, __half* __restrict__ s, int k) {
    extern __shared__ __align__(16) __half rotated[];  // k halves
    __shared__ float scratch[THREADS / 64];
    const int row = blockIdx.x;
    float amax = rotate_row_to_lds<SWIGLU, THREADS>(x, signs, rotated, row, k);
    amax = block_max(amax, scratch);  // includes the barrier that publishes `rotated`
    quantise_row(rotated, amax, q, s, row, k);
}

// rotate_expert_a8 (kernels/cuda/model/rotation_a8.py:386-422, body :452-531, entry points :558-604):
// the rotation and the A8 rule of rotate_a8_kernel with the routed hand-over to the expert GEMMs in the
// same launch.  The reference's kernel leaves the codes as two nibble planes plus their sum for its INT4
// expert GEMMs (Low, High: u32 words, row-major, or K64-major under group_major); the int8 expert GEMMs here
// take whole rows, so the kernel can write those instead (D):
//   routing "scatter": Low/High[slot] (and D[slot]) = codes, DS[slot] = scale for each of the row's top_k slots
//                      (slot = RowOffsets[IDs[row, c]] + RelativeSlot[row, c]), SlotMap[row, c] = slot;
//   routing "shared":  Low/High[row] and Q[row] = codes, and only DS[slot] and SlotMap are written per assignment;
//   no routing:        Low/High[row], Q[row], S[row] (and Sum[row]) alone.
// S[row] is always written; Q (scatter) and Sum may be null.  Sum is the integer sum of a row's codes
// (per slot under scatter, per row otherwise), the term the reference's unsigned-nibble product needs.
constexpr int kRouteScatter = 1, kRouteShared = 2;
constexpr int kMaxRouteChoices = 64;
template <bool SWIGLU, int THREADS>
__global__ __launch_bounds__(THREADS) void rotate_expert_kernel(
    const __half* __restrict__ x, const int8_t* __restrict__ signs, int8_t* __restrict__ q, __half* __restrict__ s,
    int8_t* __restrict__ d, __half* __restrict__ ds, const int* __restrict__ ids, const int* __restrict__ relative,
    const int* __restrict__ row_offsets, int* __restrict__ slot_map, int* __restrict__ sum, uint32_t* __restrict__ low,
    uint32_t* __restrict__ high, int plane_rows, int group_major, int k, int top_k, int routing) {
    extern __shared__ __align__(16) __half rotated[];  // k halves
    __shared__ float scratch[THREADS / 64];
    __shared__ int slot_of[kMaxRouteChoices];
    __shared__ int wave_sum[THREADS / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    if (routing != 0 && tid < top_k) {  // requested first: two dependent reads, hidden behind the rotation
        const int assignment = row * top_k + tid;
        const int slot = row_offsets[ids[assignment]] + relative[assignment];
        slot_of[tid] = slot;
        slot_map[assignment] = slot;
    }
    float amax = rotate_row_to_lds<SWIGLU, THREADS>(x, signs, rotated, row, k);
    amax = block_max(amax, scratch);  // includes the barrier that publishes `rotated` and `slot_of`
    const __half stored = a8_scale(amax);
    if (tid == 0) s[row] = stored;
    if (routing != 0 && tid < top_k) ds[slot_of[tid]] = stored;
    const float scale = __half2float(stored), inverse = __frcp_rn(scale);
    int total = 0;
    for (int i = tid; i < k / 4; i += THREADS) {
        const uint2 raw = *reinterpret_cast<const uint2*>(rotated + 4 * i);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const float values[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
        const uint32_t word = quantise4(values, scale, inverse);
        total += (int)(int8_t)word + (int)(int8_t)(word >> 8) + (int)(int8_t)(word >> 16) + ((int)word >> 24);
        if (q != nullptr) *reinterpret_cast<uint32_t*>(q + (int64_t)row * k + 4 * i) = word;
        if (routing == kRouteScatter && d != nullptr)
            for (int c = 0; c < top_k; ++c) *reinterpret_cast<uint32_t*>(d + (int64_t)slot_of[c] * k + 4 * i) = word;
        if (low != nullptr) {
            // threads 2j and 2j + 1 hold the two halves of plane word j (the trip count is even, so both are here)
            const bool second = i & 1;
            uint32_t lo = second ? low_word_second(word) : low_word_first(word);
            uint32_t hi = second ? high_word_second(word) : high_word_first(word);
            lo |= __shfl_xor(lo, 1, 64), hi |= __shfl_xor(hi, 1, 64);
            if (!second) {
                if (routing == kRouteScatter) {
                    for (int c = 0; c < top_k; ++c) {
                        const int64_t at = plane_index(group_major, plane_rows, k >> 3, slot_of[c], i >> 1);
                        low[at] = lo, high[at] = hi;
                    }
                } else {
                    const int64_t at = plane_index(group_major, plane_rows, k >> 3, row, i >> 1);
                    low[at] = lo, high[at] = hi;
                }
            }
        }
    }
    if (sum == nullptr) return;  // uniform: one pointer for the whole launch
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) total += __shfl_xor(total, offset, 64);
    if ((tid & 63) == 0) wave_sum[tid >> 6] = total;
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < THREADS / 64; ++w) total += wave_sum[w];
        if (routing == kRouteScatter)
            for (int c = 0; c < top_k; ++c) sum[slot_of[c]] = total;
        else
            sum[row] = total;
    }
}

// The rotation and the quantiser as two launches over tiles of block_k channels, for few long rows
// (kernels/cuda/model/rotation_a8.py:266-365): rotate_activation_tiles writes the rotated fp16 values and each tile's
// largest magnitude, quantize_rotation_tiles takes the row maximum of the tile maxima and quantises its tile.
// grid (rows, ceil(K / block_k)).  With plane_rows the up rows follow the gate rows as a second plane of X.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void rotate_tiles_kernel(const __half* __restrict__ x, const int8_t* __restrict__ signs,
                                                           __half* __restrict__ rotated, float* __restrict__ maxima, int k,
                                                           int block_k, int64_t row_stride, int64_t up_delta) {
    __shared__ float scratch[4];
    const int row = blockIdx.x, tile = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half_wave = lane >> 5, l32 = lane & 31;
    const int first_block = tile * (block_k / 128), end_block = min(first_block + block_k / 128, k / 128);
    const int64_t in_base = (int64_t)row * row_stride;
    float amax = 0.f;
    for (int pair = wave; first_block + 2 * pair < end_block; pair += 4) {  // wave-uniform trip count
        const int block = first_block + 2 * pair + half_wave;
        const bool live = block < end_block;
        const int first = (live ? block : first_block) * 128 + 4 * l32;
        const uint2 raw = *reinterpret_cast<const uint2*>(x + in_base + first);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const uint32_t sign_word = *reinterpret_cast<const uint32_t*>(signs + first);
        uint2 raw_up = make_uint2(0u, 0u);
        if (SWIGLU) raw_up = *reinterpret_cast<const uint2*>(x + in_base + up_delta + first);
        const __half* up = reinterpret_cast<const __half*>(&raw_up);
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float value = SWIGLU ? swiglu_value(h[j], up[j]) : __half2float(h[j]);
            v[j] = live ? value * (float)(int8_t)(sign_word >> (8 * j)) : 0.f;
        }
        __half out[4];
        amax = fmaxf(amax, rotate_block(v, l32, out));
        if (live) *reinterpret_cast<uint2*>(rotated + (int64_t)row * k + first) = *reinterpret_cast<const uint2*>(out);
    }
    amax = block_max(amax, scratch);
    if (tid == 0) maxima[(int64_t)row * gridDim.y + tile] = amax;
}

__global__ __launch_bounds__(256) void quantize_tiles_kernel(const __half* __restrict__ rotated, const float* __restrict__ maxima,
                                                             int8_t* __restrict__ q, __half* __restrict__ s, int k, int block_k) {
    __shared__ float scratch[4];
    const int row = blockIdx.x, tile = blockIdx.y, tiles = gridDim.y, tid = threadIdx.x;
    float amax = 0.f;
    for (int j = tid; j < tiles; j += 256) amax = fmaxf(amax, maxima[(int64_t)row * tiles + j]);
    amax = block_max(amax, scratch);
    const __half stored = a8_scale(amax);
    if (tile == 0 && tid == 0) s[row] = stored;
    const float scale = __half2float(stored), inverse = __frcp_rn(scale);
    const int first = tile * block_k, width = min(block_k, k - first);
    for (int i = tid; i < width / 4; i += 256) {
        const uint2 raw = *reinterpret_cast<const uint2*>(rotated + (int64_t)row * k + first + 4 * i);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const float values[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
        *reinterpret_cast<uint32_t*>(q + (int64_t)row * k + first + 4 * i) = quantise4(values, scale, inverse);
    }
}

// The rotation alone (kernels/cuda/model/integer_vq.py:447-486): Y = fp16(rotated * 128^-1/2), the
// values rotate_a8_kernel quantises.  Same lane layout; nothing is kept in LDS.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void rotate_kernel(const __half* __restrict__ x, const int8_t* __restrict__ signs,
                                                     __half* __restrict__ y, int k) {
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half_wave = lane >> 5, l32 = lane & 31;
    const int blocks = k / 128;
    const int64_t in_base = (int64_t)row * (SWIGLU ? 2 * k : k);
    for (int pair = wave; 2 * pair < blocks; pair += 4) {  // wave-uniform trip count
        const int block = 2 * pair + half_wave;
        const bool live = block < blocks;
        const int first = (live ? block : 0) * 128 + 4 * l32;
        const uint2 raw = *reinterpret_cast<const uint2*>(x + in_base + first);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const uint32_t sign_word = *reinterpret_cast<const uint32_t*>(signs + first);
        uint2 raw_up = make_uint2(0u, 0u);
        if (SWIGLU) raw_up = *reinterpret_cast<const uint2*>(x + in_base + k + first);
        const __half* up = reinterpret_cast<const __half*>(&raw_up);
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float value = SWIGLU ? swiglu_value(h[j], up[j]) : __half2float(h[j]);
            v[j] = live ? value * (float)(int8_t)(sign_word >> (8 * j)) : 0.f;
        }
        __half out[4];
        rotate_block(v, l32, out);
        if (live) *reinterpret_cast<uint2*>(y + (int64_t)row * k + first) = *reinterpret_cast<const uint2*>(out);
    }
}

__device__ __forceinline__ float block_sum(float v, float* scratch) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

// Residual add + RMSNorm in front of the rotation, one workgroup per row, same lane layout as
// rotate_a8_kernel.  First pass: RO = fp32(X) + R, sum of squares.  Second pass: the fp32 sum (kept
// in registers, or read back by the thread that wrote it where the row is longer than the registers
// hold), Y = fp16((sum * rsqrt(mean + eps)) * (W + offset)), and that fp16 value goes through signs,
// butterflies and A8 as if rotate_a8_kernel had read Y.
__global__ __launch_bounds__(256) void residual_norm_rotate_a8_kernel(
    const __half* __restrict__ x, const float* __restrict__ r, const __half* __restrict__ w, __half* __restrict__ y,
    float* __restrict__ ro, const int8_t* __restrict__ signs, int8_t* __restrict__ q, __half* __restrict__ s, int k,
    float epsilon, float weight_offset) {
    extern __shared__ __align__(16) __half rotated[];  // k halves
    __shared__ float scratch[4], sum_scratch[4];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half_wave = lane >> 5, l32 = lane & 31;
    const int blocks = k / 128;  // even: k is a multiple of 256
    const int64_t base = (int64_t)row * k;
    float squares = 0.f;
    // The first kHeld steps of a wave (all of them up to K = 5120): every load of both passes leaves
    // at once, and the fp32 sums stay in registers for the second pass.  Longer rows go on in the
    // loops below, which read their sums back.
    constexpr int kHeld = 5;
    float4 kept[kHeld];
    uint2 held_w[kHeld];
    uint32_t held_sign[kHeld];
    {
        uint2 raw[kHeld];
        float4 residual[kHeld];
#pragma unroll
        for (int u = 0; u < kHeld; ++u) {  // clamped, so unconditional (blocks is even: a pair is live or not as a whole)
            const int first = (min(2 * (wave + 4 * u), blocks - 2) + half_wave) * 128 + 4 * l32;
            raw[u] = *reinterpret_cast<const uint2*>(x + base + first);
            residual[u] = *reinterpret_cast<const float4*>(r + base + first);
            held_w[u] = *reinterpret_cast<const uint2*>(w + first);
            held_sign[u] = *reinterpret_cast<const uint32_t*>(signs + first);
        }
#pragma unroll
        for (int u = 0; u < kHeld; ++u) {
            if (2 * (wave + 4 * u) >= blocks) break;  // wave-uniform
            const int first = (2 * (wave + 4 * u) + half_wave) * 128 + 4 * l32;
            const __half* h = reinterpret_cast<const __half*>(&raw[u]);
            float4 sum;
            sum.x = __half2float(h[0]) + residual[u].x;
            sum.y = __half2float(h[1]) + residual[u].y;
            sum.z = __half2float(h[2]) + residual[u].z;
            sum.w = __half2float(h[3]) + residual[u].w;
            *reinterpret_cast<float4*>(ro + base + first) = sum;
            kept[u] = sum;
            squares += sum.x * sum.x;
            squares += sum.y * sum.y;
            squares += sum.z * sum.z;
            squares += sum.w * sum.w;
        }
    }
    for (int pair = wave + 4 * kHeld; 2 * pair < blocks; pair += 4) {
        const int first = (2 * pair + half_wave) * 128 + 4 * l32;
        const uint2 raw = *reinterpret_cast<const uint2*>(x + base + first);
        const __half* h = reinterpret_cast<const __half*>(&raw);
        const float4 residual = *reinterpret_cast<const float4*>(r + base + first);
        float4 sum;
        sum.x = __half2float(h[0]) + residual.x;
        sum.y = __half2float(h[1]) + residual.y;
        sum.z = __half2float(h[2]) + residual.z;
        sum.w = __half2float(h[3]) + residual.w;
        *reinterpret_cast<float4*>(ro + base + first) = sum;
        squares += sum.x * sum.x;
        squares += sum.y * sum.y;
        squares += sum.z * sum.z;
        squares += sum.w * sum.w;
    }
    const float total = block_sum(squares, sum_scratch);
    const float inverse = rsqrtf(__fdiv_rn(total, (float)k) + epsilon);
    float amax = 0.f;
    auto second_pass = [&](int first, const float4& sum, const uint2& raw_w, uint32_t sign_word) {
        const __half* weight = reinterpret_cast<const __half*>(&raw_w);
        const float values[4] = {sum.x, sum.y, sum.z, sum.w};
        __half normalized[4];
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float scaled = values[j] * inverse;
            asm volatile("" : "+v"(scaled));  // two roundings, as written: (sum * inverse) * weight
            float product = scaled * (__half2float(weight[j]) + weight_offset);
            asm volatile("" : "+v"(product));
            normalized[j] = __float2half_rn(product);
            v[j] = __half2float(normalized[j]) * (float)(int8_t)(sign_word >> (8 * j));
        }
        *reinterpret_cast<uint2*>(y + base + first) = *reinterpret_cast<const uint2*>(normalized);
        __half out[4];
        amax = fmaxf(amax, rotate_block(v, l32, out));
        *reinterpret_cast<uint2*>(rotated + first) = *reinterpret_cast<const uint2*>(out);
    };
#pragma unroll
    for (int u = 0; u < kHeld; ++u) {
        if (2 * (wave + 4 * u) >= blocks) break;  // wave-uniform
        second_pass((2 * (wave + 4 * u) + half_wave) * 128 + 4 * l32, kept[u], held_w[u], held_sign[u]);
    }
    for (int pair = wave + 4 * kHeld; 2 * pair < blocks; pair += 4) {
        const int first = (2 * pair + half_wave) * 128 + 4 * l32;
        const float4 sum = *reinterpret_cast<const float4*>(ro + base + first);  // written above by this thread
        const uint2 raw_w = *reinterpret_cast<const uint2*>(w + first);
        const uint32_t sign_word = *reinterpret_cast<const uint32_t*>(signs + first);
        second_pass(first, sum, raw_w, sign_word);
    }
    amax = block_max(amax, scratch);  // includes the barrier that publishes `rotated`
    quantise_row(rotated, amax, q, s, row, k);
}

// One workgroup per token; same lane layout as the rotation above (4 consecutive channels per lane,
// two blocks of 128 per wave step).  The bank is (hidden/128, vocab, 16) u32: one code holds 8
// channels, so a lane needs one half of one code.
__global__ __launch_bounds__(256) void q4_embedding_kernel(const int32_t* __restrict__ ids, const uint32_t* __restrict__ bank,
                                                           const uint32_t* __restrict__ book, const __half* __restrict__ scale,
                                                           const int8_t* __restrict__ signs, __half* __restrict__ out,
                                                           int vocab, int hidden) {
    __shared__ Q4ByteTables tables;
    build_tables(tables, book, threadIdx.x, 256);
    __syncthreads();
    const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half_wave = lane >> 5, l32 = lane & 31;
    const int blocks = hidden / 128;
    const int id = ids[row];
    const bool valid = id >= 0 && id < vocab;
    const float row_scale = valid ? __half2float(scale[id]) : 0.f;
    for (int pair = wave; 2 * pair < blocks; pair += 4) {
        const int block = 2 * pair + half_wave;
        const bool live = block < blocks;
        const int first = (live ? block : 0) * 128 + 4 * l32;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (valid && live) {
            const uint32_t code = bank[((int64_t)block * vocab + id) * 16 + (l32 >> 1)];
            const uint2 weights = decode_q4(tables, code);
            const uint32_t word = (l32 & 1) ? weights.y : weights.x;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (float)(int8_t)(word >> (8 * j));
        }
        {
            const float a = v[0] + v[1], b = v[0] - v[1], c = v[2] + v[3], d = v[2] - v[3];
            v[0] = a + c, v[2] = a - c, v[1] = b + d, v[3] = b - d;
        }
#pragma unroll
        for (int bit = 0; bit < 5; ++bit) {
            const bool upper = (l32 >> bit) & 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float other = __shfl_xor(v[j], 1 << bit, 64);
                v[j] = upper ? other - v[j] : other + v[j];
            }
        }
        if (live) {
            const uint32_t sign_word = *reinterpret_cast<const uint32_t*>(signs + first);
            __half result[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float value = ((v[j] * 0.08838834764831845f) * row_scale) * (float)(int8_t)(sign_word >> (8 * j));
                asm volatile("" : "+v"(value));  // the cast rounds the fp32 value, never a fused multiply-convert
                result[j] = __float2half_rn(value);
            }
            *reinterpret_cast<uint2*>(out + (int64_t)row * hidden + first) = *reinterpret_cast<const uint2*>(result);
        }
    }
}

// fp16 [rows, 2I] -> fp16 [rows, I].  grid (rows, ceil(I/256)).
__global__ __launch_bounds__(256) void swiglu_kernel(const __half* __restrict__ x, __half* __restrict__ y, int width) {
    const int row = blockIdx.x;
    const int col = blockIdx.y * 256 + threadIdx.x;
    if (col < width) {
        const int64_t base = (int64_t)row * 2 * width;
        y[(int64_t)row * width + col] = __float2half_rn(swiglu_value(x[base + col], x[base + width + col]));
    }
}

// ---- host side -----------------------------------------------------------------------------
// slots used: K, group, flags (bit0 masked, bit1 fused), capacity
// few rows of long groups (decode): 16 waves per group, one 16-byte piece per thread
bool a8_wide(const orx_function& f, int rows) { return f.flags == 0 && rows <= 256 && f.group >= 4096; }
// short groups, no mask: one wave per group
bool a8_per_wave(const orx_function& f) { return !(f.flags & 1) && f.group <= 512; }
// many rows of long groups: the pieces wait in LDS between the two passes (9 to 48 KiB per group: at least three of the four pieces a thread requests at once are real)
bool a8_staged(const orx_function& f, int rows) {
    return f.flags == 0 && !a8_wide(f, rows) && f.group % 8 == 0 && f.group >= 4608 && f.group <= 24576;
}

int a8_geometry(const orx_function& f, int rows, Geometry* g) {
    const uint32_t groups = ceil_div((uint32_t)f.K, (uint32_t)f.group);
    if (a8_per_wave(f)) {
        g->grid[0] = ceil_div((uint32_t)rows * groups, 4u);
        g->block[0] = 256;
        return ORX_OK;
    }
    g->grid[0] = (uint32_t)rows;
    g->grid[1] = groups;
    g->block[0] = a8_wide(f, rows) ? 1024 : 256;
    g->shared = a8_staged(f, rows) ? (uint32_t)f.group * 2u : 0u;
    return ORX_OK;
}

int a8_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    const uint8_t* mask = pointer_arg<const uint8_t>(args, 0);
    int8_t* q = pointer_arg<int8_t>(args, 1);
    __half* s = pointer_arg<__half>(args, 2);
    const __half* x = pointer_arg<const __half>(args, 3);
    const dim3 grid(g.grid[0], g.grid[1]), block(256);
    const int groups = (int)ceil_div((uint32_t)f.K, (uint32_t)f.group);
    const bool masked = f.flags & 1, fused = f.flags & 2;
    if (a8_per_wave(f)) {
        if (fused)
            ORX_LAUNCH((a8_wave_kernel<true>), grid, block, 0, stream, x, q, s, f.K, f.group, groups, rows);
        else
            ORX_LAUNCH((a8_wave_kernel<false>), grid, block, 0, stream, x, q, s, f.K, f.group, groups, rows);
    } else if (g.block[0] == 1024)
        ORX_LAUNCH((a8_kernel<false, false, 1024>), grid, dim3(1024), 0, stream, x, mask, q, s, f.K, f.group, groups);
    else if (g.shared > 0)
        ORX_LAUNCH((a8_kernel<false, false, 256, true>), grid, block, g.shared, stream, x, mask, q, s, f.K, f.group, groups);
    else if (fused && masked)
        ORX_LAUNCH((a8_kernel<true, true>), grid, block, 0, stream, x, mask, q, s, f.K, f.group, groups);
    else if (fused)
        ORX_LAUNCH((a8_kernel<true, false>), grid, block, 0, stream, x, mask, q, s, f.K, f.group, groups);
    else if (masked)
        ORX_LAUNCH((a8_kernel<false, true>), grid, block, 0, stream, x, mask, q, s, f.K, f.group, groups);
    else
        ORX_LAUNCH((a8_kernel<false, false>), grid, block, 0, stream, x, mask, q, s, f.K, f.group, groups);
    return hip_check(hipGetLastError(), "launch activation_quantization");
}

int make_a8(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("K", 0, &bad);
    f->group = (int)v.integer("group_size", f->K, &bad);
    const bool masked = v.boolean("masked", false, &bad);
    const bool fused = v.boolean("fused", false, &bad);
    f->capacity = (int)v.integer("M", 1 << 24, &bad);
    // op30_activation_quantization.py:84: a block size of the reference's kernel; the block here follows the row
    const int threads = (int)v.integer("threads", 256, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->K <= 0 || f->group <= 0 || f->group > f->K || f->capacity < 1) {
        set_error("activation_quantization: need K > 0 and 0 < group_size <= K");
        return ORX_ERR_BAD_VARIANT;
    }
    if (threads != 128 && threads != 256 && threads != 512) {
        set_error("activation_quantization: threads is 128, 256 or 512");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = (masked ? 1 : 0) | (fused ? 2 : 0);
    f->dynamic_rows = true;
    // Mask may be null unless masked (the reference ignores it then, op30:75-76)
    f->args = {{"Mask", ArgPointer, masked ? 1u : 0x80000001u}, {"Q", ArgPointer, 1}, {"S", ArgPointer, 2},
               {"X", ArgPointer, 2}, {"rows", ArgI32, 4}};
    f->device_function = nullptr;  // kernels with 256 and 1024 threads serve this symbol
    f->geometry = a8_geometry;
    f->launch = a8_launch;
    return ORX_OK;
}

// slots used: K, flags (bit1 swiglu), capacity
int rotate_a8_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    // few rows (decode): 16 waves share one row, so that a row is one or two steps per wave
    g->block[0] = rows <= kRotateWideRows && f.K >= 2048 ? 1024 : 256;
    g->shared = (uint32_t)f.K * 2;
    return ORX_OK;
}

// Q, S, Signs, X[, m]   (crates/orinfer-models/src/flash_next/q4.rs:176-196 binds rotation as Q, S, Signs, X)
int rotate_a8_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    int8_t* q = pointer_arg<int8_t>(args, 0);
    __half* s = pointer_arg<__half>(args, 1);
    const int8_t* signs = pointer_arg<const int8_t>(args, 2);
    const __half* x = pointer_arg<const __half>(args, 3);
    const dim3 grid(g.grid[0]), block(g.block[0]);
    if (g.block[0] == 1024) {
        if (f.flags & 2)
            ORX_LAUNCH((rotate_a8_kernel<true, 1024>), grid, block, g.shared, stream, x, signs, q, s, f.K);
        else
            ORX_LAUNCH((rotate_a8_kernel<false, 1024>), grid, block, g.shared, stream, x, signs, q, s, f.K);
    } else if (f.flags & 2) {
        ORX_LAUNCH((rotate_a8_kernel<true>), grid, block, g.shared, stream, x, signs, q, s, f.K);
    } else {
        ORX_LAUNCH((rotate_a8_kernel<false>), grid, block, g.shared, stream, x, signs, q, s, f.K);
    }
    return hip_check(hipGetLastError(), "launch rotate_activation_a8");
}

int make_rotate_a8(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("K", 0, &bad);
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const bool swiglu = v.boolean("swiglu", false, &bad);
    // rotation_a8.py:373-383: reciprocal picks one of two roundings that give the same codes (the reciprocal one
    // divides near ties), registers picks where the reference's kernel keeps the butterflies
    v.boolean("reciprocal", true, &bad);
    v.boolean("registers", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    // rotation_a8.py:425-427: K a positive multiple of 128; the row has to fit LDS as fp16
    if (f->M <= 0 || f->K <= 0 || f->K % 128 || f->K > 32768) {
        set_error("rotate_activation_a8: need M > 0 and K a multiple of 128 up to 32768");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = swiglu ? 2 : 0;
    // 8-byte loads of X, 4-byte loads of Signs and stores of Q
    f->args = {{"Q", ArgPointer, 4}, {"S", ArgPointer, 2}, {"Signs", ArgPointer, 4}, {"X", ArgPointer, 8}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    // kernels with 256 and 1024 threads serve this symbol: report the device-wide limits
    f->device_function = nullptr;
    f->geometry = rotate_a8_geometry;
    f->launch = rotate_a8_launch;
    return ORX_OK;
}

// rotate_expert_a8: buffers in ASCII order, looked up by name (the list depends on the routing and on the hand-over).
// slots used: K, top_k, E, flags (bit1 swiglu, bit2 K64-major planes), algorithm (routing).
int rotate_expert_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    auto find = [&](const char* name) -> void* {
        for (size_t i = 0; i < f.args.size(); ++i)
            if (!strcmp(f.args[i].name, name)) return pointer_arg<void>(args, (int)i);
        return nullptr;
    };
    int8_t* q = static_cast<int8_t*>(find("Q"));
    int8_t* d = static_cast<int8_t*>(find("D"));
    __half* s = static_cast<__half*>(find("S"));
    __half* ds = static_cast<__half*>(find("DS"));
    const int* ids = static_cast<const int*>(find("IDs"));
    const int* relative = static_cast<const int*>(find("RelativeSlot"));
    const int* row_offsets = static_cast<const int*>(find("RowOffsets"));
    int* slot_map = static_cast<int*>(find("SlotMap"));
    int* sum = static_cast<int*>(find("Sum"));
    uint32_t* low = static_cast<uint32_t*>(find("Low"));
    uint32_t* high = static_cast<uint32_t*>(find("High"));
    const int8_t* signs = static_cast<const int8_t*>(find("Signs"));
    const __half* x = static_cast<const __half*>(find("X"));
    // planes have one row per slot under scatter, one per token otherwise; K64-major strides follow the live rows
    const int plane_rows = f.algorithm == kRouteScatter ? rows * f.top_k : rows;
    const int group_major = (f.flags & 4) ? 1 : 0;
    const dim3 grid(g.grid[0]), block(g.block[0]);
#define ORX_ROTATE_EXPERT(SW, TH)                                                                                      \
    ORX_LAUNCH((rotate_expert_kernel<SW, TH>), grid, block, g.shared, stream, x, signs, q, s, d, ds, ids,      \
                       relative, row_offsets, slot_map, sum, low, high, plane_rows, group_major, f.K, f.top_k, f.algorithm)
    if (g.block[0] == 1024) {
        if (f.flags & 2) ORX_ROTATE_EXPERT(true, 1024);
        else ORX_ROTATE_EXPERT(false, 1024);
    } else if (f.flags & 2) {
        ORX_ROTATE_EXPERT(true, 256);
    } else {
        ORX_ROTATE_EXPERT(false, 256);
    }
#undef ORX_ROTATE_EXPERT
    return hip_check(hipGetLastError(), "launch rotate_expert_a8");
}

int make_rotate_expert(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("K", 0, &bad);
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    f->top_k = (int)v.integer("top_k", 1, &bad);
    f->E = (int)v.integer("experts", 1, &bad);
    const bool swiglu = v.boolean("swiglu", false, &bad);
    v.boolean("reciprocal", true, &bad);  // both forms of the reference give the same codes (the reciprocal one divides near ties)
    const bool group_major = v.boolean("group_major", false, &bad);
    const std::string routing = v.string("routing", "none", &bad);
    // planes: the reference's buffers (Low, High for its INT4 expert GEMMs); int8: whole rows for the int8 expert GEMMs
    const std::string hand_over = v.string("hand_over", "planes", &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->K <= 0 || f->K % 128 || f->K > 32768) {
        set_error("rotate_expert_a8: need M > 0 and K a multiple of 128 up to 32768");
        return ORX_ERR_BAD_VARIANT;
    }
    if (routing != "none" && routing != "shared" && routing != "scatter") {
        set_error("rotate_expert_a8: routing must be none, shared or scatter");
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->top_k < 1 || f->top_k > f->E || f->top_k > kMaxRouteChoices) {
        set_error("rotate_expert_a8: need 1 <= top_k <= experts and top_k <= %d", kMaxRouteChoices);
        return ORX_ERR_BAD_VARIANT;
    }
    if (hand_over != "planes" && hand_over != "int8") {
        set_error("rotate_expert_a8: hand_over must be planes or int8");
        return ORX_ERR_BAD_VARIANT;
    }
    const bool planes = hand_over == "planes";
    if (group_major && (routing != "none" || !planes)) {  // rotation_a8.py:409-410
        set_error("rotate_expert_a8: K64-major planes need contiguous expert rows (no routing) and hand_over=planes");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = (swiglu ? 2 : 0) | (group_major ? 4 : 0);
    f->algorithm = routing == "scatter" ? kRouteScatter : routing == "shared" ? kRouteShared : 0;
    const uint32_t nullable = 0x80000000u;
    const ArgSpec high = {"High", ArgPointer, 4}, low = {"Low", ArgPointer, 4};
    if (f->algorithm == 0) {
        // rotate_split_a8: X, Signs, Q, S, Low, High, Sum; rotate_pack_a8 (K64-major) has no Q (rotation_a8.py:536-571)
        if (planes) f->args = {high, low};
        if (!group_major) f->args.push_back({"Q", ArgPointer, 4});
        for (const ArgSpec& a : std::initializer_list<ArgSpec>{{"S", ArgPointer, 2}, {"Signs", ArgPointer, 4},
                                                               {"Sum", ArgPointer, nullable | 4u}, {"X", ArgPointer, 8}})
            f->args.push_back(a);
    } else {
        // rotate_dispatch_a8 (rotation_a8.py:573-604); the int8 hand-over has D (scatter) in place of Low and High
        if (!planes && f->algorithm == kRouteScatter) f->args.push_back({"D", ArgPointer, 4});
        f->args.push_back({"DS", ArgPointer, 2});
        if (planes) f->args.push_back(high);
        f->args.push_back({"IDs", ArgPointer, 4});
        if (planes) f->args.push_back(low);
        const uint32_t q_align = f->algorithm == kRouteScatter ? nullable | 4u : 4u;
        for (const ArgSpec& a : std::initializer_list<ArgSpec>{{"Q", ArgPointer, q_align}, {"RelativeSlot", ArgPointer, 4},
                                                               {"RowOffsets", ArgPointer, 4}, {"S", ArgPointer, 2},
                                                               {"Signs", ArgPointer, 4}, {"SlotMap", ArgPointer, 4},
                                                               {"Sum", ArgPointer, nullable | 4u}, {"X", ArgPointer, 8}})
            f->args.push_back(a);
    }
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = nullptr;  // 256- and 1024-thread kernels serve this symbol
    f->geometry = rotate_a8_geometry;
    f->launch = rotate_expert_launch;
    return ORX_OK;
}

// slots used: K, flags (bit1 swiglu)
int rotate_geometry(const orx_function&, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->block[0] = 256;
    return ORX_OK;
}
// Signs, X, Y (integer_vq.py:454-458 in generated-ABI order)
int rotate_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    const int8_t* signs = pointer_arg<const int8_t>(args, 0);
    const __half* x = pointer_arg<const __half>(args, 1);
    __half* y = pointer_arg<__half>(args, 2);
    if (f.flags & 2)
        ORX_LAUNCH((rotate_kernel<true>), dim3(g.grid[0]), dim3(256), 0, stream, x, signs, y, f.K);
    else
        ORX_LAUNCH((rotate_kernel<false>), dim3(g.grid[0]), dim3(256), 0, stream, x, signs, y, f.K);
    return hip_check(hipGetLastError(), "launch rotate_activation");
}
int make_rotate(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("K", 0, &bad);
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    const bool swiglu = v.boolean("swiglu", false, &bad);
    if (bad || f->M <= 0 || f->K <= 0 || f->K % 128) {
        set_error("rotate_activation: invalid block-128 activation rotation");  // integer_vq.py:449-450
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = swiglu ? 2 : 0;
    f->args = {{"Signs", ArgPointer, 4}, {"X", ArgPointer, 8}, {"Y", ArgPointer, 8}};
    f->device_function = reinterpret_cast<const void*>(&rotate_kernel<false>);
    f->geometry = rotate_geometry;
    f->launch = rotate_launch;
    return ORX_OK;
}

// slots used: K, flags (bit0: weights stored zero-centred), capacity
int residual_rotate_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->block[0] = 256;
    g->shared = (uint32_t)f.K * 2;
    return ORX_OK;
}

// Q, R, RO, S, Signs, W, X, Y[, m]: the buffers of rotation_a8.py:621-630 in generated-ABI order
int residual_rotate_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    int8_t* q = pointer_arg<int8_t>(args, 0);
    const float* r = pointer_arg<const float>(args, 1);
    float* ro = pointer_arg<float>(args, 2);
    __half* s = pointer_arg<__half>(args, 3);
    const int8_t* signs = pointer_arg<const int8_t>(args, 4);
    const __half* w = pointer_arg<const __half>(args, 5);
    const __half* x = pointer_arg<const __half>(args, 6);
    __half* y = pointer_arg<__half>(args, 7);
    ORX_LAUNCH(residual_norm_rotate_a8_kernel, dim3(g.grid[0]), dim3(256), g.shared, stream, x, r, w, y, ro, signs,
                       q, s, f.K, 1e-6f, (f.flags & 1) ? 1.0f : 0.0f);
    return hip_check(hipGetLastError(), "launch residual_norm_rotate_a8");
}

// rotate_activation_tiles / quantize_rotation_tiles.  slots used: K, group (block_k), flags (bit1 swiglu), slots (plane_rows)
int tiles_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->grid[1] = ceil_div((uint32_t)f.K, (uint32_t)f.group);
    g->block[0] = 256;
    return ORX_OK;
}
// Maxima, Rotated, Signs, X[, m]
int rotate_tiles_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    float* maxima = pointer_arg<float>(args, 0);
    __half* rotated = pointer_arg<__half>(args, 1);
    const int8_t* signs = pointer_arg<const int8_t>(args, 2);
    const __half* x = pointer_arg<const __half>(args, 3);
    const dim3 grid(g.grid[0], g.grid[1]), block(256);
    if (f.flags & 2) {
        const int64_t stride = f.slots ? f.K : 2 * (int64_t)f.K, up = f.slots ? (int64_t)f.slots * f.K : f.K;
        ORX_LAUNCH((rotate_tiles_kernel<true>), grid, block, 0, stream, x, signs, rotated, maxima, f.K, f.group, stride, up);
    } else {
        ORX_LAUNCH((rotate_tiles_kernel<false>), grid, block, 0, stream, x, signs, rotated, maxima, f.K, f.group,
                           (int64_t)f.K, (int64_t)0);
    }
    return hip_check(hipGetLastError(), "launch rotate_activation_tiles");
}
// Maxima, Q, Rotated, S[, m]
int quantize_tiles_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    ORX_LAUNCH(quantize_tiles_kernel, dim3(g.grid[0], g.grid[1]), dim3(256), 0, stream, pointer_arg<const __half>(args, 2),
                       pointer_arg<const float>(args, 0), pointer_arg<int8_t>(args, 1), pointer_arg<__half>(args, 3), f.K, f.group);
    return hip_check(hipGetLastError(), "launch quantize_rotation_tiles");
}
bool tile_shape_ok(const orx_function& f) {
    const int bk = f.group;
    return f.M > 0 && f.K > 0 && f.K % 128 == 0 && (bk == 128 || bk == 256 || bk == 512 || bk == 1024 || bk == 2048);
}
int make_rotate_tiles(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->group = (int)v.integer("block_k", 512, &bad);
    const bool swiglu = v.boolean("swiglu", false, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    f->slots = (int)v.integer("plane_rows", 0, &bad);
    const bool registers = v.boolean("registers", false, &bad);
    const int threads = (int)v.integer("threads", 128, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!tile_shape_ok(*f)) {  // rotation_a8.py:279-280
        set_error("rotate_activation_tiles: need M > 0, K a multiple of 128 and block_k 128, 256, 512, 1024 or 2048");
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->slots < 0 || (f->slots && (!swiglu || f->slots < f->M))) {  // rotation_a8.py:281-286
        set_error("rotate_activation_tiles: plane_rows needs swiglu and at least M rows");
        return ORX_ERR_BAD_VARIANT;
    }
    // rotation_a8.py:227-228, :287-288: block sizes of the reference's two kernels; the block here is 256 threads
    if ((!registers && threads != 128) ||
        (registers && ((threads != 64 && threads != 128 && threads != 256 && threads != 512) || f->group % (threads * 4)))) {
        set_error("rotate_activation_tiles: threads is 128, or with registers 64..512 with block_k a multiple of 4 threads");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = swiglu ? 2 : 0;
    f->args = {{"Maxima", ArgPointer, 4}, {"Rotated", ArgPointer, 8}, {"Signs", ArgPointer, 4}, {"X", ArgPointer, 8}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = swiglu ? reinterpret_cast<const void*>(&rotate_tiles_kernel<true>)
                                : reinterpret_cast<const void*>(&rotate_tiles_kernel<false>);
    f->geometry = tiles_geometry;
    f->launch = rotate_tiles_launch;
    return ORX_OK;
}
int make_quantize_tiles(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->group = (int)v.integer("block_k", 512, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!tile_shape_ok(*f)) {  // rotation_a8.py:332-333
        set_error("quantize_rotation_tiles: need M > 0, K a multiple of 128 and block_k 128, 256, 512, 1024 or 2048");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"Maxima", ArgPointer, 4}, {"Q", ArgPointer, 4}, {"Rotated", ArgPointer, 8}, {"S", ArgPointer, 2}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = reinterpret_cast<const void*>(&quantize_tiles_kernel);
    f->geometry = tiles_geometry;
    f->launch = quantize_tiles_launch;
    return ORX_OK;
}

int make_residual_rotate(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("K", 5120, &bad);
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const bool zero_centered = v.boolean("zero_centered", true, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    // rotation_a8.py:612-613: complete 256-column tiles; the row has to fit LDS as fp16
    if (f->M <= 0 || f->K <= 0 || f->K % 256 || f->K > 32768) {
        set_error("residual_norm_rotate_a8: need M > 0 and K a multiple of 256 up to 32768");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = zero_centered ? 1 : 0;
    // 16-byte accesses of R and RO, 8-byte of X, W and Y, 4-byte of Signs and Q
    f->args = {{"Q", ArgPointer, 4},     {"R", ArgPointer, 16}, {"RO", ArgPointer, 16}, {"S", ArgPointer, 2},
               {"Signs", ArgPointer, 4}, {"W", ArgPointer, 8},  {"X", ArgPointer, 8},   {"Y", ArgPointer, 8}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = reinterpret_cast<const void*>(&residual_norm_rotate_a8_kernel);
    f->geometry = residual_rotate_geometry;
    f->launch = residual_rotate_launch;
    return ORX_OK;
}

// slots used: N (vocab), K (hidden), capacity
int q4_embedding_geometry(const orx_function&, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->block[0] = 256;
    return ORX_OK;
}

// Book, IDs, Output, Scale, Signs, Weight, m   (e8p_q4.py:95-102 in generated-ABI order)
int q4_embedding_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    ORX_LAUNCH(q4_embedding_kernel, dim3(g.grid[0]), dim3(256), 0, stream, pointer_arg<const int32_t>(args, 1),
                       pointer_arg<const uint32_t>(args, 5), pointer_arg<const uint32_t>(args, 0),
                       pointer_arg<const __half>(args, 3), pointer_arg<const int8_t>(args, 4), pointer_arg<__half>(args, 2),
                       f.N, f.K);
    return hip_check(hipGetLastError(), "launch e8p_q4_embedding");
}

int make_q4_embedding(const Variant& v, orx_function* f) {
    if (!two_stage_coefficients_ok(v, "e8p_q4_embedding")) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    // the reference's factory calls the row capacity `capacity` (kernels/cuda/model/e8p_q4.py:84)
    f->capacity = f->M = (int)v.integer(v.has("capacity") ? "capacity" : "M", 0, &bad);
    f->N = (int)v.integer("vocab", 0, &bad);
    f->K = (int)v.integer("hidden", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->N <= 0 || f->K <= 0 || f->K % 128) {
        set_error("e8p_q4_embedding: need M > 0, vocab > 0 and hidden a multiple of 128");
        return ORX_ERR_BAD_VARIANT;
    }
    f->dynamic_rows = true;  // the reference kernel always takes the live row count
    f->args = {{"Book", ArgPointer, 4}, {"IDs", ArgPointer, 4}, {"Output", ArgPointer, 8}, {"Scale", ArgPointer, 2},
               {"Signs", ArgPointer, 4}, {"Weight", ArgPointer, 4}, {"m", ArgI32, 4}};
    f->device_function = reinterpret_cast<const void*>(&q4_embedding_kernel);
    f->geometry = q4_embedding_geometry;
    f->launch = q4_embedding_launch;
    return ORX_OK;
}

int swiglu_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->grid[1] = ceil_div((uint32_t)f.N, 256u);
    g->block[0] = 256;
    return ORX_OK;
}

int swiglu_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    ORX_LAUNCH(swiglu_kernel, dim3(g.grid[0], g.grid[1]), dim3(256), 0, stream,
                       pointer_arg<const __half>(args, 0), pointer_arg<__half>(args, 1), f.N);
    return hip_check(hipGetLastError(), "launch swiglu");
}

int make_swiglu(const Variant& v, orx_function* f) {
    bool bad = false;
    f->N = (int)v.integer("I", 0, &bad);
    f->capacity = (int)v.integer("M", 1 << 24, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->N <= 0) {
        set_error("swiglu: need I > 0");
        return ORX_ERR_BAD_VARIANT;
    }
    f->dynamic_rows = true;
    f->args = {{"X", ArgPointer, 2}, {"Y", ArgPointer, 2}, {"rows", ArgI32, 4}};
    f->device_function = reinterpret_cast<const void*>(&swiglu_kernel);
    f->geometry = swiglu_geometry;
    f->launch = swiglu_launch;
    return ORX_OK;
}

}  // namespace

const Registration* quant_registrations(int* count) {
    static const Registration rows[] = {
    {"activation_quantization", make_a8, "K, group_size=null, masked=false, fused=false, threads=256, M=capacity",
     "Mask,Q,S,X,rows"},
    {"swiglu", make_swiglu, "I, M=capacity", "X,Y,rows"},
    {"rotate_activation_a8", make_rotate_a8, "M, K, swiglu=false, reciprocal=true, dynamic_rows=false, registers=false", "Q,S,Signs,X[,m]"},
    {"rotate_expert_a8", make_rotate_expert,
     "M, K, swiglu=false, reciprocal=true, dynamic_rows=false, routing=none|shared|scatter, top_k=1, experts=1, "
     "group_major=false, hand_over=planes|int8",
     "DS,High,IDs,Low,Q,RelativeSlot,RowOffsets,S,Signs,SlotMap,Sum,X[,m] (no routing: High,Low,Q,S,Signs,Sum,X[,m]; "
     "group_major: no Q; hand_over=int8: no High, Low and D first under scatter)"},
    {"rotate_activation", make_rotate, "M, K, swiglu=false", "Signs,X,Y"},
    {"rotate_activation_tiles", make_rotate_tiles,
     "M, K, block_k=512, swiglu=false, dynamic_rows=false, plane_rows=0, registers=false, threads=128", "Maxima,Rotated,Signs,X[,m]"},
    {"quantize_rotation_tiles", make_quantize_tiles, "M, K, block_k=512, dynamic_rows=false", "Maxima,Q,Rotated,S[,m]"},
    {"residual_norm_rotate_a8", make_residual_rotate, "M, K=5120, dynamic_rows=false, zero_centered=true",
     "Q,R,RO,S,Signs,W,X,Y[,m]"},
    {"e8p_q4_embedding", make_q4_embedding, "M (or capacity), vocab, hidden", "Book,IDs,Output,Scale,Signs,Weight,m"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
