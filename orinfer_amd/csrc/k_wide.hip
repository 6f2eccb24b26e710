// Two-stage (Q4) projections for 65..128 token rows (any row count by name): one resident workgroup per CU,
// no split over K.
//
// Reference counterparts: the Tensor Core schedules of kernels/cuda/model/integer_core.py:162-272 at
// block_m = 64..256 behind kernels/cuda/model/e8p_q4.py:143-264 (the row ranges a package asks for:
// python/orinfer_build/contracts/projection_policy.py:40-101).  Arithmetic: exact int32 accumulation
// over the full K, then (float(acc) * ws) * as.
//
// MI355X design.  At these row counts the output has a few hundred 128 x 128 tiles at most, fewer
// than two per CU, so tiles leave CUs idle and tiles cut over K leave partial sums to add.  Here
//  * output channels are dealt to the CUs in equal contiguous runs (N / CUs each, 68 at N = 17408);
//    a CU multiplies all token rows (128 per pass) by its run over the whole K: every code is read
//    and decoded once per 128 rows, nothing is summed across workgroups, and the activation tile,
//    which every CU reads, comes out of the L2 (85-110 GB/s per CU measured for data all CUs share);
//  * the twelve waves have roles.  Eight decoder waves keep the CU's codes of the next ten K steps in
//    registers, decode one step ahead (two 8-byte lookups per stage in tables stored 16 times, as in
//    k_dense.hip) and write int8 weights to LDS; four MFMA waves, one per SIMD, own 32 token rows
//    each: a row block belongs to one wave only, so its fragments never pass through LDS (a lane
//    loads the 64 bytes it needs of every K step straight from memory, three steps ahead), and the
//    wave multiplies them with up to 96 channels read from LDS (v_mfma_i32_32x32x32_i8).  One
//    barrier per K step.  A step takes 0.4-0.55 us (10 us of set-up and output per pass beside it):
//    ablations put that on the token loads (16 bytes of 32 different rows per instruction take a
//    memory-pipe slot per lane; with the loads or the decode alone switched off nothing changes,
//    with both 0.33 us) and equally on the decode of the SIMD that hosts two busy decoder waves.
//    A form with loader waves (global_load_lds into four LDS stages), four decoder waves with
//    balanced shares and MFMA waves that split a step over its K halves measured slower (37.9
//    against 32.0 us at N = 17408, K = 5120, 128 rows) and is not kept;
//  * the weight tile uses the 16-byte chunk swizzle of k_gemm_big.hip, so fragment reads of sixteen
//    consecutive rows fall into sixteen bank groups;
//  * the rescaled results of a pass go through an LDS image and are stored by all waves, four
//    channels of a row per thread: a CU's run is narrow (136 bytes of fp16 per row at N = 17408),
//    and element-wise stores straight from the accumulators cost 8 us per pass.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kRows = 128;      // token rows per pass
constexpr int kStep = 128;      // K per step
constexpr int kChannels = 96;   // channels per pass: three MFMA blocks
constexpr int kMfmaWaves = 4, kDecoderWaves = 8;
constexpr int kThreads = (kMfmaWaves + kDecoderWaves) * 64;
constexpr uint32_t kMaskOffset = 128;            // tables: entry i at i*256 (basis) and i*256 + 128 (mask), 16 copies of 8 bytes
constexpr uint32_t kTableBytes = 65536;
constexpr int kWeightStages = 2;
constexpr uint32_t kWeightStage = kChannels * kStep;  // 12 KiB
constexpr uint32_t kWeightBase = kTableBytes;
constexpr int kImagePitch = kChannels + 4;       // floats per row of the output image
constexpr uint32_t kImageBase = kWeightBase + kWeightStages * kWeightStage;
constexpr uint32_t kWideLdsBytes = kImageBase + kRows * kImagePitch * 4;
constexpr int kRing = 10;       // K steps of codes a decoder lane holds (4-6 KiB per step and CU: the stream needs about 48 KiB in flight per CU)
constexpr int kTokenRing = 3;   // K steps of token fragments an MFMA lane holds (four would spill)
static_assert(kWideLdsBytes <= 160 * 1024, "tables, two weight stages and the output image share the LDS");

struct WideParams {
    const int8_t* a;
    const uint8_t* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, m, out_f32, k_major;
};

// 16-byte chunk c of row r lives in slot c ^ ((r >> 1) & 7) of the row's 128 bytes
__device__ __forceinline__ int chunk_swizzle(int row) { return (row >> 1) & 7; }

// Every wave's LDS reads and writes have finished when it passes; loads from memory stay in flight.
__device__ __forceinline__ void step_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
template <bool KM>
__global__ __launch_bounds__(kThreads) void wide_kernel(WideParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int groups = (int)gridDim.x, group = (int)blockIdx.x;
    const int run = (p.n + groups - 1) / groups;  // channels per CU
    const int first_channel = group * run;
    const int channels_here = min(run, p.n - first_channel);
    if (channels_here <= 0) return;               // same for the whole workgroup
    const int steps = p.k / kStep;
    const bool is_mfma = wave < kMfmaWaves;

    // ---- tables (decoder waves 0-3 the basis table, 4-7 the mask table) ---------------------------
    if (!is_mfma) {
        const int dt = tid - kMfmaWaves * 64, entry = dt & 255;
        const bool basis = dt < 256;
        const uint32_t selector = basis ? p.book[entry] : 0u;
        const uint2 value = basis ? byte_basis_biased(selector, 0) : byte_mask_biased((uint32_t)entry, 0);
        const uint4 pair = make_uint4(value.x, value.y, value.x, value.y);
        uint8_t* dst = lds + entry * 256 + (basis ? 0 : kMaskOffset);
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(dst + 16 * i) = pair;
    }

    // decode of one u32 two-stage code to 8 int8 weights: w + 128 = 8 (v0 + 8) + 2 (v1 + 8) + 53 in every byte
    const uint32_t copy = (uint32_t)(lane & 15) * 8;
    const uint32_t columns = copy | (kMaskOffset | copy) << 8;
    constexpr uint32_t kBasisLow = 0x0C0C0500u, kMaskLow = 0x0C0C0401u, kBasisHigh = 0x0C0C0700u, kMaskHigh = 0x0C0C0601u;
    auto lookup = [&](uint32_t code, uint32_t selector) {
        return *reinterpret_cast<const uint2*>(lds + __builtin_amdgcn_perm(code, columns, selector));
    };
    auto decode = [&](uint32_t code) {
        const uint2 b0 = lookup(code, kBasisLow), m0 = lookup(code, kMaskLow);
        const uint2 b1 = lookup(code, kBasisHigh), m1 = lookup(code, kMaskHigh);
        uint2 w;
        w.x = ((((b0.x ^ m0.x) << 3) + ((b1.x ^ m1.x) << 1)) + 0x35353535u) ^ 0x80808080u;
        w.y = ((((b0.y ^ m0.y) << 3) + ((b1.y ^ m1.y) << 1)) + 0x35353535u) ^ 0x80808080u;
        return w;
    };

    // ---- output: the image of a pass, stored by all waves ------------------------------------------------
    float* image = reinterpret_cast<float*>(lds + kImageBase);
    auto store_image = [&](int row0, int rows, int channel0, int channels) {
        const int pieces = (channels + 3) / 4;
        const int element = p.out_f32 ? 4 : 2;
        for (int task = tid; task < rows * pieces; task += kThreads) {
            const int local = task / pieces, first = (task - local * pieces) * 4;
            const float4 v = *reinterpret_cast<const float4*>(image + local * kImagePitch + first);
            const int64_t index = (int64_t)(row0 + local) * p.stride + channel0 + first;
            char* dst = static_cast<char*>(p.out) + index * element;
            const bool whole = first + 3 < channels && (reinterpret_cast<uintptr_t>(dst) & (uintptr_t)(4 * element - 1)) == 0;
            const float values[4] = {v.x, v.y, v.z, v.w};
            if (p.out_f32) {
                if (whole) {
                    *reinterpret_cast<float4*>(dst) = v;
                } else {
                    for (int i = 0; i < 4; ++i)
                        if (first + i < channels) reinterpret_cast<float*>(dst)[i] = values[i];
                }
            } else {
                __half h[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) h[i] = __float2half_rn(values[i]);
                if (whole) {
                    uint2 packed;
                    packed.x = (uint32_t)__half_as_ushort(h[0]) | (uint32_t)__half_as_ushort(h[1]) << 16;
                    packed.y = (uint32_t)__half_as_ushort(h[2]) | (uint32_t)__half_as_ushort(h[3]) << 16;
                    *reinterpret_cast<uint2*>(dst) = packed;
                } else {
                    for (int i = 0; i < 4; ++i)
                        if (first + i < channels) reinterpret_cast<__half*>(dst)[i] = h[i];
                }
            }
        }
    };

    // Both roles run the same passes (128 token rows x up to 96 of the CU's channels) and the same
    // barriers; the roles branch first so that a wave carries only its own role's addresses.
#define ORX_WIDE_PASSES                                                  \
    for (int row0 = 0; row0 < p.m; row0 += kRows)                        \
        for (int c0 = 0; c0 < channels_here; c0 += kChannels)
    if (!is_mfma) {
        ORX_WIDE_PASSES {
            const int rows = min(kRows, p.m - row0);
            const int channels = min(kChannels, channels_here - c0);
            const int channel0 = first_channel + c0;
            (void)rows, (void)channels, (void)channel0;
            // ---- decoder waves: lane (channel, quarter of the K step) owns four codes = 32 weights -----
            int dl = tid - kMfmaWaves * 64;
            asm volatile("" : "+v"(dl));  // per pass, as in the MFMA waves below
            const int channel = dl >> 2, quarter = dl & 3;
            const bool active = channel < channels;
            const int source_channel = channel0 + min(channel, channels - 1);
            // (K-major blocks of 64: the two halves of a K step lie N rows x 32 bytes apart)
            const uint8_t* codes = !KM              ? p.w + (int64_t)source_channel * (p.k / 2) + quarter * 16
                                   : p.k_major == 2 ? p.w + (int64_t)source_channel * 32 + (quarter & 1) * 16 + (int64_t)(quarter >> 1) * p.n * 32
                                                    : p.w + (int64_t)source_channel * 64 + quarter * 16;
            const int64_t step_bytes = KM ? (int64_t)p.n * 64 : 64;
            const int swz = chunk_swizzle(channel);
            uint8_t* mine = lds + kWeightBase + channel * kStep;
            const int first_slot = ((2 * quarter) ^ swz) * 16, second_slot = ((2 * quarter + 1) ^ swz) * 16;
            v4u ring[kRing];
            auto decode_step = [&](const v4u& held, int step) {
                const uint2 d0 = decode(held.x), d1 = decode(held.y), d2 = decode(held.z), d3 = decode(held.w);
                uint8_t* stage = mine + (step % kWeightStages) * kWeightStage;
                if (active) {
                    *reinterpret_cast<uint4*>(stage + first_slot) = make_uint4(d0.x, d0.y, d1.x, d1.y);
                    *reinterpret_cast<uint4*>(stage + second_slot) = make_uint4(d2.x, d2.y, d3.x, d3.y);
                }
            };
            if ((dl & ~63) * 16 / 64 >= channels) {
                // a wave whose 16 channels are all beyond this pass's only keeps the barriers (same for the wave)
                for (int t = 0; t < steps + 3; ++t) step_barrier();
                store_image(row0, rows, channel0, channels);
                continue;
            }
#pragma unroll
            for (int s = 0; s < kRing; ++s) ring[s] = *reinterpret_cast<const v4u*>(codes + min(s, steps - 1) * step_bytes);
            step_barrier();  // tables built (first pass); everyone is done with the pass before
            decode_step(ring[0], 0);
            ring[0] = *reinterpret_cast<const v4u*>(codes + min(kRing, steps - 1) * step_bytes);
            step_barrier();
            // Whole groups of kRing steps run without a branch, so that the compiler counts the loads in
            // flight (it waits for all of them at a branch); the last steps take the slow way.
            int t = 0;
            for (; t + kRing < steps; t += kRing) {
#pragma unroll
                for (int u = 0; u < kRing; ++u) {
                    // ring slot (t + u + 1) % kRing holds the codes of step t + u + 1
                    decode_step(ring[(u + 1) % kRing], t + u + 1);
                    ring[(u + 1) % kRing] = *reinterpret_cast<const v4u*>(codes + min(t + u + 1 + kRing, steps - 1) * step_bytes);
                    step_barrier();
                }
            }
#pragma unroll
            for (int u = 0; u < kRing; ++u) {
                if (t + u < steps) {  // same for the whole workgroup
                    if (t + u + 1 < steps) decode_step(ring[(u + 1) % kRing], t + u + 1);
                    step_barrier();
                }
            }
            step_barrier();  // the image is written
            store_image(row0, rows, channel0, channels);
        }
    } else {
        ORX_WIDE_PASSES {
            const int rows = min(kRows, p.m - row0);
            const int channels = min(kChannels, channels_here - c0);
            const int channel0 = first_channel + c0;
            (void)rows, (void)channels, (void)channel0;
            // ---- MFMA waves: 32 token rows x up to 96 channels --------------------------------------
            // Lane (row, half) multiplies K bytes [64 half + 16 ks, + 16) of the step in MFMA ks: the order of K
            // inside a step is free as long as both operands agree, and this one makes a lane's four token
            // fragments of a step 64 consecutive bytes of its row.
            // (the lane number is made opaque per pass: the compiler otherwise hoists every address of a pass,
            // the 48 image positions included, out of the pass loops and spills them)
            int pass_lane = lane;
            asm volatile("" : "+v"(pass_lane));
            const int frag_row = pass_lane & 31, half = pass_lane >> 5;
            const bool live = wave * 32 < rows;  // a row block without rows only keeps the barriers (same for the wave)
            const int8_t* tokens = p.a + (int64_t)(row0 + min(wave * 32 + frag_row, rows - 1)) * p.k + half * 64;
            const int blocks = (channels + 31) / 32;
            // byte offset of this lane's fragment ks inside a weight stage: weight_lane[j] ^ (ks << 4)
            // (the swizzle is an XOR on the chunk number, and ks only touches its two low bits)
            uint32_t weight_lane[3];
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int channel = j * 32 + frag_row;
                weight_lane[j] = kWeightBase + channel * kStep + (((half * 4) ^ chunk_swizzle(channel)) << 4);
            }
            v16i acc[3];
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[j][r] = 0;
            v4i ring[kTokenRing][4];
            auto request = [&](int slot, int step) {
                const v4i* src = reinterpret_cast<const v4i*>(tokens + (int64_t)min(step, steps - 1) * kStep);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) ring[slot][ks] = src[ks];
            };
            auto multiply = [&](int slot, int step, auto block_count) {
                constexpr int BLOCKS = decltype(block_count)::value;
                const uint32_t stage = (step % kWeightStages) * kWeightStage;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                    for (int j = 0; j < BLOCKS; ++j) {
                        const v4i fb = *reinterpret_cast<const v4i*>(lds + stage + (weight_lane[j] ^ (uint32_t)(ks << 4)));
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[slot][ks], fb, acc[j], 0, 0, 0);
                    }
                }
            };
            // whole groups of kTokenRing steps without a branch (see the decoder waves), then the last steps
            auto run = [&](auto block_count) {
#pragma unroll
                for (int s = 0; s < kTokenRing; ++s) request(s, s);
                step_barrier();
                step_barrier();
                int t = 0;
                for (; t + kTokenRing <= steps; t += kTokenRing) {
#pragma unroll
                    for (int u = 0; u < kTokenRing; ++u) {
                        multiply(u, t + u, block_count);
                        request(u, t + u + kTokenRing);
                        step_barrier();
                    }
                }
#pragma unroll
                for (int u = 0; u < kTokenRing; ++u) {
                    if (t + u < steps) {  // same for the whole workgroup
                        multiply(u, t + u, block_count);
                        step_barrier();
                    }
                }
            };
            if (!live) {
                for (int t = 0; t < steps + 2; ++t) step_barrier();
            } else if (blocks == 3) {
                run(std::integral_constant<int, 3>());
            } else if (blocks == 2) {
                run(std::integral_constant<int, 2>());
            } else {
                run(std::integral_constant<int, 1>());
            }
            // epilogue: a lane holds channel (lane & 31) and token rows 8 (r / 4) + 4 half + r % 4 of each block
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int channel = j * 32 + frag_row;
                if (live && j < blocks) {
                    const float weight_scale = __half2float(p.ws[channel0 + min(channel, channels - 1)]);
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int local = wave * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                        const float token_scale = __half2float(p.as[row0 + min(local, rows - 1)]);
                        image[local * kImagePitch + channel] = rescale(acc[j][r], weight_scale, token_scale);
                    }
                }
            }
            step_barrier();  // the image is written
            store_image(row0, rows, channel0, channels);
        }
    }
#undef ORX_WIDE_PASSES
}

}  // namespace

// Shapes: two-stage codes, row-major or K-major in blocks of 128.
bool dense_wide_eligible(int n, int k, int packed_k) {
    return n > 0 && k > 0 && k % kStep == 0 && (packed_k == 0 || packed_k == 128 || packed_k == 64);
}

void dense_wide_geometry(int n, Geometry* g) {
    g->grid[0] = (uint32_t)std::min(device_compute_units(), n);
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kThreads;
    g->shared = kWideLdsBytes;
}

int dense_wide_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out,
                      int rows, int n, int k, int stride, int packed_k, int out_f32, const Geometry& g, hipStream_t stream) {
    static DeviceOnce opted_in;  // dynamic LDS above 64 KiB needs an opt-in per kernel and device
    const int ready = opted_in.run([] {
        const void* kernels[] = {reinterpret_cast<const void*>(&wide_kernel<false>), reinterpret_cast<const void*>(&wide_kernel<true>)};
        for (const void* kernel : kernels) {
            const int code = hip_check(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLdsBytes),
                                       "hipFuncSetAttribute");
            if (code != ORX_OK) return code;
        }
        return (int)ORX_OK;
    });
    if (ready != ORX_OK) return ready;
    WideParams p;
    p.a = a, p.w = static_cast<const uint8_t*>(w), p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.out_f32 = out_f32, p.k_major = packed_k == 64 ? 2 : packed_k != 0;  // 1: blocks of 128, 2: blocks of 64
    if (packed_k != 0)
        ORX_LAUNCH(wide_kernel<true>, dim3(g.grid[0]), dim3(kThreads), kWideLdsBytes, stream, p);
    else
        ORX_LAUNCH(wide_kernel<false>, dim3(g.grid[0]), dim3(kThreads), kWideLdsBytes, stream, p);
    return hip_check(hipGetLastError(), "launch projection (channel runs)");
}

}  // namespace orx
