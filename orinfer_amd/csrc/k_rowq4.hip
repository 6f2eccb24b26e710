// Row-scaled scalar Q4 at one or two token rows: a plain streaming GEMV (kernels/cuda/model/q4_projection.py:38-78 is
// the reference's DP4A form of the same product).
//
// The nibbles need no table: four weights come out of one v_perm_b32 (row_q4_device.h), so the kernel is a read of
// N K / 2 bytes with about 5 vector-ALU operations per byte beside it (they, not the bytes, bound it: 3.2 TB/s).  Sixteen lanes share one output channel (256 bytes of
// its nibbles per step, 16 per lane), a wave takes four channels at a time; the token rows sit in LDS as int8, every
// group of eight in the order of the even and the odd nibbles of a word, and a lane reads the 32 activations of its 16
// bytes from there.  A wave keeps two chunks of four steps in flight (128 bytes
// per lane), so sixteen waves per CU hold 128 KiB of requests: what a CU needs to keep HBM busy.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>

#include "e8p_device.h"
#include "orx_internal.h"
#include "row_q4_device.h"

namespace orx {
namespace {

constexpr int kGemvThreads = 512;
constexpr int kGemvWaves = kGemvThreads / 64;
constexpr int kChunk = 4;            // steps of 256 bytes per channel requested together
constexpr int kMaxRowBytes = 65536;  // token rows kept in LDS

struct RowQ4GemvParams {
    const int8_t* a;
    const uint8_t* w;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, out_f32;
    uint32_t low, high;
};

template <int ROWS>
__global__ __launch_bounds__(kGemvThreads) void row_q4_gemv_kernel(RowQ4GemvParams p) {
    extern __shared__ __align__(16) int8_t rows_lds[];  // ROWS x K
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int part = lane & 15, quarter = lane >> 4;  // 16 lanes per channel, four channels per wave
    // the eight activations of a group wait as [0, 2, 4, 6 | 1, 3, 5, 7]: the even and the odd nibbles of a u32 of weights
    // are then two masks away from their bytes (a dot product does not care about the order)
    for (int i = tid; i < ROWS * p.k / 16; i += kGemvThreads) {
        const uint4 v = reinterpret_cast<const uint4*>(p.a)[i];
        reinterpret_cast<uint4*>(rows_lds)[i] =
            make_uint4(__builtin_amdgcn_perm(v.y, v.x, 0x06040200u), __builtin_amdgcn_perm(v.y, v.x, 0x07050301u),
                       __builtin_amdgcn_perm(v.w, v.z, 0x06040200u), __builtin_amdgcn_perm(v.w, v.z, 0x07050301u));
    }
    __syncthreads();

    const int row_bytes = p.k / 2;                       // nibbles of one channel
    const int steps = (row_bytes + 255) / 256;
    const int chunks = (steps + kChunk - 1) / kChunk;
    const int tasks = (p.n + 3) / 4;
    const int first_task = blockIdx.x * kGemvWaves + wave, task_stride = gridDim.x * kGemvWaves;
    if (first_task >= tasks) return;
    const int my_tasks = (tasks - first_task + task_stride - 1) / task_stride;
    const int total = my_tasks * chunks;  // (task, chunk) pairs of this wave, in order

    auto request = [&](int flat, uint4 (&buffer)[kChunk]) {
        const int task = first_task + (flat / chunks) * task_stride, chunk = flat % chunks;
        const int channel = min(task * 4 + quarter, p.n - 1);
        const uint8_t* row = p.w + (int64_t)channel * row_bytes;
#pragma unroll
        for (int s = 0; s < kChunk; ++s) {
            const int byte = ((chunk * kChunk + s) * 16 + part) * 16;
            buffer[s] = *reinterpret_cast<const uint4*>(row + min(byte, row_bytes - 16));  // clamped: unconditional
        }
    };

    int acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0;

    auto consume = [&](int flat, const uint4 (&buffer)[kChunk]) {
        const int chunk = flat % chunks;
#pragma unroll
        for (int s = 0; s < kChunk; ++s) {
            const int byte = ((chunk * kChunk + s) * 16 + part) * 16;
            if (byte < row_bytes) {
                const uint32_t words[4] = {buffer[s].x, buffer[s].y, buffer[s].z, buffer[s].w};
                uint32_t weights[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    weights[2 * j] = decode_row_q4_bytes(words[j] & 0x0F0F0F0Fu, p.low, p.high);
                    weights[2 * j + 1] = decode_row_q4_bytes((words[j] >> 4) & 0x0F0F0F0Fu, p.low, p.high);
                }
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const uint4* tokens = reinterpret_cast<const uint4*>(rows_lds + r * p.k + byte * 2);
                    const uint4 t0 = tokens[0], t1 = tokens[1];
                    const uint32_t t[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[r] = __builtin_amdgcn_sdot4((int)weights[j], (int)t[j], acc[r], false);
                }
            }
        }
        if (chunk == chunks - 1) {  // the channel is complete: add the 16 lanes, rescale, store
            const int task = first_task + (flat / chunks) * task_stride;
            const int channel = task * 4 + quarter;
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                int sum = acc[r];
#pragma unroll
                for (int offset = 8; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, 64);
                acc[r] = 0;
                if (part == 0 && channel < p.n) {
                    const float value = rescale(sum, __half2float(p.ws[channel]), __half2float(p.as[r]));
                    if (p.out_f32)
                        reinterpret_cast<float*>(p.out)[(int64_t)r * p.stride + channel] = value;
                    else
                        reinterpret_cast<__half*>(p.out)[(int64_t)r * p.stride + channel] = __float2half_rn(value);
                }
            }
        }
    };

    uint4 even[kChunk], odd[kChunk];
    request(0, even);
    for (int flat = 0; flat < total; flat += 2) {
        if (flat + 1 < total) request(flat + 1, odd);
        consume(flat, even);
        if (flat + 1 >= total) break;
        if (flat + 2 < total) request(flat + 2, even);
        consume(flat + 1, odd);
    }
}

}  // namespace

// one and two rows (N = 17408, K = 5120: 14.1 and 16.1 us against 17.4 and 17.9 for the MFMA streaming kernel; at four rows
// 20.2 against 18: the dot products grow with the rows, the MFMAs do not)
bool row_q4_gemv_serves(int rows, int k) { return rows >= 1 && rows <= 2 && (int64_t)rows * k <= kMaxRowBytes; }

void row_q4_gemv_geometry(int rows, int n, int k, Geometry* g) {
    const uint32_t tasks = ((uint32_t)n + 3) / 4;
    g->grid[0] = std::max(1u, std::min(2u * (uint32_t)device_compute_units(), (tasks + kGemvWaves - 1) / kGemvWaves));
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kGemvThreads;
    g->shared = (uint32_t)(rows * k);
}

int row_q4_gemv_launch(const int8_t* a, const void* w, uint32_t low, uint32_t high, const __half* ws, const __half* as, void* out,
                       int rows, int n, int k, int stride, bool out_f32, const Geometry& g, hipStream_t stream) {
    static DeviceOnce once;
    const int ready = once.run([] {
        hipError_t code = hipSuccess;
        const void* kernels[4] = {reinterpret_cast<const void*>(&row_q4_gemv_kernel<1>), reinterpret_cast<const void*>(&row_q4_gemv_kernel<2>),
                                  reinterpret_cast<const void*>(&row_q4_gemv_kernel<3>), reinterpret_cast<const void*>(&row_q4_gemv_kernel<4>)};
        for (const void* kernel : kernels)
            if (code == hipSuccess) code = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxRowBytes);
        return hip_check(code, "scalar Q4 GEMV: LDS size");
    });
    if (ready != ORX_OK) return ready;
    RowQ4GemvParams p = {};
    p.a = a, p.w = static_cast<const uint8_t*>(w), p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.out_f32 = out_f32, p.low = low, p.high = high;
    const dim3 grid(g.grid[0]), block(g.block[0]);
    switch (rows) {
        case 1: ORX_LAUNCH(row_q4_gemv_kernel<1>, grid, block, g.shared, stream, p); break;
        case 2: ORX_LAUNCH(row_q4_gemv_kernel<2>, grid, block, g.shared, stream, p); break;
        case 3: ORX_LAUNCH(row_q4_gemv_kernel<3>, grid, block, g.shared, stream, p); break;
        default: ORX_LAUNCH(row_q4_gemv_kernel<4>, grid, block, g.shared, stream, p); break;
    }
    return hip_check(hipGetLastError(), "launch scalar Q4 GEMV");
}

}  // namespace orx
