// Weight-streaming MFMA projections for small token counts (5..64 rows): batched decode and the
// routed single-stage experts.  Bandwidth-bound: the weight stream is read exactly once.
//
// Reference counterparts: the small-row Tensor Core schedules of kernels/cuda/model/integer_core.py
// (block_m 8..32), the warp-owned routed decode kernels/cuda/model/e8p_decode.py:36-245 (codes go
// from global memory through a LUT straight into MMA operand registers, split-K through shared
// memory) and integer_vq.py:58-260.  Arithmetic: exact int32 over full K, (float(acc)*ws)*as.
//
// MI355X design.  A workgroup owns 32 output channels; its waves split K between them.  A wave
// streams its code rows with 16/32-byte per-lane loads (whole 64-byte or 2-KiB runs per wave),
// decodes them with two 8-byte LDS table reads and XORs per code directly into the 16-byte,
// K-contiguous row-operand fragments of v_mfma_i32_32x32x32_i8 and multiplies against activation
// fragments fetched straight from L2 (the activations are tiny and shared by everybody).  There
// is no operand staging in LDS and no barrier in the K loop, so waves run fully decoupled and
// hide HBM latency by occupancy.  The K-split partial sums are added through LDS at the end
// (exact integers, fixed order).  The MFMA K order is free as long as both operands agree: lane
// half h owns bytes [64h, 64h+64) of every 128-byte K block, sub-step s the 16 bytes at 16s.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "a8_device.h"
#include "e8p_device.h"
#include "orx_internal.h"
#include "row_q4_device.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum Codec { kQ4 = 0, kQ2 = 1, kW8 = 2, kS4 = 3 };  // kS4: row-scaled scalar Q4 nibbles

struct StreamParams {
    const int8_t* a;
    const void* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, m;
    int packed_k;
    int out_f32;
    // grouped only
    const int* counts;
    const int* offsets;
    const int* tile_expert;
    const int* tile_row;
    const int* tile_count;
    int64_t expert_weight_stride;  // bytes between experts in w
    uint32_t magnitudes_low, magnitudes_high;  // scalar Q4: the eight magnitudes, one per byte
    // PLANES: activations as two planes of nibble words with the rows' sums (e8p_exact.py, e8p_prefill.py)
    const uint32_t* low;
    const uint32_t* high;
    const int* sum;
    int plane_rows, group_major, selector_book, tile_rows, list_rows;
};

template <int CODEC>
struct StreamTables {
    typedef Q4ByteTables type;
};
template <>
struct StreamTables<kQ2> {
    typedef Q2ByteTables type;
};
template <>
struct StreamTables<kW8> {
    struct type {};
};
template <>
struct StreamTables<kS4> {
    struct type {};
};

constexpr int kWaves = 8;             // waves per workgroup
constexpr int kThreads = kWaves * 64;

// bytes of weight stream per output row per 128-wide K block
template <int CODEC>
__host__ __device__ constexpr int block_bytes() {
    return CODEC == kQ4 || CODEC == kS4 ? 64 : CODEC == kQ2 ? 32 : 128;
}

// CB = column blocks of 32 token rows (1 or 2); SPLITS = waves that share one group of 32 output
// channels, each taking a slice of K (8 for long K and few channels, 2 for the short K of experts).
// PLANES (routed codes only): the INT4-exact expert kernels' operands.  Activations come as low / high nibble planes and are
// put back together in registers; weights are decoded as y = (w - 1) / 2 from the nibble Book; the integer is
// 2 acc + c Sum[row] with the caller's Sum (c = 1, or 5 for two-stage codes; kernels/cuda/model/e8p_core.py:154-189).
// The bytes of a group of eight keep the order (even nibbles, odd nibbles) on both operands.
template <int CODEC, int CB, bool GROUPED, int SPLITS, bool PLANES = false>
__global__ __launch_bounds__(kThreads) void stream_kernel(StreamParams p) {
    static_assert(!PLANES || (GROUPED && CB == 1 && (CODEC == kQ2 || CODEC == kQ4)), "planes feed the routed tiles");
    constexpr int kSplits = SPLITS;
    constexpr int GROUPS = kWaves / SPLITS;   // channel groups per workgroup
    constexpr int kRows = 32;
    __shared__ typename std::conditional<PLANES, StreamTables<kW8>, StreamTables<CODEC>>::type::type tables;
    __shared__ uint2 half_value[PLANES ? 256 : 1], half_change[PLANES ? 256 : 1];
    __shared__ int partial[kWaves][kRows][33];  // one column block at a time; +1 keeps column reads conflict-free

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = wave % SPLITS, group = wave / SPLITS;
    const int half = lane >> 5, frag = lane & 31;
    const int n0 = (blockIdx.x * GROUPS + group) * kRows;

    int row0 = 0, rows_here = p.m;
    const int8_t* w_base = reinterpret_cast<const int8_t*>(p.w);
    const __half* ws = p.ws;
    if (GROUPED) {
        const int tile = blockIdx.y;
        if (tile >= p.tile_count[0]) return;
        const int expert = p.tile_expert[tile];
        const int first = p.tile_row[tile];
        // a tile list in steps of fewer rows than a workgroup takes: the workgroup of the first tile of a stretch takes
        // them all (tiles of one expert are adjacent and start at multiples of the list's step)
        if (p.list_rows != p.tile_rows && first % p.tile_rows != 0) return;
        row0 = p.offsets[expert] + first;
        rows_here = min(p.tile_rows, p.counts[expert] - first);
        if (rows_here <= 0) return;
        w_base += (int64_t)expert * p.expert_weight_stride;
        ws += (int64_t)expert * p.n;
    }

    if constexpr (PLANES) {
        if (tid < 256) build_half_tables(half_value, half_change, p.book, p.selector_book != 0, tid);
    } else if constexpr (CODEC == kQ4 || CODEC == kQ2) {
        build_tables(tables, p.book, tid, kThreads);
    }

    // K blocks of this wave
    const int k_blocks = p.k / 128;
    const int kb_first = (int)((int64_t)k_blocks * split / SPLITS);
    const int kb_last = (int)((int64_t)k_blocks * (split + 1) / SPLITS);

    // weight row of this lane (clamped: rows beyond N are computed on row N-1 and never stored)
    const int w_row = min(n0 + frag, p.n - 1);
    constexpr int BB = block_bytes<CODEC>();
    constexpr int LANE_BYTES = BB / 2;          // this lane's half of a K block
    constexpr int LOADS = LANE_BYTES / 16;      // 16-byte loads per K block: Q4 2, Q2 1, W8 4
    auto weight_pointer = [&](int kb) -> const uint4* {
        int64_t byte;
        if (CODEC == kW8 || CODEC == kS4 || p.packed_k == 0)
            byte = ((int64_t)w_row * k_blocks + kb) * BB + half * LANE_BYTES;
        else if (p.packed_k == 64)  // two-stage codes in 64-wide K blocks: this lane's half is one block row
            byte = ((int64_t)(kb * 2 + half) * p.n + w_row) * LANE_BYTES;
        else
            byte = ((int64_t)kb * p.n + w_row) * BB + half * LANE_BYTES;
        return reinterpret_cast<const uint4*>(w_base + byte);
    };
    // activation rows of this lane, one per column block
    const int8_t* a_rows[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c)
        a_rows[c] = PLANES ? nullptr : p.a + (int64_t)(row0 + min(c * 32 + frag, rows_here - 1)) * p.k + half * 64;
    // PLANES: the lane's 64 activations of a K block are words [16 kb + 8 half, + 8) of its plane row
    const int64_t plane_row = row0 + min(frag, rows_here - 1);

    v16i acc[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0;

    uint4 codes[LOADS], next_codes[LOADS];
    uint4 act[CB][4], next_act[CB][4];
    auto fetch = [&](int kb, uint4 (&c)[LOADS], uint4 (&a)[CB][4]) {
        const uint4* src = weight_pointer(kb);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) c[i] = src[i];
        if constexpr (PLANES) {
            // a[0][0..1] hold the low words, a[0][2..3] the high words; they are combined when they are used
            const int64_t at = plane_index(p.group_major, p.plane_rows, p.k >> 3, plane_row, kb * 16 + half * 8);
            const uint4* low = reinterpret_cast<const uint4*>(p.low + at);
            const uint4* high = reinterpret_cast<const uint4*>(p.high + at);
            a[0][0] = low[0], a[0][1] = low[1], a[0][2] = high[0], a[0][3] = high[1];
            return;
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const uint4* arow = reinterpret_cast<const uint4*>(a_rows[cb] + (int64_t)kb * 128);
#pragma unroll
            for (int s = 0; s < 4; ++s) a[cb][s] = arow[s];
        }
    };
    if (kb_first < kb_last) fetch(kb_first, next_codes, next_act);
    __syncthreads();  // tables

    for (int kb = kb_first; kb < kb_last; ++kb) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) codes[i] = next_codes[i];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int s = 0; s < 4; ++s) act[cb][s] = next_act[cb][s];
        if (kb + 1 < kb_last) fetch(kb + 1, next_codes, next_act);
        // four row-operand fragments of 16 weights each
        uint4 wf[4];
        if constexpr (PLANES) {
            const uint32_t low[8] = {act[0][0].x, act[0][0].y, act[0][0].z, act[0][0].w, act[0][1].x, act[0][1].y, act[0][1].z, act[0][1].w};
            const uint32_t high[8] = {act[0][2].x, act[0][2].y, act[0][2].z, act[0][2].w, act[0][3].x, act[0][3].y, act[0][3].z, act[0][3].w};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint2 first = plane_bytes(low[2 * s], high[2 * s]), second = plane_bytes(low[2 * s + 1], high[2 * s + 1]);
                act[0][s] = make_uint4(first.x, first.y, second.x, second.y);
            }
            if constexpr (CODEC == kQ4) {
                const uint32_t c[8] = {codes[0].x, codes[0].y, codes[0].z, codes[0].w, codes[1].x, codes[1].y, codes[1].z, codes[1].w};
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint2 y0 = decode_half_q4(half_value, half_change, c[2 * s]), y1 = decode_half_q4(half_value, half_change, c[2 * s + 1]);
                    wf[s] = make_uint4(y0.x, y0.y, y1.x, y1.y);
                }
            } else {
                const uint32_t c[4] = {codes[0].x, codes[0].y, codes[0].z, codes[0].w};
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint2 y0 = decode_half(half_value, half_change, c[s] & 0xFFFFu), y1 = decode_half(half_value, half_change, c[s] >> 16);
                    wf[s] = make_uint4(y0.x, y0.y, y1.x, y1.y);
                }
            }
        } else if constexpr (CODEC == kQ4) {
            const uint32_t c[8] = {codes[0].x, codes[0].y, codes[0].z, codes[0].w,
                                   codes[1].x, codes[1].y, codes[1].z, codes[1].w};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint2 lo = decode_q4(tables, c[2 * s]), hi = decode_q4(tables, c[2 * s + 1]);
                wf[s] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        } else if constexpr (CODEC == kQ2) {
            const uint32_t c[4] = {codes[0].x, codes[0].y, codes[0].z, codes[0].w};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint2 lo = decode_q2(tables, c[s] & 0xFFFFu), hi = decode_q2(tables, c[s] >> 16);
                wf[s] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        } else if constexpr (CODEC == kS4) {
            // a lane's 32 bytes are 64 nibbles: 16 weights per fragment are one 8-byte run
            const uint32_t c[8] = {codes[0].x, codes[0].y, codes[0].z, codes[0].w,
                                   codes[1].x, codes[1].y, codes[1].z, codes[1].w};
#pragma unroll
            for (int s = 0; s < 4; ++s)
                wf[s] = make_uint4(decode_row_q4(c[2 * s], p.magnitudes_low, p.magnitudes_high),
                                   decode_row_q4(c[2 * s] >> 16, p.magnitudes_low, p.magnitudes_high),
                                   decode_row_q4(c[2 * s + 1], p.magnitudes_low, p.magnitudes_high),
                                   decode_row_q4(c[2 * s + 1] >> 16, p.magnitudes_low, p.magnitudes_high));
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) wf[s] = codes[s];
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const v4i row_operand = {(int)wf[s].x, (int)wf[s].y, (int)wf[s].z, (int)wf[s].w};
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const v4i col_operand = {(int)act[cb][s].x, (int)act[cb][s].y, (int)act[cb][s].z, (int)act[cb][s].w};
                acc[cb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(row_operand, col_operand, acc[cb], 0, 0, 0);
            }
        }
    }

    // ---- K-split reduction through LDS, then rescale and store ----
    // accumulator register r of a lane: channel 8*(r/4) + 4*half + r%4, token row `frag`
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        if (cb > 0) __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) partial[wave][8 * (r >> 2) + 4 * half + (r & 3)][frag] = acc[cb][r];
        __syncthreads();
        for (int e = tid; e < GROUPS * kRows * 32; e += kThreads) {
            const int channel = e % kRows, g = (e / kRows) % GROUPS, local_token = e / (kRows * GROUPS);
            const int token = cb * 32 + local_token;
            const int col = (blockIdx.x * GROUPS + g) * kRows + channel;
            if (token >= rows_here || col >= p.n) continue;
            int total = 0;
#pragma unroll
            for (int s = 0; s < kSplits; ++s) total += partial[g * SPLITS + s][channel][local_token];
            const int64_t row = row0 + token;
            if constexpr (PLANES) total = (int)(2u * (uint32_t)total + (CODEC == kQ4 ? 5u : 1u) * (uint32_t)p.sum[row]);
            const float value = rescale(total, __half2float(ws[col]), __half2float(p.as[row]));
            if (p.out_f32)
                reinterpret_cast<float*>(p.out)[row * p.stride + col] = value;
            else
                reinterpret_cast<__half*>(p.out)[row * p.stride + col] = __float2half_rn(value);
        }
    }
}

template <int CODEC, bool GROUPED, int SPLITS>
int launch_codec(int cb, const StreamParams& p, dim3 grid, hipStream_t stream) {
    if (cb == 1)
        ORX_LAUNCH((stream_kernel<CODEC, 1, GROUPED, SPLITS>), grid, dim3(kThreads), 0, stream, p);
    else
        ORX_LAUNCH((stream_kernel<CODEC, 2, GROUPED, SPLITS>), grid, dim3(kThreads), 0, stream, p);
    return hip_check(hipGetLastError(), "launch projection (stream)");
}

constexpr int kDenseSplits = 8;    // dense decode: K is long, 32 channels per workgroup
constexpr int kGroupedSplits = 2;  // routed experts: K is short, 128 channels per workgroup

}  // namespace

// Dense: rows <= 64.  codec: 0 Q4 (u32 codes), 1 Q2 (u16 codes), 2 W8.
void stream_geometry(int n, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)n, (uint32_t)(32 * kWaves / kDenseSplits));
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kThreads;
    g->shared = 0;
}

int stream_launch(int codec, const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                  void* out, int rows, int n, int k, int stride, int packed_k, bool out_f32, hipStream_t stream) {
    StreamParams p = {};
    p.a = a, p.w = w, p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.packed_k = packed_k, p.out_f32 = out_f32;
    Geometry g;
    stream_geometry(n, &g);
    const dim3 grid(g.grid[0]);
    const int cb = rows <= 32 ? 1 : 2;
    if (codec == kQ4) return launch_codec<kQ4, false, kDenseSplits>(cb, p, grid, stream);
    if (codec == kQ2) return launch_codec<kQ2, false, kDenseSplits>(cb, p, grid, stream);
    return launch_codec<kW8, false, kDenseSplits>(cb, p, grid, stream);
}

// Routed experts on nibble planes (e8p_exact_grouped, e8p_prefill_grouped): tiles of up to 32 rows; single-stage codes in
// K-major blocks of 64 (two-stage: blocks of 128)
int stream_planes_launch(bool two_stage, const uint32_t* low, const uint32_t* high, const int* sum, const void* w,
                         const uint32_t* book, bool selector_book, const __half* ws, const __half* as, void* out,
                         const int* counts, const int* offsets, const int* tile_expert, const int* tile_row, const int* tile_count,
                         int n, int k, int rows, bool group_major, int tile_rows, int list_rows, const Geometry& g,
                         hipStream_t stream) {
    StreamParams p = {};
    p.w = w, p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = n, p.m = 0, p.packed_k = two_stage ? 128 : 64, p.out_f32 = 0;
    p.counts = counts, p.offsets = offsets, p.tile_expert = tile_expert, p.tile_row = tile_row, p.tile_count = tile_count;
    p.expert_weight_stride = (int64_t)n * k / (two_stage ? 2 : 4);
    p.low = low, p.high = high, p.sum = sum, p.plane_rows = rows, p.group_major = group_major, p.selector_book = selector_book;
    p.tile_rows = tile_rows, p.list_rows = list_rows;
    const dim3 grid(g.grid[0], g.grid[1]);
    if (two_stage)
        ORX_LAUNCH((stream_kernel<kQ4, 1, true, kGroupedSplits, true>), grid, dim3(kThreads), 0, stream, p);
    else
        ORX_LAUNCH((stream_kernel<kQ2, 1, true, kGroupedSplits, true>), grid, dim3(kThreads), 0, stream, p);
    return hip_check(hipGetLastError(), "launch routed projection on nibble planes (stream)");
}

// Row-scaled scalar Q4 (kernels/cuda/model/q4_projection.py): W is (N, K/4) u16, rows <= 64
int stream_row_q4_launch(const int8_t* a, const void* w, uint32_t magnitudes_low, uint32_t magnitudes_high, const __half* ws,
                         const __half* as, void* out, int rows, int n, int k, int stride, bool out_f32, hipStream_t stream) {
    StreamParams p = {};
    p.a = a, p.w = w, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.out_f32 = out_f32;
    p.magnitudes_low = magnitudes_low, p.magnitudes_high = magnitudes_high;
    Geometry g;
    stream_geometry(n, &g);
    return launch_codec<kS4, false, kDenseSplits>(rows <= 32 ? 1 : 2, p, dim3(g.grid[0]), stream);
}

// Routed single-stage experts: one tile = (expert, first row, count <= block_m), block_m 32 or 64.
void stream_grouped_geometry(int n, int tiles, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)n, (uint32_t)(32 * kWaves / kGroupedSplits));
    g->grid[1] = (uint32_t)tiles;
    g->grid[2] = 1;
    g->block[0] = kThreads;
    g->shared = 0;
}

int stream_grouped_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                          void* out, const int* counts, const int* offsets, const int* tile_expert, const int* tile_row,
                          const int* tile_count, int n, int k, int tiles, int block_m, int packed_k,
                          hipStream_t stream) {
    StreamParams p = {};
    p.a = a, p.w = w, p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = n, p.m = 0, p.packed_k = packed_k, p.out_f32 = 0;
    p.counts = counts, p.offsets = offsets, p.tile_expert = tile_expert, p.tile_row = tile_row, p.tile_count = tile_count;
    p.expert_weight_stride = (int64_t)n * (k / 8) * 2;
    // lists in steps of 8 or 16 rows (the reference's own decode kernels take 8: e8p_decode.py:36-58): 32 rows per workgroup
    p.tile_rows = block_m <= 32 ? 32 : 64, p.list_rows = block_m < 32 ? block_m : p.tile_rows;
    Geometry g;
    stream_grouped_geometry(n, tiles, &g);
    return launch_codec<kQ2, true, kGroupedSplits>(block_m <= 32 ? 1 : 2, p, dim3(g.grid[0], g.grid[1]), stream);
}

}  // namespace orx
