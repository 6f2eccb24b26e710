// Nibble planes: the A8 hand-over of the reference's INT4 expert kernels, and the grouped GEMMs that take it.
//
// The reference's SM87 expert kernels multiply signed 4-bit weights y = (w - 1) / 2 with the two nibbles of an
// int8 activation, a = low_u4 + 16 * high_s4, and add the row's sum back: w . a = 2 (y . low + 16 y . high) + sum(a)
// (kernels/cuda/model/e8p_exact.py:1-7).  Their activations therefore travel as two planes of u32 words, eight
// nibbles each, nibble i holding code {0,2,1,3,4,6,5,7}[i] of its group of eight (e8p_core.py:63-78), row-major
// (rows, K/8) or K64-major (K/64, rows, 8) (e8p_prefill.py:79-80), together with the int32 row sums.
//
// CDNA4 multiplies int8 directly, so the GEMMs here put the two nibbles back together on the way into LDS
// (one OR per four codes) and feed v_mfma_i32_32x32x32_i8 with y as int8; the result is the same integer
// 2 (y . a) + c Sum with Sum taken from the caller's buffer as the reference's kernels take it, and the same
// rescale follows.  Within a group of eight the bytes keep a fixed order of their own (even nibbles, then odd
// ones) on both operands: a dot product does not care.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>

#include "a8_device.h"
#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {

// from k_stream.hip
void stream_grouped_geometry(int n, int tiles, Geometry* g);
int stream_planes_launch(bool two_stage, const uint32_t* low, const uint32_t* high, const int* sum, const void* w,
                         const uint32_t* book, bool selector_book, const __half* ws, const __half* as, void* out,
                         const int* counts, const int* offsets, const int* tile_expert, const int* tile_row, const int* tile_count,
                         int n, int k, int rows, bool group_major, int tile_rows, int list_rows, const Geometry& g,
                         hipStream_t stream);

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kPlaneThreads = 256;
constexpr int kPlaneWaves = kPlaneThreads / 64;
constexpr int kMaxChoices = 64;  // routes of one token: one lane each

// ---- packing ------------------------------------------------------------------------------------

enum PlaneMode { kSplitRows = 0, kSplitTiles = 1, kDispatchSlots = 2, kPackTokens = 3 };

struct PlaneParams {
    const int8_t* a;
    uint32_t* low;
    uint32_t* high;
    int* sum;
    int k, rows, plane_rows, group_major, mode;
    // routed tiles
    const int *counts, *offsets, *tile_expert, *tile_row, *tile_count;
    int block_m;
    // routed slots
    const __half* scale;
    const int *ids, *relative, *row_offsets;
    __half* ds;
    int *slot_map, *sources;
    int top_k;
};

// One wave packs row `src` of A into the plane rows `dst` (lane r holds the r-th of `copies` destinations,
// or every lane the one destination when copies == 0) and returns the row's sum in every lane.
// (v_readlane reads a lane whether or not it still takes part in the loop)
__device__ __forceinline__ int pack_row(const PlaneParams& p, int64_t src, int dst, int copies, int lane) {
    const int words = p.k >> 3;
    const uint2* row = reinterpret_cast<const uint2*>(p.a + src * p.k);
    int partial = 0;
    for (int j = lane; j < words; j += 64) {
        const uint2 v = row[j];
        const uint32_t lo = low_word(v.x, v.y), hi = high_word(v.x, v.y);
        partial = __builtin_amdgcn_sdot4((int)v.x, 0x01010101, partial, false);
        partial = __builtin_amdgcn_sdot4((int)v.y, 0x01010101, partial, false);
        if (copies == 0) {
            const int64_t at = plane_index(p.group_major, p.plane_rows, words, dst, j);
            p.low[at] = lo, p.high[at] = hi;
        } else {
            for (int r = 0; r < copies; ++r) {
                const int64_t at = plane_index(p.group_major, p.plane_rows, words, __builtin_amdgcn_readlane(dst, r), j);
                p.low[at] = lo, p.high[at] = hi;
            }
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) partial += __shfl_xor(partial, offset, 64);
    return partial;
}

// grid: ceil(rows / 4) workgroups of four waves (tiles: one workgroup per routed tile), one row per wave at a time
__global__ __launch_bounds__(kPlaneThreads) void plane_split_kernel(PlaneParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (p.mode == kSplitTiles) {
        // e8p_prefill.py:89-129: the rows of every routed tile, nothing else
        const int tile = blockIdx.x;
        if (tile >= p.tile_count[0]) return;
        const int expert = p.tile_expert[tile], first = p.tile_row[tile];
        const int begin = p.offsets[expert] + first, count = min(p.block_m, p.counts[expert] - first);
        for (int i = wave; i < count; i += kPlaneWaves) {
            const int row = begin + i;
            if (row < 0 || row >= p.rows) continue;
            const int total = pack_row(p, row, row, 0, lane);
            if (lane == 0) p.sum[row] = total;
        }
        return;
    }
    const int row = blockIdx.x * kPlaneWaves + wave;
    if (row >= p.rows) return;
    if (p.mode == kSplitRows) {
        const int total = pack_row(p, row, row, 0, lane);
        if (lane == 0) p.sum[row] = total;
        return;
    }
    int slot = 0;
    if (lane < p.top_k) slot = p.row_offsets[p.ids[(int64_t)row * p.top_k + lane]] + p.relative[(int64_t)row * p.top_k + lane];
    if (p.mode == kDispatchSlots) {
        // e8p_prefill.py:565-622: the planes, the sum and the scale of a token at each of its slots
        const int total = pack_row(p, row, slot, p.top_k, lane);
        if (lane < p.top_k) {
            p.sum[slot] = total;
            p.ds[slot] = p.scale[row];
            p.slot_map[(int64_t)row * p.top_k + lane] = slot;
        }
        return;
    }
    // e8p_prefill.py:625-652: each token once, and the inverse map of its slots
    const int total = pack_row(p, row, row, 0, lane);
    if (lane == 0) p.sum[row] = total;
    if (lane < p.top_k) {
        p.slot_map[(int64_t)row * p.top_k + lane] = slot;
        p.sources[slot] = row;
    }
}

// e8p_prefill.py:655-690: K64-major planes of `tokens` rows copied to `slots` rows by Sources
// grid (ceil(slots / 32), K / 64), 256 threads: one plane word each
__global__ __launch_bounds__(kPlaneThreads) void plane_expand_kernel(const uint32_t* __restrict__ src_low,
                                                                     const uint32_t* __restrict__ src_high,
                                                                     const int* __restrict__ src_sum,
                                                                     const __half* __restrict__ scale,
                                                                     const int* __restrict__ sources, uint32_t* low,
                                                                     uint32_t* high, int* sum, __half* ds, int tokens,
                                                                     int slots) {
    const int slot = blockIdx.x * 32 + (threadIdx.x >> 3), word = threadIdx.x & 7, group = blockIdx.y;
    if (slot >= slots) return;
    const int token = sources[slot];
    if (token < 0 || token >= tokens) return;
    const int64_t from = ((int64_t)group * tokens + token) * 8 + word, to = ((int64_t)group * slots + slot) * 8 + word;
    low[to] = src_low[from];
    high[to] = src_high[from];
    if (group == 0 && word == 0) {
        sum[slot] = src_sum[token];
        ds[slot] = scale[token];
    }
}

// ---- grouped GEMM on planes -----------------------------------------------------------------------

constexpr int kStepK = 128;
constexpr int kRowPitch = kStepK + 16;  // bytes between rows in LDS
constexpr int kTileRows = 32, kTileChannels = 128;

struct PlaneGemmParams {
    const uint32_t* low;
    const uint32_t* high;
    const int* sum;
    const void* codes;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    __half* out;
    const int *counts, *offsets, *tile_expert, *tile_row, *tile_count;
    int n, k, rows;
    int tile_rows;       // rows a workgroup takes from its expert (8, 16 or 32)
    int list_rows;       // row step of the caller's tile list (tile_rows, or half of it when adjacent tiles merge)
    int group_major;     // planes (K/64, rows, 8) instead of (rows, K/8)
    int selector_book;   // Book holds selector words (two-stage codes) instead of nibble words
    int64_t expert_stride;  // bytes between the experts' codes
};

// Q4: codes are u32 (coarse in the low half, weight 4; fine in the high half, weight 1) in blocks (K/128, N, 16);
// else u16 in blocks (K/64, N, 8).
template <bool Q4>
__global__ __launch_bounds__(kPlaneThreads) void plane_gemm_kernel(PlaneGemmParams p) {
    __shared__ __align__(16) int8_t lds_a[kTileRows * kRowPitch];
    __shared__ __align__(16) int8_t lds_w[kTileChannels * kRowPitch];
    // y = (w - 1) / 2 as sign-extended bytes, even nibbles of the reference's nibble word in .x, odd ones in .y: the value
    // at even parity without sign bits per basis row, and what a code's low byte changes in it.  Sign extension
    // commutes with xor, so a code is two 8-byte lookups and two xors.
    __shared__ uint2 book[256];
    __shared__ uint2 flips[256];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile = blockIdx.y;
    if (tile >= p.tile_count[0]) return;
    const int expert = p.tile_expert[tile], first = p.tile_row[tile];
    if (p.list_rows != p.tile_rows && first % p.tile_rows != 0) return;  // the second of two merged tiles
    const int row0 = p.offsets[expert] + first;
    // a tile never reaches past the live rows, whatever Counts and Offsets say (e8p_exact.py:127-150 clamps every
    // plane load to rows - 1 and predicates it on the row being live)
    const int rows_here = min(min(p.tile_rows, p.counts[expert] - first), p.rows - row0);
    if (row0 < 0 || rows_here <= 0) return;
    const int n0 = blockIdx.x * kTileChannels;
    const int8_t* codes = reinterpret_cast<const int8_t*>(p.codes) + (int64_t)expert * p.expert_stride;
    const __half* ws = p.ws + (int64_t)expert * p.n;

    build_half_tables(book, flips, p.book, p.selector_book != 0, tid);

    const int k_steps = p.k / kStepK;
    const int words = p.k >> 3;
    const int a_row = tid >> 3, a_piece = tid & 7;
    const int64_t plane_row = row0 + min(a_row, rows_here - 1);
    constexpr int W_PIECES = Q4 ? 2 : 1;
    uint2 held_low, held_high;
    uint4 held_w[W_PIECES];

    auto load_step = [&](int step) {
        const int j = step * 16 + a_piece * 2;
        const int64_t at = plane_index(p.group_major, p.rows, words, plane_row, j);
        held_low = *reinterpret_cast<const uint2*>(p.low + at);
        held_high = *reinterpret_cast<const uint2*>(p.high + at);
#pragma unroll
        for (int i = 0; i < W_PIECES; ++i) {
            const int c = tid + kPlaneThreads * i;
            int64_t byte;
            if (Q4) {
                const int channel = min(n0 + (c >> 2), p.n - 1), q = c & 3;
                byte = ((int64_t)step * p.n + channel) * 64 + q * 16;
            } else {
                const int channel = min(n0 + (c >> 1), p.n - 1), q = c & 1;
                byte = ((int64_t)(step * 2 + q) * p.n + channel) * 16;
            }
            held_w[i] = *reinterpret_cast<const uint4*>(codes + byte);
        }
    };

    auto store_step = [&]() {
        {
            const uint2 first = plane_bytes(held_low.x, held_high.x), second = plane_bytes(held_low.y, held_high.y);
            *reinterpret_cast<uint4*>(lds_a + a_row * kRowPitch + a_piece * 16) = make_uint4(first.x, first.y, second.x, second.y);
        }
#pragma unroll
        for (int i = 0; i < W_PIECES; ++i) {
            const int c = tid + kPlaneThreads * i;
            const uint32_t in[4] = {held_w[i].x, held_w[i].y, held_w[i].z, held_w[i].w};
            if (Q4) {
                // four two-stage codes: y = 4 y_coarse + y_fine
                uint32_t out[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint2 y = decode_half_q4(book, flips, in[j]);
                    out[2 * j] = y.x, out[2 * j + 1] = y.y;
                }
                uint4* dst = reinterpret_cast<uint4*>(lds_w + (c >> 2) * kRowPitch + (c & 3) * 32);
                dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
                dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
            } else {
                uint4* dst = reinterpret_cast<uint4*>(lds_w + (c >> 1) * kRowPitch + (c & 1) * 64);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint2 y0 = decode_half(book, flips, in[j] & 0xFFFFu), y1 = decode_half(book, flips, in[j] >> 16);
                    dst[j] = make_uint4(y0.x, y0.y, y1.x, y1.y);
                }
            }
        }
    };

    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;

    load_step(0);
    __syncthreads();  // tables ready
    for (int step = 0; step < k_steps; ++step) {
        store_step();
        __syncthreads();
        if (step + 1 < k_steps) load_step(step + 1);
        const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
#pragma unroll
        for (int ks = 0; ks < kStepK / 32; ++ks) {
            const v4i fa = *reinterpret_cast<const v4i*>(lds_a + frag_row * kRowPitch + ks * 32 + frag_k);
            const v4i fb = *reinterpret_cast<const v4i*>(lds_w + (wave * 32 + frag_row) * kRowPitch + ks * 32 + frag_k);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
        }
        __syncthreads();
    }

    // lane holds channel (lane & 31) and rows 8 (r / 4) + 4 (lane >> 5) + r % 4 of the wave's 32 x 32 block
    const int col = n0 + wave * 32 + (lane & 31);
    if (col >= p.n) return;
    const float wscale = __half2float(ws[col]);
    const int coefficient_sum = Q4 ? 5 : 1;  // e8p_core.py:154-189
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int local = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (local < rows_here) {
            const int64_t row = row0 + local;
            const int value = (int)(2u * (uint32_t)acc[r] + (uint32_t)coefficient_sum * (uint32_t)p.sum[row]);
            p.out[row * p.n + col] = __float2half_rn(rescale(value, wscale, __half2float(p.as[row])));
        }
    }
}

// ---- host side --------------------------------------------------------------------------------------

bool plane_shape_ok(const char* symbol, int rows, int k) {
    if (rows > 0 && k > 0 && k % 128 == 0) return true;
    set_error("%s: need rows > 0 and K a positive multiple of 128", symbol);
    return false;
}

// slots used: K, M (rows), algorithm (mode), flags (bit0 K64-major), E, top_k, block_m, tiles (capacity)
int split_geometry(const orx_function& f, int rows, Geometry* g) {
    g->block[0] = kPlaneThreads;
    if (f.algorithm == kSplitTiles)
        g->grid[0] = (uint32_t)std::max(1, std::min(f.tiles, (rows + f.block_m - 1) / f.block_m + std::min(f.E, rows)));
    else
        g->grid[0] = ceil_div((uint32_t)rows, kPlaneWaves);
    return ORX_OK;
}

int split_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    PlaneParams p = {};
    p.k = f.K, p.rows = rows, p.group_major = f.flags & 1, p.mode = f.algorithm, p.block_m = f.block_m, p.top_k = f.top_k;
    p.plane_rows = rows;
    switch (f.algorithm) {
        case kSplitRows:  // A, High, Low, Sum
            p.a = pointer_arg<const int8_t>(args, 0), p.high = pointer_arg<uint32_t>(args, 1);
            p.low = pointer_arg<uint32_t>(args, 2), p.sum = pointer_arg<int>(args, 3);
            break;
        case kSplitTiles:  // A, Counts, High, Low, Offsets, Sum, TC, TE, TR
            p.a = pointer_arg<const int8_t>(args, 0), p.counts = pointer_arg<const int>(args, 1);
            p.high = pointer_arg<uint32_t>(args, 2), p.low = pointer_arg<uint32_t>(args, 3);
            p.offsets = pointer_arg<const int>(args, 4), p.sum = pointer_arg<int>(args, 5);
            p.tile_count = pointer_arg<const int>(args, 6), p.tile_expert = pointer_arg<const int>(args, 7);
            p.tile_row = pointer_arg<const int>(args, 8);
            break;
        case kDispatchSlots:  // A, DS, High, IDs, Low, RelativeSlot, RowOffsets, Scale, SlotMap, Sum
            p.a = pointer_arg<const int8_t>(args, 0), p.ds = pointer_arg<__half>(args, 1);
            p.high = pointer_arg<uint32_t>(args, 2), p.ids = pointer_arg<const int>(args, 3);
            p.low = pointer_arg<uint32_t>(args, 4), p.relative = pointer_arg<const int>(args, 5);
            p.row_offsets = pointer_arg<const int>(args, 6), p.scale = pointer_arg<const __half>(args, 7);
            p.slot_map = pointer_arg<int>(args, 8), p.sum = pointer_arg<int>(args, 9);
            p.plane_rows = rows * f.top_k;
            break;
        default:  // A, High, IDs, Low, RelativeSlot, RowOffsets, SlotMap, Sources, Sum
            p.a = pointer_arg<const int8_t>(args, 0), p.high = pointer_arg<uint32_t>(args, 1);
            p.ids = pointer_arg<const int>(args, 2), p.low = pointer_arg<uint32_t>(args, 3);
            p.relative = pointer_arg<const int>(args, 4), p.row_offsets = pointer_arg<const int>(args, 5);
            p.slot_map = pointer_arg<int>(args, 6), p.sources = pointer_arg<int>(args, 7);
            p.sum = pointer_arg<int>(args, 8);
            break;
    }
    ORX_LAUNCH(plane_split_kernel, dim3(g.grid[0]), dim3(g.block[0]), 0, stream, p);
    return hip_check(hipGetLastError(), "launch plane split");
}

int finish_split(orx_function* f) {
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = reinterpret_cast<const void*>(&plane_split_kernel);
    f->geometry = split_geometry;
    f->launch = split_launch;
    return ORX_OK;
}

// split_a8 (kernels/cuda/model/e8p_exact.py:17-46) and split_prefill_a8 (e8p_prefill.py:69-86)
int make_split(const Variant& v, orx_function* f, bool group_major) {
    const char* symbol = group_major ? "split_prefill_a8" : "split_a8";
    bool bad = false;
    f->capacity = f->M = (int)v.integer("rows", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!plane_shape_ok(symbol, f->M, f->K)) return ORX_ERR_BAD_VARIANT;
    f->algorithm = kSplitRows, f->flags = group_major ? 1 : 0;
    f->args = {{"A", ArgPointer, 8}, {"High", ArgPointer, 4}, {"Low", ArgPointer, 4}, {"Sum", ArgPointer, 4}};
    return finish_split(f);
}
int make_split_a8(const Variant& v, orx_function* f) { return make_split(v, f, false); }
int make_split_prefill_a8(const Variant& v, orx_function* f) { return make_split(v, f, true); }

// split_routed_prefill_a8 (e8p_prefill.py:89-129)
int make_split_routed(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("rows", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->E = (int)v.integer("experts", 0, &bad);
    f->block_m = (int)v.integer("block_m", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!plane_shape_ok("split_routed_prefill_a8", f->M, f->K)) return ORX_ERR_BAD_VARIANT;
    if (f->E <= 0 || f->block_m <= 0 || f->block_m % 4) {
        set_error("split_routed_prefill_a8: need experts > 0 and block_m a positive multiple of 4");
        return ORX_ERR_BAD_VARIANT;
    }
    f->tiles = (f->M + f->block_m - 1) / f->block_m + std::min(f->E, f->M);  // e8p_prefill.py:97
    f->algorithm = kSplitTiles, f->flags = 1;
    f->args = {{"A", ArgPointer, 8},       {"Counts", ArgPointer, 4}, {"High", ArgPointer, 4},
               {"Low", ArgPointer, 4},     {"Offsets", ArgPointer, 4}, {"Sum", ArgPointer, 4},
               {"TC", ArgPointer, 4},      {"TE", ArgPointer, 4},      {"TR", ArgPointer, 4}};
    return finish_split(f);
}

bool routed_shape_ok(const char* symbol, const orx_function& f) {
    if (f.E > 0 && f.top_k >= 1 && f.top_k <= f.E && f.top_k <= kMaxChoices) return true;
    set_error("%s: need E > 0 and 1 <= top_k <= min(E, %d)", symbol, kMaxChoices);
    return false;
}

// dispatch_prefill_a8 (e8p_prefill.py:564-622)
int make_dispatch_prefill(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->K = (int)v.integer("K", 2560, &bad);
    f->E = (int)v.integer("E", 512, &bad);
    f->top_k = (int)v.integer("top_k", 10, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!plane_shape_ok("dispatch_prefill_a8", f->M, f->K) || !routed_shape_ok("dispatch_prefill_a8", *f))
        return ORX_ERR_BAD_VARIANT;
    f->algorithm = kDispatchSlots, f->flags = 1;
    f->args = {{"A", ArgPointer, 8},          {"DS", ArgPointer, 2},           {"High", ArgPointer, 4},
               {"IDs", ArgPointer, 4},        {"Low", ArgPointer, 4},          {"RelativeSlot", ArgPointer, 4},
               {"RowOffsets", ArgPointer, 4}, {"Scale", ArgPointer, 2},        {"SlotMap", ArgPointer, 4},
               {"Sum", ArgPointer, 4}};
    return finish_split(f);
}

// pack_expert_tokens (e8p_prefill.py:625-652): always takes the live row count
int make_pack_tokens(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->top_k = (int)v.integer("top_k", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!plane_shape_ok("pack_expert_tokens", f->M, f->K) || !routed_shape_ok("pack_expert_tokens", *f))
        return ORX_ERR_BAD_VARIANT;
    f->dynamic_rows = true;
    f->algorithm = kPackTokens, f->flags = 1;
    f->args = {{"A", ArgPointer, 8},       {"High", ArgPointer, 4},         {"IDs", ArgPointer, 4},
               {"Low", ArgPointer, 4},     {"RelativeSlot", ArgPointer, 4}, {"RowOffsets", ArgPointer, 4},
               {"SlotMap", ArgPointer, 4}, {"Sources", ArgPointer, 4},      {"Sum", ArgPointer, 4}};
    return finish_split(f);
}

// expand_expert_slots (e8p_prefill.py:655-690).  slots used: K, top_k
int expand_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)rows * (uint32_t)f.top_k, 32);
    g->grid[1] = (uint32_t)f.K / 64;
    g->block[0] = kPlaneThreads;
    return ORX_OK;
}

// DS, High, Low, Scale, Sources, SrcHigh, SrcLow, SrcSum, Sum, m
int expand_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    ORX_LAUNCH(plane_expand_kernel, dim3(g.grid[0], g.grid[1]), dim3(g.block[0]), 0, stream,
                       pointer_arg<const uint32_t>(args, 6), pointer_arg<const uint32_t>(args, 5),
                       pointer_arg<const int>(args, 7), pointer_arg<const __half>(args, 3),
                       pointer_arg<const int>(args, 4), pointer_arg<uint32_t>(args, 2), pointer_arg<uint32_t>(args, 1),
                       pointer_arg<int>(args, 8), pointer_arg<__half>(args, 0), rows, rows * f.top_k);
    return hip_check(hipGetLastError(), "launch expand_expert_slots");
}

int make_expand_slots(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->top_k = (int)v.integer("top_k", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (!plane_shape_ok("expand_expert_slots", f->M, f->K)) return ORX_ERR_BAD_VARIANT;
    if (f->top_k < 1) {
        set_error("expand_expert_slots: need top_k >= 1");
        return ORX_ERR_BAD_VARIANT;
    }
    f->dynamic_rows = true;
    f->args = {{"DS", ArgPointer, 2},      {"High", ArgPointer, 4},   {"Low", ArgPointer, 4},
               {"Scale", ArgPointer, 2},   {"Sources", ArgPointer, 4}, {"SrcHigh", ArgPointer, 4},
               {"SrcLow", ArgPointer, 4},  {"SrcSum", ArgPointer, 4},  {"Sum", ArgPointer, 4},
               {"m", ArgI32, 4}};
    f->device_function = reinterpret_cast<const void*>(&plane_expand_kernel);
    f->geometry = expand_geometry;
    f->launch = expand_launch;
    return ORX_OK;
}

// slots used: N, K, E, tiles, block_m (rows per workgroup), group (row step of the tile list), flags (bit0 K64-major
// planes, bit1 two-stage codes)
int plane_gemm_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)f.N, kTileChannels);
    int tiles = f.tiles;
    // e8p_exact.py:76, e8p_prefill.py:189-192: no more tiles than the live rows can fill
    if (f.dynamic_rows) tiles = std::min(tiles, (rows + f.group - 1) / f.group + std::min(f.E, rows));
    if (f.algorithm == 0) {  // the weight-streaming kernel
        stream_grouped_geometry(f.N, std::max(tiles, 1), g);
        return ORX_OK;
    }
    g->grid[1] = (uint32_t)std::max(tiles, 1);
    g->block[0] = kPlaneThreads;
    return ORX_OK;
}

// AS, Book, Counts, High, Low, Offsets, Out, P, Sum, TC, TE, TR, WS[, m]
// (crates/orinfer-models/src/flash_next/experts.rs:207-210 binds the exact kernel in this order)
int plane_gemm_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    PlaneGemmParams p = {};
    p.as = pointer_arg<const __half>(args, 0), p.book = pointer_arg<const uint32_t>(args, 1);
    p.counts = pointer_arg<const int>(args, 2), p.high = pointer_arg<const uint32_t>(args, 3);
    p.low = pointer_arg<const uint32_t>(args, 4), p.offsets = pointer_arg<const int>(args, 5);
    p.out = pointer_arg<__half>(args, 6), p.codes = pointer_arg<const void>(args, 7);
    p.sum = pointer_arg<const int>(args, 8), p.tile_count = pointer_arg<const int>(args, 9);
    p.tile_expert = pointer_arg<const int>(args, 10), p.tile_row = pointer_arg<const int>(args, 11);
    p.ws = pointer_arg<const __half>(args, 12);
    p.n = f.N, p.k = f.K, p.rows = rows, p.tile_rows = f.block_m, p.list_rows = f.group;
    p.group_major = f.flags & 1, p.selector_book = (f.flags & 2) ? 1 : 0;
    p.expert_stride = (int64_t)f.N * f.K / ((f.flags & 2) ? 2 : 4);  // 4 or 2 bits per weight
    if (f.algorithm == 0)
        return stream_planes_launch((f.flags & 2) != 0, p.low, p.high, p.sum, p.codes, p.book, p.selector_book != 0, p.ws, p.as, p.out,
                                    p.counts, p.offsets, p.tile_expert, p.tile_row, p.tile_count, f.N, f.K, rows, p.group_major != 0,
                                    p.tile_rows, p.list_rows, g, stream);
    const dim3 grid(g.grid[0], g.grid[1]), block(g.block[0]);
    if (f.flags & 2)
        ORX_LAUNCH(plane_gemm_kernel<true>, grid, block, 0, stream, p);
    else
        ORX_LAUNCH(plane_gemm_kernel<false>, grid, block, 0, stream, p);
    return hip_check(hipGetLastError(), "launch grouped GEMM on planes");
}

int finish_plane_gemm(const Variant& v, const char* symbol, orx_function* f) {
    bool bad = false;
    // stream: codes decoded straight into MFMA operands, K split over two waves (k_stream.hip); tiles: operands staged in
    // LDS (plane_gemm_kernel).  Measured at 2048 slots in 177 tiles of 16 rows: N = 1024, K = 2048: 35.5 against 43.2 us;
    // N = 2048, K = 512: 29.2 against 25.4 us (the streaming kernel's set-up is paid per 128 channels and tile).
    const std::string algorithm = v.string("algorithm", "auto", &bad);
    if (bad || (algorithm != "auto" && algorithm != "stream" && algorithm != "tiles")) {
        set_error("%s: algorithm is auto, stream or tiles", symbol);
        return ORX_ERR_BAD_VARIANT;
    }
    f->algorithm = algorithm == "tiles" || (algorithm == "auto" && f->K < 1024) ? 1 : 0;
    if (f->M <= 0 || f->E <= 0 || f->tiles <= 0 || f->N <= 0 || f->K <= 0 || f->K % 128 ||
        (int64_t)f->K * 128 * 128 > 2147483647ll) {  // e8p_exact.py:60-61: the int32 accumulator holds a whole row
        set_error("%s: need rows, E, tiles, N > 0 and K a multiple of 128 with K * 128 * 128 < 2^31", symbol);
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"AS", ArgPointer, 2},     {"Book", ArgPointer, 4},   {"Counts", ArgPointer, 4}, {"High", ArgPointer, 8},
               {"Low", ArgPointer, 8},    {"Offsets", ArgPointer, 4}, {"Out", ArgPointer, 2},    {"P", ArgPointer, 16},
               {"Sum", ArgPointer, 4},    {"TC", ArgPointer, 4},      {"TE", ArgPointer, 4},     {"TR", ArgPointer, 4},
               {"WS", ArgPointer, 2}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = f->algorithm == 0 ? nullptr  // 512 threads: the device's own limit
                         : (f->flags & 2)  ? reinterpret_cast<const void*>(&plane_gemm_kernel<true>)
                                           : reinterpret_cast<const void*>(&plane_gemm_kernel<false>);
    f->geometry = plane_gemm_geometry;
    f->launch = plane_gemm_launch;
    return ORX_OK;
}

// e8p_exact_grouped (kernels/cuda/model/e8p_exact.py:49-316): row-major planes, single-stage codes in K-major
// blocks of 64, Book = nibble words
int make_exact_grouped(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("rows", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->tiles = (int)v.integer("tiles", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->block_m = (int)v.integer("block_m", 16, &bad);
    const int stages = (int)v.integer("stages", 2, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    v.boolean("warp_private", false, &bad);  // a schedule of the reference's kernel
    if (bad) return ORX_ERR_BAD_VARIANT;
    if ((f->block_m != 8 && f->block_m != 16) || stages < 2 || stages > 4 || f->K / 64 < stages - 1) {
        set_error("e8p_exact_grouped: block_m is 8 or 16, stages 2..4 with K / 64 >= stages - 1");
        return ORX_ERR_BAD_VARIANT;
    }
    f->group = f->block_m, f->flags = 0;
    return finish_plane_gemm(v, "e8p_exact_grouped", f);
}

// e8p_prefill_grouped (e8p_prefill.py:132-561): K64-major planes (row-major on request), single-stage codes in
// blocks of 64 with nibble words as Book, or two-stage codes in blocks of 128 with selector words
int make_prefill_grouped(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("rows", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->tiles = (int)v.integer("tiles", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    v.boolean("sparse_rows", false, &bad);  // skips empty row stripes: a schedule, the results are the same
    const bool row_major = v.boolean("row_major", false, &bad);
    const std::string codec = v.string("codec", "e8p_q2", &bad);
    const int minimum_blocks = (int)v.integer("minimum_blocks", 1, &bad);
    f->block_m = (int)v.integer("block_m", 16, &bad);
    const int block_n = (int)v.integer("block_n", 128, &bad);
    const bool tails = v.boolean("specialize_tails", false, &bad);
    const bool merge = v.boolean("merge_routed_tiles", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    const bool q4 = codec == "e8p_q4";
    if ((!q4 && codec != "e8p_q2") || minimum_blocks < 1 || minimum_blocks > 16 || (f->block_m != 16 && f->block_m != 32) ||
        (block_n != 64 && block_n != 128) || (block_n != 128 && q4) || (tails && (f->block_m != 32 || q4)) ||
        (merge && !tails)) {  // e8p_prefill.py:163-183
        set_error("e8p_prefill_grouped: codec e8p_q2|e8p_q4, minimum_blocks 1..16, block_m 16|32, block_n 64|128 (128 with "
                  "e8p_q4), specialize_tails with block_m 32 and e8p_q2 only, merge_routed_tiles with specialize_tails only");
        return ORX_ERR_BAD_VARIANT;
    }
    f->group = merge ? f->block_m / 2 : f->block_m;  // e8p_prefill.py:188
    f->flags = (row_major ? 0 : 1) | (q4 ? 2 : 0);
    return finish_plane_gemm(v, "e8p_prefill_grouped", f);
}

}  // namespace

const Registration* plane_registrations(int* count) {
    static const Registration rows[] = {
        {"split_a8", make_split_a8, "rows, K, dynamic_rows=false", "A,High,Low,Sum[,m]"},
        {"split_prefill_a8", make_split_prefill_a8, "rows, K, dynamic_rows=false", "A,High,Low,Sum[,m]"},
        {"split_routed_prefill_a8", make_split_routed, "rows, K, experts, block_m, dynamic_rows=false",
         "A,Counts,High,Low,Offsets,Sum,TC,TE,TR[,m]"},
        {"dispatch_prefill_a8", make_dispatch_prefill, "M, K=2560, E=512, top_k=10, dynamic_rows=false",
         "A,DS,High,IDs,Low,RelativeSlot,RowOffsets,Scale,SlotMap,Sum[,m]"},
        {"pack_expert_tokens", make_pack_tokens, "M, K, E, top_k", "A,High,IDs,Low,RelativeSlot,RowOffsets,SlotMap,Sources,Sum,m"},
        {"expand_expert_slots", make_expand_slots, "M, K, top_k", "DS,High,Low,Scale,Sources,SrcHigh,SrcLow,SrcSum,Sum,m"},
        {"e8p_exact_grouped", make_exact_grouped,
         "rows, E, tiles, N, K, block_m=16|8, stages=2..4, dynamic_rows=false, warp_private=false, algorithm=auto|stream|tiles",
         "AS,Book,Counts,High,Low,Offsets,Out,P,Sum,TC,TE,TR,WS[,m]"},
        {"e8p_prefill_grouped", make_prefill_grouped,
         "rows, E, tiles, N, K, dynamic_rows=false, sparse_rows=false, row_major=false, codec=e8p_q2|e8p_q4, "
         "minimum_blocks=1, block_m=16|32, block_n=128|64, specialize_tails=false, merge_routed_tiles=false, algorithm=auto|stream|tiles",
         "AS,Book,Counts,High,Low,Offsets,Out,P,Sum,TC,TE,TR,WS[,m]"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
