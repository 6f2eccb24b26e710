// Routed single-stage (Q2) expert projections when the routed tiles are many enough to occupy the
// whole chip: one resident workgroup of 16 waves per CU.
//
// Reference counterpart: the warp-owned routed decode kernels/cuda/model/e8p_decode.py:36-245 (codes
// go from global memory through a lookup table straight into MMA operand registers) behind the tile
// metadata of kernels/cuda/model/routing.py.  Arithmetic: exact int32 over the full K,
// (float(acc) * ws) * as, rounded to fp16 once.
//
// MI355X design.  The work is a weight stream (2 bits per weight, every expert's matrix read once
// per routed tile) against at most 32 token rows per tile, so it is bound by HBM and by the decode.
//  * A unit is (tile, 512 output channels): each of the 16 waves owns 32 channels over the full K,
//    so there is no split-K reduction and no barrier inside a unit.  A wave streams its codes with
//    one 16-byte load per lane and 128-wide K block through a register ring that is refilled right
//    after use, also across the end of a unit into the first blocks of the next one.
//  * The tile's activations are staged once per workgroup into LDS with coalesced 16-byte loads
//    (rows padded by 16 bytes, so the per-lane 16-byte fragment reads do not collide); fetching
//    them per lane from L1 costs one cache access per lane and instruction and was the limit of the
//    streaming kernel this one replaces for large routed batches.
//  * The two 8-byte table lookups per code are random; each table entry is stored 16 times (entry i
//    for lane l at byte i*128 + (l%16)*8) so the lanes of one access group never share a bank.
//  * Units are dealt to workgroups in contiguous runs (a run mostly stays inside one tile, so the
//    staged rows are reused).  What does not divide evenly is finished in a second phase where a
//    32-channel block is split over K between the waves and summed with LDS integer atomics
//    (integer addition is exact in any order), so no CU has to run a whole extra unit.
//  * Three launches of the expert layer can disappear into this kernel (INPUT, EPILOGUE):
//    - the dispatch copy: int8 token rows are gathered through the slot -> token map while a tile is
//      staged (kInputGather), so nobody copies a token's row top_k times into slot order;
//    - the SwiGLU -> A8 launch between the two projections: with kEpilogueSwiglu a wave owns 16 gate
//      and the 16 matching up channels, so gate and up of one (token, channel) sit in one lane; the
//      epilogue writes fp16(silu(gate) * up) and raises the slot's largest magnitude with an
//      integer atomic max (non-negative fp32 bits order like integers).  The next projection
//      (kInputAct) reads those fp16 rows and maxima and quantises them while it stages a tile.
//    The arithmetic of every value is that of the separate launches, so the bits are the same.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>

#include "a8_device.h"
#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kSpan = kWaves * 32;             // output channels of one unit
constexpr uint32_t kBasisBase = 0;             // 256 entries x 16 copies x 8 bytes
constexpr uint32_t kMaskBase = 32768;
constexpr uint32_t kInfoBase = 65536;          // (expert, first row, rows) of every routed tile
constexpr int kMaxTiles = 1024;
constexpr uint32_t kRowStatBase = kInfoBase + kMaxTiles * 12;  // fp16 rows quantised while staged: the scale of every staged row
constexpr uint32_t kSumBase = kRowStatBase + 256;          // phase-two sums, then the staged token rows
constexpr int kRowPad = 16;
constexpr int kSumStride = 33;                 // ints per token row of a phase-two sum block
constexpr int kSumBlock = 32 * kSumStride;     // ints
constexpr int kMaxPieces = 5;                  // 16-byte pieces a thread stages per tile (K <= 2560)
constexpr int kMaxHalfPieces = 4;              // fp16 input: 16-byte pieces of 8 values per thread and tile (K <= 1024)
constexpr int kMaxSlots = 8192;                // rows gathered by slot: the slot -> token map sits in LDS as u16
enum { kInputInt8 = 0, kInputGather = 1, kInputAct = 2 };
enum { kEpiloguePlain = 0, kEpilogueSwiglu = 1 };

struct GroupedParams {
    const int8_t* a;               // kInputInt8: (slots, K) int8; kInputGather: (tokens, K) int8
    const __half* x;               // kInputAct: (slots, K) fp16
    const int* slot_token;         // kInputGather: token of every slot
    const int* row_max_in;         // kInputAct: fp32 bits of every slot's largest magnitude
    __half* as_out;                // kInputAct: the row scales, written once per slot (may be null)
    int8_t* q_out;                 // kInputAct: the codes, written once per slot (may be null)
    __half* act;                   // kEpilogueSwiglu: (slots, N/2) fp16(silu(gate) * up)
    int* row_max_out;              // kEpilogueSwiglu: raised to the fp32 bits of the slot's largest |act|
    int slots;
    const uint8_t* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    __half* out;
    const int* counts;
    const int* offsets;
    const int* tile_expert;
    const int* tile_row;
    const int* tile_count;
    int n, k, k_major, tile_capacity;
    int64_t expert_weight_stride;  // bytes
};

struct Tile {
    int expert, row0, rows;
};

// The split of K between waves in phase two: K blocks per wave, waves per 32-channel block, blocks
// a workgroup sums at once.
struct Split {
    int slice, ways, per_pass;
};
__host__ __device__ inline Split phase_two_split(int kb_count) {
    Split s;
    s.slice = (kb_count + kWaves - 1) / kWaves;
    s.ways = (kb_count + s.slice - 1) / s.slice;
    s.per_pass = kWaves / s.ways;
    return s;
}

// D: K blocks per ring group (the ring depth); K/128 is a multiple of it.
template <int D, int INPUT = kInputInt8, int EPILOGUE = kEpiloguePlain>
__global__ __launch_bounds__(kThreads) void grouped_resident_kernel(GroupedParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, frag = lane & 31;
    const int kb_count = p.k / 128;
    // channels a unit covers: 512 outputs, or 256 gate + the 256 matching up channels
    const int inner = p.n / 2;  // kEpilogueSwiglu: N = gate | up
    const int spans = EPILOGUE == kEpilogueSwiglu ? (inner + kSpan / 2 - 1) / (kSpan / 2) : (p.n + kSpan - 1) / kSpan;
    const int groups = (int)gridDim.x, group = (int)blockIdx.x;
    const Split split = phase_two_split(kb_count);
    // forms without a phase two (see below) have no sum blocks, and the staged rows start where those would
    constexpr bool kPhaseTwo = INPUT != kInputAct && EPILOGUE == kEpiloguePlain;
    const uint32_t tile_base = kSumBase + (kPhaseTwo ? (uint32_t)split.per_pass * kSumBlock * 4 : 0u);
    const int tile_stride = p.k + kRowPad;
    int* sums = reinterpret_cast<int*>(lds + kSumBase);
    __half* row_scale = reinterpret_cast<__half*>(lds + kRowStatBase);     // kInputAct: scales of the staged rows
    uint16_t* slot_tokens = reinterpret_cast<uint16_t*>(lds + tile_base + 32 * tile_stride);  // kInputGather

    // ---- set-up: two round trips to memory, then one barrier ------------------------------------
    // First trip: the selector table (waves 0-3 build the basis table from it, waves 4-7 the mask
    // table, which needs no load), the tile count and, one tile per thread, every tile's expert and
    // first row.  Second trip: that expert's row count and offset.  The tile list then sits in LDS,
    // so nothing later in the kernel waits for a chain of dependent loads.
    uint32_t selector = 0;
    if (wave < 4) selector = p.book[tid];
    const int listed = min(p.tile_capacity, kMaxTiles);
    const int my_tile = min(tid, listed - 1);
    const int my_expert = p.tile_expert[my_tile], my_first = p.tile_row[my_tile];
    const int tile_count = min(p.tile_count[0], listed);
    const bool listed_here = tid < tile_count;
    const int safe_expert = listed_here ? my_expert : 0;  // entries beyond the count are not initialised
    const int my_count = p.counts[safe_expert], my_offset = p.offsets[safe_expert];
    if (wave < 8) {
        const int entry = tid & 255;
        const uint2 value = wave < 4 ? byte_basis_signed(selector) : byte_mask_signed((uint32_t)entry);
        const uint4 pair = make_uint4(value.x, value.y, value.x, value.y);
        uint8_t* dst = lds + (wave < 4 ? kBasisBase : kMaskBase) + entry * 128;
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(dst + 16 * i) = pair;
    }
    if (kPhaseTwo)
        for (int i = tid; i < split.per_pass * kSumBlock; i += kThreads) sums[i] = 0;
    if constexpr (INPUT == kInputGather)  // same trip as the tile list: nothing below waits for slot -> token -> row
        for (int i = tid; i < p.slots; i += kThreads) slot_tokens[i] = (uint16_t)p.slot_token[i];
    if (listed_here) {
        int* info = reinterpret_cast<int*>(lds + kInfoBase) + 3 * tid;
        info[0] = my_expert, info[1] = my_offset + my_first, info[2] = min(32, my_count - my_first);
    }
    __syncthreads();
    auto tile_info = [&](int tile) {
        const int* info = reinterpret_cast<const int*>(lds + kInfoBase) + 3 * tile;
        Tile t;
        t.expert = __builtin_amdgcn_readfirstlane(info[0]);
        t.row0 = __builtin_amdgcn_readfirstlane(info[1]);
        t.rows = __builtin_amdgcn_readfirstlane(info[2]);
        return t;
    };

    // ---- how the units are dealt -----------------------------------------------------------
    // Every workgroup runs `full` units; the rest is either one more unit for the first
    // workgroups or, when that rest is small, split over K in phase two.  Runs are contiguous, so
    // a run mostly stays inside one tile and its staged rows are reused.
    const int units = tile_count * spans;
    const int full = units / groups;
    int leftover = units - full * groups;
    const int passes = (leftover * kWaves + groups * split.per_pass - 1) / (groups * split.per_pass);
    int my_units = full, first_unit = group * full;
    // (phase two reads int8 rows from memory and has the plain epilogue)
    if (!kPhaseTwo || passes > max(1, kb_count / 8)) {
        first_unit += min(group, leftover);
        if (group < leftover) ++my_units;
        leftover = 0;
    }

    // ---- weight stream of this lane ----------------------------------------------------------
    const int64_t kb_step = p.k_major ? (int64_t)p.n * 32 : 32;
    // kEpilogueSwiglu: n0 is the wave's first inner channel; lanes 0-15 of a half wave stream the gate
    // rows n0.., lanes 16-31 the up rows inner + n0..
    auto lane_weights = [&](int expert, int n0) -> const uint8_t* {
        const int64_t row = EPILOGUE == kEpilogueSwiglu ? (frag < 16 ? n0 + frag : inner + n0 + frag - 16) : n0 + frag;
        const int64_t offset = p.k_major ? row * 32 : row * kb_count * 32;
        return p.w + (int64_t)expert * p.expert_weight_stride + offset + half * 16;
    };
    auto fetch = [&](const uint8_t* base, int kb) { return *reinterpret_cast<const uint4*>(base + kb * kb_step); };

    // ---- decode ------------------------------------------------------------------------------
    const uint32_t copy = (uint32_t)(lane & 15) * 8;
    auto lookup = [&](uint32_t byte) { return *reinterpret_cast<const uint2*>(lds + byte); };
    auto decode_pair = [&](uint32_t word) -> v4i {  // two codes -> the 16 weights of one MFMA sub-step
        const uint2 b0 = lookup(kBasisBase + (((word & 0xFF00u) >> 1) | copy));
        const uint2 m0 = lookup(kMaskBase + (((word & 0xFFu) << 7) | copy));
        const uint2 b1 = lookup(kBasisBase + (((word >> 17) & 0x7F80u) | copy));
        const uint2 m1 = lookup(kMaskBase + (((word >> 9) & 0x7F80u) | copy));
        return v4i{(int)(b0.x ^ m0.x), (int)(b0.y ^ m0.y), (int)(b1.x ^ m1.x), (int)(b1.y ^ m1.y)};
    };

    // ---- staging of a tile's token rows ------------------------------------------------------
    // Register arrays hold the native vector type: an array of HIP's uint4 struct that is filled in
    // one lambda and read in another is kept in scratch memory by the compiler.
    v4u held[kMaxPieces];
    int held_max[INPUT == kInputAct ? kMaxHalfPieces : 1];
    const int row_pieces = p.k / 16;
    const int half_pieces = p.k / 8;  // kInputAct: pieces of 8 fp16 values per row
    auto stage_load = [&](const Tile& t) {
        // unconditional loads of clamped pieces, so that all of them are in flight together
        const int first_row = t.rows > 0 ? t.row0 : 0;
        if constexpr (INPUT == kInputInt8) {
            const v4u* src = reinterpret_cast<const v4u*>(p.a + (int64_t)first_row * p.k);
            const int last_piece = max(t.rows * row_pieces, 1) - 1;
#pragma unroll
            for (int i = 0; i < kMaxPieces; ++i) held[i] = src[min(tid + i * kThreads, last_piece)];
        } else if constexpr (INPUT == kInputGather) {
            const int last_piece = max(t.rows * row_pieces, 1) - 1;
#pragma unroll
            for (int i = 0; i < kMaxPieces; ++i) {
                const int piece = min(tid + i * kThreads, last_piece);
                const int row = piece / row_pieces, col = piece - row * row_pieces;
                const int64_t token = slot_tokens[first_row + row];
                held[i] = *reinterpret_cast<const v4u*>(p.a + token * p.k + col * 16);
            }
        } else {
            const int last_piece = max(t.rows * half_pieces, 1) - 1;
#pragma unroll
            for (int i = 0; i < kMaxHalfPieces; ++i) {
                const int piece = min(tid + i * kThreads, last_piece);
                const int row = piece / half_pieces;
                held[i] = reinterpret_cast<const v4u*>(p.x + (int64_t)first_row * p.k)[piece];
                held_max[i] = p.row_max_in[first_row + row];
            }
        }
    };
    // `publish`: this workgroup holds the tile's first span, so it is the one that writes the
    // tile's scales (and codes) to memory for whoever wants to look at them.
    auto stage_store = [&](const Tile& t, bool publish) {
        if constexpr (INPUT != kInputAct) {
            const int pieces = t.rows * row_pieces;
#pragma unroll
            for (int i = 0; i < kMaxPieces; ++i) {
                const int piece = tid + i * kThreads;
                if (piece < pieces) {
                    const int row = piece / row_pieces, col = piece - row * row_pieces;
                    *reinterpret_cast<v4u*>(lds + tile_base + row * tile_stride + col * 16) = held[i];
                }
            }
        } else {
            const int pieces = t.rows * half_pieces;
#pragma unroll
            for (int i = 0; i < kMaxHalfPieces; ++i) {
                const int piece = tid + i * kThreads;
                if (piece < pieces) {
                    const int row = piece / half_pieces, col = piece - row * half_pieces;
                    const __half stored = a8_scale(__int_as_float(held_max[i]));
                    const float scale = __half2float(stored), inverse = __frcp_rn(scale);
                    const __half* h = reinterpret_cast<const __half*>(&held[i]);
                    const float low[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
                    const float high[4] = {__half2float(h[4]), __half2float(h[5]), __half2float(h[6]), __half2float(h[7])};
                    const uint2 codes = make_uint2(quantise4(low, scale, inverse), quantise4(high, scale, inverse));
                    *reinterpret_cast<uint2*>(lds + tile_base + row * tile_stride + col * 8) = codes;
                    if (col == 0) row_scale[row] = stored;
                    if (publish) {
                        if (col == 0 && p.as_out != nullptr) p.as_out[t.row0 + row] = stored;
                        if (p.q_out != nullptr)
                            *reinterpret_cast<uint2*>(p.q_out + (int64_t)(t.row0 + row) * p.k + col * 8) = codes;
                    }
                }
            }
        }
    };
    // scale of the token in slot `row`
    auto token_scale_of = [&](int64_t row) -> __half {
        if constexpr (INPUT == kInputGather) return p.as[slot_tokens[row]];
        return p.as[row];
    };

    // accumulator register r of a lane: channel 8*(r/4) + 4*half + r%4 of the block, token `frag`
    // (kEpilogueSwiglu: channels 0-15 of the block are gate channels n0.., 16-31 the up channels
    // inner + n0.., so registers r and r + 8 hold gate and up of one inner channel)
    struct Scales {
        uint2 weight[4];  // four fp16 channel scales per 8-channel step
        __half token;
    };
    auto load_scales = [&](int expert, int64_t row, int n0) {
        Scales s;
        const __half* scales = p.ws + (int64_t)expert * p.n + n0 + 4 * half;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int at = EPILOGUE == kEpilogueSwiglu ? (j < 2 ? 8 * j : inner + 8 * (j - 2)) : 8 * j;
            s.weight[j] = *reinterpret_cast<const uint2*>(scales + at);
        }
        if constexpr (INPUT != kInputAct) s.token = token_scale_of(row);
        return s;
    };
    auto channel_scales = [](const uint2& bits, float (&s)[4]) {
        const __half2 s01 = *reinterpret_cast<const __half2*>(&bits.x), s23 = *reinterpret_cast<const __half2*>(&bits.y);
        s[0] = __low2float(s01), s[1] = __high2float(s01), s[2] = __low2float(s23), s[3] = __high2float(s23);
    };
    auto pack4 = [](const __half (&h)[4]) {
        uint2 packed;
        packed.x = (uint32_t)__half_as_ushort(h[0]) | (uint32_t)__half_as_ushort(h[1]) << 16;
        packed.y = (uint32_t)__half_as_ushort(h[2]) | (uint32_t)__half_as_ushort(h[3]) << 16;
        return packed;
    };
    auto store_block = [&](const v16i& acc, const Scales& scales, int64_t row, int n0, bool live) {
        const float token_scale = __half2float(scales.token);
        if constexpr (EPILOGUE == kEpiloguePlain) {
            if (!live) return;
            __half* dst = p.out + row * p.n + n0 + 4 * half;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float s[4];
                channel_scales(scales.weight[j], s);
                __half h[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) h[i] = __float2half_rn(rescale(acc[4 * j + i], s[i], token_scale));
                *reinterpret_cast<uint2*>(dst + 8 * j) = pack4(h);
            }
        } else {
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float sg[4], su[4];
                channel_scales(scales.weight[j], sg);
                channel_scales(scales.weight[j + 2], su);
                __half gate[4], up[4], value[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    gate[i] = __float2half_rn(rescale(acc[4 * j + i], sg[i], token_scale));
                    up[i] = __float2half_rn(rescale(acc[4 * (j + 2) + i], su[i], token_scale));
                    const float v = swiglu_value(gate[i], up[i]);  // already rounded to fp16
                    value[i] = __float2half_rn(v);
                    amax = fmaxf(amax, fabsf(v));
                }
                if (live) {
                    const int64_t at = n0 + 8 * j + 4 * half;
                    *reinterpret_cast<uint2*>(p.act + row * inner + at) = pack4(value);
                    if (p.out != nullptr) {
                        *reinterpret_cast<uint2*>(p.out + row * p.n + at) = pack4(gate);
                        *reinterpret_cast<uint2*>(p.out + row * p.n + inner + at) = pack4(up);
                    }
                }
            }
            // the two half waves hold different channels of the same token
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            if (live && half == 0) atomicMax(p.row_max_out + row, __float_as_int(amax));
        }
    };

    struct Unit {
        int tile, n0, expert, row0, rows;  // n0: first channel of this wave; rows <= 0: nothing to do
    };
    auto unit_at = [&](int u) {
        Unit unit = {-1, 0, 0, 0, 0};
        if (u < my_units) {
            const int index = first_unit + u;
            unit.tile = index / spans;
            const int span = index - unit.tile * spans;
            unit.n0 = EPILOGUE == kEpilogueSwiglu ? span * (kSpan / 2) + wave * 16 : span * kSpan + wave * 32;
            const Tile t = tile_info(unit.tile);
            unit.expert = t.expert, unit.row0 = t.row0;
            unit.rows = unit.n0 < (EPILOGUE == kEpilogueSwiglu ? inner : p.n) ? t.rows : 0;
        }
        return unit;
    };

    // ---- phase two's work of this wave (first pass), requested now and used at the very end --------
    const int blocks = leftover * kWaves, first_leftover = full * groups;
    const int local = wave / split.ways, part = wave - local * split.ways;
    struct Piece {
        int n0, kb_first, kb_last;
        Tile tile;
        bool active;
    };
    auto piece_of = [&](int pass) {
        Piece piece = {0, 0, 0, {0, 0, 0}, false};
        const int block = (pass * groups + group) * split.per_pass + local;
        if (local < split.per_pass && block < blocks) {
            const int unit = first_leftover + block / kWaves;
            const int tile = unit / spans;
            piece.n0 = (unit - tile * spans) * kSpan + (block % kWaves) * 32;
            piece.tile = tile_info(tile);
            piece.kb_first = part * split.slice;
            piece.kb_last = min(kb_count, piece.kb_first + split.slice);
            piece.active = piece.n0 < p.n && piece.tile.rows > 0 && piece.kb_first < piece.kb_last;
        }
        return piece;
    };
    auto piece_rows = [&](const Piece& piece) {
        int64_t row = piece.tile.row0 + min(frag, piece.tile.rows - 1);
        if constexpr (INPUT == kInputGather) row = slot_tokens[row];
        return p.a + row * p.k + half * 64;
    };
    const Piece early = piece_of(0);
    uint4 early_codes = make_uint4(0, 0, 0, 0), early_tokens[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) early_tokens[s] = make_uint4(0, 0, 0, 0);

    // ---- phase one: whole units ------------------------------------------------------------------
    Tile staged_tile = {0, 0, 0};
    int staged = -1;
    uint4 ring[D];
    bool ring_ready = false;
    for (int u = 0; u < my_units; ++u) {
        const Unit cur = unit_at(u), nxt = unit_at(u + 1);
        if (cur.tile != staged) {
            staged_tile = tile_info(cur.tile);
            stage_load(staged_tile);
            if (u == 0) {
                // the first codes and phase two's operands travel together with the first tile's rows
                if (cur.rows > 0) {
                    const uint8_t* weights = lane_weights(cur.expert, cur.n0);
#pragma unroll
                    for (int d = 0; d < D; ++d) ring[d] = fetch(weights, d);
                    ring_ready = true;
                }
            } else {
                __syncthreads();  // every wave has finished with the rows staged before
            }
            stage_store(staged_tile, (first_unit + u) % spans == 0);
            staged = cur.tile;
            __syncthreads();
        }
        // the same wave's block in the next unit, for the refill that crosses the unit's end
        const bool have_next = nxt.rows > 0;
        const uint8_t* next_weights = lane_weights(have_next ? nxt.expert : 0, have_next ? nxt.n0 : 0);
        if (cur.rows <= 0) {
            ring_ready = false;
            if (have_next) {
#pragma unroll
                for (int d = 0; d < D; ++d) ring[d] = fetch(next_weights, d);
                ring_ready = true;
            }
        } else {
            const uint8_t* weights = lane_weights(cur.expert, cur.n0);
            if (!ring_ready) {
#pragma unroll
                for (int d = 0; d < D; ++d) ring[d] = fetch(weights, d);
            }
            const int64_t row = cur.row0 + min(frag, cur.rows - 1);
            Scales scales = load_scales(cur.expert, row, cur.n0);
            if constexpr (INPUT == kInputAct) scales.token = row_scale[min(frag, cur.rows - 1)];
            const uint8_t* rows = lds + tile_base + min(frag, cur.rows - 1) * tile_stride + half * 64;
            v16i acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0;
            for (int g = 0; g < kb_count; g += D) {
                const bool last = g + D >= kb_count;
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    const uint4 codes = ring[d];
                    const uint8_t* refill = last ? next_weights : weights + (g + D) * kb_step;
                    if (!last || have_next) ring[d] = fetch(refill, d);
                    const uint32_t word[4] = {codes.x, codes.y, codes.z, codes.w};
                    const uint8_t* fragment = rows + (g + d) * 128;
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const v4i weight_operand = decode_pair(word[s]);
                        const v4i token_operand = *reinterpret_cast<const v4i*>(fragment + 16 * s);
                        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(weight_operand, token_operand, acc, 0, 0, 0);
                    }
                }
            }
            ring_ready = have_next;
            if (u + 1 == my_units && early.active) {
                // last unit: phase two's first operands are requested before the stores are waited for
                early_codes = fetch(lane_weights(early.tile.expert, early.n0), early.kb_first);
                const uint4* fragment = reinterpret_cast<const uint4*>(piece_rows(early) + early.kb_first * 128);
#pragma unroll
                for (int s = 0; s < 4; ++s) early_tokens[s] = fragment[s];
            }
            store_block(acc, scales, row, cur.n0, frag < cur.rows);
        }
    }

    // ---- phase two: the rest, 32-channel blocks split over K between waves ----------------------
    if (leftover == 0) return;
    const bool early_loaded = my_units > 0 && unit_at(my_units - 1).rows > 0;
    for (int pass = 0; (pass * groups + group) * split.per_pass < blocks; ++pass) {
        const int first_block = (pass * groups + group) * split.per_pass;
        if (pass > 0) {
            __syncthreads();  // the previous pass's sums have been read
            for (int i = tid; i < split.per_pass * kSumBlock; i += kThreads) sums[i] = 0;
            __syncthreads();
        }
        const Piece piece = pass == 0 ? early : piece_of(pass);
        if (piece.active) {
            const uint8_t* weights = lane_weights(piece.tile.expert, piece.n0);
            const int8_t* rows = piece_rows(piece);
            v16i acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0;
            auto multiply = [&](const uint4& codes, const uint4 (&tokens)[4]) {
                const uint32_t word[4] = {codes.x, codes.y, codes.z, codes.w};
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const v4i weight_operand = decode_pair(word[s]);
                    const v4i token_operand = {(int)tokens[s].x, (int)tokens[s].y, (int)tokens[s].z, (int)tokens[s].w};
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(weight_operand, token_operand, acc, 0, 0, 0);
                }
            };
            int kb = piece.kb_first;
            if (pass == 0 && early_loaded) {
                multiply(early_codes, early_tokens);
                ++kb;
            }
            for (; kb < piece.kb_last; ++kb) {
                const uint4 codes = fetch(weights, kb);
                const uint4* fragment = reinterpret_cast<const uint4*>(rows + kb * 128);
                const uint4 tokens[4] = {fragment[0], fragment[1], fragment[2], fragment[3]};
                multiply(codes, tokens);
            }
            int* mine = sums + local * kSumBlock + frag * kSumStride + 4 * half;
#pragma unroll
            for (int r = 0; r < 16; ++r) atomicAdd(mine + 8 * (r >> 2) + (r & 3), acc[r]);
        }
        __syncthreads();
        for (int e = 0; e < split.per_pass; ++e) {
            const int done = first_block + e;
            if (done >= blocks) break;
            const int unit = first_leftover + done / kWaves;
            const int tile = unit / spans;
            const int n0 = (unit - tile * spans) * kSpan + (done % kWaves) * 32;
            const Tile t = tile_info(tile);
            const int token = tid >> 5, channel = tid & 31;
            if (n0 >= p.n || token >= t.rows) continue;
            const int64_t row = t.row0 + token;
            const int total = sums[e * kSumBlock + token * kSumStride + channel];
            const float value = rescale(total, __half2float(p.ws[(int64_t)t.expert * p.n + n0 + channel]),
                                        __half2float(token_scale_of(row)));
            p.out[row * p.n + n0 + channel] = __float2half_rn(value);
        }
    }
}


int ring_depth(int k) {
    const int kb = k / 128;
    return kb % 2 == 0 ? 2 : kb % 3 == 0 ? 3 : 0;
}

uint32_t resident_lds_bytes(int k, int input, int epilogue, int slots) {
    const Split split = phase_two_split(k / 128);
    const bool phase_two = input != kInputAct && epilogue == kEpiloguePlain;  // the others have no sum blocks
    const uint32_t rows = kSumBase + (phase_two ? (uint32_t)split.per_pass * kSumBlock * 4u : 0u) + 32u * (uint32_t)(k + kRowPad);
    return rows + (input == kInputGather ? (((uint32_t)slots * 2u + 15u) & ~15u) : 0u);
}

constexpr uint32_t kLdsLimit = 160 * 1024;

}  // namespace

// Shapes the resident kernel takes: tiles of at most 32 rows, whole 32-channel blocks, a K whose
// blocks divide into ring groups and whose staged rows fit beside the tables.  Gathered rows keep
// the slot -> token map in LDS; fp16 rows are held in registers while a tile is quantised, which
// bounds K; the SwiGLU epilogue pairs 16 gate with 16 up channels per wave.
bool grouped_resident_eligible(int n, int k, int block_m, int tiles, int input, int epilogue, int slots) {
    if (input == kInputGather && slots > kMaxSlots) return false;
    if (input == kInputAct && k > kMaxHalfPieces * kThreads * 8 / 32) return false;
    if (epilogue == kEpilogueSwiglu && n % 32 != 0) return false;  // inner = N/2 a multiple of 16
    return block_m == 32 && n % 32 == 0 && k % 128 == 0 && ring_depth(k) > 0 && tiles <= kMaxTiles &&
           k / 16 <= kMaxPieces * kThreads / 32 && resident_lds_bytes(k, input, epilogue, slots) <= kLdsLimit;
}

// Worth it once the routed tiles give most CUs a unit of their own; below that the streaming
// kernel's many small workgroups spread better (measured crossover: about 32 tokens x top-8 over 128
// experts).  The tile count is only known on the device; with uniform routing `rows` assignments hit
// about E (1 - exp(-rows / E)) experts.
bool grouped_resident_preferred(int rows, int experts, int n) {
    const double hit = experts * (1.0 - std::exp(-(double)rows / experts));
    const double tiles = std::max((double)((rows + 31) / 32), hit);
    return tiles * ((n + kSpan - 1) / kSpan) >= 0.8 * device_compute_units();
}

void grouped_resident_geometry(int k, int input, int epilogue, int slots, Geometry* g) {
    g->grid[0] = (uint32_t)device_compute_units();
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kThreads;
    g->shared = resident_lds_bytes(k, input, epilogue, slots);
}

int grouped_resident_launch(const GroupedBuffers& b, int n, int k, int tiles, int packed_k, int input, int epilogue,
                            int slots, hipStream_t stream) {
    static DeviceOnce opted_in;  // dynamic LDS above 64 KiB needs an opt-in per kernel and device
    const int ready = opted_in.run([] {
        const void* kernels[] = {reinterpret_cast<const void*>(&grouped_resident_kernel<3, kInputInt8, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<2, kInputInt8, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<3, kInputGather, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<2, kInputGather, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<3, kInputAct, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<2, kInputAct, kEpiloguePlain>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<3, kInputInt8, kEpilogueSwiglu>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<2, kInputInt8, kEpilogueSwiglu>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<3, kInputGather, kEpilogueSwiglu>),
                                 reinterpret_cast<const void*>(&grouped_resident_kernel<2, kInputGather, kEpilogueSwiglu>)};
        for (const void* kernel : kernels) {
            const int code = hip_check(
                hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit), "hipFuncSetAttribute");
            if (code != ORX_OK) return code;
        }
        return (int)ORX_OK;
    });
    if (ready != ORX_OK) return ready;
    const int depth = ring_depth(k);
    if (depth == 0 || input < 0 || input > 2 || epilogue < 0 || epilogue > 1 || (input == kInputAct && epilogue != 0)) {
        set_error("routed projection: K=%d, input %d, epilogue %d is not a form of the resident kernel", k, input, epilogue);
        return ORX_ERR_BAD_VARIANT;
    }
    GroupedParams p = {};
    if (input == kInputAct) {
        p.x = reinterpret_cast<const __half*>(b.a), p.as_out = reinterpret_cast<__half*>(const_cast<void*>(b.as));
        p.row_max_in = b.row_max, p.q_out = reinterpret_cast<int8_t*>(b.q);
    } else {
        p.a = reinterpret_cast<const int8_t*>(b.a), p.as = reinterpret_cast<const __half*>(b.as);
        p.slot_token = b.slot_token;
    }
    if (epilogue == kEpilogueSwiglu) p.act = reinterpret_cast<__half*>(b.act), p.row_max_out = const_cast<int*>(b.row_max);
    p.slots = slots;
    p.w = reinterpret_cast<const uint8_t*>(b.w), p.book = b.book, p.ws = reinterpret_cast<const __half*>(b.ws);
    p.out = reinterpret_cast<__half*>(b.out);
    p.counts = b.counts, p.offsets = b.offsets, p.tile_expert = b.tile_expert, p.tile_row = b.tile_row;
    p.tile_count = b.tile_count;
    p.n = n, p.k = k, p.k_major = packed_k != 0, p.tile_capacity = tiles;
    p.expert_weight_stride = (int64_t)n * (k / 8) * 2;
    Geometry g;
    grouped_resident_geometry(k, input, epilogue, slots, &g);
    const dim3 grid(g.grid[0]), block(kThreads);
#define ORX_GROUPED(D, IN, EP) ORX_LAUNCH((grouped_resident_kernel<D, IN, EP>), grid, block, g.shared, stream, p)
#define ORX_GROUPED_DEPTH(IN, EP)           \
    do {                                    \
        if (depth == 3) ORX_GROUPED(3, IN, EP); \
        else ORX_GROUPED(2, IN, EP);        \
    } while (0)
    if (epilogue == kEpiloguePlain) {
        if (input == kInputInt8) ORX_GROUPED_DEPTH(kInputInt8, kEpiloguePlain);
        else if (input == kInputGather) ORX_GROUPED_DEPTH(kInputGather, kEpiloguePlain);
        else ORX_GROUPED_DEPTH(kInputAct, kEpiloguePlain);
    } else {
        if (input == kInputInt8) ORX_GROUPED_DEPTH(kInputInt8, kEpilogueSwiglu);
        else ORX_GROUPED_DEPTH(kInputGather, kEpilogueSwiglu);
    }
#undef ORX_GROUPED_DEPTH
#undef ORX_GROUPED
    return hip_check(hipGetLastError(), "launch routed projection (resident)");
}

}  // namespace orx
