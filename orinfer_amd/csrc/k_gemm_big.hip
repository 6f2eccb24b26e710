// Large-M int8 MFMA projections (prefill): 256 x 256 output tile per workgroup, K step 128.
//
// Reference counterparts: the Tensor Core schedules of kernels/cuda/model/integer_core.py:162-272
// at block_m = 128/256 with grouped tile order (:31-39) for W8A8 (int8_projection.py:15-62) and
// E8P-Q4 (e8p_q4.py:143-264).  Arithmetic is identical: exact int32 accumulation over full K,
// then (float(acc)*ws)*as.
//
// MI355X design.  Eight wave64 (2 per SIMD) share one 256x256 tile; each wave owns 128x64 of it
// as 4x2 blocks of v_mfma_i32_32x32x32_i8 (128 accumulator registers).  Both operand tiles are
// double buffered in LDS (2 x 64 KiB of the 160 KiB).  int8 operands that already exist in HBM
// (activations, W8 weights) go HBM -> LDS directly with global_load_lds_dwordx4, without touching
// VGPRs: each wave instruction moves 8 rows x 128 bytes, so global access is whole 128-byte lines,
// and the 16-byte chunk a lane fetches is XOR-swizzled with its row so that the later
// ds_read_b128 fragment reads of sixteen consecutive rows fall in sixteen different bank groups.
// E8P-Q4 weights are decoded from codes in registers (two 8-byte LDS table reads and XORs per
// code, e8p_device.h) and stored to the same swizzled layout.  Loads for K step t+1 are issued
// right after the barrier that publishes step t, so they fly under the 32 MFMAs of step t.
// Workgroup ids are remapped so that the workgroups resident on one XCD (ids congruent mod 8)
// work on neighbouring tiles and share operand panels in that XCD's L2.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "e8p_device.h"
#include "orx_internal.h"

#ifndef ORX_BIG_TM
#define ORX_BIG_TM 4
#define ORX_BIG_TN 2
#endif

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTile = 256;     // output tile edge
constexpr int kStep = 128;     // K bytes per step
constexpr int kTileBytes = kTile * kStep;  // 32 KiB per operand per stage
constexpr int kImagePitch = kTile + 8;     // halves per row of the fp16 output image (bank skew)
constexpr int kEpilogueTile = kTile * kImagePitch * 2;  // bytes of the output image in LDS

struct BigParams {
    const int8_t* a;
    const void* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, m;
    int packed_k;
    int out_f32;
    int tiles_m, tiles_n;
};

// 16-byte chunk swizzle: chunk c of row r lives in slot c ^ ((r >> 1) & 7) of the row's 128 bytes.
__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ void direct_load_16(const void* global, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// The compiler does not count direct-to-LDS loads as pending at a barrier (they have no register
// destination), so every barrier that publishes them is preceded by this explicit wait.
__device__ __forceinline__ void wait_direct_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Same, but lets the N youngest vector-memory requests stay in flight (requests retire in order):
// used when N ordinary loads (weight codes for a later step) were issued after the direct loads.
template <int N>
__device__ __forceinline__ void wait_direct_loads_except() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// 16-byte LDS read whose wait is placed by hand.  The compiler waits for EVERY outstanding LDS read before the first
// multiply that follows a batch of reads (s_waitcnt lgkmcnt(0)), also when those multiplies use fragments that were
// requested a whole sub-step earlier, which undoes the software pipeline; a read issued from an asm statement is
// invisible to that pass, and the wait is an asm statement of its own that names how many younger LDS requests may still
// be in flight (LDS requests of a wave complete in order).
template <int OFFSET>
__device__ __forceinline__ v4i lds_read_16(uint32_t lds_address) {
    v4i value;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(value) : "v"(lds_address), "n"(OFFSET));
    return value;
}
__device__ __forceinline__ uint32_t lds_address_of(const void* pointer) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)pointer;
}
// before a barrier: this wave's direct-to-LDS requests have landed and its fragment reads have returned
__device__ __forceinline__ void wait_loads_and_reads() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }

// XCD-aware tile order: hardware hands consecutive workgroup ids to the 8 XCDs in turn.  Logical
// id = (id % 8) * per_xcd + id / 8 gives each XCD one contiguous run of logical tiles; inside a
// run, tiles advance down M in groups of 8 for each N, so concurrent workgroups of one XCD share
// one weight panel and eight activation panels.
__device__ __forceinline__ void tile_of(int id, int tiles_m, int tiles_n, int* tm, int* tn) {
    const int total = tiles_m * tiles_n;
    // (id % 8, id / 8) -> contiguous run per XCD; a bijection only when total is a multiple of 8
    const int logical = (total % 8 == 0) ? (id % 8) * (total / 8) + id / 8 : id;
    constexpr int GROUP = 8;
    const int group_size = GROUP * tiles_n;
    const int first = (logical / group_size) * GROUP;
    const int rows_in_group = min(GROUP, tiles_m - first);
    const int within = logical % group_size;
    *tm = first + within % rows_in_group;
    *tn = within / rows_in_group;
}

// TM x TN blocks of 32x32 per wave: <4,2> = eight waves of 128x64 (two per SIMD),
// <4,4> = four waves of 128x128 (one per SIMD, accumulators spill over into AGPRs).
template <bool Q4, int TM, int TN>
__global__ __launch_bounds__((8 / TM) * (8 / TN) * 64) void gemm_big_kernel(BigParams p) {
    constexpr int WAVES_N = 8 / TN;
    constexpr int WAVES = (8 / TM) * WAVES_N;
    constexpr int kThreads = WAVES * 64;
    constexpr int BLOCKS_PER_WAVE = 32 / WAVES;  // 1 KiB blocks of each operand tile per wave
    constexpr int CODE_CHUNKS = 1024 / kThreads; // 16-byte code chunks per thread per K step
    extern __shared__ __align__(16) int8_t lds[];  // [2 stages][A 32 KiB | W 32 KiB] (+ Q4 tables)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

    int tile_m, tile_n;
    tile_of(blockIdx.x, p.tiles_m, p.tiles_n, &tile_m, &tile_n);
    const int row0 = tile_m * kTile, col0 = tile_n * kTile;
    const int rows_here = min(kTile, p.m - row0);
    const int cols_here = min(kTile, p.n - col0);

    // Scales of this tile, one or two per thread, fetched now as raw bits so that the epilogue
    // does not pay a memory round trip: entries 0..255 token scales, 256..511 weight scales.
    constexpr int SCALES_PER_THREAD = 2 * kTile / kThreads;
    unsigned short scale_bits[SCALES_PER_THREAD];
#pragma unroll
    for (int e = 0; e < SCALES_PER_THREAD; ++e) {
        const int i = tid + e * kThreads;
        scale_bits[e] = i < kTile ? reinterpret_cast<const unsigned short*>(p.as)[row0 + min(i, rows_here - 1)]
                                  : reinterpret_cast<const unsigned short*>(p.ws)[col0 + min(i - kTile, cols_here - 1)];
    }

    Q4ByteTables* tables = reinterpret_cast<Q4ByteTables*>(lds + 4 * kTileBytes);
    if (Q4) build_tables(*tables, p.book, tid, kThreads);

    // ---- global -> LDS: one wave instruction = 8 rows x 128 bytes (1 KiB block) ----
    // wave w owns BLOCKS_PER_WAVE consecutive blocks of each operand tile (32 blocks of 8 rows)
    const int load_r8 = lane >> 3, load_slot = lane & 7;
    auto issue_direct = [&](const int8_t* base, int limit, int origin, int kt, int8_t* stage) {
#pragma unroll
        for (int b = 0; b < BLOCKS_PER_WAVE; ++b) {
            const int block = wave * BLOCKS_PER_WAVE + b;
            const int row = block * 8 + load_r8;
            const int chunk = load_slot ^ swizzle(row);
            const int source_row = origin + min(row, limit - 1);
            direct_load_16(base + (int64_t)source_row * p.k + kt * kStep + chunk * 16, stage + block * 1024);
        }
    };
    // Q4: one K step of the weight tile is 256 rows x 64 bytes of codes = 1024 chunks of 16 bytes
    // (4 codes = 32 weights each): CODE_CHUNKS chunks per thread.
    // Two register sets so that the codes of step t+1 can be in flight while step t is decoded.
    v4u code_regs[2][CODE_CHUNKS];  // native vectors: an array of HIP's uint4 struct would live in scratch memory
    auto load_codes = [&](int kt, int set) {
#pragma unroll
        for (int i = 0; i < CODE_CHUNKS; ++i) {
            const int c = tid + kThreads * i;      // chunk id: row = c / 4, quarter = c % 4
            const int row = min(c >> 2, cols_here - 1), q = c & 3;
            int64_t byte;
            if (p.packed_k != 0)
                byte = q4_k_major_chunk(p.packed_k, p.n, col0 + row, kt, q);
            else
                byte = ((int64_t)(col0 + row) * (p.k / kStep) + kt) * 64 + q * 16;
            code_regs[set][i] = *reinterpret_cast<const v4u*>(reinterpret_cast<const int8_t*>(p.w) + byte);
        }
    };
    // Decode the codes of one K step (4 codes -> 32 weights -> two 16-byte LDS stores per chunk).
    auto decode_step = [&](int8_t* stage, int set) {
#pragma unroll
        for (int i = 0; i < CODE_CHUNKS; ++i) {
            const int c = tid + kThreads * i;
            const int row = c >> 2, q = c & 3;
            const v4u codes = code_regs[set][i];
            const uint2 d0 = decode_q4(*tables, codes.x), d1 = decode_q4(*tables, codes.y);
            const uint2 d2 = decode_q4(*tables, codes.z), d3 = decode_q4(*tables, codes.w);
            int8_t* row_base = stage + row * kStep;
            const int s = swizzle(row);
            *reinterpret_cast<uint4*>(row_base + (((2 * q) ^ s) * 16)) = make_uint4(d0.x, d0.y, d1.x, d1.y);
            *reinterpret_cast<uint4*>(row_base + (((2 * q + 1) ^ s) * 16)) = make_uint4(d2.x, d2.y, d3.x, d3.y);
        }
    };

    // ---- fragment addressing ----
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int swz = swizzle(frag_row);  // identical for every 32-row block
    int frag_offset[4];                 // byte offset inside a row for K sub-step ks
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) frag_offset[ks] = ((2 * ks + frag_half) ^ swz) * 16;
    const int a_lane = (wave_m * TM * 32 + frag_row) * kStep;
    const int w_lane = (wave_n * TN * 32 + frag_row) * kStep;

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int k_tiles = p.k / kStep;
    auto stage_a = [&](int stage) { return lds + stage * 2 * kTileBytes; };
    auto stage_w = [&](int stage) { return lds + kTileBytes + stage * 2 * kTileBytes; };

    // Software pipeline over K steps (two LDS stages, two fragment register slots):
    //   prologue   steps 0 and 1 requested, step 0 published, its first fragments read
    //   step kt    sub-steps 0..2: read fragments ks+1, issue MFMAs ks
    //              barrier: step kt+1 is complete in LDS and nobody reads stage `cur` any more
    //              read fragments 0 of step kt+1, issue MFMAs of sub-step 3 (their operands are
    //              already in registers), request step kt+2 into stage `cur`
    // so the matrix pipe always holds queued work while waves meet at the barrier.
    const int8_t* w8 = reinterpret_cast<const int8_t*>(p.w);
    issue_direct(p.a, rows_here, row0, 0, stage_a(0));
    if (!Q4) issue_direct(w8, cols_here, col0, 0, stage_w(0));
    if (k_tiles > 1) {
        issue_direct(p.a, rows_here, row0, 1, stage_a(1));
        if (!Q4) issue_direct(w8, cols_here, col0, 1, stage_w(1));
    }
    if (Q4) {
        load_codes(0, 0);
        if (k_tiles > 1) load_codes(1, 1);
        __syncthreads();  // tables
        decode_step(stage_w(0), 0);
        if (k_tiles > 2) load_codes(2, 0);
        if (k_tiles > 1) decode_step(stage_w(1), 1);
        if (k_tiles > 3) load_codes(3, 1);
    }
    wait_direct_loads();
    __syncthreads();

    v4i fa[2][TM], fb[2][TN];
    auto read_fragments = [&](int stage, int ks, int slot) {
        const int8_t* la = stage_a(stage) + a_lane;
        const int8_t* lw = stage_w(stage) + w_lane;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[slot][i] = *reinterpret_cast<const v4i*>(la + i * 32 * kStep + frag_offset[ks]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[slot][j] = *reinterpret_cast<const v4i*>(lw + j * 32 * kStep + frag_offset[ks]);
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
    };
    // W8: a wave's 2*BLOCKS_PER_WAVE load instructions per K step are threaded one by one between
    // MFMAs and spread over three MFMA groups.  A wave cannot issue anything while a vector-memory
    // instruction waits for a slot in the CU's memory pipeline, and eight waves that all request
    // their 8 KiB right after the barrier queue up there for most of an MFMA group; a single
    // request at a time leaves the wave's next MFMAs issuable almost at once.
    constexpr int LOADS = 2 * BLOCKS_PER_WAVE;
    constexpr int PART0 = (LOADS + 2) / 3, PART1 = (LOADS - PART0 + 1) / 2, PART2 = LOADS - PART0 - PART1;
    static_assert(PART0 <= TM * TN / 2 && PART1 <= TM * TN / 2, "one request after every second MFMA of a group");
    auto issue_one = [&](int id, int kt_target, int stage) {  // id < BLOCKS_PER_WAVE: activations, else weights
        const bool weights = id >= BLOCKS_PER_WAVE;
        const int block = wave * BLOCKS_PER_WAVE + (weights ? id - BLOCKS_PER_WAVE : id);
        const int row = block * 8 + load_r8;
        const int chunk = load_slot ^ swizzle(row);
        const int source_row = weights ? col0 + min(row, cols_here - 1) : row0 + min(row, rows_here - 1);
        direct_load_16((weights ? w8 : p.a) + (int64_t)source_row * p.k + kt_target * kStep + chunk * 16,
                       (weights ? stage_w(stage) : stage_a(stage)) + block * 1024);
    };
    // Requests are unconditional: a step past the end is clamped to the last one and lands in a
    // stage that is not read again (the epilogue waits for it before it reuses LDS), which keeps
    // branches out of the MFMA stream.
    auto multiply_loading = [&](int slot, int first, int count, int kt_target, int stage) {
        kt_target = min(kt_target, k_tiles - 1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
                const int index = i * TN + j;
                if ((index & 1) == 1 && index / 2 < count) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (!Q4) issue_one(first + index / 2, kt_target, stage);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
    };
    // Q4: the whole weight tile of step kt+2 is decoded in one piece right after MFMA group 3 of
    // step kt, into the stage the barrier of step kt has just released.  (Threading the decode
    // between the MFMAs of a group, with or without pipelined table reads, measured 20 % slower:
    // the LDS waits of the decode then sit in the MFMA issue stream.)
    read_fragments(0, 0, 0);
    for (int kt = 0; kt < k_tiles; ++kt) {
        const int cur = kt & 1, nxt = cur ^ 1;
        // the rest of step kt+1 (its first part went out behind the previous barrier; in step 0 this
        // repeats part of the prologue's request for step 1, byte for byte)
        read_fragments(cur, 1, 1);
        __builtin_amdgcn_sched_barrier(0);  // reads above stay ahead of the MFMAs below
        multiply_loading(0, PART0, PART1, kt + 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        read_fragments(cur, 2, 0);
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(1, PART0 + PART1, PART2, kt + 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        read_fragments(cur, 3, 1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(0);
        __builtin_amdgcn_sched_barrier(0);
        // this wave's part of step kt+1; the code loads issued after it (Q4, step kt+3) may stay
        // in flight: a barrier should not wait for HBM
        if (Q4 && kt + 3 < k_tiles)
            wait_direct_loads_except<CODE_CHUNKS>();
        else
            wait_direct_loads();
        __syncthreads();
        if (Q4 && kt + 2 < k_tiles) issue_direct(p.a, rows_here, row0, kt + 2, stage_a(cur));
        if (kt + 1 < k_tiles) read_fragments(nxt, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(1, 0, PART0, kt + 2, cur);
        __builtin_amdgcn_sched_barrier(0);
        if (Q4 && kt + 2 < k_tiles) {
            decode_step(stage_w(cur), cur);
            if (kt + 4 < k_tiles) load_codes(kt + 4, cur);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue ----
    // the clamped requests of the last two steps may still be writing LDS (and a workgroup must
    // not end with direct-to-LDS loads in flight)
    if (!Q4) wait_direct_loads();
    // Weights are the MFMA row operand, so a lane holds token row (lane & 31) of each 32x32 block
    // and, per group of four accumulator registers, four CONSECUTIVE output channels
    // 8*q + 4*(lane >> 5) + {0..3}.
    const int half = lane >> 5;
    if (p.out_f32) {
        // fp32 heads are rare: 16-byte stores straight from the accumulators
        const bool vector_ok = p.stride % 4 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int local_row = (wave_m * TM + i) * 32 + (lane & 31);
            if (local_row >= rows_here) continue;
            const int64_t row = row0 + local_row;
            const float token_scale = __half2float(p.as[row]);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int local_col = (wave_n * TN + j) * 32 + 8 * q + 4 * half;
                    if (local_col >= cols_here) continue;
                    const int col = col0 + local_col;
                    float value[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        value[r] = rescale(acc[i][j][4 * q + r], __half2float(p.ws[min(col + r, p.n - 1)]), token_scale);
                    float* dst = reinterpret_cast<float*>(p.out) + row * p.stride + col;
                    if (local_col + 4 <= cols_here && vector_ok && (col & 3) == 0) {
                        *reinterpret_cast<float4*>(dst) = make_float4(value[0], value[1], value[2], value[3]);
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (local_col + r < cols_here) dst[r] = value[r];
                    }
                }
            }
        }
        return;
    }
    // fp16: rescale into an LDS image of the tile (8-byte writes), then store whole 16-byte pieces
    // of output rows.  The operand stages are dead after the last K step, so their LDS is reused.
    __syncthreads();
    float* lds_as = reinterpret_cast<float*>(lds + kEpilogueTile);  // 256 token scales
    float* lds_ws = lds_as + kTile;                                  // 256 weight scales
#pragma unroll
    for (int e = 0; e < SCALES_PER_THREAD; ++e)
        lds_as[tid + e * kThreads] = __half2float(__ushort_as_half(scale_bits[e]));  // lds_ws follows lds_as
    __syncthreads();
    __half* image = reinterpret_cast<__half*>(lds);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int local_row = (wave_m * TM + i) * 32 + (lane & 31);
        const float token_scale = lds_as[local_row];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int local_col = (wave_n * TN + j) * 32 + 8 * q + 4 * half;
                const float4 wscale = *reinterpret_cast<const float4*>(lds_ws + local_col);
                const __half2 lo = __halves2half2(__float2half_rn(rescale(acc[i][j][4 * q + 0], wscale.x, token_scale)),
                                                  __float2half_rn(rescale(acc[i][j][4 * q + 1], wscale.y, token_scale)));
                const __half2 hi = __halves2half2(__float2half_rn(rescale(acc[i][j][4 * q + 2], wscale.z, token_scale)),
                                                  __float2half_rn(rescale(acc[i][j][4 * q + 3], wscale.w, token_scale)));
                uint2 packed;
                packed.x = *reinterpret_cast<const uint32_t*>(&lo);
                packed.y = *reinterpret_cast<const uint32_t*>(&hi);
                *reinterpret_cast<uint2*>(image + local_row * kImagePitch + local_col) = packed;
            }
        }
    }
    __syncthreads();
    // each thread moves 16 bytes: kThreads/32 rows x 512 bytes per pass
    const bool aligned = (p.stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0) && (col0 % 8 == 0);
    const int piece = tid & 31, piece_row = tid >> 5;
    constexpr int ROWS_PER_PASS = kThreads / 32;
#pragma unroll 4
    for (int pass = 0; pass < kTile / ROWS_PER_PASS; ++pass) {
        const int local = pass * ROWS_PER_PASS + piece_row;
        if (local >= rows_here) break;
        const uint4 value = *reinterpret_cast<const uint4*>(image + local * kImagePitch + piece * 8);
        __half* dst = reinterpret_cast<__half*>(p.out) + (int64_t)(row0 + local) * p.stride + col0 + piece * 8;
        if (aligned && piece * 8 + 8 <= cols_here) {
            *reinterpret_cast<uint4*>(dst) = value;
        } else {
            const __half* h = reinterpret_cast<const __half*>(&value);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (piece * 8 + e < cols_here) dst[e] = h[e];
        }
    }
}

// ---- int8 weights: persistent workgroups ------------------------------------------------------------
// One workgroup per CU walks a static list of tiles (tile r of workgroup w is number w + r * gridDim.x of the
// XCD-aware order), and the K steps of all its tiles form ONE software pipeline: the operand requests of the
// next tile's first steps go out while the current tile's last steps multiply, so no tile after the first pays a
// prologue.  The epilogue is private to a wave and stays in registers: lanes that hold neighbouring channels of a
// row trade words (v_permlane16_swap), after which every lane stores 16-byte pieces of output rows.  It needs no
// LDS, no workgroup barrier, and leaves both operand stages alone (they already hold the next tile's first
// steps); its stores are not waited for and drain under the next tile's multiplies.
//
// The kernel is bound by power, not by issue slots: on random int8 data the clock inside the K loop settles near
// 1.2-1.3 GHz, the same launch on zero operands is 30 % shorter, and taking out stalls alone changes nothing at
// large K.  What pays is less energy per multiply.  v_mfma_i32_16x16x64_i8 does the same work per cycle as
// v_mfma_i32_32x32x32_i8 with half the accumulator traffic per multiply and sustains 3.83 POP/s on random
// operands where the 32 x 32 shape sustains 3.37 (back-to-back issue from registers, whole chip); the fragment
// bytes read from LDS per multiply are the same, so the tile, the stages and the swizzle stay as they were.
constexpr uint32_t kPersistentLds = 4 * kTileBytes + 2 * kTile * 4;
constexpr int kPersistentThreads = 512;

struct TileState {
    int row0, col0, rows_here, cols_here;
};

typedef float v2f __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

// two fp32 values rounded to nearest even and packed (one v_cvt_pk_f16_f32)
__device__ __forceinline__ uint32_t pack_halves(float low, float high) {
    const v2f pair = {low, high};
    const v2h rounded = __builtin_convertvector(pair, v2h);
    return *reinterpret_cast<const uint32_t*>(&rounded);
}

// The four fragments pass through the statement, so no multiply that uses them can move in front of the wait: at
// most N younger LDS requests of this wave may still be in flight behind them (they complete in order).
template <int N>
__device__ __forceinline__ void wait_four(v4i (&f)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_eight(v4i (&f)[4], v4i (&g)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(g[0]), "+v"(g[1]), "+v"(g[2]), "+v"(g[3])
                 : "n"(N));
}

__device__ __forceinline__ const int8_t* uniform_pointer(const int8_t* pointer) {
    const uint64_t bits = reinterpret_cast<uint64_t>(pointer);
    const uint32_t low = __builtin_amdgcn_readfirstlane((uint32_t)bits), high = __builtin_amdgcn_readfirstlane((uint32_t)(bits >> 32));
    return reinterpret_cast<const int8_t*>(((uint64_t)high << 32) | low);
}

// F32: fp32 output (heads); its own instantiation, so that either kernel holds one epilogue.
//
// Eight waves share the 256 x 256 tile, 128 token rows x 64 channels each: 8 x 4 blocks of 16 x 16, 128 accumulator
// registers.  A K step of 128 is two MFMA K slices of 64; a slice is multiplied in two phases of 16 multiplies
// (token blocks 0-3, then 4-7, against the slice's four channel blocks), so that only four token fragments and four
// weight fragments are live per phase and a second set is on its way from LDS: 64 fragment registers.
template <bool F32>
__global__ __launch_bounds__(kPersistentThreads) void gemm_big_persistent_kernel(BigParams p) {
    constexpr int WAVES_N = 4, kThreads = kPersistentThreads, BLOCKS_PER_WAVE = 4;
    extern __shared__ __align__(16) int8_t lds[];  // [2 stages][A 32 KiB | W 32 KiB], 512 scales
    float* const lds_as = reinterpret_cast<float*>(lds + 4 * kTileBytes);  // 256 token scales, then 256 weight scales
    float* const lds_ws = lds_as + kTile;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

    const int total_tiles = p.tiles_m * p.tiles_n;
    const int my_tiles = (total_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;  // >= 1: grid <= tiles
    const int k_tiles = p.k / kStep;
    const int total_steps = my_tiles * k_tiles;
    auto tile_state = [&](int r) {
        int tm, tn;
        tile_of((int)blockIdx.x + min(r, my_tiles - 1) * (int)gridDim.x, p.tiles_m, p.tiles_n, &tm, &tn);
        TileState t;
        t.row0 = tm * kTile, t.col0 = tn * kTile;
        t.rows_here = min(kTile, p.m - t.row0), t.cols_here = min(kTile, p.n - t.col0);
        return t;
    };

    auto stage_a = [&](int stage) { return lds + stage * 2 * kTileBytes; };
    auto stage_w = [&](int stage) { return lds + kTileBytes + stage * 2 * kTileBytes; };
    const int8_t* const w8 = reinterpret_cast<const int8_t*>(p.w);

    // ---- load cursor: the step whose operands are being requested (clamped at this workgroup's last step) ----
    const int load_r8 = lane >> 3, load_slot = lane & 7;
    int load_tile = 0, load_kt = 0;
    // A request is a uniform 64-bit base (the tile's first row, the K step) plus a 32-bit lane offset, computed when
    // it is issued from two lane registers rather than kept per request: block b of this wave starts 8 b rows below the
    // lane's first row, and the swizzled chunk of odd blocks is that of even blocks with bit 2 flipped.
    const int load_row = wave * (BLOCKS_PER_WAVE * 8) + load_r8;                 // row of block 0
    const uint32_t load_chunk = (uint32_t)((load_slot ^ swizzle(load_row)) * 16);
    int load_rows = 0, load_cols = 0;  // live rows and channels of the tile being requested
    const int8_t* a_base = nullptr;
    const int8_t* w_base = nullptr;
    auto aim = [&](const TileState& t) {
        load_rows = t.rows_here, load_cols = t.cols_here;
        // (said to be uniform in so many words: the bases then live in scalar registers)
        a_base = uniform_pointer(p.a + (int64_t)t.row0 * p.k);
        w_base = uniform_pointer(w8 + (int64_t)t.col0 * p.k);
    };
    auto advance = [&]() {
        if (load_kt + 1 < k_tiles) {
            ++load_kt;
        } else if (load_tile + 1 < my_tiles) {
            ++load_tile, load_kt = 0;
            aim(tile_state(load_tile));
        }
    };
    auto issue_one = [&](int id, int stage) {  // id < BLOCKS_PER_WAVE: activations, else weights
        const bool weights = id >= BLOCKS_PER_WAVE;
        const int b = weights ? id - BLOCKS_PER_WAVE : id;
        // (the row is made opaque, or every request's offset is computed once and kept in a register for the whole loop)
        int row = load_row;
        asm volatile("" : "+v"(row));
        const uint32_t offset = (uint32_t)(min(row + 8 * b, (weights ? load_cols : load_rows) - 1) * p.k) + (load_chunk ^ (uint32_t)((b & 1) * 64));
        direct_load_16((weights ? w_base : a_base) + load_kt * kStep + (uint64_t)offset,
                       (weights ? stage_w(stage) : stage_a(stage)) + (wave * BLOCKS_PER_WAVE + b) * 1024);
    };

    // ---- fragment addressing: a lane reads K bytes [16 (lane / 16), +16) of K slice s for row lane % 16 of a block ----
    const int frag_row = lane & 15, frag_chunk = lane >> 4;
    const int swz = swizzle(frag_row);  // the same in every block of 16 rows
    // LDS byte address of that piece for K slice 0 in stage 0, first block of the wave; slice 1 is the same address
    // with bit 6 flipped (chunk 4 + c swizzles to the chunk of c with bit 2 flipped, and rows start at multiples of 128)
    const uint32_t a_frag = lds_address_of(lds) + (wave_m * 128 + frag_row) * kStep + ((frag_chunk ^ swz) * 16);
    const uint32_t w_frag = lds_address_of(lds) + kTileBytes + (wave_n * 64 + frag_row) * kStep + ((frag_chunk ^ swz) * 16);

    v4i acc[8][4];  // [token block][channel block]: channels 4 (lane / 16) + {0..3} of the block, token lane % 16
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    };
    clear();

    v4i ft[2][4], fw[2][4];  // token fragments of a phase, weight fragments of a K slice; two sets each
    constexpr int kBlockBytes = 16 * kStep;
    auto read_tokens = [&](int stage, int phase) {  // phase = 2 * slice + half; into set phase % 2
        const uint32_t a = (a_frag ^ (uint32_t)((phase >> 1) * 64)) + stage * (2 * kTileBytes) + (phase & 1) * 4 * kBlockBytes;
        v4i(&f)[4] = ft[phase & 1];
        f[0] = lds_read_16<0>(a);
        f[1] = lds_read_16<kBlockBytes>(a);
        f[2] = lds_read_16<2 * kBlockBytes>(a);
        f[3] = lds_read_16<3 * kBlockBytes>(a);
    };
    auto read_weights = [&](int stage, int slice) {  // into set `slice`
        const uint32_t w = (w_frag ^ (uint32_t)(slice * 64)) + stage * (2 * kTileBytes);
        v4i(&f)[4] = fw[slice];
        f[0] = lds_read_16<0>(w);
        f[1] = lds_read_16<kBlockBytes>(w);
        f[2] = lds_read_16<2 * kBlockBytes>(w);
        f[3] = lds_read_16<3 * kBlockBytes>(w);
    };
    // a wave's requests of a K step go out one at a time behind every second multiply of three phases (a wave cannot
    // issue anything while a vector-memory instruction waits for a slot in the CU's memory pipeline)
    constexpr int LOADS = 2 * BLOCKS_PER_WAVE;
    constexpr int PART0 = (LOADS + 2) / 3, PART1 = (LOADS - PART0 + 1) / 2, PART2 = LOADS - PART0 - PART1;
    auto multiply_loading = [&](int phase, int first, int count, int stage) {
        v4i(&tokens)[4] = ft[phase & 1];
        v4i(&weights)[4] = fw[phase >> 1];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int jj = (i & 1) ? 3 - j : j;  // boustrophedon: one operand changes between consecutive multiplies
                v4i& sum = acc[4 * (phase & 1) + i][jj];
                sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(weights[jj], tokens[i], sum, 0, 0, 0);
                const int index = i * 4 + j;
                if ((index & 1) == 1 && index / 2 < count) {
                    __builtin_amdgcn_sched_barrier(0);
                    issue_one(first + index / 2, stage);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
    };

    // ---- epilogue of one tile, wave-private, in registers ----
    auto epilogue = [&](const TileState& t) {
        // the lane number is made opaque here: addresses and bounds that depend only on it would otherwise be
        // computed once in front of the K loop and held in registers (or spilled) for the whole kernel
        int lane = threadIdx.x & 63;
        asm volatile("" : "+v"(lane));
        const int group = lane >> 4;
        if constexpr (F32) {
            // fp32 heads are rare: 16-byte stores straight from the accumulators
            const bool vector_ok = p.stride % 4 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int local_row = wave_m * 128 + i * 16 + (lane & 15);
                if (local_row >= t.rows_here) continue;
                const int64_t row = t.row0 + local_row;
                const float token_scale = lds_as[local_row];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int local_col = wave_n * 64 + j * 16 + 4 * group;
                    if (local_col >= t.cols_here) continue;
                    const int col = t.col0 + local_col;
                    const float4 wscale = *reinterpret_cast<const float4*>(lds_ws + local_col);
                    const float value[4] = {rescale(acc[i][j][0], wscale.x, token_scale), rescale(acc[i][j][1], wscale.y, token_scale),
                                            rescale(acc[i][j][2], wscale.z, token_scale), rescale(acc[i][j][3], wscale.w, token_scale)};
                    float* dst = reinterpret_cast<float*>(p.out) + row * p.stride + col;
                    if (local_col + 4 <= t.cols_here && vector_ok && (col & 3) == 0) {
                        *reinterpret_cast<float4*>(dst) = make_float4(value[0], value[1], value[2], value[3]);
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (local_col + r < t.cols_here) dst[r] = value[r];
                    }
                }
            }
            return;
        } else {
            // Weights are the MFMA row operand, so a lane holds token lane % 16 of each 16 x 16 block and four consecutive
            // output channels 4 (lane / 16) + {0..3}: two words of fp16.  One swap of the odd rows of 16 lanes of channel
            // block j with the even rows of block j + 1 leaves lane groups 0 and 2 with channels 0-7 and 8-15 of block j
            // and groups 1 and 3 with those of block j + 1: 16 contiguous bytes of an output row per lane and store, and a
            // store instruction covers 16 rows x 64 bytes.
            const bool aligned = (p.stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
            const bool whole = aligned && t.rows_here == kTile && t.cols_here == kTile;  // no bounds inside this tile
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int local_row = wave_m * 128 + i * 16 + (lane & 15);
                const float token_scale = lds_as[local_row];
                __half* const row_out = reinterpret_cast<__half*>(p.out) + (int64_t)(t.row0 + local_row) * p.stride + t.col0;
#pragma unroll
                for (int pair = 0; pair < 2; ++pair) {  // channel blocks (0, 1), then (2, 3)
                    uint32_t words[2][2];
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        const int j = 2 * pair + b;
                        const float4 wscale = *reinterpret_cast<const float4*>(lds_ws + wave_n * 64 + j * 16 + 4 * group);
                        words[b][0] = pack_halves(rescale(acc[i][j][0], wscale.x, token_scale), rescale(acc[i][j][1], wscale.y, token_scale));
                        words[b][1] = pack_halves(rescale(acc[i][j][2], wscale.z, token_scale), rescale(acc[i][j][3], wscale.w, token_scale));
                    }
                    const v2u low = __builtin_amdgcn_permlane16_swap(words[0][0], words[1][0], false, false);
                    const v2u high = __builtin_amdgcn_permlane16_swap(words[0][1], words[1][1], false, false);
                    const uint4 piece = make_uint4(low.x, high.x, low.y, high.y);
                    const int local_col = wave_n * 64 + (2 * pair + (group & 1)) * 16 + (group >> 1) * 8;
                    if (whole) {
                        *reinterpret_cast<uint4*>(row_out + local_col) = piece;
                    } else if (local_row < t.rows_here && local_col < t.cols_here) {
                        if (aligned && local_col + 8 <= t.cols_here) {
                            *reinterpret_cast<uint4*>(row_out + local_col) = piece;
                        } else {
                            const uint32_t parts[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (local_col + e < t.cols_here)
                                    row_out[local_col + e] = __ushort_as_half((unsigned short)(parts[e >> 1] >> (16 * (e & 1))));
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);  // one pair at a time: interleaved pairs cost registers, not time
                }
            }
        }
    };

    // ---- prologue: steps 0 and 1 requested, step 0 published, its first fragments read ----
    TileState tile = tile_state(0);
    aim(tile);
#pragma unroll
    for (int id = 0; id < LOADS; ++id) issue_one(id, 0);
    if (total_steps > 1) {
        advance();
#pragma unroll
        for (int id = 0; id < LOADS; ++id) issue_one(id, 1);
    }
    wait_direct_loads();
    __syncthreads();
    read_tokens(0, 0);
    read_weights(0, 0);

    // Step g, four phases: each requests the fragments of the next phase, waits for its own (requested a phase
    // earlier: only the younger batch may still be in flight) and multiplies.  Behind phase 2 comes the barrier (step
    // g+1 is complete in LDS and nobody reads stage `cur` any more); then the fragments of step g+1's first phase,
    // and phase 3, whose operands are already in registers, while the requests of step g+2 start into stage `cur`.
    // The load cursor points at step g+1 until the second group of requests is out, then at step g+2; at the end of
    // the list it stays on the last step, whose repeated requests land in a stage that is not read again.  A tile's
    // last step (LAST) also brings the tile's scales into LDS and keeps its first requests of step g+2 back until the
    // epilogue has read them (a read of LDS waits for every direct-to-LDS request in flight).
    int g = 0;
    auto k_step = [&](auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const int cur = g & 1, nxt = cur ^ 1;
        // this tile's scales, token scales by the first 256 threads and weight scales by the rest: in LDS before the
        // barrier below, read by the epilogue after it
        // (which of the two is the same for a whole wave, so the base stays in scalar registers; the lane number is
        // opaque so that no part of the address is carried through the K loop)
        uint32_t scale_bits = 0;
        int scale_index = 0;
        if constexpr (LAST) {
            int own = threadIdx.x & 63;
            asm volatile("" : "+v"(own));
            scale_index = (wave & 3) * 64 + own;
            if (wave < 4)
                scale_bits = reinterpret_cast<const unsigned short*>(p.as)[tile.row0 + min(scale_index, tile.rows_here - 1)];
            else
                scale_bits = reinterpret_cast<const unsigned short*>(p.ws)[tile.col0 + min(scale_index, tile.cols_here - 1)];
        }
        read_tokens(cur, 1);                  // 4 younger requests
        wait_eight<4>(ft[0], fw[0]);
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(0, PART0, PART1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        read_tokens(cur, 2);                  // 8 younger requests
        read_weights(cur, 1);
        wait_four<8>(ft[1]);
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(1, PART0 + PART1, PART2, nxt);
        __builtin_amdgcn_sched_barrier(0);
        advance();
        read_tokens(cur, 3);                  // 4 younger requests
        wait_eight<4>(ft[0], fw[1]);
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(2, 0, 0, nxt);
        __builtin_amdgcn_sched_barrier(0);
        wait_loads_and_reads();
        wait_four<0>(ft[1]);
        if constexpr (LAST) {
            // (the raw bits stay opaque up to here, or the conversion and with it the wait for the load would move up
            // to the request itself)
            asm volatile("" : "+v"(scale_bits));
            (wave < 4 ? lds_as : lds_ws)[scale_index] = __half2float(__ushort_as_half((unsigned short)scale_bits));
        }
        __syncthreads();
        // (a tile's last step leaves these reads to the tile loop, behind the epilogue: 32 registers less to carry
        // through it, for one LDS latency per tile)
        if (!LAST) {
            read_tokens(nxt, 0);
            read_weights(nxt, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        multiply_loading(3, 0, LAST ? 0 : PART0, cur);
        __builtin_amdgcn_sched_barrier(0);
        ++g;
    };
    for (int tile_index = 0; tile_index < my_tiles; ++tile_index) {
        for (int kt = 0; kt + 1 < k_tiles; ++kt) k_step(std::false_type{});
        k_step(std::true_type{});
        epilogue(tile);
        clear();
        tile = tile_state(tile_index + 1);
        const int cur = (g - 1) & 1;
#pragma unroll
        for (int id = 0; id < PART0; ++id) issue_one(id, cur);
        if (g < total_steps) {  // the next tile's first fragments (its first step was published by the last barrier)
            read_tokens(g & 1, 0);
            read_weights(g & 1, 0);
        }
    }
    // a workgroup must not end with direct-to-LDS requests in flight
    wait_direct_loads();
}

// operand stages (128 KiB, + 8 KiB of decode tables for Q4) or the epilogue's output image + scales
constexpr uint32_t kBigLdsEpilogue = kEpilogueTile + 2 * kTile * 4;
constexpr uint32_t kBigLds = 4 * kTileBytes > kBigLdsEpilogue ? 4 * kTileBytes : kBigLdsEpilogue;
constexpr uint32_t kBigLdsQ4 = 4 * kTileBytes + sizeof(Q4ByteTables) > kBigLdsEpilogue
                                   ? 4 * kTileBytes + sizeof(Q4ByteTables)
                                   : kBigLdsEpilogue;

// wave shape of the shipped kernels
constexpr int kTM = ORX_BIG_TM, kTN = ORX_BIG_TN;
constexpr int kBigThreads = (8 / kTM) * (8 / kTN) * 64;

int prepare_device() {
    int code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_persistent_kernel<false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPersistentLds),
                         "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_persistent_kernel<true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPersistentLds),
                     "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_kernel<true, kTM, kTN>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLdsQ4),
                     "hipFuncSetAttribute");
    return code;
}
int prepare() {
    static DeviceOnce done;  // once per device, safe from several session threads
    return done.run(prepare_device);
}

}  // namespace

// ---- two-stage codes -> int8 weights, once per launch ------------------------------------------
// A prefill GEMM decodes every weight tile once per 256-row tile of activations; with many row
// tiles it is cheaper to decode the whole matrix once into scratch (1.5 bytes of HBM traffic per
// weight) and run the plain int8 kernel on it.  One thread turns 16 bytes of codes (4 codes, 32
// weights) into 32 consecutive bytes of a row-major (N, K) int8 matrix.
namespace {
__global__ __launch_bounds__(512) void q4_expand_kernel(const uint4* __restrict__ codes, const uint32_t* __restrict__ book,
                                                        int8_t* __restrict__ out, int n, int k, int packed_k) {
    __shared__ Q4ByteTables tables;
    build_tables(tables, book, threadIdx.x, 512);
    __syncthreads();
    const int64_t total = (int64_t)n * (k / 32);
    const int per_row = k / 32;
    for (int64_t c = (int64_t)blockIdx.x * 512 + threadIdx.x; c < total; c += (int64_t)gridDim.x * 512) {
        int64_t row, k0;
        if (packed_k == 128) {  // (K/128, N, 16) u32: four chunks per row and K block
            const int64_t kt = c / ((int64_t)n * 4), rest = c % ((int64_t)n * 4);
            row = rest >> 2, k0 = kt * 128 + (rest & 3) * 32;
        } else if (packed_k == 64) {  // (K/64, N, 8) u32: two chunks per row and K block
            const int64_t kb = c / ((int64_t)n * 2), rest = c % ((int64_t)n * 2);
            row = rest >> 1, k0 = kb * 64 + (rest & 1) * 32;
        } else {
            row = c / per_row, k0 = (c % per_row) * 32;
        }
        const uint4 four = codes[c];
        const uint2 w0 = decode_q4(tables, four.x), w1 = decode_q4(tables, four.y);
        const uint2 w2 = decode_q4(tables, four.z), w3 = decode_q4(tables, four.w);
        uint4* dst = reinterpret_cast<uint4*>(out + row * k + k0);
        dst[0] = make_uint4(w0.x, w0.y, w1.x, w1.y);
        dst[1] = make_uint4(w2.x, w2.y, w3.x, w3.y);
    }
}
}  // namespace

int q4_expand_launch(const void* codes, const uint32_t* book, void* weights, int n, int k, int packed_k,
                     hipStream_t stream) {
    const int64_t chunks = (int64_t)n * (k / 32);
    const int blocks = (int)std::min<int64_t>((chunks + 511) / 512, 2048);
    ORX_LAUNCH(q4_expand_kernel, dim3(blocks), dim3(512), 0, stream, reinterpret_cast<const uint4*>(codes), book,
                       reinterpret_cast<int8_t*>(weights), n, k, packed_k);
    return hip_check(hipGetLastError(), "launch two-stage weight expansion");
}

void gemm_big_geometry(int rows, int n, bool q4, Geometry* g) {
    const uint32_t tiles = ceil_div((uint32_t)rows, (uint32_t)kTile) * ceil_div((uint32_t)n, (uint32_t)kTile);
    // int8 weights: one persistent workgroup per CU walks the tiles; two-stage codes decoded in the loop: one per tile
    g->grid[0] = q4 ? tiles : std::min(tiles, (uint32_t)device_compute_units());
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = q4 ? kBigThreads : kPersistentThreads;
    g->shared = q4 ? kBigLdsQ4 : kPersistentLds;
}

int gemm_big_launch(bool q4, const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                    void* out, int rows, int n, int k, int stride, int packed_k, bool out_f32, const Geometry& g,
                    hipStream_t stream) {
    const int ready = prepare();
    if (ready != ORX_OK) return ready;
    BigParams p = {};
    p.a = a, p.w = w, p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.packed_k = packed_k, p.out_f32 = out_f32;
    p.tiles_m = (rows + kTile - 1) / kTile, p.tiles_n = (n + kTile - 1) / kTile;
    if (!q4 && k < 2 * kStep) {
        set_error("projection (mfma 256x256): the persistent int8 kernel needs K >= 256");
        return ORX_ERR_BAD_VARIANT;
    }
    if (q4)
        ORX_LAUNCH((gemm_big_kernel<true, kTM, kTN>), dim3(g.grid[0]), dim3(kBigThreads), g.shared, stream, p);
    else
        if (out_f32)
            ORX_LAUNCH((gemm_big_persistent_kernel<true>), dim3(g.grid[0]), dim3(kPersistentThreads), g.shared, stream, p);
        else
            ORX_LAUNCH((gemm_big_persistent_kernel<false>), dim3(g.grid[0]), dim3(kPersistentThreads), g.shared, stream, p);
    return hip_check(hipGetLastError(), "launch projection (mfma 256x256)");
}

}  // namespace orx
