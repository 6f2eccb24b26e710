// Many-row int8 MFMA projections (prefill).
//
// Reference counterparts: the Tensor Core schedules of kernels/cuda/model/integer_core.py:162-272
// at block_m = 128/256 with grouped tile order (:31-39) for W8A8 (int8_projection.py:15-62) and
// E8P-Q4 (e8p_q4.py:143-264).  Arithmetic is identical: exact int32 accumulation over full K,
// then (float(acc)*ws)*as.
//
// Two kernels.  int8 weights (W8A8, and two-stage weights that q4_expand_kernel has decoded once into the
// caller's scratch): gemm_big_persistent_kernel, one workgroup per CU walking 256 x 256 tiles, eight wave64 of
// 128 token rows x 64 channels each.  Two-stage codes without scratch: gemm_q4_tall_kernel, 512 token rows x a run
// of up to 80 channels per workgroup with the decode in the K loop, eight wave64 of 64 rows x the run.  Both
// multiply with v_mfma_i32_16x16x64_i8 from two waves per SIMD; int8 operands that already exist in HBM go
// HBM -> LDS directly with global_load_lds_dwordx4, without touching VGPRs, and the 16-byte chunk a lane fetches is
// XOR-swizzled with its row so that the later ds_read_b128 fragment reads of sixteen consecutive rows fall in
// different bank groups.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

constexpr int kTile = 256;     // output tile edge
constexpr int kStep = 128;     // K bytes per step
constexpr int kTileBytes = kTile * kStep;  // 32 KiB per operand per stage

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

// ---- int8 weights: persistent workgroups ------------------------------------------------------------
// One workgroup per CU walks a static list of tiles (tile r of workgroup w is number w + r * gridDim.x of the
// XCD-aware order), and the K steps of all its tiles form ONE software pipeline: the operand requests of the
// next tile's first steps go out while the current tile's last steps multiply, so no tile after the first pays a
// prologue.  The epilogue is private to a wave and stays in registers: lanes that hold neighbouring channels of a
// row trade words (v_permlane16_swap), after which every lane stores 16-byte pieces of output rows.  It needs no
// LDS, no workgroup barrier, and leaves both operand stages alone (they already hold the next tile's first
// steps); its stores are not waited for and drain under the next tile's multiplies.
//
// The kernel is bound by power, not by issue slots: on random int8 data the clock inside the K loop is 1.9 GHz in a
// sustained run (1.2-1.3 GHz in a launch that follows a pause), the same launch on zero operands is 30 % shorter, and
// taking out stalls alone changes nothing at large K.  What pays is less energy per multiply.  v_mfma_i32_16x16x64_i8 does the same work per cycle as
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
    constexpr int WAVES_N = 4, BLOCKS_PER_WAVE = 4;
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

// ---- two-stage codes without scratch: 512 rows x a run of channels, the decode in the K loop ---------------------
// From 257 rows on the other kernels either decode every weight once per 128- or 256-row tile, or need the weights
// decoded once into scratch first (1.5 bytes of HBM traffic per weight, a launch of its own).  Here a workgroup owns
// up to 512 token rows and a run of at most five blocks of 16 channels over the whole K; the blocks of the matrix
// are dealt evenly to whole rounds of the CUs (N = 17408 on 256 CUs: 1088 blocks, 4 or 5 per workgroup, one
// round), so every weight is decoded once per 512 rows and nothing goes through scratch.
//
// Eight waves; wave w owns token rows [64 w, +64) and all channels of the run: 4 x 5 blocks of
// v_mfma_i32_16x16x64_i8 (80 accumulator registers), weights as the row operand, so a lane holds four consecutive
// channels of one token.  K advances in MFMA slices of 64.
//   token rows   two slots of 512 rows x 128 bytes of K (64 KiB each): a wave requests its own 64 rows of a K chunk
//                of 128 with eight direct-to-LDS loads of 8 rows x 128 bytes, whole cache lines (requests of half
//                lines, one 64-byte slice per step, cost twice the traffic between L2 and the CU: the other half
//                of a line has left the L1 by the next step).  Nobody but the wave itself reads those rows, so
//                they need no barrier, only the wave's own wait.
//   weights      a thread of the first five waves owns one 16-byte chunk of the decoded stage per step (channel
//                tid / 4, K bytes [16 (tid % 4), +16) of the slice: two code words); it holds the four words of
//                its channel and quarter for a K block of 128 in registers, a second set for the block after it.
//                Every code word costs four 8-byte lookups in the compact byte tables (8 KiB at the start of the
//                LDS, so a lookup's address is its entry's offset and the table is the instruction's offset
//                field) and four byte-parallel operations per output word.  Four stages of 5 KiB.
//   step s       between its 20 multiplies the wave issues the eight lookups for the weights of step s + 2, combines
//                them and writes its chunk, then requests the nine fragments of step s + 1, which cross the
//                step's barrier and are waited for in front of the next step's first multiply; in odd steps the
//                eight requests for the token rows of steps s + 3 and s + 4 (the slot that steps s - 1 and s have
//                left); in even steps the codes two blocks ahead (every wave does, so that all count the same
//                requests).  One barrier per step publishes the decoded stage.
// All LDS traffic and the code loads of the loop are asm statements with hand-placed waits: the compiler would
// wait for every direct-to-LDS request in flight before an LDS access it can see.  Per step and CU the LDS pipe
// serves 72 fragment reads of 1 KiB (8 clocks each), 32 KiB of token rows landing, 5 KiB written and 40 wave
// lookups whose random addresses collide in the banks, and no unit is full: the matrix pipe is busy in 0.35 of
// the cycles, the LDS pipe in about 0.6.  Taking out any one part of a step shortens the loop by 5-25 % (the
// decode most), while lookups made cheaper (4-byte nibble tables, also stored 8 and 4 times) measure the same:
// what a step issues has to come back within the step, and the parts queue behind one another.  The floor under
// it is what the token rows cost: every CU reads all of them once, 2.6 MB per CU at 512 x 5120, which 256 CUs
// together pull out of the L2 in 37 us.
constexpr int kTallBlocks = 5;  // blocks of 16 channels per workgroup, at most
constexpr int kTallRows = 512, kTallCols = 16 * kTallBlocks, kTallStep = 64, kTallThreads = 512, kTallStagesW = 4;
constexpr uint32_t kTallSlotA = kTallRows * 128;  // token rows of a K chunk of 128
constexpr uint32_t kTallStageW = kTallCols * kTallStep;
// byte offsets in dynamic LDS: the tables first, so that a lookup's address is its table index alone
constexpr uint32_t kTallTokens = (uint32_t)sizeof(Q4ByteTables);
constexpr uint32_t kTallWeights = kTallTokens + 2 * kTallSlotA;
constexpr uint32_t kTallScales = kTallWeights + kTallStagesW * kTallStageW;
constexpr uint32_t kTallLds = kTallScales + (kTallRows + kTallCols) * 4;

typedef unsigned int v2w __attribute__((ext_vector_type(2)));

template <int OFFSET>
__device__ __forceinline__ v2w lds_read_8(uint32_t lds_address) {
    v2w value;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(value) : "v"(lds_address), "n"(OFFSET));
    return value;
}
// 8 bytes from global memory that the compiler keeps no count for: whoever uses them waits by hand
__device__ __forceinline__ void load_8(v2w& destination, uint32_t lane_offset, const int8_t* uniform_base) {
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(destination) : "v"(lane_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void lds_write_16(uint32_t lds_address, v4u value) {
    asm volatile("ds_write_b128 %0, %1" ::"v"(lds_address), "v"(value) : "memory");
}
// rows of 64 bytes: four chunks of 16; chunk c of row r sits at position c ^ ((r / 4) % 4), so that the 16 rows a
// fragment read touches per chunk spread over all banks
__device__ __forceinline__ int tall_swizzle(int row) { return (row >> 2) & 3; }

template <bool F32>
__global__ __launch_bounds__(kTallThreads) void gemm_q4_tall_kernel(BigParams p) {
    extern __shared__ __align__(16) int8_t lds[];
    float* const lds_as = reinterpret_cast<float*>(lds + kTallScales);
    float* const lds_ws = lds_as + kTallRows;
    Q4ByteTables* const tables = reinterpret_cast<Q4ByteTables*>(lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // unit u of a row tile owns the channel blocks [u B / U, (u + 1) B / U) of the B blocks of 16 channels
    const int unit = (int)blockIdx.x % p.tiles_n, tm = (int)blockIdx.x / p.tiles_n;
    const int channel_blocks = (p.n + 15) >> 4;
    const int first_block = (int)((int64_t)unit * channel_blocks / p.tiles_n);
    const int end_block = (int)((int64_t)(unit + 1) * channel_blocks / p.tiles_n);
    TileState t;
    t.row0 = tm * kTallRows, t.col0 = first_block * 16;
    t.rows_here = min(kTallRows, p.m - t.row0), t.cols_here = min((end_block - first_block) * 16, p.n - t.col0);
    const bool decoder = wave < kTallBlocks;  // threads 0 .. 64 blocks - 1 own the chunks of the weight stage
    const int steps = p.k / kTallStep, blocks = p.k / 128;
    const uint32_t lds_base = lds_address_of(lds);

    // ---- codes: words 2q, 2q+1 (first step of a K block) and 8+2q, 8+2q+1 (second step) of channel tid / 4 ----
    const int channel = tid >> 2, quarter = tid & 3;
    const int code_row = t.col0 + min(channel, t.cols_here - 1);
    // The loads are asm statements: the compiler then keeps no count for them, and the waits in front of the barriers
    // (which let only the youngest requests stay in flight) are what guarantees that a set has arrived two steps
    // after it was requested.  Sets and halves are compile-time indices everywhere, so that no select or copy
    // touches a register whose load is still in flight.
    v2w codes[2][2];  // [set][half of the K block]
    // address = uniform base of the K block (+ uniform step to its second half) + a lane offset, for all three layouts:
    // row-major (N, K/8) words, K-major blocks of 128 (K/128, N, 16) and of 64 (K/64, N, 8)
    const uint32_t piece = (uint32_t)((quarter >> 1) * 16 + (quarter & 1) * 8);
    const uint32_t code_lane = (uint32_t)code_row * (uint32_t)(p.packed_k == 0 ? blocks * 64 : p.packed_k == 128 ? 64 : 32) + piece;
    const int64_t block_stride = p.packed_k == 0 ? 64 : (int64_t)p.n * 64;
    const int64_t half_stride = p.packed_k == 64 ? (int64_t)p.n * 32 : 32;
    auto load_codes = [&](int block, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
        const int8_t* const base = uniform_pointer(reinterpret_cast<const int8_t*>(p.w) + (int64_t)min(block, blocks - 1) * block_stride);
        load_8(codes[SET][0], code_lane, base);
        load_8(codes[SET][1], code_lane, base + half_stride);
    };
    load_codes(0, std::integral_constant<int, 0>{});
    load_codes(1, std::integral_constant<int, 1>{});

    // ---- tables and scales, written before any direct-to-LDS request is in flight ----
    build_tables(*tables, p.book, tid, kTallThreads);
    lds_as[tid] = __half2float(p.as[t.row0 + min(tid, t.rows_here - 1)]);
    if (tid < kTallCols) lds_ws[tid] = __half2float(p.ws[t.col0 + min(tid, t.cols_here - 1)]);
    __syncthreads();

    // ---- token rows: K chunks of 128 (whole cache lines), two slots of 512 rows x 128 bytes; a wave requests its own
    // rows [64 wave, +64) of a chunk as eight 1 KiB blocks of 8 rows; 16-byte piece c of row r sits at position
    // c ^ ((r / 2) % 8) of the row, as in the persistent kernel ----
    const int load_row = wave * 64 + (lane >> 3);
    const uint32_t load_chunk = (uint32_t)(((lane & 7) ^ swizzle(load_row)) * 16);
    const int8_t* const a_base = uniform_pointer(p.a + (int64_t)t.row0 * p.k);
    // (the eight offsets stay in registers: computing them on issue is a multiply and five more instructions per
    // request)
    uint32_t load_offset[8];
#pragma unroll
    for (int b = 0; b < 8; ++b)
        load_offset[b] = (uint32_t)(min(load_row + 8 * b, t.rows_here - 1) * p.k) + (load_chunk ^ (uint32_t)((b & 1) * 64));
    auto issue_tokens = [&](int b, int chunk, int slot) {
        direct_load_16(a_base + min(chunk, blocks - 1) * 128 + (uint64_t)load_offset[b],
                       lds + kTallTokens + slot * kTallSlotA + (wave * 8 + b) * 1024);
    };

    // ---- fragments: a lane reads K bytes [16 (lane / 16), +16) of the slice for row lane % 16 of a block ----
    const int frag_row = lane & 15, frag_chunk = lane >> 4;
    const uint32_t a_frag = lds_base + kTallTokens + (wave * 64 + frag_row) * 128 + ((frag_chunk ^ swizzle(frag_row)) * 16);
    const uint32_t w_frag = lds_base + kTallWeights + (uint32_t)(frag_row * kTallStep + ((frag_chunk ^ tall_swizzle(frag_row)) * 16));
    v4i ft[2][4], fw[2][kTallBlocks];  // token and weight fragments of even and odd steps
    constexpr int kBlock = 16 * kTallStep;
    // slice step % 2 of chunk step / 2, which sits in slot (step / 2) % 2; the second slice of a row is the first
    // with address bit 6 flipped (piece 4 + c swizzles to the position of piece c with bit 2 flipped)
    auto read_tokens = [&](int step, int parity) {
        const uint32_t a = (a_frag ^ (uint32_t)((step & 1) * 64)) + ((step >> 1) & 1) * kTallSlotA;
        v4i(&f)[4] = ft[parity];
        f[0] = lds_read_16<0>(a);
        f[1] = lds_read_16<2048>(a);
        f[2] = lds_read_16<4096>(a);
        f[3] = lds_read_16<6144>(a);
    };
    auto read_weights = [&](int stage, int parity) {  // register set by the parity of the step
        const uint32_t w = w_frag + stage * kTallStageW;
        v4i(&f)[kTallBlocks] = fw[parity];
        f[0] = lds_read_16<0>(w);
        f[1] = lds_read_16<kBlock>(w);
        f[2] = lds_read_16<2 * kBlock>(w);
        f[3] = lds_read_16<3 * kBlock>(w);
        f[4] = lds_read_16<4 * kBlock>(w);
    };

    // ---- decode: this thread's chunk of a weight stage ----
    const uint32_t write_offset = kTallWeights + (uint32_t)(channel * kTallStep + ((quarter ^ tall_swizzle(channel)) * 16));
    // (the dynamic LDS of a kernel without static LDS starts at address 0, where the tables sit: a lookup's address
    // is the byte offset of its entry, the table chosen by the instruction's offset field)
    v2w looked[8];
    auto lookups = [&](v2w pair) {  // two code words: basis0, mask0, basis1, mask1 of each
        asm volatile("" : "+v"(pair));  // nothing computed from the words moves above this point
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t code = pair[i];
            looked[4 * i + 0] = lds_read_8<0>(lds_base + ((code >> 5) & 0x7F8u));       // basis0[(code >> 8) & 255]
            looked[4 * i + 1] = lds_read_8<2048>(lds_base + ((code << 3) & 0x7F8u));    // mask0[code & 255]
            looked[4 * i + 2] = lds_read_8<4096>(lds_base + ((code >> 21) & 0x7F8u));   // basis1[code >> 24]
            looked[4 * i + 3] = lds_read_8<6144>(lds_base + ((code >> 13) & 0x7F8u));   // mask1[(code >> 16) & 255]
        }
    };
    v4u chunk;
    // (LDS requests of a wave return in order)
    auto wait_lookups = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(looked[0]), "+v"(looked[1]), "+v"(looked[2]), "+v"(looked[3]), "+v"(looked[4]), "+v"(looked[5]),
                       "+v"(looked[6]), "+v"(looked[7]));
    };
    // code word i -> 8 weights, as decode_q4 combines the four entries
    auto combine = [&](int i) {
        chunk[2 * i + 0] = ((looked[4 * i][0] ^ looked[4 * i + 1][0]) + (looked[4 * i + 2][0] ^ looked[4 * i + 3][0]) + 0x35353535u) ^ 0x80808080u;
        chunk[2 * i + 1] = ((looked[4 * i][1] ^ looked[4 * i + 1][1]) + (looked[4 * i + 2][1] ^ looked[4 * i + 3][1]) + 0x35353535u) ^ 0x80808080u;
    };
    auto write_chunk = [&](int stage) { lds_write_16(lds_base + write_offset + stage * kTallStageW, chunk); };
    auto write_decoded = [&](int stage) {
        wait_lookups();
        combine(0);
        combine(1);
        write_chunk(stage);
    };

    v4i acc[4][kTallBlocks];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < kTallBlocks; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    // 4 x 5 multiplies of a step, one operand changing between consecutive instructions
    auto multiply = [&](int parity, auto between) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < kTallBlocks; ++j) {
                const int jj = (i & 1) ? kTallBlocks - 1 - j : j;
                v4i& sum = acc[i][jj];
                sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[parity][jj], ft[parity][i], sum, 0, 0, 0);
                between(i * kTallBlocks + j);
            }
    };

    // ---- prologue: K chunks 0 and 1 requested, the weights of steps 0 and 1 decoded (block 0), step 0's fragments requested ----
#pragma unroll
    for (int b = 0; b < 8; ++b) issue_tokens(b, 0, 0);
#pragma unroll
    for (int b = 0; b < 8; ++b) issue_tokens(b, 1, 1);
    asm volatile("s_waitcnt vmcnt(16)" : "+v"(codes[0][0]), "+v"(codes[0][1]), "+v"(codes[1][0]), "+v"(codes[1][1]));
    if (decoder) {
        lookups(codes[0][0]);
        write_decoded(0);
        lookups(codes[0][1]);
        write_decoded(1);
    }
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    read_tokens(0, 0);
    read_weights(0, 0);

    // Step s.  On entry the fragments of step s are on their way into registers (requested late in step s - 1, waited
    // for here), the rows of step s + 1 (this wave's own requests) have landed and its weights were written in front
    // of the last barrier.  Everything else of the step sits between its 20 multiplies, so that the matrix pipe works
    // while the LDS pipe and the vector ALU serve the rest: the lookups for the weights of step s + 2 first, behind
    // the fifth multiply their combination and the write of the chunk, and only then the nine fragment reads of step
    // s + 1.  LDS requests of a wave return in order, so the wait in front of the barrier can name the nine reads as
    // what may stay in flight: the chunk has landed, which is all the barrier has to publish, and the reads cross the
    // barrier (the LDS pipe has work while the waves meet; with the reads waited for in front of the barrier the
    // loop measured 5 % longer).  The stages they read are not written again before two more barriers.
    // K chunk c (steps 2 c, 2 c + 1) is requested in step 2 c - 3 into the slot that chunk c - 2 left when step
    // 2 c - 3 waited for its last fragments, and has two steps to land.  The vector-memory part of the wait names
    // how many younger requests may stay in flight (vector memory retires in order): behind an even step its 2 code
    // requests, behind an odd step its 8 row requests.
    auto wait_fragments_even = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(ft[0][0]), "+v"(ft[0][1]), "+v"(ft[0][2]), "+v"(ft[0][3]), "+v"(fw[0][0]), "+v"(fw[0][1]), "+v"(fw[0][2]),
                       "+v"(fw[0][3]), "+v"(fw[0][4])
                     :
                     : "memory");
    };
    auto wait_fragments_odd = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(ft[1][0]), "+v"(ft[1][1]), "+v"(ft[1][2]), "+v"(ft[1][3]), "+v"(fw[1][0]), "+v"(fw[1][1]), "+v"(fw[1][2]),
                       "+v"(fw[1][3]), "+v"(fw[1][4])
                     :
                     : "memory");
    };
    auto step = [&](int s, auto set_tag, auto odd_tag) {
        constexpr int SET = decltype(set_tag)::value, ODD = decltype(odd_tag)::value;  // SET: of the block being decoded
        const int next_stage = (s + 1) % kTallStagesW, decode_stage = (s + 2) % kTallStagesW;
        if constexpr (ODD) wait_fragments_odd(); else wait_fragments_even();
        __builtin_amdgcn_sched_barrier(0);
        multiply(ODD, [&](int index) {
            __builtin_amdgcn_sched_barrier(0);
            if (index == 0 && decoder) lookups(codes[SET][ODD]);
            if (ODD && (index & 1) == 1 && index < 16)  // chunk (s + 3) / 2 into the slot that chunk (s - 1) / 2 has left
                issue_tokens(index >> 1, (s + 3) >> 1, ((s + 3) >> 1) & 1);
            if (index >= 4 && index <= 8 && (index & 1) == 0 && decoder) {
                if (index == 4) wait_lookups();
                if (index == 4) combine(0);
                if (index == 6) combine(1);
                if (index == 8) write_chunk(decode_stage);
            }
            if (index == 10) read_tokens(s + 1, 1 - ODD);
            if (index == 12) read_weights(next_stage, 1 - ODD);
            __builtin_amdgcn_sched_barrier(0);
        });
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!ODD) load_codes((s >> 1) + 2, std::integral_constant<int, 1 - SET>{});
        // the 9 fragment reads may stay in flight over the barrier; the chunk written before them has landed
        if constexpr (!ODD)
            asm volatile("s_waitcnt vmcnt(2) lgkmcnt(9)\n\ts_barrier" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(8) lgkmcnt(9)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    // steps 4 g .. 4 g + 3 decode blocks 2 g + 1 (set 1: steps 4 g, 4 g + 1) and 2 g + 2 (set 0: steps 4 g + 2, 4 g + 3)
    std::integral_constant<int, 0> zero;
    std::integral_constant<int, 1> one;
    int s = 0;
    for (; s + 3 < steps; s += 4) {
        step(s, one, zero);       // requests block 2 g + 2 into set 0
        step(s + 1, one, one);
        step(s + 2, zero, zero);  // requests block 2 g + 3 into set 1
        step(s + 3, zero, one);
    }
    if (s < steps) {  // K = 128 x an odd number: one block left
        step(s, one, zero);
        step(s + 1, one, one);
    }
    // The last steps request code words, token rows and fragments that nobody consumes (clamped addresses; the waits above
    // count on every step issuing the same requests).  Their destination registers are named here, behind the wait:
    // a register whose value the compiler believes dead is free for reuse while its load is still in flight, and the
    // data would land on whatever lives there by then.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)"
                 : "+v"(ft[0][0]), "+v"(ft[0][1]), "+v"(ft[0][2]), "+v"(ft[0][3]), "+v"(ft[1][0]), "+v"(ft[1][1]), "+v"(ft[1][2]),
                   "+v"(ft[1][3]), "+v"(fw[0][0]), "+v"(fw[0][1]), "+v"(fw[0][2]), "+v"(fw[0][3]), "+v"(fw[0][4]), "+v"(fw[1][0]),
                   "+v"(fw[1][1]), "+v"(fw[1][2]), "+v"(fw[1][3]), "+v"(fw[1][4])
                 :
                 : "memory");
    asm volatile("" : "+v"(codes[0][0]), "+v"(codes[0][1]), "+v"(codes[1][0]), "+v"(codes[1][1]));

    // ---- epilogue: private to a wave and in registers; a lane holds four consecutive channels of one token ----
    int own = threadIdx.x & 63;
    asm volatile("" : "+v"(own));
    const int group = own >> 4;
    if constexpr (F32) {
        const bool vector_ok = p.stride % 4 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int local_row = wave * 64 + i * 16 + (own & 15);
            if (local_row >= t.rows_here) continue;
            const int64_t row = t.row0 + local_row;
            const float token_scale = lds_as[local_row];
#pragma unroll
            for (int j = 0; j < kTallBlocks; ++j) {
                const int local_col = j * 16 + 4 * group;
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
    } else {
        const bool aligned = (p.stride % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int local_row = wave * 64 + i * 16 + (own & 15);
            const float token_scale = lds_as[local_row];
            __half* const row_out = reinterpret_cast<__half*>(p.out) + (int64_t)(t.row0 + local_row) * p.stride + t.col0;
            // blocks 0..3 in pairs: a lane swap turns two 4-channel pieces into one of 8 channels (16 bytes)
#pragma unroll
            for (int pair = 0; pair < 2; ++pair) {
                uint32_t words[2][2];
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const int j = 2 * pair + b;
                    const float4 wscale = *reinterpret_cast<const float4*>(lds_ws + j * 16 + 4 * group);
                    words[b][0] = pack_halves(rescale(acc[i][j][0], wscale.x, token_scale), rescale(acc[i][j][1], wscale.y, token_scale));
                    words[b][1] = pack_halves(rescale(acc[i][j][2], wscale.z, token_scale), rescale(acc[i][j][3], wscale.w, token_scale));
                }
                const v2u low = __builtin_amdgcn_permlane16_swap(words[0][0], words[1][0], false, false);
                const v2u high = __builtin_amdgcn_permlane16_swap(words[0][1], words[1][1], false, false);
                const uint4 piece = make_uint4(low.x, high.x, low.y, high.y);
                const int local_col = (2 * pair + (group & 1)) * 16 + (group >> 1) * 8;
                if (local_row < t.rows_here && local_col < t.cols_here) {
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
                __builtin_amdgcn_sched_barrier(0);
            }
            // the fifth block: four channels (8 bytes) per lane
            {
                constexpr int j = kTallBlocks - 1;
                const int local_col = j * 16 + 4 * group;
                const float4 wscale = *reinterpret_cast<const float4*>(lds_ws + local_col);
                const uint2 piece = make_uint2(pack_halves(rescale(acc[i][j][0], wscale.x, token_scale), rescale(acc[i][j][1], wscale.y, token_scale)),
                                               pack_halves(rescale(acc[i][j][2], wscale.z, token_scale), rescale(acc[i][j][3], wscale.w, token_scale)));
                if (local_row < t.rows_here && local_col < t.cols_here) {
                    if (aligned && local_col + 4 <= t.cols_here) {
                        *reinterpret_cast<uint2*>(row_out + local_col) = piece;
                    } else {
                        const uint32_t parts[2] = {piece.x, piece.y};
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (local_col + e < t.cols_here)
                                row_out[local_col + e] = __ushort_as_half((unsigned short)(parts[e >> 1] >> (16 * (e & 1))));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

int prepare_device() {
    int code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_persistent_kernel<false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPersistentLds),
                         "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_persistent_kernel<true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPersistentLds),
                     "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_q4_tall_kernel<false>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTallLds),
                     "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_q4_tall_kernel<true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTallLds),
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

// int8 weights: one persistent workgroup per CU walks the 256 x 256 tiles
void gemm_big_geometry(int rows, int n, Geometry* g) {
    const uint32_t tiles = ceil_div((uint32_t)rows, (uint32_t)kTile) * ceil_div((uint32_t)n, (uint32_t)kTile);
    g->grid[0] = std::min(tiles, (uint32_t)device_compute_units());
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kPersistentThreads;
    g->shared = kPersistentLds;
}

int gemm_big_launch(const int8_t* a, const void* w, const __half* ws, const __half* as, void* out, int rows, int n,
                    int k, int stride, bool out_f32, const Geometry& g, hipStream_t stream) {
    const int ready = prepare();
    if (ready != ORX_OK) return ready;
    BigParams p = {};
    p.a = a, p.w = w, p.book = nullptr, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.packed_k = 0, p.out_f32 = out_f32;
    p.tiles_m = (rows + kTile - 1) / kTile, p.tiles_n = (n + kTile - 1) / kTile;
    if (k < 2 * kStep) {
        set_error("projection (mfma 256x256): the persistent int8 kernel needs K >= 256");
        return ORX_ERR_BAD_VARIANT;
    }
    if (out_f32)
        ORX_LAUNCH((gemm_big_persistent_kernel<true>), dim3(g.grid[0]), dim3(kPersistentThreads), g.shared, stream, p);
    else
        ORX_LAUNCH((gemm_big_persistent_kernel<false>), dim3(g.grid[0]), dim3(kPersistentThreads), g.shared, stream, p);
    return hip_check(hipGetLastError(), "launch projection (mfma 256x256)");
}

// Two-stage codes on 512 rows x channel runs with the decode in the K loop (K a multiple of 128).
// Workgroups per row tile: the blocks of 16 channels are dealt evenly over whole rounds of the CUs, at most kTallBlocks
// to a workgroup.
uint32_t gemm_tall_units(int n) {
    const uint32_t blocks = ceil_div((uint32_t)n, 16u), cus = (uint32_t)device_compute_units();
    const uint32_t rounds = ceil_div(blocks, (uint32_t)kTallBlocks * cus);
    return std::min(blocks, rounds * cus);
}
void gemm_tall_geometry(int rows, int n, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)rows, (uint32_t)kTallRows) * gemm_tall_units(n);
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kTallThreads;
    g->shared = kTallLds;
}

int gemm_tall_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out,
                     int rows, int n, int k, int stride, int packed_k, bool out_f32, const Geometry& g, hipStream_t stream) {
    const int ready = prepare();
    if (ready != ORX_OK) return ready;
    if (k % 128 != 0 || k < 256) {
        set_error("projection (mfma, 512-row channel runs): K must be a multiple of 128, at least 256");
        return ORX_ERR_BAD_VARIANT;
    }
    BigParams p = {};
    p.a = a, p.w = w, p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.packed_k = packed_k, p.out_f32 = out_f32;
    p.tiles_m = (rows + kTallRows - 1) / kTallRows, p.tiles_n = (int)gemm_tall_units(n);
    if (out_f32)
        ORX_LAUNCH((gemm_q4_tall_kernel<true>), dim3(g.grid[0]), dim3(kTallThreads), g.shared, stream, p);
    else
        ORX_LAUNCH((gemm_q4_tall_kernel<false>), dim3(g.grid[0]), dim3(kTallThreads), g.shared, stream, p);
    return hip_check(hipGetLastError(), "launch projection (mfma, 512-row channel runs, decode in the loop)");
}

}  // namespace orx
