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

#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTile = 256;     // output tile edge
constexpr int kStep = 128;     // K bytes per step
constexpr int kThreads = 512;  // 8 waves
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

template <bool Q4>
__global__ __launch_bounds__(kThreads, 2) void gemm_big_kernel(BigParams p) {
    extern __shared__ __align__(16) int8_t lds[];  // [2 stages][A 32 KiB | W 32 KiB] (+ Q4 tables)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2, wave_n = wave & 3;  // 2 x 4 waves, wave tile 128 x 64

    int tile_m, tile_n;
    tile_of(blockIdx.x, p.tiles_m, p.tiles_n, &tile_m, &tile_n);
    const int row0 = tile_m * kTile, col0 = tile_n * kTile;
    const int rows_here = min(kTile, p.m - row0);
    const int cols_here = min(kTile, p.n - col0);

    Q4ByteTables* tables = reinterpret_cast<Q4ByteTables*>(lds + 4 * kTileBytes);
    if (Q4) build_tables(*tables, p.book, tid, kThreads);

    // ---- global -> LDS: one wave instruction = 8 rows x 128 bytes (1 KiB block) ----
    // wave w owns blocks w*4 .. w*4+3 of each operand tile (32 blocks of 8 rows)
    const int load_r8 = lane >> 3, load_slot = lane & 7;
    auto issue_direct = [&](const int8_t* base, int limit, int origin, int kt, int8_t* stage) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int block = wave * 4 + b;
            const int row = block * 8 + load_r8;
            const int chunk = load_slot ^ swizzle(row);
            const int source_row = origin + min(row, limit - 1);
            direct_load_16(base + (int64_t)source_row * p.k + kt * kStep + chunk * 16, stage + block * 1024);
        }
    };
    // Q4: one K step of the weight tile is 256 rows x 64 bytes of codes = 1024 chunks of 16 bytes
    // (4 codes = 32 weights each): two chunks per thread.
    uint4 code_regs[2];
    auto load_codes = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + kThreads * i;      // chunk id: row = c / 4, quarter = c % 4
            const int row = min(c >> 2, cols_here - 1), q = c & 3;
            int64_t byte;
            if (p.packed_k == 128)
                byte = ((int64_t)kt * p.n + col0 + row) * 64 + q * 16;
            else
                byte = ((int64_t)(col0 + row) * (p.k / kStep) + kt) * 64 + q * 16;
            code_regs[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const int8_t*>(p.w) + byte);
        }
    };
    auto store_decoded = [&](int8_t* stage) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + kThreads * i;
            const int row = c >> 2, q = c & 3;
            const uint2 d0 = decode_q4(*tables, code_regs[i].x), d1 = decode_q4(*tables, code_regs[i].y);
            const uint2 d2 = decode_q4(*tables, code_regs[i].z), d3 = decode_q4(*tables, code_regs[i].w);
            // 32 weights = chunks 2q and 2q+1 of the row
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
    const int a_lane = (wave_m * 128 + frag_row) * kStep;
    const int w_lane = (wave_n * 64 + frag_row) * kStep;

    v16i acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int k_tiles = p.k / kStep;
    auto stage_a = [&](int stage) { return lds + stage * 2 * kTileBytes; };
    auto stage_w = [&](int stage) { return lds + kTileBytes + stage * 2 * kTileBytes; };

    issue_direct(p.a, rows_here, row0, 0, stage_a(0));
    if (Q4) {
        load_codes(0);
        __syncthreads();  // tables
        store_decoded(stage_w(0));
        if (k_tiles > 1) load_codes(1);
    } else {
        issue_direct(reinterpret_cast<const int8_t*>(p.w), cols_here, col0, 0, stage_w(0));
    }

    for (int kt = 0; kt < k_tiles; ++kt) {
        const int cur = kt & 1, nxt = cur ^ 1;
        __syncthreads();  // step kt is in LDS for everybody; everybody is done reading stage nxt
        if (kt + 1 < k_tiles) {
            issue_direct(p.a, rows_here, row0, kt + 1, stage_a(nxt));
            if (!Q4) issue_direct(reinterpret_cast<const int8_t*>(p.w), cols_here, col0, kt + 1, stage_w(nxt));
        }
        const int8_t* la = stage_a(cur) + a_lane;
        const int8_t* lw = stage_w(cur) + w_lane;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            v4i fa[4], fb[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const v4i*>(la + i * 32 * kStep + frag_offset[ks]);
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = *reinterpret_cast<const v4i*>(lw + j * 32 * kStep + frag_offset[ks]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (Q4 && kt + 1 < k_tiles) {
            store_decoded(stage_w(nxt));  // stage nxt was released by the barrier above
            if (kt + 2 < k_tiles) load_codes(kt + 2);
        }
    }

    // ---- epilogue ----
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int local_col = wave_n * 64 + j * 32 + (lane & 31);
        if (local_col >= cols_here) continue;
        const int col = col0 + local_col;
        const float wscale = __half2float(p.ws[col]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int local = wave_m * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (local < rows_here) {
                    const int64_t row = row0 + local;
                    const float value = rescale(acc[i][j][r], wscale, __half2float(p.as[row]));
                    if (p.out_f32)
                        reinterpret_cast<float*>(p.out)[row * p.stride + col] = value;
                    else
                        reinterpret_cast<__half*>(p.out)[row * p.stride + col] = __float2half_rn(value);
                }
            }
        }
    }
}

constexpr uint32_t kBigLds = 4 * kTileBytes;                       // 128 KiB
constexpr uint32_t kBigLdsQ4 = 4 * kTileBytes + sizeof(Q4ByteTables);  // + 8 KiB

int prepare() {
    static bool done = false;
    if (done) return ORX_OK;
    int code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_kernel<false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLds),
                         "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_big_kernel<true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLdsQ4),
                     "hipFuncSetAttribute");
    if (code != ORX_OK) return code;
    done = true;
    return ORX_OK;
}

}  // namespace

void gemm_big_geometry(int rows, int n, bool q4, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)rows, (uint32_t)kTile) * ceil_div((uint32_t)n, (uint32_t)kTile);
    g->grid[1] = g->grid[2] = 1;
    g->block[0] = kThreads;
    g->shared = q4 ? kBigLdsQ4 : kBigLds;
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
    if (q4)
        hipLaunchKernelGGL((gemm_big_kernel<true>), dim3(g.grid[0]), dim3(kThreads), g.shared, stream, p);
    else
        hipLaunchKernelGGL((gemm_big_kernel<false>), dim3(g.grid[0]), dim3(kThreads), g.shared, stream, p);
    return hip_check(hipGetLastError(), "launch projection (mfma 256x256)");
}

}  // namespace orx
