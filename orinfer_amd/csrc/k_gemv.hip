// Bandwidth-bound projections for 1..4 token rows (batch-1 decode and tiny batches).
//
// Reference counterparts: the DP4A schedules kernels/cuda/model/integer_core.py:275-388
// (E8P-Q4 and W8), kernels/cuda/model/int8_projection.py:66-107 and the single-token Q2
// route kernel kernels/cuda/model/integer_vq.py:380-444.  Arithmetic is the same exact
// int32 dot over full K followed by (float(acc)*ws)*as (integer_core.py:19-22).
//
// MI355X design.  The weight stream (4 bits/weight) is the only HBM traffic that matters,
// so each lane pulls 16-byte chunks of codes with global_load_dwordx4 and the whole decode
// is two LDS table reads and one XOR per u16 code: q = 2v+1 with v = nib[b] ^ msk[u] as
// eight signed nibbles.  Activations are split once per workgroup into nibble planes
// a = 16*hi + lo + 8 (hi, lo signed 4-bit), so the dot with a code is three v_dot8_i32_i4:
//     sum q*a = 2*(16*sum v*hi + sum v*lo + 8*sum v) + sum a.
// Two-stage Q4 (w = 4*q0 + q1 = 8*v0 + 2*v1 + 5) keeps one accumulator set per stage.
// Lanes of a row group own fixed k-chunks; LPR lanes share one output row and are
// reduced with cross-lane shuffles at the end.  The only atomics are integer adds into LDS for the
// per-row activation sums (order-independent, so results stay bit-exact); no global atomics, no
// scratch memory, no host reads.
#include <hip/hip_fp16.h>

#include "a8_device.h"
#include "e8p_device.h"
#include "moe_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

enum Codec { kQ4 = 0, kQ2 = 1, kW8 = 2 };

constexpr int kThreads = 512;       // 8 waves
constexpr int kLanesPerRow = 16;    // lanes that share one output row
constexpr int kRowsPerWave = 64 / kLanesPerRow;
constexpr int kRowsPerPass = (kThreads / 64) * kRowsPerWave;  // 32 rows per workgroup pass

__device__ __forceinline__ int sdot8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot8((int)a, (int)b, c, false);
}
__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// LDS: static nib[256], msk[256], sums[4]; dynamic activation planes.  For Q4/Q2 the planes are hi
// then lo nibble words, MR x K/8 each; for W8 they are the raw int8 rows, MR x K bytes.
template <int CODEC, int MR>
__global__ __launch_bounds__(kThreads) void gemv_rowmajor_kernel(
    const int8_t* __restrict__ a, const uint4* __restrict__ w, const uint32_t* __restrict__ book,
    const __half* __restrict__ ws, const __half* __restrict__ as, void* __restrict__ out, int n, int k, int stride,
    int m, int passes, int out_f32) {
    extern __shared__ __align__(16) uint32_t planes[];
    __shared__ uint32_t nib[256];
    __shared__ uint32_t msk[256];
    __shared__ int sums[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int sub = lane & (kLanesPerRow - 1);  // which chunks of the row
    const int row_in_wave = lane / kLanesPerRow;
    // bytes per row of the weight stream and number of 16-byte chunks
    const int row_bytes = CODEC == kQ4 ? k / 2 : CODEC == kQ2 ? k / 4 : k;
    const int chunks = row_bytes / 16;
    const int groups = k / 8;

    // Row owned by this lane group in the first pass; its first chunks are requested right after
    // the small setup reads below (the memory counter retires in order, so the setup reads must
    // be older than the bulk stream to be waited on alone) and land while the tables are built.
    // Stream loads are never predicated:
    // indices beyond the row are clamped to its last chunk (a cache hit) and simply not consumed,
    // which keeps the loop free of divergent branches and lets the hardware counters track
    // exactly which request each consume step waits for.
    // register ring of 16-byte chunks per lane; int8 weights have four times the bytes per row and no
    // decode between the loads, so twice the ring keeps the memory system busier (N = 5120, K = 17408:
    // 22.4 -> 21.0 us at one row)
    constexpr int D = CODEC == kW8 ? 8 : 4;
    const int per_lane = (chunks - sub + kLanesPerRow - 1) / kLanesPerRow;       // chunks this lane owns
    const int steps = (chunks + kLanesPerRow - 1) / kLanesPerRow;                // wave-uniform trip count
    auto row_of = [&](int pass) {
        return (blockIdx.x * passes + pass) * kRowsPerPass + wave * kRowsPerWave + row_in_wave;
    };
    auto fetch = [&](const uint4* src, int step) { return src[min(sub + step * kLanesPerRow, chunks - 1)]; };
    uint4 ring[D];

    // ---- workgroup setup: tables, activation planes, activation sums ----
    // Every global read of the setup is issued up front (selector word, activation groups, the
    // row's scales) so that the kernel pays one memory latency, not one per dependent step.
    const int first_row = row_of(0);
    // raw bits now, conversion in the epilogue: a conversion here would wait for the load at once
    // (unconditional, clamped indices: a conditional load would merge with a constant and be
    // waited for at the merge)
    const unsigned short ws_first = reinterpret_cast<const unsigned short*>(ws)[min(first_row, n - 1)];
    unsigned short as_bits[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) as_bits[r] = reinterpret_cast<const unsigned short*>(as)[min(r, m - 1)];
    const uint32_t selector = CODEC != kW8 ? book[tid & 255] : 0u;
    if (tid < 4) sums[tid] = 0;
    if (CODEC != kW8) {
        uint32_t* hi = planes;
        uint32_t* lo = planes + MR * groups;
        constexpr int GR = 2;  // activation groups per thread per round
        for (int g0 = 0; g0 < groups; g0 += GR * kThreads) {
            uint2 raw[MR][GR];
#pragma unroll
            for (int r = 0; r < MR; ++r)
#pragma unroll
                for (int i = 0; i < GR; ++i) {
                    const int g = g0 + i * kThreads + tid;
                    raw[r][i] = (r < m && g < groups) ? *reinterpret_cast<const uint2*>(a + (int64_t)r * k + 8 * g)
                                                     : make_uint2(0u, 0u);
                }
            if (g0 == 0) {  // bulk stream behind the setup reads, ahead of any wait
                const uint4* src = w + (int64_t)(first_row < n ? first_row : 0) * chunks;
#pragma unroll
                for (int d = 0; d < D; ++d) ring[d] = fetch(src, d);
            }
            if (g0 == 0 && tid < 256) {  // table entries while the loads are in flight
                nib[tid] = nibble_basis_word(selector, 0u);
                msk[tid] = nibble_mask_word((uint32_t)tid);
            }
            if (g0 == 0) __syncthreads();  // sums[] is zero before the first add below
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                int partial = 0;
#pragma unroll
                for (int i = 0; i < GR; ++i) {
                    const int g = g0 + i * kThreads + tid;
                    const uint2 v = raw[r][i];
                    if (g < groups) {
                        // hi nibbles: coordinates 0..3 to even nibble slots, 4..7 to odd slots
                        hi[r * groups + g] = ((v.x >> 4) & 0x0F0F0F0Fu) | (v.y & 0xF0F0F0F0u);
                        lo[r * groups + g] = ((v.x & 0x0F0F0F0Fu) | ((v.y << 4) & 0xF0F0F0F0u)) ^ 0x88888888u;
                    }
                    partial = sdot4(v.x, 0x01010101u, partial);
                    partial = sdot4(v.y, 0x01010101u, partial);
                }
#pragma unroll
                for (int offset = 32; offset > 0; offset >>= 1) partial += __shfl_xor(partial, offset, 64);
                if (lane == 0 && partial != 0) atomicAdd(&sums[r], partial);
            }
        }
    } else {
        {
            const uint4* src = w + (int64_t)(first_row < n ? first_row : 0) * chunks;
#pragma unroll
            for (int d = 0; d < D; ++d) ring[d] = fetch(src, d);
        }
        for (int r = 0; r < MR; ++r)
            for (int i = tid; i < k / 4; i += kThreads)
                planes[r * (k / 4) + i] = r < m ? reinterpret_cast<const uint32_t*>(a + (int64_t)r * k)[i] : 0u;
    }
    __syncthreads();

    // One 16-byte chunk of the weight stream against every activation row.
    int acc_h0[MR], acc_l0[MR], acc_h1[MR], acc_l1[MR];
    int acc_v0, acc_v1;
    auto consume = [&](const uint4& cur, int j) {
        if (CODEC == kQ4) {
            const uint32_t code[4] = {cur.x, cur.y, cur.z, cur.w};
            uint4 ph[MR], pl[MR];
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                ph[r] = *reinterpret_cast<const uint4*>(planes + r * groups + 4 * j);
                pl[r] = *reinterpret_cast<const uint4*>(planes + (MR + r) * groups + 4 * j);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t c = code[i];
                const uint32_t v0 = nib[(c >> 8) & 255u] ^ msk[c & 255u];
                const uint32_t v1 = nib[c >> 24] ^ msk[(c >> 16) & 255u];
                acc_v0 = sdot8(v0, 0x11111111u, acc_v0);
                acc_v1 = sdot8(v1, 0x11111111u, acc_v1);
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    const uint32_t h = reinterpret_cast<const uint32_t*>(&ph[r])[i];
                    const uint32_t l = reinterpret_cast<const uint32_t*>(&pl[r])[i];
                    acc_h0[r] = sdot8(v0, h, acc_h0[r]);
                    acc_l0[r] = sdot8(v0, l, acc_l0[r]);
                    acc_h1[r] = sdot8(v1, h, acc_h1[r]);
                    acc_l1[r] = sdot8(v1, l, acc_l1[r]);
                }
            }
        } else if (CODEC == kQ2) {
            const uint32_t pair[4] = {cur.x, cur.y, cur.z, cur.w};
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                uint4 ph[MR], pl[MR];
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    ph[r] = *reinterpret_cast<const uint4*>(planes + r * groups + 8 * j + 4 * half);
                    pl[r] = *reinterpret_cast<const uint4*>(planes + (MR + r) * groups + 8 * j + 4 * half);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t c = (pair[2 * half + (i >> 1)] >> (16 * (i & 1))) & 0xFFFFu;
                    const uint32_t v0 = nib[c >> 8] ^ msk[c & 255u];
                    acc_v0 = sdot8(v0, 0x11111111u, acc_v0);
#pragma unroll
                    for (int r = 0; r < MR; ++r) {
                        acc_h0[r] = sdot8(v0, reinterpret_cast<const uint32_t*>(&ph[r])[i], acc_h0[r]);
                        acc_l0[r] = sdot8(v0, reinterpret_cast<const uint32_t*>(&pl[r])[i], acc_l0[r]);
                    }
                }
            }
        } else {
            const uint32_t word[4] = {cur.x, cur.y, cur.z, cur.w};
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                const uint4 act = *reinterpret_cast<const uint4*>(planes + r * (k / 4) + 4 * j);
                const uint32_t aw[4] = {act.x, act.y, act.z, act.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) acc_h0[r] = sdot4(word[i], aw[i], acc_h0[r]);
            }
        }
    };

    for (int pass = 0; pass < passes; ++pass) {
        const int row = row_of(pass);
        const bool live = row < n;
        const uint4* src = w + (int64_t)(live ? row : 0) * chunks;
        acc_v0 = acc_v1 = 0;
#pragma unroll
        for (int r = 0; r < MR; ++r) acc_h0[r] = acc_l0[r] = acc_h1[r] = acc_l1[r] = 0;
        if (pass > 0) {
#pragma unroll
            for (int d = 0; d < D; ++d) ring[d] = fetch(src, d);
        }
        for (int base = 0; base < steps; base += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const uint4 cur = ring[d];
                ring[d] = fetch(src, base + D + d);
                if (base + d < per_lane) consume(cur, sub + (base + d) * kLanesPerRow);
            }
        }

        // per-lane totals, then reduce over the lanes of the row
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            int total;
            if (CODEC == kQ4)
                total = 8 * (16 * acc_h0[r] + acc_l0[r] + 8 * acc_v0) + 2 * (16 * acc_h1[r] + acc_l1[r] + 8 * acc_v1);
            else if (CODEC == kQ2)
                total = 2 * (16 * acc_h0[r] + acc_l0[r] + 8 * acc_v0);
            else
                total = acc_h0[r];
#pragma unroll
            for (int offset = kLanesPerRow / 2; offset > 0; offset >>= 1) total += __shfl_xor(total, offset, 64);
            if (live && sub == 0 && r < m) {
                if (CODEC == kQ4) total += 5 * sums[r];
                if (CODEC == kQ2) total += sums[r];
                const unsigned short ws_bits = pass == 0 ? ws_first : reinterpret_cast<const unsigned short*>(ws)[row];
                const float value = rescale(total, __half2float(__ushort_as_half(ws_bits)),
                                            __half2float(__ushort_as_half(as_bits[r])));
                if (out_f32)
                    reinterpret_cast<float*>(out)[(int64_t)r * stride + row] = value;
                else
                    reinterpret_cast<__half*>(out)[(int64_t)r * stride + row] = __float2half_rn(value);
            }
        }
    }
}

// ---- bank-replicated tables -----------------------------------------------------------------
// The two lookups per code are random reads of 1 KiB tables: 64 lanes collide in the LDS banks
// and the lookups, not HBM, bound the kernel above.  This variant stores every table entry once
// per lane column (entry i of lane l at byte i*256 + l*4), so lane l only ever touches bank l and
// every lookup is conflict-free.  Two tables take 128 KiB; a 16-wave workgroup owns a whole CU,
// stays resident and walks its rows wave by wave (wave g takes row tasks g, g + waves, ...), which
// spreads a ragged tail evenly over the CUs.  The lookup address is one v_perm_b32: byte 0 and
// byte 2 come from the lane's column address, byte 1 is the code byte.  That needs the tables at
// LDS byte 0 and 65536, so the kernel uses dynamic LDS only (no static LDS ahead of it).
constexpr uint32_t kMskBase = 65536u, kBankedPlanes = 131072u;
constexpr int kBankedThreads = 1024;
typedef __attribute__((address_space(3))) const uint32_t lds_word;

// Sum over the 64 lanes with data-parallel-primitive moves only (no LDS traffic); the total lands
// in lane 63.  Quad swaps, half-row and row mirrors give every lane its row's sum, the two
// broadcasts carry row sums across rows.
__device__ __forceinline__ int wave_sum_to_last_lane(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);  // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);  // row_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false); // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false); // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ uint32_t wave_or_to_last_lane(uint32_t bits) {
    int v = (int)bits;
    v |= __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v |= __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    v |= __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
    v |= __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);
    v |= __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);
    v |= __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);
    return (uint32_t)v;
}

__device__ __forceinline__ uint32_t banked_lookup(uint32_t code, uint32_t column, uint32_t selector) {
    const uint32_t address = __builtin_amdgcn_perm(code, column, selector);
    return *reinterpret_cast<lds_word*>(address);
}
// selectors: result byte 0 = column byte 0, byte 1 = code byte k, byte 2 = column byte 2 (mask
// table, base 65536) or zero (basis table, base 0), byte 3 = zero
constexpr uint32_t kSelNib1 = 0x0C0C0500u, kSelNib3 = 0x0C0C0700u, kSelMsk0 = 0x0C020400u, kSelMsk2 = 0x0C020600u;

// Activations are split differently from the kernel above: a = 16*hi + lo with both nibbles
// signed, hi = (a + 8) >> 4 and lo = the two's complement low nibble.  That needs no bias term
// (no third dot product per code), but hi reaches +8 for a >= 120, which a signed nibble reads
// as -8.  Those few positions (the row maximum and values within 6 % of it) are marked in a
// third plane, ov = 1, worth 256 each; a chunk whose 32 activations hold such a value is flagged
// per lane and step, and only flagged chunks pay for the extra dot products.
//
// LDS (dynamic only): [0,64K) basis words, [64K,128K) mask words, then the activation planes
// (hi, lo, ov; MR x K/8 words each), one partial activation sum per wave and row, and one flag
// byte per chunk of a row (does it hold an overflow; 64 steps per lane at most).
// LPR lanes share one output row (64/LPR rows per wave task); D is the depth of the per-lane
// ring of 16-byte chunks.  Two-stage Q4 only.  HOLD (one activation row, a row's steps equal to D):
// a lane meets the same chunk positions in every output row, so it keeps their hi and lo words in
// registers for the whole kernel and the main loop reads LDS for table lookups only.
// LAYOUT: lanes per row, + 64 for K-major codes.
constexpr int kKMajorLayout = 64;
// X16 (one activation row, K up to 8192): `a` holds the row as fp16 and the kernel quantises it
// itself during set-up, by the rule of the activation quantiser (row maximum over 127, fp16 scale,
// round to nearest even); every workgroup does so for itself, the first one also writes the scale
// to `as`.  That saves the separate launch in front of a single-row projection.
template <int CODEC, int MR, int D, int LAYOUT, bool HOLD, bool X16 = false>
__global__ __launch_bounds__(kBankedThreads) void gemv_banked_kernel(
    const int8_t* __restrict__ a, const uint4* __restrict__ w, const uint32_t* __restrict__ book,
    const __half* __restrict__ ws, const __half* __restrict__ as, void* __restrict__ out, int n, int k, int stride,
    int m, int flags, const int8_t* __restrict__ signs) {
    extern __shared__ __align__(16) uint32_t lds[];
    const bool out_f32 = flags & 1;  // bit 1: K-major blocks of 64 instead of 128
    constexpr int LPR = LAYOUT & (kKMajorLayout - 1);
    constexpr bool kKMajor = LAYOUT >= kKMajorLayout;
    constexpr int kRows = 64 / LPR;  // rows per wave task
    const int groups = k / 8;
    uint32_t* planes = lds + kBankedPlanes / 4;
    static_assert(CODEC == kQ4, "the replicated-table kernel decodes two-stage codes");
    int* wave_sums = reinterpret_cast<int*>(planes + 3 * MR * groups);          // [MR][16 waves]
    uint8_t* chunk_flags = reinterpret_cast<uint8_t*>(wave_sums + 4 * 16);      // [chunks]: chunk holds an overflow
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int sub = lane & (LPR - 1);
    const int row_in_wave = lane / LPR;
    const int row_bytes = CODEC == kQ4 ? k / 2 : k / 4;
    const int chunks = row_bytes / 16;
    const int steps = HOLD ? D : chunks / LPR;   // the host guarantees chunks % LPR == 0 (HOLD: and a quotient of D)
    const int padded = (steps + D - 1) / D * D;  // ring refills happen in whole groups of D
    const int tasks = (n + kRows - 1) / kRows;
    const int task_stride = gridDim.x * (kBankedThreads / 64);
    // Wave-uniform values are kept in scalar registers so that a stream address is a scalar base
    // plus one 32-bit lane offset: no vector arithmetic per load.
    const int first_task = __builtin_amdgcn_readfirstlane(wave) * gridDim.x + blockIdx.x;
    const char* stream = reinterpret_cast<const char*>(w);
    // K-major codes (K/128 blocks of N rows x 64 bytes, or K/64 blocks of N rows x 32 bytes): a task is still
    // 64/LPR adjacent rows, a step is LPR/4 (LPR/2) K blocks, and the lanes of one K block read the task's rows as
    // one contiguous run of 64 (32) bytes per row.  A lane still owns chunk sub + step * LPR of its row, so
    // everything below the addressing is shared with the row-major form.
    const int block_shift = (flags & 2) ? 1 : 2;  // log2 of the 16-byte chunks a row holds per K block
    const int block_bytes = 16 << block_shift;
    const size_t task_bytes = kKMajor ? (size_t)kRows * block_bytes : (size_t)kRows * row_bytes;
    const size_t step_bytes = kKMajor ? (size_t)n * 16 * LPR : (size_t)LPR * 16;
    auto base_of = [&](int task) { return stream + (size_t)min(task, tasks - 1) * task_bytes; };
    auto lane_offset = [&](int task) {  // rows past the end re-read the task's first row and are not stored
        const int row = min(task, tasks - 1) * kRows + row_in_wave;
        const int local_row = row < n ? row_in_wave : 0;
        if (kKMajor)
            return (uint32_t)(((sub >> block_shift) * n + local_row) * block_bytes + (sub & ((1 << block_shift) - 1)) * 16);
        return (uint32_t)(local_row * row_bytes + sub * 16);
    };
    auto fetch = [&](const char* base, uint32_t offset, int step) {
        return *reinterpret_cast<const uint4*>(base + (size_t)min(step, steps - 1) * step_bytes + offset);
    };
    uint4 ring[D];

    // ---- setup: one barrier ----
    // Every global read is issued before anything waits: scales, selector word, this thread's
    // activation groups, then the first chunks of the bulk stream.  The memory counter retires in
    // order, so the small reads can be waited for without waiting for the stream behind them.
    // Each wave then builds its own 16 entries of both tables and its own slice of the planes;
    // nothing is accumulated across waves with atomics, so nothing has to be cleared first and
    // the only barrier is the one that publishes the finished tables and planes.  Waves launched
    // early do this work while the dispatcher is still launching the rest of the workgroup.
    uint32_t* hi = planes;
    uint32_t* lo = planes + MR * groups;
    uint32_t* ov = planes + 2 * MR * groups;
    static_assert(!X16 || MR == 1, "the fp16 input form serves one activation row");
    unsigned short as_bits[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) as_bits[r] = X16 ? (unsigned short)0 : reinterpret_cast<const unsigned short*>(as)[min(r, m - 1)];
    const int entry_in_wave = lane >> 2, quarter = lane & 3;
    const int entry = wave * 16 + entry_in_wave;  // 16 waves x 16 entries
    uint32_t selector = book[entry];
    uint2 raw[MR];
    uint4 raw_x16 = make_uint4(0u, 0u, 0u, 0u);
    uint2 sign_bytes = make_uint2(0u, 0u);
    if (X16) {
        raw_x16 = *reinterpret_cast<const uint4*>(reinterpret_cast<const __half*>(a) + 8 * min(tid, groups - 1));
        if (signs != nullptr) sign_bytes = *reinterpret_cast<const uint2*>(signs + 8 * min(tid, groups - 1));
    } else
#pragma unroll
        for (int r = 0; r < MR; ++r)  // unconditional, clamped: a predicated load would be waited for at once
            raw[r] = *reinterpret_cast<const uint2*>(a + (int64_t)min(r, m - 1) * k + 8 * min(tid, groups - 1));
    // The first chunks of the stream are requested in two instalments (when the small reads are back,
    // and after the barrier) rather than all at once: a workgroup's full ring is 80 KiB, and the small
    // reads of workgroups that start later would wait behind the bursts of the early ones.
    const char* first_base = base_of(first_task);
    const uint32_t first_offset = lane_offset(first_task);
    auto prefetch = [&](int from, int to) {
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (d >= from && d < to) ring[d] = fetch(first_base, first_offset, d);
    };
    // Lane `quarter` of a quad makes byte `quarter` of the entry's word (coordinates quarter and
    // quarter + 4 share that byte); two quad swaps OR the four bytes together.  Every lane then
    // writes four of the entry's sixteen 16-byte pieces, rotated by the entry so that the 64
    // lanes of one write spread over all banks.
    auto quad_or = [](uint32_t v) {
        v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);
        v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);
        return v;
    };
    auto replicate = [&](uint32_t table_byte_base, uint32_t value) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t piece = (uint32_t)(entry_in_wave + 4 * quarter + i) & 15u;
            *reinterpret_cast<uint4*>(reinterpret_cast<char*>(lds) + table_byte_base + entry * 256 + piece * 16) =
                make_uint4(value, value, value, value);
        }
    };
    {   // mask table: needs no load, built while the reads are in flight
        const uint32_t u = (uint32_t)entry;
        const uint32_t parity = __popc(u) & 1u, flips = u ^ parity;
        const uint32_t low = (sign_bit(flips, quarter) ? 0xEu : 0u) ^ parity;
        const uint32_t high = (sign_bit(flips, quarter + 4) ? 0xEu : 0u) ^ parity;
        replicate(kMskBase, quad_or((low | high << 4) << (8 * quarter)));
    }
    // First use of a loaded value.  The empty statements pin that use here: without them the
    // compiler schedules the basis words ahead of the mask table and waits for the read at once.
    asm volatile("" : "+v"(selector));
    if (!X16) {
#pragma unroll
        for (int r = 0; r < MR; ++r) asm volatile("" : "+v"(raw[r].x), "+v"(raw[r].y));
    }
    // The wave's small reads are back: two chunks of the stream go out now and are in flight while the
    // tables are built (measured against one chunk just before the barrier: 6.8 -> 6.4 us at N=9728,
    // K=2560, 13.4 -> 12.8 us for the fp16-input form at N=17408, K=5120).  Earlier, or more of them,
    // and the small reads of workgroups that start later wait behind the bursts in the L2 queues
    // (set-up data back after 2.1-3.9 us instead of 1.2-2.0 us) and nothing is gained.
    prefetch(0, 2);
    {
        const uint32_t low = (uint32_t)selector_half(selector, quarter) & 15u;
        const uint32_t high = (uint32_t)selector_half(selector, quarter + 4) & 15u;
        replicate(0u, quad_or((low | high << 4) << (8 * quarter)));
    }
    if (X16) {
        // row maximum: per thread, per wave, then over the 16 waves through LDS (one more barrier)
        float* wave_max = reinterpret_cast<float*>(wave_sums + 3 * 16);  // the fourth row of sums is unused with one row
        const __half* h = reinterpret_cast<const __half*>(&raw_x16);
        // Waves past the end of the row (K / 8 pieces, one per thread) skip the per-value work: with
        // four waves per SIMD in the same phase, their instructions would take issue slots from the rest.
        const bool wave_live = __builtin_amdgcn_readfirstlane(wave) * 64 < groups;
        float value[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) value[j] = wave_live ? __half2float(h[j]) : 0.f;
        if (signs != nullptr && wave_live) {
            // Signed block-128 rotation in front of the quantiser (kernels/cuda/model/rotation_a8.py:188-224):
            // a block is the 8 values of each of 16 adjacent threads, so distances 1, 2 and 4 are inside
            // the thread and 8..64 are lane exchanges at distance 1..8 inside a row of 16 lanes.  Every
            // stage is one fp32 add or subtract in the reference's order; then one multiply by
            // fp32(128^-1/2) and the fp16 boundary.
#pragma unroll
            for (int j = 0; j < 8; ++j)
                value[j] *= (float)(int8_t)((j < 4 ? sign_bytes.x : sign_bytes.y) >> (8 * (j & 3)));
#pragma unroll
            for (int distance = 1; distance < 8; distance <<= 1) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if (j & distance) continue;
                    const float left = value[j], right = value[j + distance];
                    value[j] = left + right;
                    value[j + distance] = left - right;
                }
            }
#pragma unroll
            for (int bit = 0; bit < 4; ++bit) {
                const uint32_t flip = ((uint32_t)(lane >> bit) & 1u) << 31;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int own = __float_as_int(value[j]);
                    int partner;
                    if (bit == 0)
                        partner = __builtin_amdgcn_update_dpp(0, own, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
                    else if (bit == 1)
                        partner = __builtin_amdgcn_update_dpp(0, own, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
                    else if (bit == 2) {
                        partner = __builtin_amdgcn_update_dpp(own, own, 0x104, 0xF, 0x5, false);      // row_shl:4, banks 0, 2
                        partner = __builtin_amdgcn_update_dpp(partner, own, 0x114, 0xF, 0xA, false);  // row_shr:4, banks 1, 3
                    } else
                        partner = __builtin_amdgcn_update_dpp(0, own, 0x128, 0xF, 0xF, true);  // row_ror:8
                    value[j] = __int_as_float(partner) + __int_as_float(own ^ (int)flip);
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float scaled = value[j] * 0.08838834764831845f;
                asm volatile("" : "+v"(scaled));  // the fp16 cast rounds the fp32 product, not a fused multiply-convert
                value[j] = __half2float(__float2half_rn(scaled));
            }
        }
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (tid < groups) amax = fmaxf(amax, fabsf(value[j]));
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
        if (lane == 0) wave_max[wave] = amax;
        __syncthreads();
        // the 16 wave maxima, one per lane of a row, reduced with lane controls (no LDS round trips):
        // quad permutes, then the mirror of each half row, then the mirror of the row
        amax = wave_max[lane & 15];
        amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0xB1, 0xF, 0xF, true)));
        amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x4E, 0xF, 0xF, true)));
        amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x141, 0xF, 0xF, true)));
        amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(amax), 0x140, 0xF, 0xF, true)));
        const float raw_scale = fmaxf(__fdiv_rn(amax, 127.0f), 5.9604644775390625e-08f);
        const __half stored = amax > 0.f ? __float2half_rn(raw_scale) : __float2half_rn(1.0f);
        as_bits[0] = __half_as_ushort(stored);
        if (blockIdx.x == 0 && tid == 0) *const_cast<__half*>(as) = stored;
        const float scale = __half2float(stored);
        const float inverse = __builtin_amdgcn_rcpf(scale);  // within one unit in the last place: inside the margin below
        // the product with the reciprocal decides, except within 2^-14 of a tie, where the correctly
        // rounded quotient does (the product is within 2^-15 of the quotient)
        uint32_t packed[2] = {0u, 0u};
        if (wave_live) {
            float r[8];
            float farthest = 0.f;  // a product is at most 0.5 from its rounded value: 0.5 at a tie
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float guess = value[j] * inverse;
                r[j] = rintf(guess);
                farthest = fmaxf(farthest, fabsf(guess - r[j]));
            }
            if (farthest > 0.49993896484375f) {
#pragma unroll
                for (int j = 0; j < 8; ++j) r[j] = rintf(__fdiv_rn(value[j], scale));
            }
            // clamped integer + 1.5 * 2^23: the low byte of the word is the int8 code
            uint32_t word[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) word[j] = __float_as_uint(__builtin_amdgcn_fmed3f(r[j], -127.f, 127.f) + 12582912.0f);
#pragma unroll
            for (int half = 0; half < 2; ++half)
                packed[half] = __builtin_amdgcn_perm(word[4 * half + 1], word[4 * half], 0x0C0C0400u) |
                               (__builtin_amdgcn_perm(word[4 * half + 3], word[4 * half + 2], 0x0C0C0400u) << 16);
        }
        raw[0] = make_uint2(packed[0], packed[1]);
    }
    int wave_total[MR];  // sum of this wave's activations, valid in lane 63
#pragma unroll
    for (int r = 0; r < MR; ++r) wave_total[r] = 0;
    auto add_groups = [&](const uint2 (&v)[MR], int g) {
        uint32_t any_overflow = 0;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const bool live = r < m && g < groups;
            const uint32_t x = live ? v[r].x : 0u, y = live ? v[r].y : 0u;
            // bytewise a + 8 (no carry between bytes); its high nibble is hi
            const uint32_t x8 = ((x & 0x7F7F7F7Fu) + 0x08080808u) ^ (x & 0x80808080u);
            const uint32_t y8 = ((y & 0x7F7F7F7Fu) + 0x08080808u) ^ (y & 0x80808080u);
            // bit 7 of a byte set iff 120 <= a <= 127, i.e. (a & 0xF8) == 0x78
            const uint32_t xd = (x ^ 0x78787878u) & 0xF8F8F8F8u, yd = (y ^ 0x78787878u) & 0xF8F8F8F8u;
            const uint32_t xo = ~(((xd & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | xd) & 0x80808080u;
            const uint32_t yo = ~(((yd & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | yd) & 0x80808080u;
            const uint32_t over = (xo >> 7) | (yo >> 3);
            if (live) {
                // coordinates 0..3 to even nibble slots, 4..7 to odd slots
                hi[r * groups + g] = ((x8 >> 4) & 0x0F0F0F0Fu) | (y8 & 0xF0F0F0F0u);
                lo[r * groups + g] = (x & 0x0F0F0F0Fu) | ((y << 4) & 0xF0F0F0F0u);
                ov[r * groups + g] = over;
            }
            any_overflow |= over;
            wave_total[r] += wave_sum_to_last_lane(sdot4(x, 0x01010101u, sdot4(y, 0x01010101u, 0)));
        }
        // one byte per chunk (4 groups = one quad of threads): does it hold an overflow?
        any_overflow = quad_or(any_overflow);
        if (quarter == 0 && g < groups) chunk_flags[g >> 2] = any_overflow ? 1 : 0;
    };
    // wave-uniform trip count; the first pass uses the groups read above, longer rows (K > 8192) loop
    if (__builtin_amdgcn_readfirstlane(wave) * 64 < groups) add_groups(raw, tid);
    for (int g = kBankedThreads + tid; g - lane < groups; g += kBankedThreads) {
        uint2 more[MR];
#pragma unroll
        for (int r = 0; r < MR; ++r)
            more[r] = *reinterpret_cast<const uint2*>(a + (int64_t)min(r, m - 1) * k + 8 * min(g, groups - 1));
        add_groups(more, g);
    }
    if (lane == 63) {
#pragma unroll
        for (int r = 0; r < MR; ++r) wave_sums[r * 16 + wave] = wave_total[r];
    }
    __syncthreads();
    prefetch(2, D);

    const uint32_t column = kMskBase + 4u * (uint32_t)lane;
    // sum of each activation row (scalar), the steps at which this lane's column holds an
    // overflow, and (scalar) the steps at which any column of the wave does
    int row_sum[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r)
        row_sum[r] = __builtin_amdgcn_readlane(wave_sum_to_last_lane(lane < 16 ? wave_sums[r * 16 + lane] : 0), 63);
    uint32_t flag_lo = 0, flag_hi = 0;
    for (int step = 0; step < steps; ++step) {
        const uint32_t bit = chunk_flags[sub + step * LPR];
        if (step < 32) flag_lo |= bit << step; else flag_hi |= bit << (step - 32);
    }
    const uint64_t flagged = (uint64_t)flag_lo | (uint64_t)flag_hi << 32;
    const uint64_t any_flagged = (uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)wave_or_to_last_lane(flag_lo), 63) |
                                 (uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)wave_or_to_last_lane(flag_hi), 63) << 32;
    int acc_h0[MR], acc_l0[MR], acc_h1[MR], acc_l1[MR], acc_o0[MR], acc_o1[MR];
    static_assert(!HOLD || MR == 1, "held planes are for a single activation row");
    uint4 held_h[HOLD ? D : 1], held_l[HOLD ? D : 1];
    if (HOLD) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            held_h[d] = *reinterpret_cast<const uint4*>(planes + 4 * (sub + d * LPR));
            held_l[d] = *reinterpret_cast<const uint4*>(planes + groups + 4 * (sub + d * LPR));
        }
    }
    // One 16-byte chunk = 4 codes (coarse code in the low half, residual code in the high half) of
    // 8 weights each, against every activation row.  `slot` is the chunk's ring slot.
    auto consume = [&](const uint4& cur, int j, int step, int slot) {
        const uint32_t word[4] = {cur.x, cur.y, cur.z, cur.w};
        uint32_t v0[4], v1[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v0[i] = banked_lookup(word[i], column, kSelNib1) ^ banked_lookup(word[i], column, kSelMsk0);
            v1[i] = banked_lookup(word[i], column, kSelNib3) ^ banked_lookup(word[i], column, kSelMsk2);
        }
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const uint4 ph = HOLD ? held_h[slot] : *reinterpret_cast<const uint4*>(planes + r * groups + 4 * j);
            const uint4 pl = HOLD ? held_l[slot] : *reinterpret_cast<const uint4*>(planes + (MR + r) * groups + 4 * j);
            const uint32_t h[4] = {ph.x, ph.y, ph.z, ph.w}, l[4] = {pl.x, pl.y, pl.z, pl.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc_h0[r] = sdot8(v0[i], h[i], acc_h0[r]);
                acc_l0[r] = sdot8(v0[i], l[i], acc_l0[r]);
                acc_h1[r] = sdot8(v1[i], h[i], acc_h1[r]);
                acc_l1[r] = sdot8(v1[i], l[i], acc_l1[r]);
            }
        }
        if ((any_flagged >> step) & 1)  // scalar test first: almost every step skips the vector one
            if ((flagged >> step) & 1) {
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                const uint4 po = *reinterpret_cast<const uint4*>(planes + (2 * MR + r) * groups + 4 * j);
                const uint32_t o[4] = {po.x, po.y, po.z, po.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc_o0[r] = sdot8(v0[i], o[i], acc_o0[r]);
                    acc_o1[r] = sdot8(v1[i], o[i], acc_o1[r]);
                }
            }
        }
    };

    for (int task = first_task; task < tasks; task += task_stride) {
        const int row = task * kRows + row_in_wave;
        const bool live = row < n;
        const char* base = base_of(task);
        const char* next_base = base_of(task + task_stride);
        const uint32_t offset = lane_offset(task), next_offset = lane_offset(task + task_stride);
        // older than this row's refills, so it has landed long before the epilogue reads it
        const unsigned short ws_bits = reinterpret_cast<const unsigned short*>(ws)[min(row, n - 1)];
#pragma unroll
        for (int r = 0; r < MR; ++r) acc_h0[r] = acc_l0[r] = acc_h1[r] = acc_l1[r] = acc_o0[r] = acc_o1[r] = 0;
        for (int group = 0; group < padded; group += D) {
            // the last group of a row refills the ring with the first chunks of the wave's next row
            const bool last = group + D >= padded;
            const char* refill = last ? next_base : base;
            const uint32_t refill_offset = last ? next_offset : offset;
            const int refill_step = last ? 0 : group + D;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                // consume, then refill the same registers: a refill issued first would need a
                // second set of registers and a copy per group
                if (group + d < steps) consume(ring[d], sub + (group + d) * LPR, group + d, d);
                ring[d] = fetch(refill, refill_offset, refill_step + d);
            }
        }
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            // w = 4*q0 + q1 = 8*v0 + 2*v1 + 5 and a = 16*hi + lo + 256*ov
            int total = 8 * (16 * acc_h0[r] + acc_l0[r] + 256 * acc_o0[r]) + 2 * (16 * acc_h1[r] + acc_l1[r] + 256 * acc_o1[r]);
#pragma unroll
            for (int offset = LPR / 2; offset > 0; offset >>= 1) total += __shfl_xor(total, offset, 64);
            if (live && sub == 0 && r < m) {
                total += 5 * row_sum[r];
                const float value = rescale(total, __half2float(__ushort_as_half(ws_bits)),
                                            __half2float(__ushort_as_half(as_bits[r])));
                if (out_f32)
                    reinterpret_cast<float*>(out)[(int64_t)r * stride + row] = value;
                else
                    reinterpret_cast<__half*>(out)[(int64_t)r * stride + row] = __float2half_rn(value);
            }
        }
    }
}

// ---- host side -----------------------------------------------------------------------------
// slots: N, K, stride, capacity, block_m (= passes), flags (= codec), out_f32
int device_cus() { return device_compute_units(); }

uint32_t gemv_lds_bytes(const orx_function& f, int mr) {
    const uint32_t planes = f.flags == kW8 ? (uint32_t)mr * f.K : (uint32_t)mr * (f.K / 8) * 8;
    return planes;
}

int mr_for(int rows) { return rows <= 1 ? 1 : rows <= 2 ? 2 : 4; }

// The bank-replicated variant is chosen per launch: it needs its planes to fit beside the 128 KiB
// of tables, so a variant can run it for 1 row and the compact kernel for 4.  f.slots packs its
// shape: ring depth | lanes per row << 8 (0 = compact-table kernel only).
constexpr uint32_t kLdsLimit = 160 * 1024 - 4096;   // compact-table kernel: its static tables take part of the 160 KiB
constexpr uint32_t kBankedLdsLimit = 160 * 1024;    // replicated-table kernel: dynamic LDS only
uint32_t banked_lds_bytes(const orx_function& f, int mr) {
    // tables, 3 planes, wave sums, one flag byte per chunk (rounded up to 16)
    return kBankedPlanes + (uint32_t)mr * (f.K / 8) * 12 + 4 * 16 * 4 + (((uint32_t)f.K / 32 + 15) & ~15u);
}
bool use_banked(const orx_function& f, int mr) {
    return f.slots > 0 && f.flags == kQ4 && banked_lds_bytes(f, mr) <= kBankedLdsLimit;
}

int gemv_geometry(const orx_function& f, int rows, Geometry* g) {
    const int mr = mr_for(rows);
    if (use_banked(f, mr)) {
        const uint32_t lanes_per_row = ((uint32_t)f.slots >> 8) & (uint32_t)(kKMajorLayout - 1);
        const uint32_t tasks = ceil_div((uint32_t)f.N, 64u / lanes_per_row);
        // every CU gets a workgroup as soon as there is a task for each: a small matrix then runs with
        // some idle waves per CU rather than with idle CUs
        g->grid[0] = std::min<uint32_t>((uint32_t)device_cus(), tasks);
        g->block[0] = kBankedThreads;
        g->shared = banked_lds_bytes(f, mr);
        return ORX_OK;
    }
    g->grid[0] = ceil_div((uint32_t)f.N, (uint32_t)(kRowsPerPass * f.block_m));
    g->block[0] = kThreads;
    g->shared = gemv_lds_bytes(f, mr);
    return ORX_OK;
}

// Sign vector of the rotation that the fp16-input form applies in front of its quantiser (null: none);
// set by gemv_launch for the launch it is about to make on this thread.
static thread_local const int8_t* pending_signs = nullptr;

template <int D, int LPR>  // LPR: the kernel's LAYOUT (lanes per row, + 64 for K-major codes)
int gemv_launch_banked(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                       const uint4* w, const uint32_t* book, const __half* ws, const __half* as, void* out) {
    const dim3 grid(g.grid[0]), block(kBankedThreads);
    const bool hold = f.K / 32 / (LPR & (kKMajorLayout - 1)) == D;  // a row's steps fill the ring exactly
    switch (mr_for(rows)) {
        case 1:
            if (f.input_f16 && hold)
                ORX_LAUNCH((gemv_banked_kernel<kQ4, 1, D, LPR, true, true>), grid, block, g.shared, stream, a, w,
                                   book, ws, as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            else if (f.input_f16)
                ORX_LAUNCH((gemv_banked_kernel<kQ4, 1, D, LPR, false, true>), grid, block, g.shared, stream, a, w,
                                   book, ws, as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            else if (hold)
                ORX_LAUNCH((gemv_banked_kernel<kQ4, 1, D, LPR, true>), grid, block, g.shared, stream, a, w, book,
                                   ws, as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            else
                ORX_LAUNCH((gemv_banked_kernel<kQ4, 1, D, LPR, false>), grid, block, g.shared, stream, a, w, book,
                                   ws, as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            break;
        case 2:
            ORX_LAUNCH((gemv_banked_kernel<kQ4, 2, D, LPR, false>), grid, block, g.shared, stream, a, w, book, ws,
                               as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            break;
        default:
            ORX_LAUNCH((gemv_banked_kernel<kQ4, 4, D, LPR, false>), grid, block, g.shared, stream, a, w, book, ws,
                               as, out, f.N, f.K, f.stride, rows, (int)f.out_f32 | (f.packed_k == 64 ? 2 : 0), pending_signs);
            break;
    }
    return hip_check(hipGetLastError(), "launch projection (gemv, replicated tables)");
}

template <int LPR>
int gemv_launch_banked_depth(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                             const uint4* w, const uint32_t* book, const __half* ws, const __half* as, void* out) {
    switch (f.slots & 255) {
        case 4: return gemv_launch_banked<4, LPR>(f, rows, g, stream, a, w, book, ws, as, out);
        case 5: return gemv_launch_banked<5, LPR>(f, rows, g, stream, a, w, book, ws, as, out);
        default: return gemv_launch_banked<6, LPR>(f, rows, g, stream, a, w, book, ws, as, out);
    }
}

template <int CODEC>
int gemv_launch_codec(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                      const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out) {
    const dim3 grid(g.grid[0]), block(kThreads);
    const uint4* wp = reinterpret_cast<const uint4*>(w);
    if constexpr (CODEC == kQ4) {
        if (use_banked(f, mr_for(rows))) {
            switch (f.slots >> 8) {
                case 32: return gemv_launch_banked_depth<32>(f, rows, g, stream, a, wp, book, ws, as, out);
                case kKMajorLayout + 16: return gemv_launch_banked_depth<kKMajorLayout + 16>(f, rows, g, stream, a, wp, book, ws, as, out);
                case kKMajorLayout + 8: return gemv_launch_banked_depth<kKMajorLayout + 8>(f, rows, g, stream, a, wp, book, ws, as, out);
                default: return gemv_launch_banked_depth<16>(f, rows, g, stream, a, wp, book, ws, as, out);
            }
        }
    }
    switch (mr_for(rows)) {
        case 1:
            ORX_LAUNCH((gemv_rowmajor_kernel<CODEC, 1>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
        case 2:
            ORX_LAUNCH((gemv_rowmajor_kernel<CODEC, 2>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
        default:
            ORX_LAUNCH((gemv_rowmajor_kernel<CODEC, 4>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
    }
    return hip_check(hipGetLastError(), "launch projection (gemv)");
}


// ---- single-token expert routes (kernels/cuda/model/integer_vq.py:380-444) ---------------------
//
// Every route indexes its expert's bank directly: no sorting, no tile list.  Book is the raw table
// as (256, 2) u32 (vq.py:199-204): eight signed even bytes per entry, any values (the reference's
// test draws random tables, tests/cuda/operators/flash_mtp_optimization.py:133), so the decode is
// the general one: byte j of the quad is +-table[b][j] by sign bit j of (u ^ parity), plus one for
// even parity, minus one for odd (vq.py:34-43).  The table is only assumed to hold bytes whose
// negation fits int8 (the reference's tables are even, within +-126).
//
// One workgroup per (route, 32 output channels).  P is (E, K/128, N, 16) u16, so the 32 channels of
// one K block are 1 KiB of consecutive codes: a wave reads them with one 16-byte load per lane
// (lane = channel * 2 + half of the block), the eight waves take K blocks round robin.  The token row
// is staged in LDS once; lanes of one half read the same 64 bytes from it (broadcast).

constexpr uint32_t kHighBits = 0x80808080u, kLowBits = 0x7f7f7f7fu;

// per byte: 0 - b, without carries between bytes
__device__ __forceinline__ uint32_t negate_bytes(uint32_t b) { return (kHighBits - (b & kLowBits)) ^ (~b & kHighBits); }

// byte masks of the coordinates whose sign bit is set: bits 0, 4, 1, 5 of `signs` (vq.py:17)
__device__ __forceinline__ uint32_t sign_mask(uint32_t signs) {
    const uint32_t flags = (signs & 1u) | ((signs & 16u) << 4) | ((signs & 2u) << 15) | ((signs & 32u) << 19);
    return flags * 255u;
}

constexpr int kRouteChannels = 32, kRouteWaves = 8, kRouteThreads = 64 * kRouteWaves, kRouteDepth = 2;
constexpr int kRouteTableBytes = 256 * 16, kRouteMaskBytes = 256 * 8, kRoutePartialBytes = kRouteWaves * kRouteChannels * 4;

// The decode is split so that the inner loop is two table reads and two selects per code:
//   q[j] = +-t[j] + c,  c = 1 - 2 * parity   =>   a . q = a . (+-t) + c * sum(a)
// with +-t picked per byte between the table entry and its negation (both prepared per entry at
// set-up), the byte masks of u prepared per u, and the sums of every 8 token bytes prepared once.
//
// Two launches of the one-token expert layer can run inside this kernel's set-up:
//   LOCAL > 0 (route_logits): `ids` is an output.  Wave 0 of every workgroup selects the token's
//     routes from `logits` (the router's rule, moe_device.h) while the others build the tables; the
//     first workgroup writes ids and probabilities for the combine.  Selecting eight routes of one
//     token costs a wave about a microsecond; a router launch in front costs three to four.
//   x16 == 2 (fused_swiglu): `a` holds fp16 gate|up rows, one per route; the row becomes
//     fp16(silu(gate) * up), then A8 codes, on its way into LDS (the SwiGLU -> A8 launch between the
//     two projections disappears); the first workgroup of a route writes its scale.
template <int LOCAL>
__global__ __launch_bounds__(kRouteThreads) void route_gemv_kernel(
    const int8_t* __restrict__ a, const __half* __restrict__ as, const uint32_t* __restrict__ book, __half* __restrict__ c,
    const int32_t* __restrict__ ids, const uint16_t* __restrict__ p, const __half* __restrict__ ws, int experts, int n,
    int k, int shared_input, int x16, const float* __restrict__ logits, float* __restrict__ prob, int renormalize) {
    extern __shared__ __align__(16) uint8_t route_lds[];
    __shared__ float route_wave_max[kRouteWaves];
    __shared__ int selected_ids[64];
    __shared__ float selected_prob[64];
    uint4* table = reinterpret_cast<uint4*>(route_lds);                                    // entry, negated entry
    uint2* masks = reinterpret_cast<uint2*>(route_lds + kRouteTableBytes);                  // per u
    int* partial = reinterpret_cast<int*>(route_lds + kRouteTableBytes + kRouteMaskBytes);  // [waves][channels]
    uint4* token = reinterpret_cast<uint4*>(route_lds + kRouteTableBytes + kRouteMaskBytes + kRoutePartialBytes);
    int* token_sums = reinterpret_cast<int*>(reinterpret_cast<uint8_t*>(token) + k);        // k / 8 sums
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int route = blockIdx.y;
    const int routes = (int)gridDim.y;
    int expert = LOCAL > 0 ? 0 : ids[route];
    if (LOCAL == 0 && (unsigned)expert >= (unsigned)experts) return;  // nothing to index: the row stays as it was
    const int row = shared_input ? 0 : route;
    const int blocks = k / 128;
    const int channel = blockIdx.x * kRouteChannels + (lane >> 1);
    const int half = lane & 1;
    const bool live = channel < n;
    // codes of this lane: 16 bytes per K block, K blocks wave, wave + 8, ...; the first kRouteDepth
    // loads leave before anything else (once the expert is known)
    const int64_t block_stride = (int64_t)n * 2;  // uint4 per K block
    const uint4* codes = nullptr;
    uint4 held[kRouteDepth];
    auto request_codes = [&]() {
        codes = reinterpret_cast<const uint4*>(p + (((int64_t)expert * blocks) * n + (live ? channel : 0)) * 16) + half;
#pragma unroll
        for (int d = 0; d < kRouteDepth; ++d) {
            const int kb = wave + d * kRouteWaves;
            held[d] = kb < blocks ? codes[kb * block_stride] : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    if (LOCAL == 0) request_codes();
    if (LOCAL > 0 && wave == 0) select_routes<LOCAL == 0 ? 1 : LOCAL>(logits, selected_ids, selected_prob, 0, experts, routes, renormalize, lane);
    if (tid < 256) {
        const uint2 entry = reinterpret_cast<const uint2*>(book)[tid];
        table[tid] = make_uint4(entry.x, entry.y, negate_bytes(entry.x), negate_bytes(entry.y));
    } else {
        const uint32_t u = tid - 256;
        const uint32_t signs = u ^ (__popc(u) & 1u);
        masks[u] = make_uint2(sign_mask(signs), sign_mask(signs >> 2));
    }
    float row_scale = 0.f;  // x16: fp32 value of the row's fp16 scale
    // the routes are known after the next barrier (the one of the row maximum where there is one)
    auto routes_published = [&]() {
        if (LOCAL == 0) return;
        expert = selected_ids[route];
        request_codes();
        if (blockIdx.x == 0 && blockIdx.y == 0 && tid < routes) {
            const_cast<int32_t*>(ids)[tid] = selected_ids[tid];
            prob[tid] = selected_prob[tid];
        }
    };
    if (x16) {
        // `a` is an fp16 row (the shared token row, or with x16 == 2 this route's gate|up row, which
        // first becomes fp16(silu(gate) * up)): every workgroup quantises it by the A8 rule (row maximum
        // over 127, fp16 scale, round to nearest even) on its way into LDS; the first one also writes
        // the scale.  Up to 4 pieces of 8 values per thread (K <= 16384) stay in registers between the
        // two passes.
        const bool swiglu_rows = x16 == 2;
        const __half* x = reinterpret_cast<const __half*>(a) + (swiglu_rows ? (int64_t)route * 2 * k : 0);
        uint4 kept[4];
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = tid + j * kRouteThreads;
            kept[j] = make_uint4(0u, 0u, 0u, 0u);
            if (i < k / 8) {
                kept[j] = reinterpret_cast<const uint4*>(x)[i];
                if (swiglu_rows) {
                    const uint4 up_bits = reinterpret_cast<const uint4*>(x + k)[i];
                    __half* gate = reinterpret_cast<__half*>(&kept[j]);
                    const __half* up = reinterpret_cast<const __half*>(&up_bits);
#pragma unroll
                    for (int e = 0; e < 8; ++e) gate[e] = __float2half_rn(swiglu_value(gate[e], up[e]));
                }
            }
            const __half2* pairs = reinterpret_cast<const __half2*>(&kept[j]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float2 f = __half22float2(pairs[e]);
                amax = fmaxf(amax, fmaxf(fabsf(f.x), fabsf(f.y)));
            }
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
        if (lane == 0) route_wave_max[wave] = amax;
        __syncthreads();
        routes_published();
        amax = route_wave_max[0];
#pragma unroll
        for (int w = 1; w < kRouteWaves; ++w) amax = fmaxf(amax, route_wave_max[w]);
        const __half stored = a8_scale(amax);
        if (blockIdx.x == 0 && (swiglu_rows || blockIdx.y == 0) && tid == 0) const_cast<__half*>(as)[swiglu_rows ? route : 0] = stored;
        row_scale = __half2float(stored);
        const float inverse = __builtin_amdgcn_rcpf(row_scale);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = tid + j * kRouteThreads;
            if (i < k / 8) {
                const __half* h = reinterpret_cast<const __half*>(&kept[j]);
                const float low[4] = {__half2float(h[0]), __half2float(h[1]), __half2float(h[2]), __half2float(h[3])};
                const float high[4] = {__half2float(h[4]), __half2float(h[5]), __half2float(h[6]), __half2float(h[7])};
                const uint2 bytes = make_uint2(quantise4(low, row_scale, inverse), quantise4(high, row_scale, inverse));
                reinterpret_cast<uint2*>(token)[i] = bytes;
                token_sums[i] = __builtin_amdgcn_sdot4((int)bytes.y, 0x01010101, __builtin_amdgcn_sdot4((int)bytes.x, 0x01010101, 0, false), false);
            }
        }
    } else {
        if (LOCAL > 0) {
            __syncthreads();
            routes_published();
        }
        for (int i = tid; i < k / 8; i += kRouteThreads) {
            const uint2 bytes = reinterpret_cast<const uint2*>(a + (int64_t)row * k)[i];
            reinterpret_cast<uint2*>(token)[i] = bytes;
            token_sums[i] = __builtin_amdgcn_sdot4((int)bytes.y, 0x01010101, __builtin_amdgcn_sdot4((int)bytes.x, 0x01010101, 0, false), false);
        }
    }
    __syncthreads();
    int acc = 0;
    for (int first = wave; first < blocks; first += kRouteDepth * kRouteWaves) {
#pragma unroll
        for (int d = 0; d < kRouteDepth; ++d) {
            const int kb = first + d * kRouteWaves;
            if (kb >= blocks) break;  // wave-uniform
            const uint4 now = held[d];
            const int next = kb + kRouteDepth * kRouteWaves;
            if (next < blocks) held[d] = codes[next * block_stride];
            const uint32_t words[4] = {now.x, now.y, now.z, now.w};
            const uint4* fragment = token + kb * 8 + half * 4;                                  // 64 token bytes
            const int4* sums = reinterpret_cast<const int4*>(token_sums + kb * 16 + half * 8);  // of 8 codes
            const int4 sums_low = sums[0], sums_high = sums[1];
            const int sum_of[8] = {sums_low.x, sums_low.y, sums_low.z, sums_low.w, sums_high.x, sums_high.y, sums_high.z, sums_high.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 values = fragment[i];  // 16 token bytes: two codes
                const uint32_t pair[4] = {values.x, values.y, values.z, values.w};
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t code = (words[i] >> (16 * j)) & 0xffffu;
                    const uint32_t u = code & 255u;
                    const uint4 entry = table[code >> 8];
                    const uint2 mask = masks[u];
                    const uint32_t low = (entry.x & ~mask.x) | (entry.z & mask.x);
                    const uint32_t high = (entry.y & ~mask.y) | (entry.w & mask.y);
                    acc = __builtin_amdgcn_sdot4((int)pair[2 * j], (int)low, acc, false);
                    acc = __builtin_amdgcn_sdot4((int)pair[2 * j + 1], (int)high, acc, false);
                    acc += (__popc(u) & 1u) ? -sum_of[2 * i + j] : sum_of[2 * i + j];
                }
            }
        }
    }
    acc += __shfl_xor(acc, 1, 64);
    if (half == 0) partial[wave * kRouteChannels + (lane >> 1)] = acc;
    __syncthreads();
    if (tid < kRouteChannels) {
        const int out_channel = blockIdx.x * kRouteChannels + tid;
        if (out_channel < n) {
            int total = 0;
#pragma unroll
            for (int w = 0; w < kRouteWaves; ++w) total += partial[w * kRouteChannels + tid];
            const float token_scale = x16 ? row_scale : __half2float(as[row]);
            const float scaled = ((float)total * __half2float(ws[(int64_t)expert * n + out_channel])) * token_scale;
            c[(int64_t)route * n + out_channel] = __float2half_rn(scaled);
        }
    }
}

// slots used: E, M (routes), N, K, flags (bit0 shared_input)
int route_gemv_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = ceil_div((uint32_t)f.N, (uint32_t)kRouteChannels);
    g->grid[1] = (uint32_t)f.M;
    g->block[0] = kRouteThreads;
    g->shared = (uint32_t)(kRouteTableBytes + kRouteMaskBytes + kRoutePartialBytes) + (uint32_t)f.K + (uint32_t)f.K / 2;
    return ORX_OK;
}

// A, AS, Book, C, IDs, [Logits,] P, [Prob,] WS: the buffers of integer_vq.py:388-395 in generated-ABI order
// slots used: flags bit0 shared_input, bit1 fused_swiglu, bit2 route_logits, bit3 renormalize
int route_gemv_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    const bool routing = f.flags & 4;
    const int8_t* a = pointer_arg<const int8_t>(args, 0);
    const __half* as = pointer_arg<const __half>(args, 1);
    const uint32_t* book = pointer_arg<const uint32_t>(args, 2);
    __half* c = pointer_arg<__half>(args, 3);
    const int32_t* ids = pointer_arg<const int32_t>(args, 4);
    const float* logits = routing ? pointer_arg<const float>(args, 5) : nullptr;
    const uint16_t* p = pointer_arg<const uint16_t>(args, routing ? 6 : 5);
    float* prob = routing ? pointer_arg<float>(args, 7) : nullptr;
    const __half* ws = pointer_arg<const __half>(args, routing ? 8 : 6);
    const int x16 = f.input_f16 ? ((f.flags & 2) ? 2 : 1) : 0;
    const dim3 grid(g.grid[0], g.grid[1]), block(kRouteThreads);
#define ORX_ROUTE_GEMV(LOCAL)                                                                                      \
    ORX_LAUNCH(route_gemv_kernel<LOCAL>, grid, block, g.shared, stream, a, as, book, c, ids, p, ws, f.E, f.N, f.K, \
                       f.flags & 1, x16, logits, prob, (f.flags >> 3) & 1)
    if (!routing) ORX_ROUTE_GEMV(0);
    else if (f.E <= 64) ORX_ROUTE_GEMV(1);
    else if (f.E <= 128) ORX_ROUTE_GEMV(2);
    else if (f.E <= 256) ORX_ROUTE_GEMV(4);
    else ORX_ROUTE_GEMV(8);
#undef ORX_ROUTE_GEMV
    return hip_check(hipGetLastError(), "launch integer_e8p_gemv");
}

int make_route_gemv(const Variant& v, orx_function* f) {
    bool bad = false;
    f->E = (int)v.integer("E", 0, &bad);
    f->capacity = f->M = (int)v.integer("routes", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    const bool shared_input = v.boolean("shared_input", false, &bad);
    const long long block_n = v.integer("block_n", 8, &bad);  // the reference's tile hint: accepted, not used
    if (bad || !v.has("shared_input")) {
        set_error("integer_e8p_gemv: needs E, routes, N, K and shared_input");
        return ORX_ERR_BAD_VARIANT;
    }
    // integer_vq.py:382-383: K in whole 128-blocks, int32-exact dots, block_n in (4, 8, 16)
    if (f->E <= 0 || f->M <= 0 || f->N <= 0 || f->K <= 0 || f->K % 128 || (long long)f->K * 128 * 128 >= (1ll << 31) ||
        (block_n != 4 && block_n != 8 && block_n != 16) || f->K > 65536) {
        set_error("integer_e8p_gemv: need E, routes, N > 0, K a multiple of 128 with K*128*128 < 2^31, block_n in 4|8|16");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = shared_input ? 1 : 0;
    // input_dtype=float16: A is fp16 and AS is written, not read.  With shared_input it is the one token row,
    // quantised by every workgroup on its way into LDS; with fused_swiglu (no shared input) it holds one
    // gate|up row of 2K values per route, which becomes fp16(silu(gate) * up) and then A8 codes.
    const std::string input = v.string("input_dtype", "int8", &bad);
    const bool fused_swiglu = v.boolean("fused_swiglu", false, &bad);
    if (bad || (input != "int8" && input != "float16") || (input == "float16" && f->K > 16384) ||
        (input == "float16" && shared_input == fused_swiglu) || (fused_swiglu && input != "float16")) {
        set_error("integer_e8p_gemv: input_dtype must be int8 or float16 (float16: the shared row, or with fused_swiglu "
                  "one gate|up row per route; K up to 16384)");
        return ORX_ERR_BAD_VARIANT;
    }
    f->input_f16 = input == "float16";
    if (fused_swiglu) f->flags |= 2;
    // route_logits=true: IDs is written, not read: every workgroup selects the token's `routes` routes from
    // Logits (1, E) by the router's rule, the first one writes IDs and Prob (renormalize as router_topk)
    const bool route_logits = v.boolean("route_logits", false, &bad);
    const bool renormalize = v.boolean("renormalize", true, &bad);
    if (bad || (route_logits && (f->E > 512 || f->M > 64 || f->M > f->E))) {
        set_error("integer_e8p_gemv: route_logits needs E <= 512 and routes <= min(E, 64)");
        return ORX_ERR_BAD_VARIANT;
    }
    if (route_logits) f->flags |= 4 | (renormalize ? 8 : 0);
    // 16-byte loads of A rows and P, 8-byte loads of Book
    f->args = {{"A", ArgPointer, 16}, {"AS", ArgPointer, 2}, {"Book", ArgPointer, 8}, {"C", ArgPointer, 2}, {"IDs", ArgPointer, 4}};
    if (route_logits) f->args.push_back({"Logits", ArgPointer, 4});
    f->args.push_back({"P", ArgPointer, 16});
    if (route_logits) f->args.push_back({"Prob", ArgPointer, 4});
    f->args.push_back({"WS", ArgPointer, 2});
    f->device_function = !route_logits  ? reinterpret_cast<const void*>(&route_gemv_kernel<0>)
                         : f->E <= 64  ? reinterpret_cast<const void*>(&route_gemv_kernel<1>)
                         : f->E <= 128 ? reinterpret_cast<const void*>(&route_gemv_kernel<2>)
                         : f->E <= 256 ? reinterpret_cast<const void*>(&route_gemv_kernel<4>)
                                       : reinterpret_cast<const void*>(&route_gemv_kernel<8>);
    f->geometry = route_gemv_geometry;
    f->launch = route_gemv_launch;
    return ORX_OK;
}

}  // namespace

int gemv_prepare_device();

// K-major two-stage codes are only served by the replicated-table kernel.
bool gemv_serves_k_major(const orx_function& f, int rows) {
    return f.flags == kQ4 && (f.packed_k == 128 || f.packed_k == 64) && ((uint32_t)f.slots >> 8) >= (uint32_t)kKMajorLayout && use_banked(f, mr_for(rows));
}

// Launchers used by the projection factories.  Argument order is the caller's business:
// they pass already-unmarshalled pointers.
int gemv_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out, const int8_t* signs) {
    // LDS opt-in needs a device, so it happens at the first launch rather than at resolve time
    const int ready = gemv_prepare_device();
    if (ready != ORX_OK) return ready;
    pending_signs = f.input_f16 ? signs : nullptr;
    if (f.packed_k != 0 && !gemv_serves_k_major(f, rows)) {
        set_error("%s: the gemv algorithm does not serve this K-major shape for %d rows", f.symbol.c_str(), rows);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f.flags == kQ4) return gemv_launch_codec<kQ4>(f, rows, g, stream, a, w, book, ws, as, out);
    if (f.flags == kQ2) return gemv_launch_codec<kQ2>(f, rows, g, stream, a, w, book, ws, as, out);
    return gemv_launch_codec<kW8>(f, rows, g, stream, a, w, book, ws, as, out);
}

int gemv_geometry_for(const orx_function& f, int rows, Geometry* g) { return gemv_geometry(f, rows, g); }

// The fp16-input form exists in the replicated-table kernel, one row, one 16-byte piece per thread.
bool gemv_serves_fp16_input(const orx_function& f) { return use_banked(f, 1) && f.K <= 8 * kBankedThreads; }

// Fills the gemv-specific slots.  codec: 0 Q4 (u32 codes), 1 Q2 (u16 codes), 2 W8.
int gemv_configure(orx_function* f, int codec, int passes_override) {
    if (f->capacity > 4) {
        set_error("%s: the gemv algorithm serves 1..4 rows, variant asks for %d", f->symbol.c_str(), f->capacity);
        return ORX_ERR_BAD_VARIANT;
    }
    const int unit = codec == kW8 ? 16 : codec == kQ2 ? 64 : 32;  // weights per 16-byte chunk
    if (f->K % unit || f->K % 8) {
        set_error("%s: gemv needs K to be a multiple of %d", f->symbol.c_str(), unit);
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = codec;
    int passes = passes_override;
    if (passes <= 0) {
        // one pass per workgroup keeps the most waves (and HBM requests) in flight; more passes
        // only pay off when N is so large that table rebuilds dominate
        passes = f->N / (kRowsPerPass * device_cus() * 16);
        if (passes < 1) passes = 1;
        if (passes > 8) passes = 8;
    }
    f->block_m = passes;
    // Shape of the replicated-table kernel (0 = compact-table kernel only, which an explicit
    // gemv_passes asks for): 32 or 16 lanes per row, whichever divides the row's chunk count (the
    // kernel keeps its step arithmetic scalar by assuming every lane owns the same number of
    // chunks), and the ring depth in {6,5,4} that pads a row's step count the least.
    f->slots = 0;
    if (passes_override <= 0 && codec == kQ4) {
        const int chunks = f->K / 2 / 16;
        int lanes_per_row = chunks % 32 == 0 ? 32 : chunks % 16 == 0 ? 16 : 0;
        // K-major codes: 16 lanes per row measure best (13.4 us at N=17408, K=5120 against 15.1 with 8
        // and 15.0 with 32), 8 for a K that is a multiple of 256 only
        if (f->packed_k != 0) lanes_per_row = chunks % 16 == 0 ? 16 : chunks % 8 == 0 ? 8 : 0;
        if (lanes_per_row) {
            const int steps = chunks / lanes_per_row;
            int best_pad = 1 << 30, depth = 4;
            for (int candidate : {6, 5, 4}) {
                const int pad = ceil_div(steps, candidate) * candidate - steps;
                if (pad < best_pad) best_pad = pad, depth = candidate;
            }
            // the overflow flags hold one bit per step in a 64-bit word per lane column
            if (steps <= 64) f->slots = depth | (lanes_per_row + (f->packed_k != 0 ? kKMajorLayout : 0)) << 8;
        }
    }
    if (gemv_lds_bytes(*f, 4) > kLdsLimit) {
        set_error("%s: K=%d does not fit the gemv activation planes in LDS", f->symbol.c_str(), f->K);
        return ORX_ERR_BAD_VARIANT;
    }
    f->device_function = reinterpret_cast<const void*>(&gemv_rowmajor_kernel<kQ4, 1>);
    return ORX_OK;
}

static int gemv_opt_in_current_device() {
    // Dynamic LDS above 64 KiB needs an opt-in per kernel (kernels.rs:171-190 does the same on CUDA).
    int limit = (int)kLdsLimit;  // the static tables take 2064 bytes of the 160 KiB
#define ORX_OPT_IN(kernel)                                                                                   \
    {                                                                                                        \
        int code = hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&kernel),                     \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, limit),        \
                             "hipFuncSetAttribute");                                                         \
        if (code != ORX_OK) return code;                                                                     \
    }
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ4, 1>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ4, 2>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ4, 4>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ2, 1>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ2, 2>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kQ2, 4>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kW8, 1>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kW8, 2>))
    ORX_OPT_IN((gemv_rowmajor_kernel<kW8, 4>))
    limit = (int)kBankedLdsLimit;
#define ORX_OPT_IN_BANKED(depth, lanes)                       \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 1, depth, lanes, true>))     \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 1, depth, lanes, false>))    \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 1, depth, lanes, true, true>))  \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 1, depth, lanes, false, true>)) \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 2, depth, lanes, false>))    \
    ORX_OPT_IN((gemv_banked_kernel<kQ4, 4, depth, lanes, false>))
    ORX_OPT_IN_BANKED(4, 16) ORX_OPT_IN_BANKED(5, 16) ORX_OPT_IN_BANKED(6, 16)
    ORX_OPT_IN_BANKED(4, 32) ORX_OPT_IN_BANKED(5, 32) ORX_OPT_IN_BANKED(6, 32)
    ORX_OPT_IN_BANKED(4, kKMajorLayout + 8) ORX_OPT_IN_BANKED(5, kKMajorLayout + 8) ORX_OPT_IN_BANKED(6, kKMajorLayout + 8)
    ORX_OPT_IN_BANKED(4, kKMajorLayout + 16) ORX_OPT_IN_BANKED(5, kKMajorLayout + 16) ORX_OPT_IN_BANKED(6, kKMajorLayout + 16)
#undef ORX_OPT_IN_BANKED
#undef ORX_OPT_IN
    return ORX_OK;
}

int gemv_prepare_device() {
    static DeviceOnce done;  // once per device, safe from several session threads
    return done.run(gemv_opt_in_current_device);
}

const Registration* gemv_registrations(int* count) {
    static const Registration rows[] = {
    {"integer_e8p_gemv", make_route_gemv,
     "E, routes, N, K, shared_input, block_n=8, input_dtype=int8|float16, fused_swiglu=false, route_logits=false, renormalize=true",
     "A,AS,Book,C,IDs[,Logits],P[,Prob],WS"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
