// MoE routing, dispatch and weighted combine around the grouped expert projections.
//
// Reference: kernels/cuda/model/moe.py -- router_topk (:413-494), expert_histogram (:177-210),
// expert_offsets (:214-244), expert_tiles (:248-282), expert_dispatch (:286-329),
// moe_combine (:498-554).  All metadata is int32, assignment order is token-major /
// rank-minor, and nothing here uses atomics: each output element has exactly one writer, so
// the result is deterministic and every kernel is replayable inside a captured graph.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "a8_device.h"
#include "moe_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

constexpr int kMaxLocal = 16;  // router keys per lane: E <= 1024

// The A8 quantiser of one row of fp16 values by one wave (the rule of a8_device.h).
__device__ __forceinline__ void wave_quantise_row(const __half* __restrict__ x, int8_t* __restrict__ q,
                                                  __half* __restrict__ s, int row, int h, int lane) {
    constexpr int kHeldPieces = 4;  // 16-byte pieces a lane keeps in registers (the whole row up to h = 2048)
    const int pieces = h / 8;
    const uint4* row_pieces = reinterpret_cast<const uint4*>(x + (int64_t)row * h);
    uint4 held[kHeldPieces];
#pragma unroll
    for (int i = 0; i < kHeldPieces; ++i) held[i] = row_pieces[min(lane + 64 * i, pieces - 1)];
    auto piece_at = [&](int i) { return i < kHeldPieces ? held[i] : row_pieces[lane + 64 * i]; };
    float amax = 0.f;
    for (int i = 0; lane + 64 * i < pieces; ++i) {
        const uint4 raw = piece_at(i);
        const __half2* pairs = reinterpret_cast<const __half2*>(&raw);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float2 f = __half22float2(pairs[j]);
            amax = fmaxf(amax, fmaxf(fabsf(f.x), fabsf(f.y)));
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
    const __half stored = a8_scale(amax);
    if (lane == 0) s[row] = stored;
    const float scale = __half2float(stored), inverse = __frcp_rn(scale);
    for (int i = 0; lane + 64 * i < pieces; ++i) {
        const uint4 raw = piece_at(i);
        const __half* v = reinterpret_cast<const __half*>(&raw);
        const float low[4] = {__half2float(v[0]), __half2float(v[1]), __half2float(v[2]), __half2float(v[3])};
        const float high[4] = {__half2float(v[4]), __half2float(v[5]), __half2float(v[6]), __half2float(v[7])};
        reinterpret_cast<uint2*>(q + (int64_t)row * h)[lane + 64 * i] =
            make_uint2(quantise4(low, scale, inverse), quantise4(high, scale, inverse));
    }
}

// QUANT (quantize_hidden): four more waves per workgroup quantise the same four tokens' hidden rows
// by the A8 rule while the first four select the routes (the expert projections gather these rows
// by slot, so a row is quantised once, not once per route, and it costs no launch of its own).
// With 16 keys per lane the selection wants more registers than a 512-thread workgroup leaves a
// wave, so there each wave quantises its own token's row after it has selected the routes.
template <int LOCAL, bool QUANT>
constexpr int router_threads() { return QUANT && LOCAL <= 8 ? 512 : 256; }
template <int LOCAL, bool QUANT>  // LOCAL keys per lane: ceil(E / 64) rounded up to a power of two
__global__ __launch_bounds__((router_threads<LOCAL, QUANT>())) void router_topk_kernel(
    const float* __restrict__ logits, int* __restrict__ ids, float* __restrict__ prob, int m, int e, int top_k,
    int renormalize, const __half* __restrict__ x, int8_t* __restrict__ q, __half* __restrict__ s, int h) {
    constexpr bool kQuantiserWaves = router_threads<LOCAL, QUANT>() == 512;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + (wave & 3);
    if (row >= m) return;
    if (kQuantiserWaves && wave >= 4) {
        wave_quantise_row(x, q, s, row, h, lane);
        return;
    }
    select_routes<LOCAL>(logits, ids, prob, row, e, top_k, renormalize, lane);
    if (QUANT && !kQuantiserWaves) wave_quantise_row(x, q, s, row, h, lane);
}

// Block-wide exclusive prefix of a 0/1 flag; returns this thread's prefix and the block total.
__device__ __forceinline__ int block_flag_scan(bool flag, int* wave_totals, int* total) {
    const unsigned long long ballot = __ballot(flag);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int within = __popcll(ballot & ((1ull << lane) - 1ull));
    __syncthreads();  // previous round's readers are done with wave_totals
    if (lane == 0) wave_totals[wave] = __popcll(ballot);
    __syncthreads();
    int before = 0, sum = 0;
    for (int w = 0; w < (int)(blockDim.x >> 6); ++w) {
        const int t = wave_totals[w];
        if (w < wave) before += t;
        sum += t;
    }
    *total = sum;
    return before + within;
}

// grid E: expert e scans every assignment in token-major order.
__global__ __launch_bounds__(256) void expert_histogram_kernel(const int* __restrict__ ids, int* __restrict__ counts,
                                                               int* __restrict__ relative, int assignments) {
    __shared__ int wave_totals[4];
    const int expert = blockIdx.x;
    int base = 0;
    for (int first = 0; first < assignments; first += 256) {
        const int i = first + threadIdx.x;
        const bool match = i < assignments && ids[i] == expert;
        int total;
        const int prefix = block_flag_scan(match, wave_totals, &total);
        if (match) relative[i] = base + prefix;
        base += total;
    }
    if (threadIdx.x == 0) counts[expert] = base;
}

// router_projection (kernels/cuda/model/moe.py:15-49): Logits[m, E] fp32 and SharedGate[m] fp16 = X[m, H] . W[E + 1, H]^T,
// fp16 operands, fp32 accumulation.  Floating point: the order of the additions is this kernel's own.
// grid (ceil(m / T), ceil((E + 1) / T)) with T = 16 up to 1024 rows and 32 above, eight waves: each takes an eighth of H,
// operands straight from global memory (a lane reads 16 contiguous bytes of its row), the eighths are added through LDS.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kProjectionWaves = 8;
constexpr int kProjectionSmallRows = 1024;  // up to here 16 x 16 tiles: four times the workgroups, each pulls half the rows
// TILE 32: v_mfma_f32_32x32x16_f16, a lane holds row (lane % 32) and 8 values of k at 8 (lane / 32);
// TILE 16: v_mfma_f32_16x16x32_f16, a lane holds row (lane % 16) and 8 values of k at 8 (lane / 16).
template <int TILE>
__global__ __launch_bounds__(kProjectionWaves * 64) void router_projection_kernel(const __half* __restrict__ x,
                                                                                  const __half* __restrict__ w,
                                                                                  float* __restrict__ logits,
                                                                                  __half* __restrict__ shared_gate, int rows,
                                                                                  int h, int experts) {
    constexpr int STEP = TILE == 32 ? 16 : 32, REGS = TILE == 32 ? 16 : 4;
    __shared__ float partial[kProjectionWaves - 1][TILE][TILE + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int frag = lane % TILE, piece = lane / TILE;
    const int row0 = blockIdx.x * TILE, col0 = blockIdx.y * TILE;
    const __half* x_row = x + (int64_t)min(row0 + frag, rows - 1) * h + piece * 8;
    const __half* w_row = w + (int64_t)min(col0 + frag, experts) * h + piece * 8;
    const int steps = h / STEP;  // H is a multiple of 128
    const int first = steps * wave / kProjectionWaves, last = steps * (wave + 1) / kProjectionWaves;
    typename std::conditional<TILE == 32, v16f, v4f>::type acc;
#pragma unroll
    for (int r = 0; r < REGS; ++r) acc[r] = 0.f;
#pragma unroll 8
    for (int step = first; step < last; ++step) {
        const v8h a = *reinterpret_cast<const v8h*>(x_row + step * STEP);
        const v8h b = *reinterpret_cast<const v8h*>(w_row + step * STEP);
        if constexpr (TILE == 32)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
    }
    // a lane holds column `frag`; TILE 32: rows 8 (r / 4) + 4 piece + r % 4, TILE 16: rows 4 piece + r
    auto local_row = [&](int r) { return TILE == 32 ? 8 * (r >> 2) + 4 * piece + (r & 3) : 4 * piece + r; };
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < REGS; ++r) partial[wave - 1][local_row(r)][frag] = acc[r];
    }
    __syncthreads();
    if (wave > 0) return;
    const int col = col0 + frag;
#pragma unroll
    for (int r = 0; r < REGS; ++r) {
        const int local = local_row(r), row = row0 + local;
        float value = acc[r];
#pragma unroll
        for (int other = 0; other < kProjectionWaves - 1; ++other) value += partial[other][local][frag];
        if (row < rows) {
            if (col < experts)
                logits[(int64_t)row * experts + col] = value;
            else if (col == experts)
                shared_gate[row] = __float2half_rn(value);
        }
    }
}

// ---- the histogram in three launches over segments of the assignment list (kernels/cuda/model/moe.py:556-656) ----
// local:   grid (segments, E).  Partial[e, s] = assignments of segment s routed to expert e, Slots[i] = rank of
//          assignment i among those of its expert inside its segment.
// offsets: grid E.  Offsets[e, s] = exclusive prefix of Partial[e, :], Counts[e] = their sum.
// finish:  Slots[i] += Offsets[IDs[i], segment of i]: the token-major stable slot of expert_histogram.
// Partial and Offsets are (E, segments) with the segments of the live rows.
__global__ __launch_bounds__(256) void histogram_local_kernel(const int* __restrict__ ids, int* __restrict__ partial,
                                                              int* __restrict__ slots, int assignments, int block,
                                                              int segments) {
    __shared__ int wave_totals[4];
    const int segment = blockIdx.x, expert = blockIdx.y;
    int base = 0;
    for (int first = 0; first < block; first += 256) {
        const int i = segment * block + first + threadIdx.x;
        const bool match = first + (int)threadIdx.x < block && i < assignments && ids[i] == expert;
        int total;
        const int prefix = block_flag_scan(match, wave_totals, &total);
        if (match) slots[i] = base + prefix;
        base += total;
    }
    if (threadIdx.x == 0) partial[(int64_t)expert * segments + segment] = base;
}

__global__ __launch_bounds__(64) void histogram_offsets_kernel(const int* __restrict__ partial, int* __restrict__ offsets,
                                                               int* __restrict__ counts, int segments) {
    const int expert = blockIdx.x, lane = threadIdx.x;
    const int per = (segments + 63) / 64;
    const int begin = min(lane * per, segments), end = min(begin + per, segments);
    const int* row = partial + (int64_t)expert * segments;
    int mine = 0;
    for (int j = begin; j < end; ++j) mine += row[j];
    int inclusive = mine;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const int other = __shfl_up(inclusive, offset, 64);
        if (lane >= offset) inclusive += other;
    }
    int running = inclusive - mine;
    for (int j = begin; j < end; ++j) {
        offsets[(int64_t)expert * segments + j] = running;
        running += row[j];
    }
    if (lane == 63) counts[expert] = inclusive;
}

__global__ __launch_bounds__(256) void histogram_finish_kernel(const int* __restrict__ ids, const int* __restrict__ offsets,
                                                               int* __restrict__ slots, int assignments, int block,
                                                               int segments) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < assignments) slots[i] += offsets[(int64_t)ids[i] * segments + i / block];
}

// one block: exclusive prefixes of counts and of ceil(counts/bm); TileCount = total tiles.
__global__ __launch_bounds__(256) void expert_offsets_kernel(const int* __restrict__ counts, int* __restrict__ row_offsets,
                                                             int* __restrict__ tile_count, int* __restrict__ tile_offsets,
                                                             int experts, int block_m) {
    __shared__ int rows_scan[256], tiles_scan[256];
    int row_base = 0, tile_base = 0;
    for (int first = 0; first < experts; first += 256) {
        const int e = first + threadIdx.x;
        const int c = e < experts ? counts[e] : 0;
        const int t = (c + block_m - 1) / block_m;
        rows_scan[threadIdx.x] = c;
        tiles_scan[threadIdx.x] = t;
        __syncthreads();
        for (int offset = 1; offset < 256; offset <<= 1) {
            const int r = threadIdx.x >= offset ? rows_scan[threadIdx.x - offset] : 0;
            const int s = threadIdx.x >= offset ? tiles_scan[threadIdx.x - offset] : 0;
            __syncthreads();
            rows_scan[threadIdx.x] += r;
            tiles_scan[threadIdx.x] += s;
            __syncthreads();
        }
        if (e < experts) {
            row_offsets[e] = row_base + rows_scan[threadIdx.x] - c;
            tile_offsets[e] = tile_base + tiles_scan[threadIdx.x] - t;
        }
        row_base += rows_scan[255];
        tile_base += tiles_scan[255];
        __syncthreads();
    }
    if (threadIdx.x == 0) tile_count[0] = tile_base;
}

// grid E
__global__ __launch_bounds__(256) void expert_tiles_kernel(const int* __restrict__ counts, int* __restrict__ tile_expert,
                                                           const int* __restrict__ tile_offsets, int* __restrict__ tile_row,
                                                           int block_m) {
    const int e = blockIdx.x;
    const int c = counts[e], base = tile_offsets[e];
    for (int tile = threadIdx.x; tile * block_m < c; tile += 256) {
        tile_expert[base + tile] = e;
        tile_row[base + tile] = tile * block_m;
    }
}

// ---- hot / cold expert partition (kernels/cuda/model/expert_partition.py:16-89) -----------------
// Experts with more than cold_rows routed rows get tiles of hot_m rows in one list, the others tiles
// of cold_m rows in a second list; row offsets are the common ones, so two grouped launches (one per
// list) write disjoint rows of the same output.
__global__ __launch_bounds__(256) void partition_offsets_kernel(const int* __restrict__ counts, int* __restrict__ row_offsets,
                                                                int* __restrict__ tile_offsets, int* __restrict__ tile_count,
                                                                int* __restrict__ cold_offsets, int* __restrict__ cold_count,
                                                                int experts, int hot_m, int cold_m, int cold_rows) {
    __shared__ int scan[3][256];
    int base[3] = {0, 0, 0};
    for (int first = 0; first < experts; first += 256) {
        const int e = first + threadIdx.x;
        const int c = e < experts ? counts[e] : 0;
        const int own[3] = {c, c > cold_rows ? (c + hot_m - 1) / hot_m : 0, c <= cold_rows ? (c + cold_m - 1) / cold_m : 0};
#pragma unroll
        for (int i = 0; i < 3; ++i) scan[i][threadIdx.x] = own[i];
        __syncthreads();
        for (int offset = 1; offset < 256; offset <<= 1) {
            int add[3];
#pragma unroll
            for (int i = 0; i < 3; ++i) add[i] = threadIdx.x >= offset ? scan[i][threadIdx.x - offset] : 0;
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 3; ++i) scan[i][threadIdx.x] += add[i];
            __syncthreads();
        }
        if (e < experts) {
            row_offsets[e] = base[0] + scan[0][threadIdx.x] - own[0];
            tile_offsets[e] = base[1] + scan[1][threadIdx.x] - own[1];
            cold_offsets[e] = base[2] + scan[2][threadIdx.x] - own[2];
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) base[i] += scan[i][255];
        __syncthreads();
    }
    if (threadIdx.x == 0) tile_count[0] = base[1], cold_count[0] = base[2];
}

// grid E
__global__ __launch_bounds__(256) void partition_tiles_kernel(const int* __restrict__ counts,
                                                              const int* __restrict__ tile_offsets,
                                                              int* __restrict__ tile_expert, int* __restrict__ tile_row,
                                                              const int* __restrict__ cold_offsets,
                                                              int* __restrict__ cold_expert, int* __restrict__ cold_row,
                                                              int hot_m, int cold_m, int cold_rows) {
    const int e = blockIdx.x;
    const int c = counts[e];
    const bool cold = c <= cold_rows;
    const int height = cold ? cold_m : hot_m;
    const int base = cold ? cold_offsets[e] : tile_offsets[e];
    int* experts_out = cold ? cold_expert : tile_expert;
    int* rows_out = cold ? cold_row : tile_row;
    for (int tile = threadIdx.x; tile * height < c; tile += 256) {
        experts_out[base + tile] = e;
        rows_out[base + tile] = tile * height;
    }
}

// ---- all routing metadata in one launch ---------------------------------------------------------
// kernels/cuda/model/moe.py:713-764: counts, stable relative slots, row and tile prefixes and the
// tile list from one workgroup, instead of three dependent launches.  16 waves; wave w owns a
// contiguous run of assignments (token-major) and walks it 64 at a time: lanes that name the same
// expert are ranked by lane order with one ballot per distinct expert (scalar loop, no memory
// traffic), on top of the expert's running count in the wave's own counter row.  A prefix over the
// 16 rows per expert then turns wave-local slots into global ones.  No atomics, one writer per
// element, token-major stable order; a token may name an expert more than once.
// LDS (dynamic): counters[16][E], wave-local slots[capacity assignments], scan totals.
constexpr int kMetaWaves = 16, kMetaThreads = kMetaWaves * 64;
__global__ __launch_bounds__(kMetaThreads) void route_metadata_kernel(
    const int* __restrict__ ids, int* __restrict__ counts, int* __restrict__ relative, int* __restrict__ row_offsets,
    int* __restrict__ tile_count, int* __restrict__ tile_expert, int* __restrict__ tile_offsets, int* __restrict__ tile_row,
    int* __restrict__ slot_map, int* __restrict__ slot_token, int* __restrict__ row_max, int m, int experts, int top_k,
    int block_m) {
    extern __shared__ int meta_lds[];
    int* counters = meta_lds;                          // [kMetaWaves][experts]
    int* wave_rows = counters + kMetaWaves * experts;  // [kMetaWaves]
    int* wave_tiles = wave_rows + kMetaWaves;          // [kMetaWaves]
    int* local = wave_tiles + kMetaWaves;              // [assignments]: id << 16 | wave-local slot... two arrays below
    const int assignments = m * top_k;
    int* local_id = local + assignments;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this wave's run of assignments, a multiple of 64 long
    const int per_wave = ((assignments + kMetaWaves - 1) / kMetaWaves + 63) & ~63;
    const int first = wave * per_wave, last = min(assignments, first + per_wave);
    // the ids of the first two steps travel while the counters are cleared (2048 assignments are two steps per wave)
    const int early_id[2] = {first + lane < last ? ids[first + lane] : -1, first + 64 + lane < last ? ids[first + 64 + lane] : -1};
    for (int i = tid; i < kMetaWaves * experts; i += kMetaThreads) counters[i] = 0;
    __syncthreads();
    int* mine = counters + wave * experts;
    const int id_bits = 32 - __builtin_clz(max(experts - 1, 1));
    for (int base = first; base < last; base += 64) {
        const int at = base + lane;
        const bool valid = at < last;
        const int step = (base - first) >> 6;
        const int id = step == 0 ? early_id[0] : step == 1 ? early_id[1] : valid ? ids[at] : -1;
        const int running = valid ? mine[id] : 0;  // nobody has written this expert in this step yet
        // the lanes that hold the same expert, found one id bit at a time
        unsigned long long same = __ballot(valid);
        for (int bit = 0; bit < id_bits; ++bit) {
            const bool set = (id >> bit) & 1;
            const unsigned long long with = __ballot(valid && set);
            same &= set ? with : ~with;
        }
        const int rank = __popcll(same & ((1ull << lane) - 1ull));
        const int group = __popcll(same);
        if (valid) {
            local[at] = running + rank;
            local_id[at] = id;
            if (rank == group - 1) mine[id] = running + group;
        }
    }
    __syncthreads();
    // per expert: exclusive prefix over the 16 wave rows, total count
    int count = 0;
    if (tid < experts) {
        for (int w = 0; w < kMetaWaves; ++w) {
            const int t = counters[w * experts + tid];
            counters[w * experts + tid] = count;
            count += t;
        }
        counts[tid] = count;
    }
    __syncthreads();
    // global relative slots, written once and coalesced
    for (int at = tid; at < assignments; at += kMetaThreads) {
        const int slot_in_expert = local[at] + counters[(at / per_wave) * experts + local_id[at]];
        relative[at] = slot_in_expert;
        local[at] = slot_in_expert;
    }
    // exclusive scans of count and ceil(count / block_m) over the experts (one per thread)
    const int tiles = (count + block_m - 1) / block_m;
    int row_scan = count, tile_scan = tiles;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const int r = __shfl_up(row_scan, offset, 64), t = __shfl_up(tile_scan, offset, 64);
        if (lane >= offset) row_scan += r, tile_scan += t;
    }
    if (lane == 63) wave_rows[wave] = row_scan, wave_tiles[wave] = tile_scan;
    __syncthreads();
    int row_base = 0, tile_base = 0, tile_total = 0;
    for (int w = 0; w < kMetaWaves; ++w) {
        if (w < wave) row_base += wave_rows[w], tile_base += wave_tiles[w];
        tile_total += wave_tiles[w];
    }
    if (tid == 0) tile_count[0] = tile_total;
    // (the barrier above also ended the reads of the counter rows: row 0 now takes the row offsets)
    if (tid < experts) {
        const int first_tile = tile_base + tile_scan - tiles;
        row_offsets[tid] = row_base + row_scan - count;
        if (slot_map != nullptr) counters[tid] = row_base + row_scan - count;
        tile_offsets[tid] = first_tile;
        for (int t = 0; t < tiles; ++t) {
            tile_expert[first_tile + t] = tid;
            tile_row[first_tile + t] = t * block_m;
        }
    }
    // slot_maps: what the dispatch would compute, slot = RowOffsets[expert] + RelativeSlot, and its
    // inverse (the token of every slot), so that no launch has to copy rows into slot order; and the
    // per-slot maxima the expert projection's SwiGLU epilogue raises start at zero
    if (slot_map == nullptr) return;
    __syncthreads();
    for (int at = tid; at < assignments; at += kMetaThreads) {
        const int slot = counters[local_id[at]] + local[at];
        slot_map[at] = slot;
        slot_token[slot] = at / top_k;
        row_max[at] = 0;
    }
}

// One token: every selected expert owns one row and one tile, in expert-id order
// (moe.py:659-709; ids distinct and inside [0, E), as router_topk leaves them).  One workgroup;
// thread e counts the ids equal to and below e, thread rank places its id.  Tiles from top_k on
// are left as they were.
__global__ __launch_bounds__(256) void single_route_metadata_kernel(const int* __restrict__ ids, int* __restrict__ counts,
                                                                    int* __restrict__ relative, int* __restrict__ offsets,
                                                                    int* __restrict__ tile_offsets,
                                                                    int* __restrict__ tile_expert, int* __restrict__ tile_row,
                                                                    int* __restrict__ tile_count, int experts, int top_k) {
    extern __shared__ int route_ids[];  // top_k
    for (int rank = threadIdx.x; rank < top_k; rank += 256) route_ids[rank] = ids[rank];
    __syncthreads();
    for (int expert = threadIdx.x; expert < experts; expert += 256) {
        int equal = 0, below = 0;
        for (int rank = 0; rank < top_k; ++rank) {
            equal += route_ids[rank] == expert;
            below += route_ids[rank] < expert;
        }
        counts[expert] = equal;
        offsets[expert] = below;
        tile_offsets[expert] = below;
    }
    for (int rank = threadIdx.x; rank < top_k; rank += 256) {
        const int mine = route_ids[rank];
        int position = 0;
        for (int other = 0; other < top_k; ++other) position += route_ids[other] < mine;
        relative[rank] = 0;
        tile_expert[position] = mine;
        tile_row[position] = 0;
    }
    if (threadIdx.x == 0) tile_count[0] = top_k;
}

// grid M*top_k: copy one int8 row and its scales to the expert-sorted slot.
__global__ __launch_bounds__(256) void expert_dispatch_kernel(const int8_t* __restrict__ a, int8_t* __restrict__ d,
                                                              __half* __restrict__ ds, const int* __restrict__ ids,
                                                              const int* __restrict__ relative,
                                                              const int* __restrict__ row_offsets,
                                                              const __half* __restrict__ scale, int* __restrict__ slot_map,
                                                              int h, int groups, int top_k) {
    const int assignment = blockIdx.x;
    const int row = assignment / top_k;
    const int slot = row_offsets[ids[assignment]] + relative[assignment];
    if (threadIdx.x == 0) slot_map[assignment] = slot;
    const int8_t* src = a + (int64_t)row * h;
    int8_t* dst = d + (int64_t)slot * h;
    if ((h & 15) == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(d)) & 15) == 0) {
        for (int i = threadIdx.x; i < h / 16; i += 256)
            reinterpret_cast<uint4*>(dst)[i] = reinterpret_cast<const uint4*>(src)[i];
    } else {
        for (int i = threadIdx.x; i < h; i += 256) dst[i] = src[i];
    }
    for (int g = threadIdx.x; g < groups; g += 256) ds[(int64_t)slot * groups + g] = scale[(int64_t)row * groups + g];
}

// The same with the quantiser in front (un-rotated activations): A is the fp16 row, every assignment
// quantises its token row by the A8 rule (one scale per row) straight into its slot.  The row is
// quantised top_k times over, which costs less than a launch of its own and a round trip of the codes.
__global__ __launch_bounds__(256) void quantize_dispatch_kernel(const __half* __restrict__ x, int8_t* __restrict__ d,
                                                                __half* __restrict__ ds, const int* __restrict__ ids,
                                                                const int* __restrict__ relative,
                                                                const int* __restrict__ row_offsets,
                                                                int* __restrict__ slot_map, int h, int top_k) {
    __shared__ float wave_max[4];
    const int assignment = blockIdx.x, tid = threadIdx.x;
    const int row = assignment / top_k;
    const __half* src = x + (int64_t)row * h;
    const int pieces = h / 8;  // the host guarantees h % 8 == 0 and 16-byte aligned rows
    // the row's first piece is requested before the slot's chain of dependent reads, and stays in
    // registers (the whole row when h <= 2048)
    uint4 kept = reinterpret_cast<const uint4*>(src)[min(tid, pieces - 1)];
    const int slot = row_offsets[ids[assignment]] + relative[assignment];
    if (tid == 0) slot_map[assignment] = slot;
    int8_t* dst = d + (int64_t)slot * h;
    float amax = 0.f;
    for (int i = tid; i < pieces; i += 256) {
        const uint4 raw = i == tid ? kept : reinterpret_cast<const uint4*>(src)[i];
        const __half2* pairs = reinterpret_cast<const __half2*>(&raw);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float2 f = __half22float2(pairs[j]);
            amax = fmaxf(amax, fmaxf(fabsf(f.x), fabsf(f.y)));
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    const __half stored = a8_scale(amax);
    if (tid == 0) ds[slot] = stored;
    const float scale = __half2float(stored), inverse = __frcp_rn(scale);
    for (int i = tid; i < pieces; i += 256) {
        const uint4 raw = i == tid ? kept : reinterpret_cast<const uint4*>(src)[i];
        const __half* v = reinterpret_cast<const __half*>(&raw);
        const float low[4] = {__half2float(v[0]), __half2float(v[1]), __half2float(v[2]), __half2float(v[3])};
        const float high[4] = {__half2float(v[4]), __half2float(v[5]), __half2float(v[6]), __half2float(v[7])};
        reinterpret_cast<uint2*>(dst)[i] = make_uint2(quantise4(low, scale, inverse), quantise4(high, scale, inverse));
    }
}

// grid (M, ceil(H/256)): fp32 accumulate in rank order, one fp16 cast.
__global__ __launch_bounds__(256) void moe_combine_kernel(const __half* __restrict__ expert, __half* __restrict__ output,
                                                          const float* __restrict__ prob, const __half* __restrict__ shared,
                                                          const __half* __restrict__ shared_gate,
                                                          const int* __restrict__ slot_map, int h, int slots, int top_k) {
    const int row = blockIdx.x;
    const int col = blockIdx.y * 256 + threadIdx.x;
    if (col >= h) return;
    float acc = 0.f;
    for (int rank = 0; rank < top_k; ++rank) {
        const int slot = slot_map[(int64_t)row * top_k + rank];
        if (slot >= 0 && slot < slots)
            acc += __half2float(expert[(int64_t)slot * h + col]) * prob[(int64_t)row * top_k + rank];
    }
    if (shared != nullptr) {
        const float gate = __fdiv_rn(1.0f, 1.0f + expf(-__half2float(shared_gate[row])));
        acc = acc + gate * __half2float(shared[(int64_t)row * h + col]);
    }
    output[(int64_t)row * h + col] = __float2half_rn(acc);
}

// H a multiple of 8: a thread owns 8 consecutive columns (one 16-byte piece per rank), a workgroup
// 2048 columns of one row.  Same operations per column as above, in the same order.
__global__ __launch_bounds__(256) void moe_combine_wide_kernel(const __half* __restrict__ expert, __half* __restrict__ output,
                                                               const float* __restrict__ prob,
                                                               const __half* __restrict__ shared,
                                                               const __half* __restrict__ shared_gate,
                                                               const int* __restrict__ slot_map, int h, int slots,
                                                               int top_k) {
    const int row = blockIdx.x;
    const int col = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (col >= h) return;
    const bool aligned = ((reinterpret_cast<uintptr_t>(expert) | reinterpret_cast<uintptr_t>(output) |
                           reinterpret_cast<uintptr_t>(shared)) & 15) == 0;
    auto load8 = [&](const __half* src, __half (&dst)[8]) {
        if (aligned) {
            *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = src[j];
        }
    };
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    // Ranks in batches of 8: all slots, then all pieces, then the sums in rank order.  A skipped slot
    // reads slot 0 and its term is not added, so the loads of a batch do not wait for one another.
    for (int first = 0; first < top_k; first += 8) {
        int slot[8];
        float weight[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int rank = min(first + i, top_k - 1);
            slot[i] = slot_map[(int64_t)row * top_k + rank];
            weight[i] = prob[(int64_t)row * top_k + rank];
        }
        __align__(16) __half values[8][8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool valid = first + i < top_k && slot[i] >= 0 && slot[i] < slots;
            load8(expert + (int64_t)(valid ? slot[i] : 0) * h + col, values[i]);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool valid = first + i < top_k && slot[i] >= 0 && slot[i] < slots;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float sum = acc[j] + __half2float(values[i][j]) * weight[i];
                acc[j] = valid ? sum : acc[j];
            }
        }
    }
    if (shared != nullptr) {
        const float gate = __fdiv_rn(1.0f, 1.0f + expf(-__half2float(shared_gate[row])));
        __align__(16) __half values[8];
        load8(shared + (int64_t)row * h + col, values);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = acc[j] + gate * __half2float(values[j]);
    }
    __align__(16) __half result[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) result[j] = __float2half_rn(acc[j]);
    __half* dst = output + (int64_t)row * h + col;
    if (aligned) {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(result);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = result[j];
    }
}

// ---- host side -----------------------------------------------------------------------------
bool geometry_fields(const Variant& v, orx_function* f, bool need_m) {
    bool bad = false;
    f->M = (int)v.integer("M", need_m ? 0 : 1, &bad);
    f->E = (int)v.integer("E", 512, &bad);
    f->top_k = (int)v.integer("top_k", 10, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    f->capacity = f->M;
    return !bad;
}

int rows_geometry_router(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)rows, 4u);
    // quantize_hidden: four more waves quantise the four tokens' rows (up to 8 keys per lane, E <= 512)
    g->block[0] = f.H > 0 && f.E <= 512 ? 512 : 256;
    return ORX_OK;
}
// IDs, Logits, Prob[, Q, S, X][, m]
int router_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    const float* logits = pointer_arg<const float>(args, 1);
    int* ids = pointer_arg<int>(args, 0);
    float* prob = pointer_arg<float>(args, 2);
    const __half* x = f.H > 0 ? pointer_arg<const __half>(args, 5) : nullptr;
    int8_t* q = f.H > 0 ? pointer_arg<int8_t>(args, 3) : nullptr;
    __half* scale = f.H > 0 ? pointer_arg<__half>(args, 4) : nullptr;
    const dim3 grid(g.grid[0]), block(g.block[0]);
#define ORX_ROUTER(LOCAL)                                                                                              \
    do {                                                                                                               \
        if (f.H > 0)                                                                                                   \
            ORX_LAUNCH((router_topk_kernel<LOCAL, true>), grid, block, 0, s, logits, ids, prob, rows, f.E,     \
                               f.top_k, f.flags, x, q, scale, f.H);                                                    \
        else                                                                                                           \
            ORX_LAUNCH((router_topk_kernel<LOCAL, false>), grid, block, 0, s, logits, ids, prob, rows, f.E,    \
                               f.top_k, f.flags, x, q, scale, f.H);                                                    \
    } while (0)
    if (f.E <= 64) ORX_ROUTER(1);
    else if (f.E <= 128) ORX_ROUTER(2);
    else if (f.E <= 256) ORX_ROUTER(4);
    else if (f.E <= 512) ORX_ROUTER(8);
    else ORX_ROUTER(16);
#undef ORX_ROUTER
    return hip_check(hipGetLastError(), "launch router_topk");
}
int make_router(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->flags = v.boolean("renormalize", true, &bad) ? 1 : 0;
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->E <= 0 || f->top_k <= 0 || f->top_k > f->E || f->top_k > 64 || f->E > 64 * kMaxLocal) {
        set_error("router_topk: invalid MoE router dimensions (need top_k <= min(E,64), E <= 1024)");
        return ORX_ERR_BAD_VARIANT;
    }
    // quantize_hidden=H: the launch also writes the A8 codes Q (M, H) and scales S (M) of the fp16 rows X (M, H)
    f->H = (int)v.integer("quantize_hidden", 0, &bad);
    if (bad || f->H < 0 || f->H % 8) {
        set_error("router_topk: quantize_hidden must be a multiple of 8");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"IDs", ArgPointer, 4}, {"Logits", ArgPointer, 4}, {"Prob", ArgPointer, 4}};
    if (f->H > 0) f->args.push_back({"Q", ArgPointer, 8}), f->args.push_back({"S", ArgPointer, 2}), f->args.push_back({"X", ArgPointer, 16});
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = rows_geometry_router;
    f->launch = router_launch;
    // the instantiation this variant launches (its thread limit is what orx_query reports)
#define ORX_ROUTER_FN(LOCAL)                                                                \
    (f->H > 0 ? reinterpret_cast<const void*>(&router_topk_kernel<LOCAL, true>)             \
              : reinterpret_cast<const void*>(&router_topk_kernel<LOCAL, false>))
    f->device_function = f->E <= 64    ? ORX_ROUTER_FN(1)
                         : f->E <= 128 ? ORX_ROUTER_FN(2)
                         : f->E <= 256 ? ORX_ROUTER_FN(4)
                         : f->E <= 512 ? ORX_ROUTER_FN(8)
                                       : ORX_ROUTER_FN(16);
#undef ORX_ROUTER_FN
    return ORX_OK;
}

// kernels/cuda/model/moe.py:332-409: the reference's one-warp-per-row form; same ids (descending
// logit, ties to the lower id, +-0 equal) and probabilities renormalised over the selected routes.
int make_router_warp(const Variant& v, orx_function* f) {
    bool bad = false;
    const long long experts = v.integer("E", 0, &bad), top_k = v.integer("top_k", 0, &bad), warps = v.integer("warps", 4, &bad);
    if (bad || !v.has("E") || !v.has("top_k") || experts % 32 || top_k > 32 || (warps != 1 && warps != 2 && warps != 4) ||
        v.has("renormalize")) {
        set_error("router_topk_warp: invalid warp router geometry (E a multiple of 32, top_k <= 32, warps 1|2|4)");
        return ORX_ERR_BAD_VARIANT;
    }
    Variant plain = v;
    plain.fields.erase("warps");
    return make_router(plain, f);
}

int histogram_geometry(const orx_function& f, int, Geometry* g) {
    g->grid[0] = (uint32_t)f.E;
    g->block[0] = 256;
    return ORX_OK;
}
int histogram_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    ORX_LAUNCH(expert_histogram_kernel, dim3(g.grid[0]), dim3(256), 0, s, pointer_arg<const int>(args, 1),
                       pointer_arg<int>(args, 0), pointer_arg<int>(args, 2), rows * f.top_k);
    return hip_check(hipGetLastError(), "launch expert_histogram");
}
int make_histogram(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->E <= 0 || f->top_k <= 0 || f->top_k > f->E) {
        set_error("expert_histogram: invalid MoE dispatch dimensions");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"Counts", ArgPointer, 4}, {"IDs", ArgPointer, 4}, {"RelativeSlot", ArgPointer, 4}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = histogram_geometry;
    f->launch = histogram_launch;
    f->device_function = reinterpret_cast<const void*>(&expert_histogram_kernel);
    return ORX_OK;
}

// router_projection: Logits, SharedGate, W, X[, m].  slots used: M, H, E
int router_projection_geometry(const orx_function& f, int rows, Geometry* g) {
    const uint32_t tile = rows <= kProjectionSmallRows ? 16u : 32u;
    g->grid[0] = ceil_div((uint32_t)rows, tile);
    g->grid[1] = ceil_div((uint32_t)f.E + 1u, tile);
    g->block[0] = kProjectionWaves * 64;
    return ORX_OK;
}
int router_projection_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    const dim3 grid(g.grid[0], g.grid[1]), block(g.block[0]);
    const __half *x = pointer_arg<const __half>(args, 3), *w = pointer_arg<const __half>(args, 2);
    float* logits = pointer_arg<float>(args, 0);
    __half* gate = pointer_arg<__half>(args, 1);
    if (rows <= kProjectionSmallRows)
        ORX_LAUNCH(router_projection_kernel<16>, grid, block, 0, s, x, w, logits, gate, rows, f.H, f.E);
    else
        ORX_LAUNCH(router_projection_kernel<32>, grid, block, 0, s, x, w, logits, gate, rows, f.H, f.E);
    return hip_check(hipGetLastError(), "launch router_projection");
}
int make_router_projection(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->H = (int)v.integer("H", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const int bm = (int)v.integer("block_m", 16, &bad), bn = (int)v.integer("block_n", 32, &bad);
    const int bk = (int)v.integer("block_k", 128, &bad), stages = (int)v.integer("stages", 2, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    // moe.py:20-28: tile choices of the reference's kernel, checked as it checks them; H in whole K steps
    if (f->M <= 0 || f->H <= 0 || f->E <= 0 || (bm != 16 && bm != 32 && bm != 64 && bm != 128) || (bn != 32 && bn != 64 && bn != 128) ||
        (bk != 128 && bk != 256) || f->H % bk || (stages != 1 && stages != 2)) {
        set_error("router_projection: need M, H, E > 0, block_m 16..128, block_n 32|64|128, block_k 128|256 dividing H, stages 1|2");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"Logits", ArgPointer, 4}, {"SharedGate", ArgPointer, 2}, {"W", ArgPointer, 16}, {"X", ArgPointer, 16}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = router_projection_geometry;
    f->launch = router_projection_launch;
    f->device_function = reinterpret_cast<const void*>(&router_projection_kernel<32>);
    return ORX_OK;
}

// expert_histogram_local / _offsets / _finish (moe.py:556-656).  slots used: M, E, top_k (the reference's K), group (block),
// algorithm (0 local, 1 offsets, 2 finish)
int segmented_geometry(const orx_function& f, int rows, Geometry* g) {
    const uint32_t assignments = (uint32_t)rows * (uint32_t)f.top_k, segments = ceil_div(assignments, (uint32_t)f.group);
    if (f.algorithm == 0) {
        g->grid[0] = segments, g->grid[1] = (uint32_t)f.E, g->block[0] = 256;
    } else if (f.algorithm == 1) {
        g->grid[0] = (uint32_t)f.E, g->block[0] = 64;
    } else {
        g->grid[0] = ceil_div(assignments, 256u), g->block[0] = 256;
    }
    return ORX_OK;
}
int segmented_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    const int assignments = rows * f.top_k, segments = (assignments + f.group - 1) / f.group;
    const dim3 grid(g.grid[0], g.grid[1]), block(g.block[0]);
    if (f.algorithm == 0)  // IDs, Partial, Slots
        ORX_LAUNCH(histogram_local_kernel, grid, block, 0, s, pointer_arg<const int>(args, 0), pointer_arg<int>(args, 1),
                           pointer_arg<int>(args, 2), assignments, f.group, segments);
    else if (f.algorithm == 1)  // Counts, Offsets, Partial
        ORX_LAUNCH(histogram_offsets_kernel, grid, block, 0, s, pointer_arg<const int>(args, 2),
                           pointer_arg<int>(args, 1), pointer_arg<int>(args, 0), segments);
    else  // IDs, Offsets, Slots
        ORX_LAUNCH(histogram_finish_kernel, grid, block, 0, s, pointer_arg<const int>(args, 0),
                           pointer_arg<const int>(args, 1), pointer_arg<int>(args, 2), assignments, f.group, segments);
    return hip_check(hipGetLastError(), "launch segmented expert histogram");
}
int make_segmented(const Variant& v, orx_function* f, int stage) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->E = (int)v.integer("E", 512, &bad);
    f->top_k = (int)v.integer("K", 10, &bad);
    f->group = (int)v.integer("block", 1024, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->E <= 0 || f->top_k <= 0 || f->top_k > f->E || (f->group != 512 && f->group != 1024 && f->group != 2048)) {
        set_error("%s: need M, E > 0, 1 <= K <= E and block 512, 1024 or 2048", f->symbol.c_str());
        return ORX_ERR_BAD_VARIANT;
    }
    f->algorithm = stage;
    if (stage == 0) f->args = {{"IDs", ArgPointer, 4}, {"Partial", ArgPointer, 4}, {"Slots", ArgPointer, 4}};
    if (stage == 1) f->args = {{"Counts", ArgPointer, 4}, {"Offsets", ArgPointer, 4}, {"Partial", ArgPointer, 4}};
    if (stage == 2) f->args = {{"IDs", ArgPointer, 4}, {"Offsets", ArgPointer, 4}, {"Slots", ArgPointer, 4}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = segmented_geometry;
    f->launch = segmented_launch;
    f->device_function = stage == 0   ? reinterpret_cast<const void*>(&histogram_local_kernel)
                         : stage == 1 ? reinterpret_cast<const void*>(&histogram_offsets_kernel)
                                      : reinterpret_cast<const void*>(&histogram_finish_kernel);
    return ORX_OK;
}
int make_histogram_local(const Variant& v, orx_function* f) { return make_segmented(v, f, 0); }
int make_histogram_offsets(const Variant& v, orx_function* f) { return make_segmented(v, f, 1); }
int make_histogram_finish(const Variant& v, orx_function* f) { return make_segmented(v, f, 2); }

int one_block_geometry(const orx_function&, int, Geometry* g) {
    g->block[0] = 256;
    return ORX_OK;
}
int offsets_launch(const orx_function& f, int, const Geometry&, hipStream_t s, void** args) {
    ORX_LAUNCH(expert_offsets_kernel, dim3(1), dim3(256), 0, s, pointer_arg<const int>(args, 0),
                       pointer_arg<int>(args, 1), pointer_arg<int>(args, 2), pointer_arg<int>(args, 3), f.E, f.block_m);
    return hip_check(hipGetLastError(), "launch expert_offsets");
}
bool valid_block_m(int bm) { return bm == 8 || bm == 16 || bm == 32 || bm == 64 || bm == 128 || bm == 256; }
int make_offsets(const Variant& v, orx_function* f) {
    bool bad = false;
    f->E = (int)v.integer("E", 512, &bad);
    f->block_m = (int)v.integer("block_m", 16, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->E <= 0 || !valid_block_m(f->block_m)) {
        set_error("expert_offsets: invalid MoE expert prefix dimensions");
        return ORX_ERR_BAD_VARIANT;
    }
    f->capacity = 1;
    f->args = {{"Counts", ArgPointer, 4}, {"RowOffsets", ArgPointer, 4}, {"TileCount", ArgPointer, 4},
               {"TileOffsets", ArgPointer, 4}};
    f->geometry = one_block_geometry;
    f->launch = offsets_launch;
    f->device_function = reinterpret_cast<const void*>(&expert_offsets_kernel);
    return ORX_OK;
}

int tiles_launch(const orx_function& f, int, const Geometry& g, hipStream_t s, void** args) {
    ORX_LAUNCH(expert_tiles_kernel, dim3(g.grid[0]), dim3(256), 0, s, pointer_arg<const int>(args, 0),
                       pointer_arg<int>(args, 1), pointer_arg<const int>(args, 2), pointer_arg<int>(args, 3), f.block_m);
    return hip_check(hipGetLastError(), "launch expert_tiles");
}
int make_tiles(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->block_m = (int)v.integer("block_m", 16, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->E <= 0 || f->top_k <= 0 || !valid_block_m(f->block_m)) {
        set_error("expert_tiles: invalid MoE tile dimensions");
        return ORX_ERR_BAD_VARIANT;
    }
    f->dynamic_rows = false;
    f->args = {{"Counts", ArgPointer, 4}, {"TileExpert", ArgPointer, 4}, {"TileOffsets", ArgPointer, 4},
               {"TileRow", ArgPointer, 4}};
    f->geometry = histogram_geometry;
    f->launch = tiles_launch;
    f->device_function = reinterpret_cast<const void*>(&expert_tiles_kernel);
    return ORX_OK;
}

int metadata_geometry(const orx_function& f, int, Geometry* g) {
    g->grid[0] = 1;
    g->block[0] = kMetaThreads;
    // counters, scan totals, wave-local slot and expert of every assignment the variant can hold
    g->shared = (uint32_t)((kMetaWaves * f.E + 2 * kMetaWaves + 2 * f.M * f.top_k) * sizeof(int));
    return ORX_OK;
}
// Counts, IDs, RelativeSlot, [RowMax,] RowOffsets, [SlotMap, SlotToken,] TileCount, TileExpert, TileOffsets, TileRow[, m]
// (moe.py:726-735 in generated-ABI order; slot_maps=true adds the two slot tables and the zeroed RowMax)
int metadata_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    static DeviceOnce opted_in;  // 64 KiB of counters at E = 1024 needs the LDS opt-in
    const int ready = opted_in.run([] {
        return hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&route_metadata_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024),
                         "hipFuncSetAttribute");
    });
    if (ready != ORX_OK) return ready;
    const bool maps = f.flags & 1;
    const int offsets_at = maps ? 4 : 3, tiles_at = maps ? 7 : 4;
    ORX_LAUNCH(route_metadata_kernel, dim3(1), dim3(kMetaThreads), g.shared, s, pointer_arg<const int>(args, 1),
                       pointer_arg<int>(args, 0), pointer_arg<int>(args, 2), pointer_arg<int>(args, offsets_at),
                       pointer_arg<int>(args, tiles_at), pointer_arg<int>(args, tiles_at + 1),
                       pointer_arg<int>(args, tiles_at + 2), pointer_arg<int>(args, tiles_at + 3),
                       maps ? pointer_arg<int>(args, 5) : nullptr, maps ? pointer_arg<int>(args, 6) : nullptr,
                       maps ? pointer_arg<int>(args, 3) : nullptr, rows, f.E, f.top_k, f.block_m);
    return hip_check(hipGetLastError(), "launch route_metadata");
}
int make_metadata(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->block_m = (int)v.integer("block_m", 8, &bad);  // moe.py:714
    if (bad) return ORX_ERR_BAD_VARIANT;
    // one expert per thread, one route per lane; the reference's own form is decode-only (M <= 1024)
    if (f->M <= 0 || f->E <= 0 || f->E > kMetaThreads || f->top_k <= 0 || f->top_k > f->E || !valid_block_m(f->block_m) ||
        (size_t)(kMetaWaves * f->E + 2 * kMetaWaves + 2 * (size_t)f->M * f->top_k) * sizeof(int) > 160 * 1024) {
        set_error("route_metadata: need E <= 1024, top_k <= E, a valid block_m and M*top_k small enough for LDS");
        return ORX_ERR_BAD_VARIANT;
    }
    const bool slot_maps = v.boolean("slot_maps", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    f->flags = slot_maps ? 1 : 0;
    f->args = {{"Counts", ArgPointer, 4}, {"IDs", ArgPointer, 4}, {"RelativeSlot", ArgPointer, 4}};
    if (slot_maps) f->args.push_back({"RowMax", ArgPointer, 4});
    f->args.push_back({"RowOffsets", ArgPointer, 4});
    if (slot_maps) f->args.push_back({"SlotMap", ArgPointer, 4}), f->args.push_back({"SlotToken", ArgPointer, 4});
    for (const ArgSpec& a : std::initializer_list<ArgSpec>{{"TileCount", ArgPointer, 4}, {"TileExpert", ArgPointer, 4},
                                                           {"TileOffsets", ArgPointer, 4}, {"TileRow", ArgPointer, 4}})
        f->args.push_back(a);
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = metadata_geometry;
    f->launch = metadata_launch;
    f->device_function = reinterpret_cast<const void*>(&route_metadata_kernel);
    return ORX_OK;
}

int single_metadata_geometry(const orx_function& f, int, Geometry* g) {
    g->grid[0] = 1;
    g->block[0] = 256;
    g->shared = (uint32_t)(f.top_k * sizeof(int));
    return ORX_OK;
}
// Counts, IDs, Offsets, Relative, TileCount, TileExpert, TileOffsets, TileRow (moe.py:674-683 in generated-ABI order)
int single_metadata_launch(const orx_function& f, int, const Geometry& g, hipStream_t s, void** args) {
    ORX_LAUNCH(single_route_metadata_kernel, dim3(1), dim3(256), g.shared, s, pointer_arg<const int>(args, 1),
                       pointer_arg<int>(args, 0), pointer_arg<int>(args, 3), pointer_arg<int>(args, 2),
                       pointer_arg<int>(args, 6), pointer_arg<int>(args, 5), pointer_arg<int>(args, 7),
                       pointer_arg<int>(args, 4), f.E, f.top_k);
    return hip_check(hipGetLastError(), "launch single_route_metadata");
}
int make_single_metadata(const Variant& v, orx_function* f) {
    bool bad = false;
    f->E = (int)v.integer("E", 512, &bad);
    f->top_k = (int)v.integer("top_k", 10, &bad);
    f->tiles = (int)v.integer("capacity", 11, &bad);
    f->M = f->capacity = 1;
    // moe.py:665-671
    if (bad || f->E <= 0 || f->top_k <= 0 || f->tiles <= 0 || f->top_k > f->E || f->tiles < f->top_k || f->top_k > 8192) {
        set_error("single_route_metadata: need 0 < top_k <= E and capacity >= top_k");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"Counts", ArgPointer, 4},    {"IDs", ArgPointer, 4},        {"Offsets", ArgPointer, 4},
               {"Relative", ArgPointer, 4},  {"TileCount", ArgPointer, 4},  {"TileExpert", ArgPointer, 4},
               {"TileOffsets", ArgPointer, 4}, {"TileRow", ArgPointer, 4}};
    f->geometry = single_metadata_geometry;
    f->launch = single_metadata_launch;
    f->device_function = reinterpret_cast<const void*>(&single_route_metadata_kernel);
    return ORX_OK;
}

// slots used: E, block_m (hot_m), block_n (cold_m), group (cold_rows)
bool partition_fields(const Variant& v, orx_function* f, const char* who) {
    bool bad = false;
    f->E = (int)v.integer("experts", 0, &bad);
    f->block_m = (int)v.integer("hot_m", 0, &bad);
    f->block_n = (int)v.integer("cold_m", 0, &bad);
    f->group = (int)v.integer("cold_rows", 0, &bad);
    // expert_partition.py:10-13
    if (bad || f->E <= 0 || f->block_m <= 0 || f->block_n <= 0 || f->group <= 0) {
        set_error("%s: need experts, hot_m, cold_m and cold_rows, all positive", who);
        return false;
    }
    return true;
}
// ColdCount, ColdOffsets, Counts, RowOffsets, TileCount, TileOffsets (expert_partition.py:21-28 in generated-ABI order)
int partition_offsets_launch(const orx_function& f, int, const Geometry&, hipStream_t s, void** args) {
    ORX_LAUNCH(partition_offsets_kernel, dim3(1), dim3(256), 0, s, pointer_arg<const int>(args, 2),
                       pointer_arg<int>(args, 3), pointer_arg<int>(args, 5), pointer_arg<int>(args, 4),
                       pointer_arg<int>(args, 1), pointer_arg<int>(args, 0), f.E, f.block_m, f.block_n, f.group);
    return hip_check(hipGetLastError(), "launch expert_partition_offsets");
}
int make_partition_offsets(const Variant& v, orx_function* f) {
    if (!partition_fields(v, f, "expert_partition_offsets")) return ORX_ERR_BAD_VARIANT;
    f->capacity = 1;
    f->args = {{"ColdCount", ArgPointer, 4},  {"ColdOffsets", ArgPointer, 4}, {"Counts", ArgPointer, 4},
               {"RowOffsets", ArgPointer, 4}, {"TileCount", ArgPointer, 4},   {"TileOffsets", ArgPointer, 4}};
    f->geometry = one_block_geometry;
    f->launch = partition_offsets_launch;
    f->device_function = reinterpret_cast<const void*>(&partition_offsets_kernel);
    return ORX_OK;
}
// ColdExpert, ColdOffsets, ColdRow, Counts, TileExpert, TileOffsets, TileRow[, m] (expert_partition.py:70-78)
int partition_tiles_launch(const orx_function& f, int, const Geometry& g, hipStream_t s, void** args) {
    ORX_LAUNCH(partition_tiles_kernel, dim3(g.grid[0]), dim3(256), 0, s, pointer_arg<const int>(args, 3),
                       pointer_arg<const int>(args, 5), pointer_arg<int>(args, 4), pointer_arg<int>(args, 6),
                       pointer_arg<const int>(args, 1), pointer_arg<int>(args, 0), pointer_arg<int>(args, 2), f.block_m,
                       f.block_n, f.group);
    return hip_check(hipGetLastError(), "launch expert_partition_tiles");
}
int make_partition_tiles(const Variant& v, orx_function* f) {
    if (!partition_fields(v, f, "expert_partition_tiles")) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->top_k = (int)v.integer("top_k", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    // expert_partition.py:64-65
    if (bad || f->M <= 0 || f->top_k <= 0 || f->top_k > f->E) {
        set_error("expert_partition_tiles: need M > 0 and 0 < top_k <= experts");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"ColdExpert", ArgPointer, 4}, {"ColdOffsets", ArgPointer, 4}, {"ColdRow", ArgPointer, 4},
               {"Counts", ArgPointer, 4},     {"TileExpert", ArgPointer, 4},  {"TileOffsets", ArgPointer, 4},
               {"TileRow", ArgPointer, 4}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = histogram_geometry;
    f->launch = partition_tiles_launch;
    f->device_function = reinterpret_cast<const void*>(&partition_tiles_kernel);
    return ORX_OK;
}

int dispatch_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)(rows * f.top_k);
    g->block[0] = 256;
    return ORX_OK;
}
int dispatch_launch(const orx_function& f, int, const Geometry& g, hipStream_t s, void** args) {
    if (f.flags & 1) {  // fp16 rows, quantised on the way (Scale is not read)
        ORX_LAUNCH(quantize_dispatch_kernel, dim3(g.grid[0]), dim3(256), 0, s, pointer_arg<const __half>(args, 0),
                           pointer_arg<int8_t>(args, 1), pointer_arg<__half>(args, 2), pointer_arg<const int>(args, 3),
                           pointer_arg<const int>(args, 4), pointer_arg<const int>(args, 5), pointer_arg<int>(args, 7), f.H,
                           f.top_k);
        return hip_check(hipGetLastError(), "launch expert_dispatch (fp16 rows)");
    }
    ORX_LAUNCH(expert_dispatch_kernel, dim3(g.grid[0]), dim3(256), 0, s, pointer_arg<const int8_t>(args, 0),
                       pointer_arg<int8_t>(args, 1), pointer_arg<__half>(args, 2), pointer_arg<const int>(args, 3),
                       pointer_arg<const int>(args, 4), pointer_arg<const int>(args, 5),
                       pointer_arg<const __half>(args, 6), pointer_arg<int>(args, 7), f.H, f.H / f.group, f.top_k);
    return hip_check(hipGetLastError(), "launch expert_dispatch");
}
int make_dispatch(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->H = (int)v.integer("H", 0, &bad);
    // moe.py:286: 64 channels share a scale unless the record says otherwise (fp16 rows, quantised here, have one per row)
    const std::string input_kind = v.string("input_dtype", "int8", &bad);
    f->group = (int)v.integer("scale_group", input_kind == "float16" ? f->H : 64, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->H <= 0 || f->E <= 0 || f->top_k <= 0 || f->top_k > f->E || f->group <= 0 || f->H % f->group) {
        set_error("expert_dispatch: invalid MoE activation dispatch dimensions");
        return ORX_ERR_BAD_VARIANT;
    }
    // input_dtype=float16: A holds fp16 rows, quantised by the A8 rule on the way to their slots (one scale
    // per row); Scale is then not read and may be null
    const std::string input = v.string("input_dtype", "int8", &bad);
    if (bad || (input != "int8" && input != "float16") || (input == "float16" && (f->group != f->H || f->H % 8))) {
        set_error("expert_dispatch: input_dtype must be int8 or float16 (float16: one scale per row, H a multiple of 8)");
        return ORX_ERR_BAD_VARIANT;
    }
    const bool fp16_rows = input == "float16";
    f->flags = fp16_rows ? 1 : 0;
    f->args = {{"A", ArgPointer, fp16_rows ? 16u : 1u}, {"D", ArgPointer, fp16_rows ? 8u : 1u}, {"DS", ArgPointer, 2},
               {"IDs", ArgPointer, 4},        {"RelativeSlot", ArgPointer, 4}, {"RowOffsets", ArgPointer, 4},
               {"Scale", ArgPointer, fp16_rows ? 0x80000002u : 2u}, {"SlotMap", ArgPointer, 4}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = dispatch_geometry;
    f->launch = dispatch_launch;
    f->device_function = reinterpret_cast<const void*>(&expert_dispatch_kernel);
    return ORX_OK;
}

int combine_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = (uint32_t)rows;
    g->grid[1] = ceil_div((uint32_t)f.H, f.H % 8 == 0 ? 2048u : 256u);
    g->block[0] = 256;
    return ORX_OK;
}
int combine_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t s, void** args) {
    // dynamic decode has exactly top_k assignments per live row (moe.py:514-517)
    const int slots = f.dynamic_rows ? rows * f.top_k : f.slots;
    if (f.H % 8 == 0) {
        ORX_LAUNCH(moe_combine_wide_kernel, dim3(g.grid[0], g.grid[1]), dim3(256), 0, s,
                           pointer_arg<const __half>(args, 0), pointer_arg<__half>(args, 1), pointer_arg<const float>(args, 2),
                           pointer_arg<const __half>(args, 3), pointer_arg<const __half>(args, 4),
                           pointer_arg<const int>(args, 5), f.H, slots, f.top_k);
        return hip_check(hipGetLastError(), "launch moe_combine");
    }
    ORX_LAUNCH(moe_combine_kernel, dim3(g.grid[0], g.grid[1]), dim3(256), 0, s,
                       pointer_arg<const __half>(args, 0), pointer_arg<__half>(args, 1), pointer_arg<const float>(args, 2),
                       pointer_arg<const __half>(args, 3), pointer_arg<const __half>(args, 4),
                       pointer_arg<const int>(args, 5), f.H, slots, f.top_k);
    return hip_check(hipGetLastError(), "launch moe_combine");
}
int make_combine(const Variant& v, orx_function* f) {
    if (!geometry_fields(v, f, true)) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->H = (int)v.integer("H", 0, &bad);
    f->slots = (int)v.integer("slots", f->M * f->top_k, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->H <= 0 || f->slots <= 0 || f->top_k <= 0) {
        set_error("moe_combine: invalid MoE mixture dimensions");
        return ORX_ERR_BAD_VARIANT;
    }
    // Shared / SharedGate may be null device pointers: then no shared expert is added
    f->args = {{"Expert", ArgPointer, 2},     {"Output", ArgPointer, 2},           {"Prob", ArgPointer, 4},
               {"Shared", ArgPointer, 0x80000002u}, {"SharedGate", ArgPointer, 0x80000002u}, {"SlotMap", ArgPointer, 4}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = combine_geometry;
    f->launch = combine_launch;
    f->device_function = reinterpret_cast<const void*>(&moe_combine_kernel);
    return ORX_OK;
}

}  // namespace

const Registration* moe_registrations(int* count) {
    static const Registration rows[] = {
    {"router_topk", make_router, "M, E=512, top_k=10, renormalize=true, dynamic_rows=false, quantize_hidden=0",
     "IDs,Logits,Prob[,Q,S,X][,m]"},
    {"router_projection", make_router_projection, "M, H, E, dynamic_rows=false, block_m=16, block_n=32, block_k=128, stages=2",
     "Logits,SharedGate,W,X[,m]"},
    {"router_topk_warp", make_router_warp, "M, E, top_k, dynamic_rows=false, warps=4", "IDs,Logits,Prob[,m]"},
    {"expert_histogram", make_histogram, "M, E=512, top_k=10, dynamic_rows=false", "Counts,IDs,RelativeSlot[,m]"},
    {"expert_histogram_local", make_histogram_local, "M, E=512, K=10 (routes per token), block=1024|512|2048, dynamic_rows=false",
     "IDs,Partial,Slots[,m]"},
    {"expert_histogram_offsets", make_histogram_offsets, "M, E=512, K=10, block=1024|512|2048, dynamic_rows=false",
     "Counts,Offsets,Partial[,m]"},
    {"expert_histogram_finish", make_histogram_finish, "M, E=512, K=10, block=1024|512|2048, dynamic_rows=false",
     "IDs,Offsets,Slots[,m]"},
    {"expert_offsets", make_offsets, "E=512, block_m=16", "Counts,RowOffsets,TileCount,TileOffsets"},
    {"expert_tiles", make_tiles, "M, E=512, top_k=10, block_m=16", "Counts,TileExpert,TileOffsets,TileRow"},
    {"route_metadata", make_metadata, "M, E=512, top_k=10, block_m=8, dynamic_rows=false, slot_maps=false",
     "Counts,IDs,RelativeSlot[,RowMax],RowOffsets[,SlotMap,SlotToken],TileCount,TileExpert,TileOffsets,TileRow[,m]"},
    {"single_route_metadata", make_single_metadata, "E=512, top_k=10, capacity=11",
     "Counts,IDs,Offsets,Relative,TileCount,TileExpert,TileOffsets,TileRow"},
    {"expert_partition_offsets", make_partition_offsets, "experts, hot_m, cold_m, cold_rows",
     "ColdCount,ColdOffsets,Counts,RowOffsets,TileCount,TileOffsets"},
    {"expert_partition_tiles", make_partition_tiles, "M, experts, top_k, hot_m, cold_m, cold_rows, dynamic_rows=false",
     "ColdExpert,ColdOffsets,ColdRow,Counts,TileExpert,TileOffsets,TileRow[,m]"},
    {"expert_dispatch", make_dispatch, "M, H, E=512, top_k=10, scale_group=64, dynamic_rows=false, input_dtype=int8|float16 (one scale per row)",
     "A,D,DS,IDs,RelativeSlot,RowOffsets,Scale,SlotMap[,m]"},
    {"moe_combine", make_combine, "M, H, slots=M*top_k, top_k=10, dynamic_rows=false",
     "Expert,Output,Prob,Shared,SharedGate,SlotMap[,m]"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
