// int8 MFMA projections: E8P-Q4 (decode fused), single-stage E8P-Q2 experts (grouped) and W8A8.
//
// Reference counterparts: kernels/cuda/model/integer_core.py:162-272 (tile loop, weight loader,
// epilogue), kernels/cuda/model/e8p_q4.py:143-264 (Q4 projection + ABI), int8_projection.py:15-62
// (W8A8 ABI), integer_vq.py:58-260 / e8p_decode.py:36-245 (routed Q2 ABI), e8p_q4.py:267-302
// (unpack).  Arithmetic: exact int32 accumulation over full K, then (float(acc)*ws)*as.
//
// MI355X design.  A workgroup of four wave64 owns a BM x BN output tile and walks K in steps
// of 128.  Activations go HBM -> registers -> LDS as int8; weight codes go HBM -> registers,
// are decoded with two 8-byte LDS table reads and XORs per code (e8p_device.h), and land in
// LDS as an int8 [BN][128] tile, so v_mfma_i32_32x32x32_i8 reads both operands as 16-byte,
// K-contiguous lane fragments.  Rows in LDS are padded to 144 bytes so that the sixteen lanes of
// one ds_read_b128 phase hit distinct banks.  Global loads for tile t+1 are issued before the
// MFMAs of tile t.  Grouped (expert) tiles take (expert, first row, count) from device lists.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "e8p_device.h"
#include "orx_internal.h"
#include "row_q4_device.h"

namespace orx {

// from k_gemv.hip
int gemv_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out,
                const int8_t* signs = nullptr);
int gemv_geometry_for(const orx_function& f, int rows, Geometry* g);
int gemv_configure(orx_function* f, int codec, int passes_override);
int gemv_prepare_device();
bool gemv_serves_k_major(const orx_function& f, int rows);
bool gemv_serves_fp16_input(const orx_function& f);
// from k_stream.hip
void stream_geometry(int n, Geometry* g);
int stream_launch(int codec, const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                  void* out, int rows, int n, int k, int stride, int packed_k, bool out_f32, hipStream_t stream);
int stream_row_q4_launch(const int8_t* a, const void* w, uint32_t magnitudes_low, uint32_t magnitudes_high, const __half* ws,
                         const __half* as, void* out, int rows, int n, int k, int stride, bool out_f32, hipStream_t stream);
// from k_rowq4.hip
bool row_q4_gemv_serves(int rows, int k);
void row_q4_gemv_geometry(int rows, int n, int k, Geometry* g);
int row_q4_gemv_launch(const int8_t* a, const void* w, uint32_t low, uint32_t high, const __half* ws, const __half* as, void* out,
                       int rows, int n, int k, int stride, bool out_f32, const Geometry& g, hipStream_t stream);
void stream_grouped_geometry(int n, int tiles, Geometry* g);
bool dense_resident_eligible(int n, int k, int packed_k);
void dense_resident_geometry(int rows, int n, int k, int packed_k, Geometry* g);
int dense_resident_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                          void* out, int rows, int n, int k, int stride, int packed_k, bool out_f32, hipStream_t stream);
bool dense_wide_eligible(int n, int k, int packed_k);
void dense_wide_geometry(int n, Geometry* g);
int dense_wide_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out,
                      int rows, int n, int k, int stride, int packed_k, int out_f32, const Geometry& g, hipStream_t stream);
bool grouped_resident_eligible(int n, int k, int block_m, int tiles, int input, int epilogue, int slots);
bool grouped_resident_preferred(int rows, int experts, int n);
void grouped_resident_geometry(int k, int input, int epilogue, int slots, Geometry* g);
int grouped_resident_launch(const GroupedBuffers& b, int n, int k, int tiles, int packed_k, int input, int epilogue,
                            int slots, hipStream_t stream);
int stream_grouped_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                          void* out, const int* counts, const int* offsets, const int* tile_expert, const int* tile_row,
                          const int* tile_count, int n, int k, int tiles, int block_m, int packed_k,
                          hipStream_t stream);
// from k_gemm_big.hip
void gemm_big_geometry(int rows, int n, Geometry* g);
int q4_expand_launch(const void* codes, const uint32_t* book, void* weights, int n, int k, int packed_k,
                     hipStream_t stream);
void gemm_tall_geometry(int rows, int n, Geometry* g);
uint32_t gemm_tall_units(int n);
int gemm_tall_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out,
                     int rows, int n, int k, int stride, int packed_k, bool out_f32, const Geometry& g, hipStream_t stream);
int gemm_big_launch(const int8_t* a, const void* w, const __half* ws, const __half* as, void* out, int rows, int n,
                    int k, int stride, bool out_f32, const Geometry& g, hipStream_t stream);

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
// Register arrays hold the native vector type: an array of HIP's uint4 struct that is filled in
// one lambda and read in another is kept in scratch memory by the compiler.
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum Codec { kQ4 = 0, kQ2 = 1, kW8 = 2, kS4 = 3 };  // kS4: row-scaled scalar Q4 nibbles (q4_projection.py)
enum Algorithm { kAuto = 0, kGemv = 1, kMfma = 2, kStream = 3, kResident = 4, kWide = 5, kTall = 6 };
// orx_function::flags2 of a projection.  kPreferGemv / kNoGemv: the reference's schedule names as hints among the
// library's own kernels (algorithm=dp4a: its dot-product schedule for few rows; tensor_core: its matrix-unit one).
enum Flags2 { kNoSplit = 1, kNoExpand = 2, kPreferGemv = 4, kNoGemv = 8 };

constexpr int kBK = 128;        // K bytes per tile step
constexpr int kPitch = kBK + 16;  // LDS row pitch in bytes

struct GemmParams {
    const int8_t* a;
    const void* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, m;
    int packed_k;  // 0 row-major codes, 128 or 64 K-major blocks
    int out_f32;
    // grouped only
    const int* counts;
    const int* offsets;
    const int* tile_expert;
    const int* tile_row;
    const int* tile_count;
    int64_t expert_weight_stride;  // bytes between experts in w
    int tile_rows;                 // rows a routed tile may hold (0: the kernel's own tile height)
    int list_split;                // workgroups per listed tile when its rows exceed the kernel's tile (0 or 1: one)
    int* partials;                 // split launches: int32 partial tiles, two slots per workgroup
    const void* w2;                // gate/up + SwiGLU: the Up matrix (w is Gate) and its scales
    const __half* ws2;
    // routed single-stage codes, general form
    const uint16_t* patch;         // (E, K/128, N) patch words or null
    int book_stride;               // words between the experts' tables (0: one table for all)
    int book_form;                 // BookForm of the general decode: selector words, raw int8 basis, signed values
    int direct_rows;               // > 0: no tile list; expert blockIdx.z owns rows [z * direct_rows, (z + 1) * direct_rows)
    uint32_t magnitudes_low, magnitudes_high;  // scalar Q4: the eight magnitudes, one per byte
};

template <int CODEC>
struct Tables {
    typedef Q4ByteTables type;
};
template <>
struct Tables<kQ2> {
    typedef Q2ByteTables type;
};
template <>
struct Tables<kW8> {
    struct type {};
};
template <>
struct Tables<kS4> {
    struct type {};
};

// Number of 16-byte global chunks of weight stream per output row per K step.
template <int CODEC>
__host__ __device__ constexpr int weight_chunks() {
    return CODEC == kQ4 || CODEC == kS4 ? 4 : CODEC == kQ2 ? 2 : 8;
}

// SWIGLU (W8 only): the tile's 128 weight rows are 64 Gate channels followed by the same 64 Up channels,
// a wave's two column blocks are gate and up of the same 32 channels, and the epilogue rounds both
// projections to fp16 and stores fp16(g / (1 + exp(-g)) * u) (int8_swiglu.py:10-57 with
// integer_core.py:19-28, 261-264): no intermediate leaves the workgroup.
//
// GENERAL (routed single-stage codes only; kernels/cuda/model/integer_vq.py:111-214): the selector table may
// hold zero coordinates and may differ per expert (`book_stride`), the K-major blocks may be 64 wide, and
// one weight per row and 128-wide K group may be overridden by a patch word: bit 15 valid, bits 7-14 the
// int8 value, bits 0-6 the position in the group (integer_vq.py:193-202, quantization/vq.py:184-194).
template <int CODEC, int BM, int BN, int WAVES_M, bool GROUPED, bool SWIGLU = false, bool GENERAL = false>
__global__ __launch_bounds__(256) void gemm_kernel(GemmParams p) {
    constexpr int WAVES_N = 4 / WAVES_M;
    static_assert(!SWIGLU || (CODEC == kW8 && !GROUPED && BN == 128 && WAVES_N == 2), "gate/up tile shape");
    static_assert(!GENERAL || (CODEC == kQ2 && GROUPED && !SWIGLU), "the general decode is the routed single-stage one");
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile must hold at least one 32x32 block");
    constexpr int A_CHUNKS = BM * 8 / 256;                        // uint4 per thread for A
    constexpr int W_CHUNKS = BN * weight_chunks<CODEC>() / 256;   // uint4 per thread for weights
    static_assert(A_CHUNKS >= 1 && W_CHUNKS >= 1, "tile too small for 256 threads");

    __shared__ __align__(16) int8_t lds_a[BM * kPitch];
    __shared__ __align__(16) int8_t lds_w[BN * kPitch];
    __shared__ typename std::conditional<GENERAL, Q2GeneralTables, typename Tables<CODEC>::type>::type tables;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int n0 = blockIdx.x * (SWIGLU ? BN / 2 : BN);
    int row0, rows_here;
    const int8_t* w_base = reinterpret_cast<const int8_t*>(p.w);
    const __half* ws = p.ws;
    const uint32_t* book = p.book;
    const uint16_t* patch = nullptr;
    if (GROUPED) {
        int expert, first;
        if (GENERAL && p.direct_rows > 0) {  // every expert has the same number of rows (integer_vq.py:217-228)
            expert = blockIdx.z, first = blockIdx.y * BM;
            row0 = expert * p.direct_rows + first;
            rows_here = min(BM, p.direct_rows - first);
        } else {
            const int split = p.list_split > 1 ? p.list_split : 1;  // a listed tile of split * BM rows: one workgroup per BM
            const int tile = split > 1 ? blockIdx.y / split : blockIdx.y;
            if (tile >= p.tile_count[0]) return;
            expert = p.tile_expert[tile];
            first = p.tile_row[tile] + (split > 1 ? (int)(blockIdx.y % split) * BM : 0);
            row0 = p.offsets[expert] + first;
            rows_here = min(p.tile_rows > 0 ? min(BM, p.tile_rows) : BM, p.counts[expert] - first);
        }
        if (rows_here <= 0) return;
        w_base += (int64_t)expert * p.expert_weight_stride;
        ws += (int64_t)expert * p.n;
        if constexpr (GENERAL) {
            book += (int64_t)expert * p.book_stride;
            if (p.patch != nullptr) patch = p.patch + (int64_t)expert * (p.k / kBK) * p.n;
        }
    } else {
        row0 = blockIdx.y * BM;
        rows_here = min(BM, p.m - row0);
    }

    if constexpr (GENERAL)
        build_tables(tables, book, p.book_form, tid, 256);
    else if constexpr (CODEC == kQ4 || CODEC == kQ2)
        build_tables(tables, book, tid, 256);

    // int8 weights may end in half a K step (K a multiple of 64, int8_projection.py:29): the missing halves of
    // both operands are zeros.  Codes always come in whole steps.
    const int k_tiles = CODEC == kW8 ? (p.k + kBK - 1) / kBK : p.k / kBK;
    v4u held_a[A_CHUNKS], held_w[W_CHUNKS];
    const v4u zero_chunk = {0u, 0u, 0u, 0u};

    auto load_tile = [&](int kt, v4u (&reg_a)[A_CHUNKS], v4u (&reg_w)[W_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            const int r = min(c >> 3, rows_here - 1), kc = c & 7;
            if (CODEC == kW8 && kt * kBK + kc * 16 >= p.k)
                reg_a[i] = zero_chunk;
            else
                reg_a[i] = *reinterpret_cast<const v4u*>(p.a + (int64_t)(row0 + r) * p.k + kt * kBK + kc * 16);
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            constexpr int PER_ROW = weight_chunks<CODEC>();
            if constexpr (SWIGLU) {
                const int r = c / PER_ROW, q = c % PER_ROW;
                const int nn = min(n0 + (r & 63), p.n - 1);
                const int8_t* side = reinterpret_cast<const int8_t*>(r < 64 ? p.w : p.w2);
                reg_w[i] = *reinterpret_cast<const v4u*>(side + (int64_t)nn * p.k + kt * kBK + q * 16);
                continue;
            }
            const int nn = min(n0 + c / PER_ROW, p.n - 1), q = c % PER_ROW;
            int64_t byte;
            if (CODEC == kW8 && kt * kBK + q * 16 >= p.k) {
                reg_w[i] = zero_chunk;
                continue;
            }
            if (CODEC == kW8)
                byte = (int64_t)nn * p.k + kt * kBK + q * 16;
            else if (p.packed_k == 128)  // (K/128, N, 16 codes): one block row is PER_ROW*16 bytes
                byte = ((int64_t)kt * p.n + nn) * (PER_ROW * 16) + q * 16;
            else if (p.packed_k == 64)  // (K/64, N, 8 codes): two block rows per K step
                byte = CODEC == kQ2 ? ((int64_t)(kt * 2 + q) * p.n + nn) * 16 : q4_k_major_chunk(64, p.n, nn, kt, q);
            else  // (N, K/8 codes)
                byte = ((int64_t)nn * k_tiles + kt) * (PER_ROW * 16) + q * 16;
            reg_w[i] = *reinterpret_cast<const v4u*>(w_base + byte);
        }
    };

    auto store_tile = [&](int kt, const v4u (&reg_a)[A_CHUNKS], const v4u (&reg_w)[W_CHUNKS]) {
        (void)kt;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            *reinterpret_cast<v4u*>(lds_a + (c >> 3) * kPitch + (c & 7) * 16) = reg_a[i];
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            constexpr int PER_ROW = weight_chunks<CODEC>();
            const int nn = c / PER_ROW, q = c % PER_ROW;
            if constexpr (CODEC == kW8) {
                *reinterpret_cast<v4u*>(lds_w + nn * kPitch + q * 16) = reg_w[i];
            } else if constexpr (CODEC == kS4) {
                // 64 nibbles -> 32 weights at k offset q*32
                const uint32_t in[4] = {reg_w[i].x, reg_w[i].y, reg_w[i].z, reg_w[i].w};
                uint32_t out[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    out[2 * j] = decode_row_q4(in[j], p.magnitudes_low, p.magnitudes_high);
                    out[2 * j + 1] = decode_row_q4(in[j] >> 16, p.magnitudes_low, p.magnitudes_high);
                }
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 32);
                dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
                dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
            } else if constexpr (CODEC == kQ4) {
                // 4 u32 codes -> 32 weights at k offset q*32
                const uint2 d0 = decode_q4(tables, reg_w[i].x), d1 = decode_q4(tables, reg_w[i].y);
                const uint2 d2 = decode_q4(tables, reg_w[i].z), d3 = decode_q4(tables, reg_w[i].w);
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 32);
                dst[0] = make_uint4(d0.x, d0.y, d1.x, d1.y);
                dst[1] = make_uint4(d2.x, d2.y, d3.x, d3.y);
            } else {
                // 8 u16 codes -> 64 weights at k offset q*64
                const uint32_t pair[4] = {reg_w[i].x, reg_w[i].y, reg_w[i].z, reg_w[i].w};
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 64);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint2 lo = decode_q2(tables, pair[j] & 0xFFFFu), hi = decode_q2(tables, pair[j] >> 16);
                    dst[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
                }
                if constexpr (GENERAL) {
                    // the thread that decoded the half group a patch points into overwrites that weight
                    // (its own earlier stores to LDS are ordered before this one)
                    if (patch != nullptr && n0 + nn < p.n) {
                        const uint32_t word = patch[(int64_t)kt * p.n + n0 + nn];
                        if ((word & 0x8000u) && ((word & 127u) >> 6) == (uint32_t)q)
                            lds_w[nn * kPitch + (word & 127u)] = (int8_t)((word >> 7) & 255u);
                    }
                }
            }
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    load_tile(0, held_a, held_w);
    __syncthreads();  // tables ready
    for (int kt = 0; kt < k_tiles; ++kt) {
        store_tile(kt, held_a, held_w);
        __syncthreads();
        if (kt + 1 < k_tiles) load_tile(kt + 1, held_a, held_w);
        const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
#pragma unroll
        for (int ks = 0; ks < kBK / 32; ++ks) {
            v4i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *reinterpret_cast<const v4i*>(lds_a + ((wave_m * TM + i) * 32 + frag_row) * kPitch + ks * 32 + frag_k);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *reinterpret_cast<const v4i*>(lds_w + ((SWIGLU ? j * 2 + wave_n : wave_n * TN + j) * 32 + frag_row) * kPitch + ks * 32 + frag_k);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane&31) and rows 8*(r/4) + 4*(lane>>5) + r%4 of each 32x32 block
    if constexpr (SWIGLU) {
        const int col = n0 + wave_n * 32 + (lane & 31);
        if (col >= p.n) return;
        const float gate_scale = __half2float(ws[col]), up_scale = __half2float(p.ws2[col]);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int local = (wave_m * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (local < rows_here) {
                    const int64_t row = row0 + local;
                    const float token = __half2float(p.as[row]);
                    const float g = __half2float(__float2half_rn(rescale(acc[i][0][r], gate_scale, token)));
                    const float u = __half2float(__float2half_rn(rescale(acc[i][1][r], up_scale, token)));
                    float value = __fdiv_rn(g, 1.0f + expf(-g)) * u;
                    asm volatile("" : "+v"(value));  // the cast rounds the fp32 product, never a fused multiply-convert
                    reinterpret_cast<__half*>(p.out)[row * p.stride + col] = __float2half_rn(value);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0 + (wave_n * TN + j) * 32 + (lane & 31);
        if (col >= p.n) continue;
        const float wscale = __half2float(ws[col]);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int local = (wave_m * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
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

// ---- the same tiles with the K steps dealt evenly to the workgroups ------------------------------
// With a few hundred output tiles for 256 CUs (N = 17408 at 128 rows: 136 tiles) whole tiles leave
// CUs idle or give some CUs twice the work, and a CU's share of the memory system bounds its tile.
// Here the (tile, K step) units are numbered tile-major and workgroup g of G takes units
// [g U / G, (g + 1) U / G): every CU pulls the same number of bytes.  A run of units that covers a
// whole tile is finished in place; any other run leaves its int32 accumulators in one of the
// workgroup's two partial slots (first run, last run), and gemm_split_finish_kernel adds the runs of
// each tile (exact: integers) and rescales.  No atomics, no waiting between workgroups.
constexpr int kSplitTile = 128;
constexpr int kSplitSlotInts = kSplitTile * kSplitTile;

__device__ __forceinline__ int64_t split_begin(int64_t units, int g, int groups) { return units * g / groups; }

template <int CODEC>
__global__ __launch_bounds__(256) void gemm_split_kernel(GemmParams p) {
    constexpr int BM = kSplitTile, BN = kSplitTile, WAVES_M = 2;
    constexpr int WAVES_N = 4 / WAVES_M;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile must hold at least one 32x32 block");
    constexpr int A_CHUNKS = BM * 8 / 256;                        // uint4 per thread for A
    constexpr int W_CHUNKS = BN * weight_chunks<CODEC>() / 256;   // uint4 per thread for weights
    static_assert(A_CHUNKS >= 1 && W_CHUNKS >= 1, "tile too small for 256 threads");

    __shared__ __align__(16) int8_t lds_a[BM * kPitch];
    __shared__ __align__(16) int8_t lds_w[BN * kPitch];
    __shared__ typename Tables<CODEC>::type tables;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int8_t* w_base = reinterpret_cast<const int8_t*>(p.w);
    const __half* ws = p.ws;
    const int tiles_n = (p.n + BN - 1) / BN, tiles_m = (p.m + BM - 1) / BM;
    const int64_t units = (int64_t)tiles_m * tiles_n * (p.k / kBK);
    const int64_t unit_begin = split_begin(units, blockIdx.x, gridDim.x), unit_end = split_begin(units, blockIdx.x + 1, gridDim.x);
    int n0 = 0, row0 = 0, rows_here = 1;

    if constexpr (CODEC == kQ4 || CODEC == kQ2) build_tables(tables, p.book, tid, 256);

    const int k_tiles = p.k / kBK;
    v4u held_a[A_CHUNKS], held_w[W_CHUNKS];

    auto load_tile = [&](int kt, v4u (&reg_a)[A_CHUNKS], v4u (&reg_w)[W_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            const int r = min(c >> 3, rows_here - 1), kc = c & 7;
            reg_a[i] = *reinterpret_cast<const v4u*>(p.a + (int64_t)(row0 + r) * p.k + kt * kBK + kc * 16);
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            constexpr int PER_ROW = weight_chunks<CODEC>();
            const int nn = min(n0 + c / PER_ROW, p.n - 1), q = c % PER_ROW;
            int64_t byte;
            if (CODEC == kW8)
                byte = (int64_t)nn * p.k + kt * kBK + q * 16;
            else if (p.packed_k == 128)  // (K/128, N, 16 codes): one block row is PER_ROW*16 bytes
                byte = ((int64_t)kt * p.n + nn) * (PER_ROW * 16) + q * 16;
            else if (p.packed_k == 64)  // (K/64, N, 8 two-stage codes): two block rows per K step
                byte = q4_k_major_chunk(64, p.n, nn, kt, q);
            else  // (N, K/8 codes)
                byte = ((int64_t)nn * k_tiles + kt) * (PER_ROW * 16) + q * 16;
            reg_w[i] = *reinterpret_cast<const v4u*>(w_base + byte);
        }
    };

    auto store_tile = [&](const v4u (&reg_a)[A_CHUNKS], const v4u (&reg_w)[W_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            *reinterpret_cast<v4u*>(lds_a + (c >> 3) * kPitch + (c & 7) * 16) = reg_a[i];
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i;
            constexpr int PER_ROW = weight_chunks<CODEC>();
            const int nn = c / PER_ROW, q = c % PER_ROW;
            if constexpr (CODEC == kW8) {
                *reinterpret_cast<v4u*>(lds_w + nn * kPitch + q * 16) = reg_w[i];
            } else if constexpr (CODEC == kS4) {
                // 64 nibbles -> 32 weights at k offset q*32
                const uint32_t in[4] = {reg_w[i].x, reg_w[i].y, reg_w[i].z, reg_w[i].w};
                uint32_t out[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    out[2 * j] = decode_row_q4(in[j], p.magnitudes_low, p.magnitudes_high);
                    out[2 * j + 1] = decode_row_q4(in[j] >> 16, p.magnitudes_low, p.magnitudes_high);
                }
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 32);
                dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
                dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
            } else if constexpr (CODEC == kQ4) {
                // 4 u32 codes -> 32 weights at k offset q*32
                const uint2 d0 = decode_q4(tables, reg_w[i].x), d1 = decode_q4(tables, reg_w[i].y);
                const uint2 d2 = decode_q4(tables, reg_w[i].z), d3 = decode_q4(tables, reg_w[i].w);
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 32);
                dst[0] = make_uint4(d0.x, d0.y, d1.x, d1.y);
                dst[1] = make_uint4(d2.x, d2.y, d3.x, d3.y);
            } else {
                // 8 u16 codes -> 64 weights at k offset q*64
                const uint32_t pair[4] = {reg_w[i].x, reg_w[i].y, reg_w[i].z, reg_w[i].w};
                uint4* dst = reinterpret_cast<uint4*>(lds_w + nn * kPitch + q * 64);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint2 lo = decode_q2(tables, pair[j] & 0xFFFFu), hi = decode_q2(tables, pair[j] >> 16);
                    dst[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
                }
            }
        }
    };

    __syncthreads();  // tables ready
    for (int64_t unit = unit_begin; unit < unit_end;) {
        const int tile = (int)(unit / k_tiles), kt_begin = (int)(unit - (int64_t)tile * k_tiles);
        const int kt_end = (int)min((int64_t)k_tiles, kt_begin + (unit_end - unit));
        n0 = (tile % tiles_n) * BN;
        row0 = (tile / tiles_n) * BM;
        rows_here = min(BM, p.m - row0);
        v16i acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

        load_tile(kt_begin, held_a, held_w);
        for (int kt = kt_begin; kt < kt_end; ++kt) {
            store_tile(held_a, held_w);
            __syncthreads();
            if (kt + 1 < kt_end) load_tile(kt + 1, held_a, held_w);
            const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
#pragma unroll
            for (int ks = 0; ks < kBK / 32; ++ks) {
                v4i fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    fa[i] = *reinterpret_cast<const v4i*>(lds_a + ((wave_m * TM + i) * 32 + frag_row) * kPitch + ks * 32 + frag_k);
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    fb[j] = *reinterpret_cast<const v4i*>(lds_w + ((wave_n * TN + j) * 32 + frag_row) * kPitch + ks * 32 + frag_k);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
            __syncthreads();
        }
        const bool whole = kt_begin == 0 && kt_end == k_tiles;
        if (!whole) {
            // accumulator (i, j, r) of thread tid at ((i TN + j) 16 + r) 256 + tid: 1 KiB per store instruction
            int* slot = p.partials + ((int64_t)blockIdx.x * 2 + (unit == unit_begin ? 0 : 1)) * kSplitSlotInts;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) slot[((i * TN + j) * 16 + r) * 256 + tid] = acc[i][j][r];
        } else {
    // epilogue: lane holds column (lane&31) and rows 8*(r/4) + 4*(lane>>5) + r%4 of each 32x32 block
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0 + (wave_n * TN + j) * 32 + (lane & 31);
        if (col >= p.n) continue;
        const float wscale = __half2float(ws[col]);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int local = (wave_m * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
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
        unit += kt_end - kt_begin;
    }
}

// Four workgroups per output tile, one per 32 x 32 block of every wave's 64 x 64: nothing to do when
// one run covered the tile, else the sum of the tile's runs (in workgroup order) goes through the same
// rescale and store as above.  A thread has 16 sums, so all loads of a run are in flight at once.
__global__ __launch_bounds__(256) void gemm_split_finish_kernel(GemmParams p, int groups) {
    constexpr int BM = kSplitTile, BN = kSplitTile, WAVES_N = 2, TM = 2, TN = 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int tiles_n = (p.n + BN - 1) / BN, tiles_m = (p.m + BM - 1) / BM;
    const int k_tiles = p.k / kBK;
    const int64_t units = (int64_t)tiles_m * tiles_n * k_tiles;
    const int tile = blockIdx.x >> 2, i = (blockIdx.x >> 1) & 1, j = blockIdx.x & 1;
    const int64_t first = (int64_t)tile * k_tiles, last = first + k_tiles;
    int g = (int)(first * groups / units);
    while (g > 0 && split_begin(units, g, groups) > first) --g;
    while (split_begin(units, g + 1, groups) <= first) ++g;
    if (split_begin(units, g, groups) <= first && split_begin(units, g + 1, groups) >= last) return;  // one run: done in place
    int acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    for (; g < groups && split_begin(units, g, groups) < last; ++g) {
        const int64_t begin = split_begin(units, g, groups);
        if (split_begin(units, g + 1, groups) == begin) continue;  // fewer units than workgroups: this one had none
        const int64_t run_start = begin > first ? begin : first;
        const int* slot = p.partials + ((int64_t)g * 2 + (run_start == begin ? 0 : 1)) * kSplitSlotInts;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] += slot[((i * TN + j) * 16 + r) * 256 + tid];
    }
    const int n0 = (tile % tiles_n) * BN, row0 = (tile / tiles_n) * BM;
    const int rows_here = min(BM, p.m - row0);
    const int col = n0 + (wave_n * TN + j) * 32 + (lane & 31);
    if (col >= p.n) return;
    const float wscale = __half2float(p.ws[col]);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int local = (wave_m * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (local < rows_here) {
            const int64_t row = row0 + local;
            const float value = rescale(acc[r], wscale, __half2float(p.as[row]));
            if (p.out_f32)
                reinterpret_cast<float*>(p.out)[row * p.stride + col] = value;
            else
                reinterpret_cast<__half*>(p.out)[row * p.stride + col] = __float2half_rn(value);
        }
    }
}

// Whole-matrix decode to int8 (diagnostic; e8p_q4.py:267-302).  One thread per code.
template <int CODEC>
__global__ __launch_bounds__(256) void unpack_kernel(const void* __restrict__ w, const uint32_t* __restrict__ book,
                                                     uint2* __restrict__ out, int n, int k, int packed_k,
                                                     const int* __restrict__ counts) {
    // banks of routed experts (grid y): only the experts that have rows are decoded (kernels/cuda/model/moe.py:147-173)
    if (counts != nullptr) {
        if (counts[blockIdx.y] <= 0) return;
        w = reinterpret_cast<const int8_t*>(w) + (int64_t)blockIdx.y * n * (k / 8) * (CODEC == kQ4 ? 4 : 2);
        out += (int64_t)blockIdx.y * n * (k / 8);
    }
    __shared__ typename Tables<CODEC>::type tables;
    build_tables(tables, book, threadIdx.x, 256);
    __syncthreads();
    const int64_t total = (int64_t)n * (k / 8);
    const int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= total) return;
    const int row = (int)(index / (k / 8)), vec = (int)(index % (k / 8));
    int64_t src = index;
    if (packed_k) {
        const int per = packed_k / 8;
        src = ((int64_t)(vec / per) * n + row) * per + vec % per;
    }
    if constexpr (CODEC == kQ4)
        out[index] = decode_q4(tables, reinterpret_cast<const uint32_t*>(w)[src]);
    else
        out[index] = decode_q2(tables, reinterpret_cast<const uint16_t*>(w)[src]);
}

// ---- host side -----------------------------------------------------------------------------
// slots: M/capacity, N, K, stride, packed_k, algorithm, block_m (gemv passes), flags (codec),
// E/tiles (grouped), out_f32.

int pick_bm(int rows) { return rows <= 32 ? 32 : rows <= 64 ? 64 : 128; }

template <int CODEC, bool GROUPED>
int launch_mfma(int bm, const GemmParams& p, const Geometry& g, hipStream_t stream) {
    const dim3 grid(g.grid[0], g.grid[1]), block(256);
    switch (bm) {
        case 32:
            ORX_LAUNCH((gemm_kernel<CODEC, 32, 128, 1, GROUPED>), grid, block, 0, stream, p);
            break;
        case 64:
            ORX_LAUNCH((gemm_kernel<CODEC, 64, 128, 2, GROUPED>), grid, block, 0, stream, p);
            break;
        default:
            ORX_LAUNCH((gemm_kernel<CODEC, 128, 128, 2, GROUPED>), grid, block, 0, stream, p);
            break;
    }
    return hip_check(hipGetLastError(), "launch projection (mfma)");
}

// routed single-stage codes, general decode (any selector table, per-expert tables, patches, 64-wide blocks)
int launch_mfma_general(int bm, const GemmParams& p, const Geometry& g, hipStream_t stream) {
    const dim3 grid(g.grid[0], g.grid[1], g.grid[2]), block(256);
    if (bm <= 32)
        ORX_LAUNCH((gemm_kernel<kQ2, 32, 128, 1, true, false, true>), grid, block, 0, stream, p);
    else if (bm == 64)
        ORX_LAUNCH((gemm_kernel<kQ2, 64, 128, 2, true, false, true>), grid, block, 0, stream, p);
    else
        ORX_LAUNCH((gemm_kernel<kQ2, 128, 128, 2, true, false, true>), grid, block, 0, stream, p);
    return hip_check(hipGetLastError(), "launch routed projection (general decode)");
}

// Row tile asked for at `rows` live rows: a block_m this library has a tile for (32, 64, 128, 256) holds at every row
// count; a reference-only tile (16, 96, 192) was chosen for launches of about that many rows, so it names the tile
// that holds it (32, 128, 256) while the live rows fit one such tile, and beyond that the row count decides.
int tile_for(const orx_function& f, int rows) {
    if (f.tiles) return f.tiles;
    return f.tile_hint && rows <= f.tile_hint ? f.tile_hint : 0;
}

// Channel runs per CU over the whole K (k_wide.hip): two-stage codes, `algorithm=wide` by name, and by
// `auto` at 65..128 rows (33..64 rows of large matrices) while K is short enough.  Its time is 10 us + 0.4..0.55 us per K step of 128 whatever
// N is (up to 96 channels per CU), where the split 128 x 128 tiles pay for N K: measured at 65-128 rows,
// K-major and row-major alike, K = 1024: 9 against 23 us (N = 1024); 2560: 16-17 against 26-28 (N = 9728);
// 4096: 20-23 against 29 (N = 11008), 17-20 against 23 (N = 4096); 5120: 31-32 against 40 (N = 17408),
// 21-25 against 27-30 (N = 5120, 7168), 55-62 against 62-63 (N = 34816); 8192: 30-36 against 32 (N = 8192),
// 70-83 against 72-74 (N = 28672); 9728 and up: slower (N = 5120, K = 17408: 56-69 against 41).  Below 65
// rows the batched-decode kernels are as fast or faster except at N = 17408 (30 against 31-34 us), above 128
// rows a second pass doubles the time (58-62 against 57 us at 160-256 rows).
bool use_wide(const orx_function& f, int rows) {
    if (f.flags != kQ4 || !dense_wide_eligible(f.N, f.K, f.packed_k)) return false;
    if (f.algorithm == kWide) return true;
    if (f.algorithm != kAuto || tile_for(f, rows) != 0 || f.K > 6144) return false;
    if (rows >= 65 && rows <= 128) return true;
    // 33..64 rows of a large matrix would be two batched-decode launches: one pass here is faster while a CU's
    // run fits one channel pass (N = 17408, K = 5120: 29.9 / 30.2 / 30.4 us at 33 / 48 / 64 rows against 31.2 / 31.8 /
    // 34.3; N = 34816, two channel passes: 51-53 against 49-54, left alone)
    return rows >= 33 && rows <= 64 && (int64_t)f.N * f.K >= ((int64_t)1 << 26) && f.N <= 96 * device_compute_units();
}

// Two-stage codes on 512 rows x channel runs with the decode in the K loop (k_gemm_big.hip): `algorithm=tall` by
// name, and `auto` from 257 (the widest matrices: 129) to 512 rows, with or without scratch, when the runs fill
// their five blocks of 16 channels well enough.  A launch costs 0.76 us per 64 of K and round of the CUs whatever N is (every CU reads all
// token rows), so it pays when the matrix gives every CU enough channels.  Measured against the kernels `auto` had
// at 384 / 512 rows (128 x 128 tiles / decode once + 256 x 256 tiles; us, 256 CUs): N x K = 17408 x 5120 (4.25
// blocks per CU) 64 / 66 against 77 / 86, 34816 x 5120 (two rounds of 4.25) 131 / 135 against 142 / 158,
// 14336 x 4096 (3.5) 52 / 53 against 64 / 65, 12288 x 3072 (3) 41 / 42 against 46 / 55, 9728 x 2560 (2.4) 35 / 34
// against 40 / 44; 7168 x 5120 (1.75) 59 / 59 against 44 / 51, 28672 x 8192 (two rounds of 3.5) 189 / 194 against
// 158 / 194.  At 129..256 rows the runs cost what they cost at 512 and the 128 x 128 tiles half as much: only a
// matrix with 4.25 blocks per CU in one round gains (17408 x 5120 at 130 / 192 / 256 rows: 56 / 57 / 56 us against
// 57 / 59 / 59 for the split tiles and 69 / 76 / 76 for whole tiles, what a handle without scratch had; 14336 x 4096
// at 3.5 blocks per CU: 51 against 45 and 47).
bool tall_runs_fill(int n, int rows) {
    const int64_t blocks = ceil_div((uint32_t)n, 16u), cus = device_compute_units();
    const int64_t rounds = (blocks + 5 * cus - 1) / (5 * cus);
    if (rows <= 256) return rounds == 1 && 4 * blocks >= 17 * cus;
    return rounds == 1 ? 4 * blocks >= 9 * cus : blocks >= 4 * rounds * cus;
}
bool use_tall(const orx_function& f, int rows) {
    if (f.flags != kQ4) return false;
    if (f.algorithm == kTall) return true;
    if (f.algorithm != kAuto || tile_for(f, rows) != 0 || f.K % 128 != 0 || f.K < 256) return false;
    return rows > 128 && rows <= 512 && tall_runs_fill(f.N, rows);
}

bool use_resident(const orx_function& f, int rows);
bool use_gemv(const orx_function& f, int rows) {
    if (use_wide(f, rows) || use_tall(f, rows)) return false;
    if (f.algorithm == kGemv) return true;
    if (f.algorithm != kAuto) return false;
    if (f.flags2 & kNoGemv) return false;  // the matrix-unit kernels were asked for: streaming / batched-decode from row 1
    if ((f.flags2 & kPreferGemv) && f.block_m > 0 && f.tiles == 0)  // the dot-product family wherever it serves the rows
        return rows <= (f.flags == kW8 ? 2 : 4) && (f.packed_k == 0 || (rows <= 2 && gemv_serves_k_major(f, rows)));
    // K-major codes: 1 row (13.4 us at N=17408, K=5120; the streaming kernel takes 17.2), and 2 rows
    // (16.4 us) where the batched-decode kernel (15.4 us) does not take the shape
    if (f.packed_k != 0) return rows <= 2 && gemv_serves_k_major(f, rows) && !use_resident(f, rows);
    // W8: 3 and 4 rows go to the streaming kernel (N = 5120, K = 17408: 25.9 us there against 32.2 us here)
    return rows <= (f.flags == kW8 ? 2 : 4) && !use_resident(f, rows);
}

// weight-streaming kernel for up to 64 rows.  Two-stage codes of 65..128 rows go to the 128x128
// MFMA tiles with the decode inside (measured at N=17408, K=5120, 128 rows: 59 us against 91 us for
// two streaming launches and 118 us for the 256x256 kernel).  W8 leaves the streaming kernel above
// 16 rows: the 32/64/128-row tiles measure 27 / 31 / 40 us at 32 / 48 / 128 rows against 29 / 43 / 94.
bool use_stream(const orx_function& f, int rows) {
    if (f.algorithm == kStream) return rows <= 64;
    if (f.algorithm != kAuto || tile_for(f, rows) != 0) return false;
    if (f.flags == kQ4) return rows <= 64;
    // W8 with weights that do not stay in cache: up to 32 rows (N = 17408, K = 5120 at 32 rows: 34.8 us
    // against 39.0 us for the 32-row tiles; at 48 rows 49.0 against 42.5), up to 64 rows for matrices of
    // at most 32 M weights (N = K = 4096 at 64 rows: 14.7 against 19.5 us)
    return rows <= 32 || (rows <= 64 && (int64_t)f.N * f.K <= (int64_t)1 << 25);
}

// Resident two-stage kernel (32 rows per launch) where the streaming kernel would run and the shape
// fits; `algorithm=resident` asks for it by name.
bool use_resident(const orx_function& f, int rows) {
    if (f.flags != kQ4 || !dense_resident_eligible(f.N, f.K, f.packed_k)) return false;
    if (f.algorithm == kResident) return rows <= 128;
    // from 2 rows: the GEMV's dot products grow with the row count (16.4 us at 2 rows, 23 us at 3 and 4
    // rows of N=17408, K=5120), this kernel's MFMAs do not (15.6 us from 2 to 16 rows)
    // up to 64 rows as two launches of 32 (36 and 39 us at 48 and 64 rows against 42 and 48 us for
    // the streaming kernel)
    // (the second launch pays for itself only on large matrices: N = 17408, K = 5120 at 48 rows 33 us
    // against 39 us for the streaming kernel, but N = K = 5120 20 against 14.5 us)
    const int limit = (int64_t)f.N * f.K >= ((int64_t)1 << 26) ? 64 : 32;
    return f.algorithm == kAuto && tile_for(f, rows) == 0 && rows > 1 && rows <= limit;
}

// 256x256 tiles once there are enough rows to fill them (or when block_m = 256 is forced)
// (from 385 rows: up to 384 the 128x128 tiles measure 73..77 us for two-stage codes at N=17408,
// K=5120 against 86..93 us for decode-once + 256x256, and 54..60 us against 58..62 us for W8; at 512
// rows the 256x256 kernel wins, 92 against 104 us and 61 against 79 us)
bool split_preferred_to_big(const orx_function& f, int rows);
// Two-stage codes above 384 rows without scratch: the 512-row channel runs against whole 128 x 128 tiles, which
// decode every weight once per 128 rows but come four to the 512 rows.  Measured at K = 5120 (times scale with K):
// the runs take 66 us per row tile and round of the CUs (N = 17408: 66 / 124 / 132 us at 512 / 768 / 1024 rows),
// the small tiles 40 us + 32 us per tile and CU (105 / 141 / 171 us); N = 5120: 61 / 113 / 113 against 55 / 56 / 77 us.
bool tall_beats_whole_tiles(const orx_function& f, int rows) {
    const int64_t cus = device_compute_units();
    const int64_t tall = (int64_t)gemm_tall_units(f.N) * ceil_div((uint32_t)rows, 512u);
    const int64_t small = (int64_t)ceil_div((uint32_t)f.N, 128u) * ceil_div((uint32_t)rows, 128u);
    return 66 * ((tall + cus - 1) / cus) * cus < 40 * cus + 32 * small;
}
bool use_big(const orx_function& f, int rows) {
    if (f.K % kBK || f.K < 2 * kBK) return false;  // half a K step at the end, or a single step: the 32-128 row tiles only
    const int tile = tile_for(f, rows);
    if (tile == 256) return true;
    if (tile != 0 || rows <= 384 || split_preferred_to_big(f, rows)) return false;
    const bool decodes_once = f.takes_workspace && (f.flags2 & kNoExpand) == 0;
    if (f.flags == kQ4 && !decodes_once) return tall_beats_whole_tiles(f, rows);
    return true;
}

// Two-stage weights are decoded once into the handle's scratch and multiplied by the int8 kernel
// when the rows need the 256-row MFMA tiles (every row tile would otherwise decode every weight
// again, and even a single tile row gains: the decode leaves the MFMA loop).
constexpr int kExpandRows = 129;
bool use_expand(const orx_function& f, int rows) {
    return f.flags == kQ4 && f.takes_workspace && (f.flags2 & kNoExpand) == 0 && use_big(f, rows) && rows >= kExpandRows;
}

// Split launches serve the 128-row tiles when whole tiles would not spread evenly: up to two tiles
// per CU.  The partial slots are in the caller's Workspace.
// two workgroups per CU: a single workgroup of four waves leaves every load latency exposed
int split_groups() { return 2 * device_compute_units(); }
// 128-row tiles of this launch, and whether their count suits a split launch: measured at K = 5120
// with N = 5120, 7168 and 17408, 40-272 tiles gain 10-40 % (two-stage codes 59 -> 44 us at 136 tiles,
// 53 -> 32 us at 80), 408 tiles lose; a handful of tiles is latency, not balance, and two launches would
// only add to it; tiles that divide evenly over the CUs are balanced as they are.
int64_t split_tiles(const orx_function& f, int rows) {
    return (int64_t)ceil_div((uint32_t)f.N, 128u) * ceil_div((uint32_t)rows, 128u);
}
bool split_shape_ok(const orx_function& f, int rows) {
    if (!f.takes_workspace || (f.flags2 & kNoSplit) || tile_for(f, rows) != 0 || (f.algorithm != kAuto && f.algorithm != kMfma)) return false;
    const int64_t tiles = split_tiles(f, rows);
    return tiles >= 8 && tiles <= (int64_t)split_groups() * 9 / 16 && tiles % (split_groups() / 2) != 0;
}
// Above 384 rows the 256 x 256 kernel is the default, but with fewer such tiles than half the CUs it
// leaves most of the chip idle (W8, N = 5120, K = 17408 at 512 rows: 40 tiles, 209 us; N = K = 4096:
// 32 tiles, 48 us against 29 us at 384 rows): the split 128-row tiles take those launches.
bool split_preferred_to_big(const orx_function& f, int rows) {
    const int64_t big_tiles = (int64_t)ceil_div((uint32_t)f.N, 256u) * ceil_div((uint32_t)rows, 256u);
    return big_tiles < split_groups() / 4 && split_shape_ok(f, rows);
}
bool use_split(const orx_function& f, int rows) {
    if (!split_shape_ok(f, rows)) return false;
    if (use_gemv(f, rows) || use_resident(f, rows) || use_stream(f, rows) || use_big(f, rows)) return false;
    // 17-64 rows: the 32- and 64-row tiles give one workgroup per 128 channels, which leaves most CUs
    // idle when N is small and K long (W8, N = 5120, K = 17408: 112 us at 32 rows as 40 whole tiles);
    // with 136 such tiles (N = 17408) the whole 32-row tiles win, 39.7 against 43.1 us
    if (pick_bm(rows) != 128 && split_tiles(f, rows) >= split_groups() / 8) return false;
    return true;
}
// Workgroups of a split launch: two per CU, but at least 8 K steps each, so that the partial tiles
// (64 KiB per run) stay small beside the operands a workgroup reads (32 KiB per K step).
int split_groups_for(const orx_function& f, int rows) {
    const int64_t units = split_tiles(f, rows) * (f.K / kBK);
    return (int)std::max<int64_t>(1, std::min<int64_t>(split_groups(), units / 8));
}

// A few 256 x 256 tiles more than there are CUs would be a second round with most of the chip idle (1024 rows of
// N = 17408: 272 tiles; int8, K = 5120: 118 us, against 75 us for the 256 tiles of the first 16384 channels).  The
// persistent launch then takes the column tiles that fill one round, and the channels behind them go to the
// 128 x 128 tiles with their K steps split over all CUs (26 us for those 1024 channels: 96 us together).  Only
// where the second round would hold at most an eighth of the CUs: with more tiles left, or more rounds in front,
// the half-empty round runs at a higher clock and the split launch gains nothing (2048 rows: 175 against 180 us;
// 8192 rows of N = 5120, K = 17408: 669 against 657 us).  Returns the channels of the persistent launch (N: all).
int big_main_channels(const orx_function& f, int rows) {
    if (!f.takes_workspace || (f.flags2 & kNoSplit) || f.algorithm != kAuto || tile_for(f, rows) != 0) return f.N;
    const int cus = device_compute_units();
    const int row_tiles = (int)ceil_div((uint32_t)rows, 256u), column_tiles = (int)ceil_div((uint32_t)f.N, 256u);
    const int tiles = row_tiles * column_tiles;
    if (tiles <= cus || tiles > cus + cus / 8 || row_tiles > cus) return f.N;
    const int main_columns = cus / row_tiles;
    return main_columns * 256;
}
int split_groups_for_channels(int channels, int rows, int k) {
    const int64_t units = (int64_t)ceil_div((uint32_t)channels, 128u) * ceil_div((uint32_t)rows, 128u) * (k / kBK);
    return (int)std::max<int64_t>(1, std::min<int64_t>(split_groups(), units / 8));
}
uint64_t big_rest_workspace(const orx_function& f, int rows) {
    const int main_channels = big_main_channels(f, rows);
    if (main_channels >= f.N) return 0;
    return (uint64_t)split_groups_for_channels(f.N - main_channels, rows, f.K) * 2 * kSplitSlotInts * sizeof(int);
}

// Workspace bytes of a launch: the partial slots of a split launch, or the decoded weights of a
// two-stage launch on the 256-row tiles (and behind them the partial slots of the channels that the
// persistent launch leaves to the split tiles).
uint64_t projection_workspace(const orx_function& f, int rows) {
    if (use_wide(f, rows) || use_tall(f, rows)) return 0;
    if (use_gemv(f, rows) || use_resident(f, rows) || use_stream(f, rows)) return 0;
    if (use_expand(f, rows)) return (uint64_t)f.N * f.K + big_rest_workspace(f, rows);
    if (use_big(f, rows)) return f.flags == kW8 ? big_rest_workspace(f, rows) : 0;
    if (use_split(f, rows)) return (uint64_t)split_groups_for(f, rows) * 2 * kSplitSlotInts * sizeof(int);
    return 0;
}

template <int CODEC>
int launch_split(const GemmParams& p, int groups, hipStream_t stream) {
    ORX_LAUNCH((gemm_split_kernel<CODEC>), dim3(groups), dim3(256), 0, stream, p);
    int code = hip_check(hipGetLastError(), "launch projection (mfma, split K steps)");
    if (code != ORX_OK) return code;
    const uint32_t tiles = ceil_div((uint32_t)p.n, 128u) * ceil_div((uint32_t)p.m, 128u);
    ORX_LAUNCH(gemm_split_finish_kernel, dim3(4 * tiles), dim3(256), 0, stream, p, groups);
    return hip_check(hipGetLastError(), "launch projection (mfma, sum of split tiles)");
}

int projection_geometry(const orx_function& f, int rows, Geometry* g) {
    if (use_wide(f, rows)) {
        dense_wide_geometry(f.N, g);
        return ORX_OK;
    }
    if (use_tall(f, rows)) {
        gemm_tall_geometry(rows, f.N, g);
        return ORX_OK;
    }
    if (use_gemv(f, rows)) return gemv_geometry_for(f, rows, g);
    if (use_resident(f, rows)) {
        dense_resident_geometry(rows, f.N, f.K, f.packed_k, g);
        return ORX_OK;
    }
    if (use_stream(f, rows)) {
        stream_geometry(f.N, g);
        return ORX_OK;
    }
    if (use_big(f, rows)) {
        if (f.flags == kQ4 && !use_expand(f, rows))  // decode in the K loop: the 512-row channel runs
            gemm_tall_geometry(rows, f.N, g);
        else
            gemm_big_geometry(rows, big_main_channels(f, rows), g);
        return ORX_OK;
    }
    if (use_split(f, rows)) {
        g->grid[0] = (uint32_t)split_groups_for(f, rows);
        g->block[0] = 256;
        g->shared = 0;
        return ORX_OK;
    }
    const int bm = tile_for(f, rows) ? tile_for(f, rows) : pick_bm(rows);
    g->grid[0] = ceil_div((uint32_t)f.N, 128u);
    g->grid[1] = ceil_div((uint32_t)rows, (uint32_t)bm);
    g->block[0] = 256;
    g->shared = 0;
    return ORX_OK;
}

// int8 weights on the 256 x 256 tiles: the persistent launch, and the split 128 x 128 tiles for the channels it
// leaves (big_main_channels).  `partials`: the workspace bytes behind whatever else the launch keeps there.
int int8_big_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const GemmParams& p,
                    const void* weights, void* partials) {
    const int main_channels = big_main_channels(f, rows);
    int code = gemm_big_launch(p.a, weights, p.ws, p.as, p.out, rows, main_channels, f.K, f.stride, f.out_f32, g, stream);
    if (code != ORX_OK || main_channels >= f.N) return code;
    GemmParams rest = p;
    rest.book = nullptr, rest.packed_k = 0;
    rest.w = static_cast<const int8_t*>(weights) + (size_t)main_channels * f.K;
    rest.ws = p.ws + main_channels;
    rest.out = static_cast<char*>(p.out) + (size_t)main_channels * (f.out_f32 ? 4 : 2);
    rest.n = f.N - main_channels;
    rest.partials = static_cast<int*>(partials);
    return launch_split<kW8>(rest, split_groups_for_channels(rest.n, rows, f.K), stream);
}

// E8P-Q4: A, AS, Book, Out, S, W[, m]   (e8p_q4.py:248-255 in generated-ABI order)
int q4_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0);
    p.as = pointer_arg<const __half>(args, 1);
    p.book = pointer_arg<const uint32_t>(args, 2);
    p.out = pointer_arg<void>(args, 3);
    p.ws = pointer_arg<const __half>(args, 4);
    const int8_t* signs = f.rotate_input ? pointer_arg<const int8_t>(args, 5) : nullptr;
    p.w = pointer_arg<const void>(args, f.rotate_input ? 6 : 5);
    void* workspace = f.takes_workspace ? pointer_arg<void>(args, f.workspace_arg) : nullptr;
    p.n = f.N, p.k = f.K, p.stride = f.stride, p.m = rows, p.packed_k = f.packed_k, p.out_f32 = f.out_f32;
    if (use_wide(f, rows))
        return dense_wide_launch(p.a, p.w, p.book, p.ws, p.as, p.out, rows, f.N, f.K, f.stride, f.packed_k, f.out_f32, g, stream);
    if (use_tall(f, rows))
        return gemm_tall_launch(p.a, p.w, p.book, p.ws, p.as, p.out, rows, f.N, f.K, f.stride, f.packed_k, f.out_f32, g, stream);
    if (use_gemv(f, rows)) return gemv_launch(f, rows, g, stream, p.a, p.w, p.book, p.ws, p.as, p.out, signs);
    if (use_resident(f, rows)) {
        for (int first = 0; first < rows; first += 32) {
            const size_t out_offset = (size_t)first * f.stride * (f.out_f32 ? 4 : 2);
            const int code = dense_resident_launch(p.a + (size_t)first * f.K, p.w, p.book, p.ws, p.as + first,
                                                   static_cast<char*>(p.out) + out_offset, std::min(32, rows - first),
                                                   f.N, f.K, f.stride, f.packed_k, f.out_f32, stream);
            if (code != ORX_OK) return code;
        }
        return ORX_OK;
    }
    if (use_stream(f, rows)) {
        for (int first = 0; first < rows; first += 64) {
            const size_t out_offset = (size_t)first * f.stride * (f.out_f32 ? 4 : 2);
            const int code = stream_launch(kQ4, p.a + (size_t)first * f.K, p.w, p.book, p.ws, p.as + first,
                                           static_cast<char*>(p.out) + out_offset, std::min(64, rows - first), f.N, f.K,
                                           f.stride, f.packed_k, f.out_f32, stream);
            if (code != ORX_OK) return code;
        }
        return ORX_OK;
    }
    if (use_expand(f, rows)) {
        const int code = q4_expand_launch(p.w, p.book, workspace, f.N, f.K, f.packed_k, stream);
        if (code != ORX_OK) return code;
        return int8_big_launch(f, rows, g, stream, p, workspace, static_cast<char*>(workspace) + (size_t)f.N * f.K);
    }
    if (use_big(f, rows))
        return gemm_tall_launch(p.a, p.w, p.book, p.ws, p.as, p.out, rows, f.N, f.K, f.stride, f.packed_k, f.out_f32, g, stream);
    if (use_split(f, rows)) {
        p.partials = static_cast<int*>(workspace);
        return launch_split<kQ4>(p, split_groups_for(f, rows), stream);
    }
    return launch_mfma<kQ4, false>(tile_for(f, rows) ? tile_for(f, rows) : pick_bm(rows), p, g, stream);
}

// W8A8: A, Output, TokenScale, Weight, WeightScale[, m]   (int8_projection.py:51-57)
int w8_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0);
    p.out = pointer_arg<void>(args, 1);
    p.as = pointer_arg<const __half>(args, 2);
    p.w = pointer_arg<const void>(args, 3);
    p.ws = pointer_arg<const __half>(args, 4);
    p.book = nullptr;
    void* workspace = f.takes_workspace ? pointer_arg<void>(args, f.workspace_arg) : nullptr;
    p.n = f.N, p.k = f.K, p.stride = f.stride, p.m = rows, p.packed_k = 0, p.out_f32 = f.out_f32;
    if (use_gemv(f, rows)) return gemv_launch(f, rows, g, stream, p.a, p.w, p.book, p.ws, p.as, p.out);
    if (use_stream(f, rows)) {
        for (int first = 0; first < rows; first += 64) {
            const size_t out_offset = (size_t)first * f.stride * (f.out_f32 ? 4 : 2);
            const int code = stream_launch(kW8, p.a + (size_t)first * f.K, p.w, p.book, p.ws, p.as + first,
                                           static_cast<char*>(p.out) + out_offset, std::min(64, rows - first), f.N, f.K,
                                           f.stride, 0, f.out_f32, stream);
            if (code != ORX_OK) return code;
        }
        return ORX_OK;
    }
    if (use_big(f, rows)) return int8_big_launch(f, rows, g, stream, p, p.w, workspace);
    if (use_split(f, rows)) {
        p.partials = static_cast<int*>(workspace);
        return launch_split<kW8>(p, split_groups_for(f, rows), stream);
    }
    return launch_mfma<kW8, false>(tile_for(f, rows) ? tile_for(f, rows) : pick_bm(rows), p, g, stream);
}

int make_projection(const Variant& v, orx_function* f, int codec) {
    bool bad = false;
    f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    f->stride = (int)v.integer("output_stride", f->N, &bad);
    f->packed_k = (int)v.integer("packed_k", 0, &bad);
    f->tiles = (int)v.integer("block_m", 0, &bad);  // forced MFMA row tile, 0 = by row count
    const int passes = (int)v.integer("gemv_passes", 0, &bad);
    const std::string dtype = v.string("output_dtype", "float16", &bad);
    std::string algorithm = v.string("algorithm", "auto", &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    const char* name = f->symbol.c_str();
    // The reference's factories name their schedules tensor_core, dp4a and int4_direct and take row tiles of
    // 1-8, 16, 96 and 192 as well (e8p_q4.py:143-215, int8_projection.py:15-48; a package's winners come from
    // contracts/projection_policy.py:40-101).  They are hints among the library's own kernels: dp4a (the dot-product
    // schedule) keeps the single-row GEMV family wherever it serves the rows, tensor_core keeps to the kernels built on
    // the matrix unit at every row count, int4_direct means no preference; a row tile of 16, 96 or 192 asks for the MFMA
    // tile that holds it (32, 128, 256) for launches whose rows fit one such tile, and tiles of 1-8 rows, which have no
    // tile kernel here, leave the choice to the row count.  Its other tile keys (block_n, block_k, stages, tail_m, group_m, cache_scales, an integer split_k) are
    // not read.
    int schedule_hint = 0;
    if (algorithm == "dp4a") schedule_hint = kPreferGemv;
    if (algorithm == "tensor_core") schedule_hint = kNoGemv;
    if (algorithm == "tensor_core" || algorithm == "dp4a" || algorithm == "int4_direct") algorithm = "auto";
    for (const char* hint : {"block_n", "block_k", "stages", "tail_m", "group_m", "cache_scales", "basis_nonzero", "minimum_blocks"}) v.accept(hint);
    if (f->tiles >= 1 && f->tiles <= 8) f->tiles = 0;
    if (f->tiles == 16) f->tile_hint = 32;
    if (f->tiles == 96) f->tile_hint = 128;
    if (f->tiles == 192) f->tile_hint = f->K % kBK == 0 && f->K >= 2 * kBK ? 256 : 128;
    if (f->tile_hint) f->tiles = 0;
    // validate_shape + K*128*127 < 2^31 (q4_projection.py:33-35, int8_projection.py:29)
    const bool half_step = codec == kW8 && f->K % kBK == 64;  // int8_projection.py:29 takes K % 64 == 0
    if (f->M <= 0 || f->N <= 0 || f->K <= 0 || (f->K % kBK && !half_step) || (int64_t)f->K * 128 * 128 > 2147483647LL) {
        set_error("%s: need M,N,K > 0, K a multiple of 128 (of 64 for int8 weights) and K*2^14 < 2^31", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->stride < f->N) {
        set_error("%s: output_stride must contain the entire row", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (dtype != "float16" && dtype != "float32") {
        set_error("%s: output_dtype must be float16 or float32", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->packed_k != 0 && ((f->packed_k != 128 && f->packed_k != 64) || codec == kW8)) {
        set_error("%s: packed_k must be 0, 64 or 128 (codes only)", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->tiles != 0 && f->tiles != 32 && f->tiles != 64 && f->tiles != 128 && f->tiles != 256) {
        set_error("%s: block_m must be 32, 64, 128 or 256", name);
        return ORX_ERR_BAD_VARIANT;
    }
    f->out_f32 = dtype == "float32";
    f->capacity = f->M;
    f->flags = codec;
    f->algorithm = algorithm == "gemv"     ? kGemv
                   : algorithm == "mfma"   ? kMfma
                   : algorithm == "stream"   ? kStream
                   : algorithm == "resident" ? kResident
                   : algorithm == "wide"     ? kWide
                   : algorithm == "tall"     ? kTall
                   : algorithm == "auto"     ? kAuto
                                             : -1;
    if (f->algorithm < 0) {
        set_error("%s: algorithm must be auto, gemv, stream, resident, wide, tall or mfma", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kTall && (codec != kQ4 || f->K % 128 != 0 || f->K < 256)) {
        set_error("%s: algorithm=tall serves two-stage codes with K a multiple of 128, at least 256", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kWide && (codec != kQ4 || !dense_wide_eligible(f->N, f->K, f->packed_k))) {
        set_error("%s: algorithm=wide serves two-stage codes, row-major or K-major", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (half_step) {
        // a K that ends in half a step is served by the 32/64/128-row MFMA tiles at every row count
        if ((f->algorithm != kAuto && f->algorithm != kMfma) || f->tiles == 256) {
            set_error("%s: K = %d is not a multiple of 128: served by the MFMA tiles (algorithm auto or mfma, block_m up to 128)", name, f->K);
            return ORX_ERR_BAD_VARIANT;
        }
        f->algorithm = kMfma;
    }
    if (f->algorithm == kResident &&
        (codec != kQ4 || f->capacity > 128 || !dense_resident_eligible(f->N, f->K, f->packed_k))) {
        set_error("%s: algorithm=resident serves two-stage row-major codes, at most 128 rows, K a multiple of 512 up to 5120 or of 1024 up to 8192",
                  name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kStream && f->capacity > 64) {
        set_error("%s: the stream algorithm serves up to 64 rows, variant asks for %d", name, f->capacity);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kGemv && f->packed_k != 0 && (codec != kQ4 || f->K % 256 != 0)) {
        set_error("%s: the gemv algorithm reads row-major codes (packed_k = 0), or K-major two-stage codes (blocks of 128 or 64) with K a multiple of 256",
                  name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kGemv || (f->algorithm == kAuto && (f->packed_k == 0 || (codec == kQ4 && f->K % 256 == 0)))) {
        orx_function probe = *f;
        if (probe.capacity > 4) probe.capacity = 4;
        int code = gemv_configure(&probe, codec, passes);
        if (code != ORX_OK) {
            if (f->algorithm == kGemv) return code;
            f->algorithm = kMfma;
        } else {
            if (f->algorithm == kGemv && f->capacity > 4) return gemv_configure(f, codec, passes);  // reports the error
            f->block_m = probe.block_m;
            f->slots = probe.slots;  // ring depth of the replicated-table gemv, 0 = compact tables
        }
    }
    // workspace=true: the launch takes a trailing `Workspace` buffer (the caller's; orx_workspace_bytes
    // gives its size) and may then split the K steps of its tiles over the CUs (int32 partial tiles) or
    // decode two-stage weights once per launch; without it the handle keeps whole tiles and decodes
    // inside the GEMM.  split_k=false and decode_in_gemm=true switch the two uses off one by one.
    {
        f->takes_workspace = v.boolean("workspace", false, &bad);
        // (an integer split_k is the reference's K partition of its direct INT4 schedule: not a request here)
        const bool split = v.has("split_k") && v.fields.at("split_k").kind == Value::Number ? true : v.boolean("split_k", true, &bad);
        const bool in_gemm = v.boolean("decode_in_gemm", false, &bad);
        if (bad) return ORX_ERR_BAD_VARIANT;
        f->flags2 = (split && !half_step ? 0 : kNoSplit) | (in_gemm ? kNoExpand : 0) | schedule_hint;
        f->workspace_need = projection_workspace;
    }
    f->geometry = projection_geometry;
    // a projection handle launches one of several kernels depending on the live rows (1024-thread
    // GEMV, 512-thread streaming and 256x256 kernels, 256-thread tiles): no single function's
    // attributes describe it: orx_query_rows reports the kernel a row count starts, orx_query the capacity's
    f->device_function = nullptr;
    return ORX_OK;
}

int make_q4_projection(const Variant& v, orx_function* f) {
    if (!two_stage_coefficients_ok(v, "e8p_q4_projection")) return ORX_ERR_BAD_VARIANT;
    int code = make_projection(v, f, kQ4);
    if (code != ORX_OK) return code;
    bool bad = false;
    // input_dtype=float16: A is the fp16 row and AS is written, not read (the kernel quantises the row)
    const std::string input = v.string("input_dtype", "int8", &bad);
    if (bad || (input != "int8" && input != "float16")) {
        set_error("e8p_q4_projection: input_dtype must be int8 or float16");
        return ORX_ERR_BAD_VARIANT;
    }
    if (input == "float16") {
        if (f->capacity != 1 || (f->algorithm != kAuto && f->algorithm != kGemv) || !gemv_serves_fp16_input(*f)) {
            set_error("e8p_q4_projection: input_dtype=float16 is served for one row by the replicated-table GEMV "
                      "(M = 1, algorithm auto or gemv, K up to 8192 with a layout that kernel reads)");
            return ORX_ERR_BAD_VARIANT;
        }
        f->input_f16 = true;
        f->algorithm = kGemv;
    }
    // rotate=true (fp16 input only): the signed block-128 rotation runs in front of the quantiser, Signs
    // joins the buffers (kernels/cuda/model/rotation_a8.py:369-383 followed by the projection, in one launch)
    f->rotate_input = v.boolean("rotate", false, &bad);
    if (bad || (f->rotate_input && !f->input_f16)) {
        set_error("e8p_q4_projection: rotate=true needs input_dtype=float16");
        return ORX_ERR_BAD_VARIANT;
    }
    f->args = {{"A", ArgPointer, 16}, {"AS", ArgPointer, 2}, {"Book", ArgPointer, 4},
               {"Out", ArgPointer, 2}, {"S", ArgPointer, 2}};
    if (f->rotate_input) f->args.push_back({"Signs", ArgPointer, 8});
    f->args.push_back({"W", ArgPointer, 16});
    if (f->takes_workspace) f->args.push_back({"Workspace", ArgPointer, 256u | 0x80000000u});  // null where no launch needs it
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->launch = q4_launch;
    return ORX_OK;
}

int make_w8_projection(const Variant& v, orx_function* f) {
    int code = make_projection(v, f, kW8);
    if (code != ORX_OK) return code;
    f->args = {{"A", ArgPointer, 16},     {"Output", ArgPointer, 2},      {"TokenScale", ArgPointer, 2},
               {"Weight", ArgPointer, 16}, {"WeightScale", ArgPointer, 2}};
    if (f->takes_workspace) f->args.push_back({"Workspace", ArgPointer, 256u | 0x80000000u});
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->launch = w8_launch;
    return ORX_OK;
}

// ---- row-scaled scalar Q4 (kernels/cuda/model/q4_projection.py; python/orinfer_build/quantization/row_q4.py) ----
// W is (N, K/4) u16: four nibbles per word, weight = +-magnitudes[nibble & 7], negative when bit 3 is set.  Same
// activations, accumulation and rescale as every other projection.  One or two rows: a streaming GEMV (k_rowq4.hip);
// up to 64 rows the weight-streaming MFMA kernel reads the nibbles once; above, the 128-wide MFMA tiles decode them into LDS; from 512 rows with a Workspace they
// are decoded once per launch and the int8 256 x 256 kernel runs.
// slots used: M/capacity, N, K, stride, out_f32, H (magnitudes 0-3 as bytes), group (magnitudes 4-7)
__global__ __launch_bounds__(256) void row_q4_unpack_kernel(const uint32_t* __restrict__ w, uint2* __restrict__ out,
                                                            int64_t pairs, uint32_t low, uint32_t high) {
    // one u32 = two words = eight weights
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pairs; i += (int64_t)gridDim.x * 256) {
        const uint32_t v = w[i];
        out[i] = make_uint2(decode_row_q4(v, low, high), decode_row_q4(v >> 16, low, high));
    }
}

int row_q4_unpack(const void* w, void* out, int n, int k, uint32_t low, uint32_t high, hipStream_t stream) {
    const int64_t pairs = (int64_t)n * (k / 8);
    const int blocks = (int)std::min<int64_t>((pairs + 255) / 256, 4096);
    ORX_LAUNCH(row_q4_unpack_kernel, dim3(blocks), dim3(256), 0, stream, reinterpret_cast<const uint32_t*>(w),
                       reinterpret_cast<uint2*>(out), pairs, low, high);
    return hip_check(hipGetLastError(), "launch unpack_q4");
}

constexpr int kRowQ4BigRows = 512;
bool row_q4_expands(const orx_function& f, int rows) { return f.takes_workspace && rows >= kRowQ4BigRows && f.K >= 2 * kBK; }
// 65..511 rows: the K steps of the 128-row tiles dealt evenly to the CUs when whole tiles would not spread evenly
// (the rule of the other codecs: 8 to 288 tiles that do not divide over the CUs)
bool row_q4_splits(const orx_function& f, int rows) { return rows > 64 && !row_q4_expands(f, rows) && split_shape_ok(f, rows); }

uint64_t row_q4_workspace(const orx_function& f, int rows) {
    if (rows == 0) {  // the most any row count needs: one probe per height in 128-row tiles
        uint64_t most = 0;
        for (int top = 128; top - 128 < std::min(f.capacity, kRowQ4BigRows); top += 128)
            most = std::max(most, row_q4_workspace(f, std::min(top, f.capacity)));
        return most;
    }
    if (row_q4_expands(f, rows)) return (uint64_t)f.N * f.K;
    if (row_q4_splits(f, rows)) return (uint64_t)split_groups_for(f, rows) * 2 * kSplitSlotInts * sizeof(int);
    return 0;
}

int row_q4_geometry(const orx_function& f, int rows, Geometry* g) {
    if (row_q4_gemv_serves(rows, f.K)) {
        row_q4_gemv_geometry(rows, f.N, f.K, g);
        return ORX_OK;
    }
    if (rows <= 64) {
        stream_geometry(f.N, g);
        return ORX_OK;
    }
    if (row_q4_expands(f, rows)) {
        gemm_big_geometry(rows, f.N, g);
        return ORX_OK;
    }
    if (row_q4_splits(f, rows)) {
        g->grid[0] = (uint32_t)split_groups_for(f, rows);
        g->block[0] = 256;
        g->shared = 0;
        return ORX_OK;
    }
    g->grid[0] = ceil_div((uint32_t)f.N, 128u);
    g->grid[1] = ceil_div((uint32_t)rows, 128u);
    g->block[0] = 256;
    g->shared = 0;
    return ORX_OK;
}

// A, AS, Out, S, W[, Workspace][, m]   (crates/orinfer-models/src/flash_next/q4.rs:176-196 binds A, AS, Out, S, W)
int row_q4_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0);
    p.as = pointer_arg<const __half>(args, 1);
    p.out = pointer_arg<void>(args, 2);
    p.ws = pointer_arg<const __half>(args, 3);
    p.w = pointer_arg<const void>(args, 4);
    p.n = f.N, p.k = f.K, p.stride = f.stride, p.m = rows, p.out_f32 = f.out_f32;
    p.magnitudes_low = (uint32_t)f.H, p.magnitudes_high = (uint32_t)f.group;
    if (row_q4_gemv_serves(rows, f.K))
        return row_q4_gemv_launch(p.a, p.w, p.magnitudes_low, p.magnitudes_high, p.ws, p.as, p.out, rows, f.N, f.K, f.stride,
                                  f.out_f32, g, stream);
    if (rows <= 64)
        return stream_row_q4_launch(p.a, p.w, p.magnitudes_low, p.magnitudes_high, p.ws, p.as, p.out, rows, f.N, f.K, f.stride,
                                    f.out_f32, stream);
    if (row_q4_expands(f, rows)) {
        void* workspace = pointer_arg<void>(args, f.workspace_arg);
        const int code = row_q4_unpack(p.w, workspace, f.N, f.K, p.magnitudes_low, p.magnitudes_high, stream);
        if (code != ORX_OK) return code;
        return gemm_big_launch(p.a, workspace, p.ws, p.as, p.out, rows, f.N, f.K, f.stride, f.out_f32, g, stream);
    }
    if (row_q4_splits(f, rows)) {
        p.partials = pointer_arg<int>(args, f.workspace_arg);
        return launch_split<kS4>(p, split_groups_for(f, rows), stream);
    }
    ORX_LAUNCH((gemm_kernel<kS4, 128, 128, 2, false>), dim3(g.grid[0], g.grid[1]), dim3(256), 0, stream, p);
    return hip_check(hipGetLastError(), "launch scalar Q4 projection (mfma)");
}

// `magnitudes`: eight strictly increasing integers in 1..127 (q4_projection.py:17-21)
bool row_q4_magnitudes(const Variant& v, const char* symbol, uint32_t* low, uint32_t* high) {
    bool bad = false;
    std::string given = v.string("magnitudes", "3,10,19,31,46,67,93,127", &bad);
    int values[8], count = 0, previous = 0;
    bool ok = !bad;
    size_t at = 0;
    while (ok && at <= given.size() && count < 9) {
        size_t end = given.find(',', at);
        if (end == std::string::npos) end = given.size();
        const std::string piece = given.substr(at, end - at);
        char* rest = nullptr;
        const long value = strtol(piece.c_str(), &rest, 10);
        if (piece.empty() || rest == piece.c_str() || value <= previous || value > 127 || count == 8) ok = false;
        while (ok && *rest == ' ') ++rest;
        if (ok && *rest != 0) ok = false;
        if (ok) values[count++] = previous = (int)value;
        at = end + 1;
        if (end == given.size()) break;
    }
    if (!ok || count != 8) {
        set_error("%s: magnitudes are eight strictly increasing integers in 1..127", symbol);
        return false;
    }
    *low = *high = 0;
    for (int i = 0; i < 4; ++i) *low |= (uint32_t)values[i] << (8 * i), *high |= (uint32_t)values[4 + i] << (8 * i);
    return true;
}

bool row_q4_shape(const char* symbol, orx_function* f) {
    // q4_projection.py:32-35: block-128 geometry, the int32 accumulator holds a whole row
    if (f->M > 0 && f->N > 0 && f->K > 0 && f->K % 128 == 0 && (int64_t)f->K * 128 * 127 <= 2147483647ll) return true;
    set_error("%s: need M, N, K > 0, K a multiple of 128 and K * 128 * 127 < 2^31", symbol);
    return false;
}

int finish_row_q4(const Variant& v, orx_function* f, const std::string& dtype) {
    const char* symbol = f->symbol.c_str();
    uint32_t low, high;
    if (!row_q4_shape(symbol, f) || !row_q4_magnitudes(v, symbol, &low, &high)) return ORX_ERR_BAD_VARIANT;
    if (dtype != "float16" && dtype != "float32") {
        set_error("%s: output_dtype must be float16 or float32", symbol);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->stride < f->N) {
        set_error("%s: output_stride must hold a whole row", symbol);
        return ORX_ERR_BAD_VARIANT;
    }
    f->capacity = f->M;
    f->out_f32 = dtype == "float32";
    f->H = (int)low, f->group = (int)high;
    f->args = {{"A", ArgPointer, 16}, {"AS", ArgPointer, 2}, {"Out", ArgPointer, f->out_f32 ? 4u : 2u}, {"S", ArgPointer, 2},
               {"W", ArgPointer, 16}};
    if (f->takes_workspace) {
        f->workspace_arg = (int)f->args.size();
        f->args.push_back({"Workspace", ArgPointer, 256u | 0x80000000u});
        f->workspace_need = row_q4_workspace;
    }
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->device_function = nullptr;  // several kernels serve the symbol
    f->geometry = row_q4_geometry;
    f->launch = row_q4_launch;
    return ORX_OK;
}

// q4_projection (q4_projection.py:125-183)
int make_row_q4_projection(const Variant& v, orx_function* f) {
    bool bad = false;
    f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    const int bn = (int)v.integer("BN", 64, &bad), bk = (int)v.integer("BK", 128, &bad);
    const std::string dtype = v.string("output_dtype", "float16", &bad);
    const int block_m = (int)v.integer("block_m", 8, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const int stages = (int)v.integer("stages", 2, &bad);
    f->stride = (int)v.integer("output_stride", f->N, &bad);
    const int tail_m = (int)v.integer("tail_m", 0, &bad), group_m = (int)v.integer("group_m", 0, &bad);
    f->takes_workspace = v.boolean("workspace", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    // tile choices of the reference's kernel, checked as it checks them (q4_projection.py:142-150); the row count picks here
    if ((bn != 32 && bn != 64 && bn != 128) || bk <= 0 || bk % 128 || (f->K > 0 && f->K % bk) ||
        (block_m != 8 && block_m != 16 && block_m != 32 && block_m != 64 && block_m != 128) || (stages != 1 && stages != 2) ||
        (group_m != 0 && group_m != 1 && group_m != 2 && group_m != 4 && group_m != 8) || tail_m < 0) {
        set_error("q4_projection: BN 32|64|128, BK a multiple of 128 that divides K, block_m 8..128, stages 1|2, group_m 0|1|2|4|8");
        return ORX_ERR_BAD_VARIANT;
    }
    return finish_row_q4(v, f, dtype);
}

// q4_gemv (q4_projection.py:38-78): the reference's DP4A form for tiles of up to 8 rows; A is the same bytes read as int32
int make_row_q4_gemv(const Variant& v, orx_function* f) {
    bool bad = false;
    f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    const int bn = (int)v.integer("BN", 16, &bad);
    const std::string dtype = v.string("output_dtype", "float16", &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const int block_m = (int)v.integer("block_m", std::max(1, std::min(f->M, 8)), &bad);
    f->stride = (int)v.integer("output_stride", f->N, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (block_m < 1 || block_m > 8 || (bn != 4 && bn != 8 && bn != 16)) {  // q4_projection.py:53-54
        set_error("q4_gemv: block_m 1..8 and BN 4, 8 or 16");
        return ORX_ERR_BAD_VARIANT;
    }
    return finish_row_q4(v, f, dtype);
}

// unpack_q4 (q4_projection.py:186-213): Output, W.  slots used: N, K, H, group
int row_q4_unpack_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = (uint32_t)std::min<int64_t>(((int64_t)f.N * (f.K / 8) + 255) / 256, 4096);
    g->block[0] = 256;
    return ORX_OK;
}
int row_q4_unpack_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows, (void)g;
    return row_q4_unpack(pointer_arg<const void>(args, 1), pointer_arg<void>(args, 0), f.N, f.K, (uint32_t)f.H, (uint32_t)f.group,
                         stream);
}
int make_row_q4_unpack(const Variant& v, orx_function* f) {
    bool bad = false;
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    f->M = 1;
    uint32_t low, high;
    if (!row_q4_shape("unpack_q4", f) || !row_q4_magnitudes(v, "unpack_q4", &low, &high)) return ORX_ERR_BAD_VARIANT;
    f->capacity = 1;
    f->H = (int)low, f->group = (int)high;
    f->args = {{"Output", ArgPointer, 8}, {"W", ArgPointer, 4}};
    f->geometry = row_q4_unpack_geometry;
    f->launch = row_q4_unpack_launch;
    f->device_function = reinterpret_cast<const void*>(&row_q4_unpack_kernel);
    return ORX_OK;
}

// kernels/cuda/model/int8_projection.py:65-107: the reference's DP4A form for up to 8-row tiles.  Same
// buffers and arithmetic as int8_projection; here the row count picks the kernel, so the tile hints
// are checked as the reference checks them and dropped.
int make_w8_small_projection(const Variant& v, orx_function* f) {
    bool bad = false;
    const long long m = v.integer("M", 0, &bad);
    const long long block_m = v.integer("block_m", m < 4 ? m : 4, &bad), block_n = v.integer("block_n", 4, &bad);
    if (bad || block_m < 1 || block_m > 8 || (block_n != 4 && block_n != 8 && block_n != 16)) {
        set_error("int8_small_projection: invalid INT8 DP4A tile (block_m 1..8, block_n 4|8|16)");
        return ORX_ERR_BAD_VARIANT;
    }
    Variant plain = v;
    plain.fields.erase("block_m");
    plain.fields.erase("block_n");
    return make_w8_projection(plain, f);
}

// ---- W8 gate/up projections with the SwiGLU boundary (shared expert) ---------------------------
// kernels/cuda/model/int8_swiglu.py:10-57 with integer_core.py:19-28: both projections are rounded
// to fp16, then out = fp16((g / (1 + exp(-g))) * u) in fp32.  One launch: a workgroup owns 64 output
// channels, holds the gate and the up accumulators of the same channels side by side (gemm_kernel's
// SWIGLU form) and applies the boundary in its epilogue; nothing goes through memory in between.
int int8_swiglu_geometry(const orx_function& f, int rows, Geometry* g) {
    const int bm = rows <= 64 ? 64 : 128;
    g->grid[0] = ceil_div((uint32_t)f.N, 64u);
    g->grid[1] = ceil_div((uint32_t)rows, (uint32_t)bm);
    g->block[0] = 256;
    g->shared = 0;
    return ORX_OK;
}

// A, Gate, GateScale, Output, TokenScale, Up, UpScale[, m]   (int8_swiglu.py:43-50 in generated-ABI order)
int int8_swiglu_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0);
    p.w = pointer_arg<const void>(args, 1);
    p.ws = pointer_arg<const __half>(args, 2);
    p.out = pointer_arg<void>(args, 3);
    p.as = pointer_arg<const __half>(args, 4);
    p.w2 = pointer_arg<const void>(args, 5);
    p.ws2 = pointer_arg<const __half>(args, 6);
    p.n = f.N, p.k = f.K, p.stride = f.N, p.m = rows, p.packed_k = 0, p.out_f32 = 0;
    const dim3 grid(g.grid[0], g.grid[1]), block(256);
    if (rows <= 64)
        ORX_LAUNCH((gemm_kernel<kW8, 64, 128, 2, false, true>), grid, block, 0, stream, p);
    else
        ORX_LAUNCH((gemm_kernel<kW8, 128, 128, 2, false, true>), grid, block, 0, stream, p);
    return hip_check(hipGetLastError(), "launch int8_swiglu");
}

int make_int8_swiglu(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    // the reference's tile hints (int8_swiglu.py:15-31): checked as it checks them, otherwise not used
    const std::string algorithm = v.string("algorithm", "tensor_core", &bad);
    const bool packed = algorithm == "dp4a";
    const long long block_n = v.integer("block_n", 64, &bad), block_m = v.integer("block_m", packed ? 4 : 16, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->M <= 0 || f->N <= 0 || f->K <= 0 || f->K % kBK || (int64_t)f->K * 128 * 128 > 2147483647LL) {
        set_error("int8_swiglu: invalid decode INT8 SwiGLU geometry (M, N, K > 0, K a multiple of 128, K*2^14 < 2^31)");
        return ORX_ERR_BAD_VARIANT;
    }
    if ((algorithm != "dp4a" && algorithm != "tensor_core" && algorithm != "auto" && algorithm != "mfma") ||
        (packed && (block_m < 1 || block_m > 8 || (block_n != 4 && block_n != 8 && block_n != 16 && block_n != 32 && block_n != 64))) ||
        (!packed && ((block_m != 16 && block_m != 32) || (block_n != 64 && block_n != 128)))) {
        set_error("int8_swiglu: invalid INT8 SwiGLU algorithm or tile");
        return ORX_ERR_BAD_VARIANT;
    }
    f->stride = f->N;
    f->flags = kW8;
    f->args = {{"A", ArgPointer, 16},         {"Gate", ArgPointer, 16}, {"GateScale", ArgPointer, 2}, {"Output", ArgPointer, 2},
               {"TokenScale", ArgPointer, 2}, {"Up", ArgPointer, 16},   {"UpScale", ArgPointer, 2}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = int8_swiglu_geometry;
    f->launch = int8_swiglu_launch;
    f->device_function = reinterpret_cast<const void*>(&gemm_kernel<kW8, 128, 128, 2, false, true>);
    return ORX_OK;
}

// ---- routed single-stage experts -----------------------------------------------------------
// A, AS, Book, C, Counts, Offsets, P, TileCount, TileExpert, TileRow, WS
// (tests/cuda/operators/e8p_decode.py:72-84; kernels/cuda/model/e8p_decode.py:60-73 without Patch)
// Resident kernel: forced by `algorithm=resident`, chosen by `auto` once the routed rows give every
// CU a unit of its own.
// flags2: input form (0 int8 rows per slot, 1 int8 token rows gathered by slot, 2 fp16 rows quantised while
// staged) + 4 * epilogue (0 plain, 1 SwiGLU).  Anything but 0 is a form of the resident kernel.
// H (integer_vq_grouped only): 1 general decode, 2 patched, 4 one selector table per expert, 8 the list has a Patch.
// bits 4-5: the BookForm of the general decode
enum GroupedForm { kGeneralDecode = 1, kPatched = 2, kExpertTables = 4, kTakesPatch = 8, kBookFormShift = 4 };

bool grouped_uses_resident(const orx_function& f) {
    if (f.H & kGeneralDecode) return false;
    if (f.algorithm == kResident || f.flags2 != 0) return true;
    return f.algorithm == kAuto && grouped_resident_eligible(f.N, f.K, f.block_m, f.tiles, 0, 0, f.capacity) &&
           grouped_resident_preferred(f.capacity, f.E, f.N);
}

int grouped_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    if (grouped_uses_resident(f)) {
        grouped_resident_geometry(f.K, f.flags2 & 3, f.flags2 >> 2, f.capacity, g);
        return ORX_OK;
    }
    if (f.block_m <= 64 && f.algorithm != kMfma && !(f.H & kGeneralDecode)) {
        stream_grouped_geometry(f.N, f.tiles, g);
        return ORX_OK;
    }
    g->grid[0] = ceil_div((uint32_t)f.N, 128u);
    g->grid[1] = (uint32_t)f.tiles;
    g->block[0] = 256;
    return ORX_OK;
}

// position of a buffer in the handle's argument list, -1 when this form has none
int grouped_arg(const orx_function& f, const char* name) {
    for (size_t i = 0; i < f.args.size(); ++i)
        if (std::string(f.args[i].name) == name) return (int)i;
    return -1;
}

int grouped_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    auto buffer = [&](const char* name) -> void* {
        const int at = grouped_arg(f, name);
        return at < 0 ? nullptr : pointer_arg<void>(args, at);
    };
    GroupedBuffers b;
    b.a = buffer("A"), b.as = buffer("AS"), b.book = reinterpret_cast<const uint32_t*>(buffer("Book"));
    b.out = buffer("C"), b.counts = reinterpret_cast<const int*>(buffer("Counts"));
    b.offsets = reinterpret_cast<const int*>(buffer("Offsets")), b.w = buffer("P");
    b.tile_count = reinterpret_cast<const int*>(buffer("TileCount"));
    b.tile_expert = reinterpret_cast<const int*>(buffer("TileExpert"));
    b.tile_row = reinterpret_cast<const int*>(buffer("TileRow")), b.ws = buffer("WS");
    b.slot_token = reinterpret_cast<const int*>(buffer("SlotToken"));
    b.row_max = reinterpret_cast<const int*>(buffer("RowMax")), b.act = buffer("Act"), b.q = buffer("Q");
    if (grouped_uses_resident(f))
        return grouped_resident_launch(b, f.N, f.K, f.tiles, f.packed_k, f.flags2 & 3, f.flags2 >> 2, f.capacity, stream);
    GemmParams p = {};
    p.a = reinterpret_cast<const int8_t*>(b.a), p.as = reinterpret_cast<const __half*>(b.as), p.book = b.book, p.out = b.out;
    p.counts = b.counts, p.offsets = b.offsets, p.w = b.w, p.tile_count = b.tile_count, p.tile_expert = b.tile_expert;
    p.tile_row = b.tile_row, p.ws = reinterpret_cast<const __half*>(b.ws);
    p.n = f.N, p.k = f.K, p.stride = f.N, p.m = f.capacity, p.packed_k = f.packed_k, p.out_f32 = 0;
    p.expert_weight_stride = (int64_t)f.N * (f.K / 8) * 2;
    if (f.H & kGeneralDecode) {
        p.patch = (f.H & kPatched) ? reinterpret_cast<const uint16_t*>(buffer("Patch")) : nullptr;
        p.book_form = (f.H >> kBookFormShift) & 3;
        p.book_stride = (f.H & kExpertTables) ? book_words(p.book_form) : 0;
        p.tile_rows = f.block_m;
        return launch_mfma_general(f.block_m, p, g, stream);
    }
    if (f.block_m <= 64 && f.algorithm != kMfma)
        return stream_grouped_launch(p.a, p.w, p.book, p.ws, p.as, p.out, p.counts, p.offsets, p.tile_expert,
                                     p.tile_row, p.tile_count, f.N, f.K, f.tiles, f.block_m, f.packed_k, stream);
    return launch_mfma<kQ2, true>(f.block_m, p, g, stream);
}

int make_q2_grouped(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("rows", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->tiles = (int)v.integer("tiles", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->block_m = (int)v.integer("block_m", f->symbol == "integer_vq_grouped" ? 16 : 32, &bad);  // integer_vq.py:314
    f->packed_k = (int)v.integer("packed_k", 128, &bad);
    const std::string grouped_algorithm = v.string("algorithm", "auto", &bad);
    const std::string input = v.string("input_dtype", "int8", &bad);
    const bool gather = v.boolean("gather", false, &bad);
    const std::string epilogue = v.string("epilogue", "none", &bad);
    // integer_vq_grouped carries the reference's Patch buffer and its decoder options (integer_vq.py:217-258)
    const bool vq = f->symbol == "integer_vq_grouped";
    const bool patched = vq && v.boolean("patched", false, &bad);
    const bool shared_table = !vq || v.boolean("shared_table", false, &bad);  // the reference's default (integer_vq.py:308)
    const std::string basis = vq ? v.string("basis", "spread29", &bad) : std::string("spread29");
    // The reference factories' other keywords (integer_vq.py:300-322, e8p_decode.py:36-58): `kind` is e8p; Book is the
    // (256, 2) table of raw basis values unless shortbook (the (512, 4) table of signed values) or shortbook +
    // selectorbook (the (256, 1) selector words) say otherwise, as in integer_vq.py:93-107; e8p_decode_grouped always
    // takes selector words (e8p_decode.py:63).  The rest chooses among its own schedules and is accepted as a hint.
    const std::string kind = v.string("kind", "e8p", &bad);
    const bool shortbook = vq ? v.boolean("shortbook", false, &bad) : true;
    const bool selectorbook = vq ? v.boolean("selectorbook", false, &bad) : true;
    const bool byte_permute = v.boolean("byte_permute", false, &bad);
    for (const char* hint : {"block_n", "num_stages", "stages", "group_n", "warp_decode", "split_k", "parity_xor", "warp_private"})
        v.accept(hint);
    // dynamic_rows: the reference's kernel then takes the live row count as a trailing `m` (integer_vq.py:234-258
    // with kernels/shared/rows.py); the tile lists already bound every row these kernels touch, so `m` is taken
    // and only checked against the capacity
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    const char* name = f->symbol.c_str();
    if (kind != "e8p" || ((selectorbook || byte_permute) && !shortbook)) {  // integer_vq.py:83-97
        set_error("%s: kind must be e8p; selectorbook and byte_permute need shortbook", name);
        return ORX_ERR_BAD_VARIANT;
    }
    const int book_form = selectorbook ? kBookSelector : shortbook ? kBookSigned : kBookRaw;
    if (basis != "spread29" && basis != "any") {
        set_error("%s: basis must be spread29 (no zero coordinates: the XOR decoders) or any (selector ids 0-7)", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if ((input != "int8" && input != "float16") || (epilogue != "none" && epilogue != "swiglu") ||
        (input == "float16" && (gather || epilogue != "none"))) {
        set_error("%s: input_dtype int8 (optionally gather=true, epilogue=swiglu) or float16 (rows with RowMax, plain epilogue)",
                  name);
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags2 = (input == "float16" ? 2 : gather ? 1 : 0) + (epilogue == "swiglu" ? 4 : 0);
    if (grouped_algorithm != "auto" && grouped_algorithm != "mfma" && grouped_algorithm != "stream" &&
        grouped_algorithm != "resident") {
        set_error("%s: algorithm must be auto, stream, resident or mfma", name);
        return ORX_ERR_BAD_VARIANT;
    }
    f->algorithm = grouped_algorithm == "mfma"       ? kMfma
                   : grouped_algorithm == "stream"   ? kStream
                   : grouped_algorithm == "resident" ? kResident
                                                     : kAuto;
    if (f->M <= 0 || f->E <= 0 || f->tiles <= 0 || f->N <= 0 || f->K <= 0 || f->K % 128 ||
        (int64_t)f->K * 128 * 128 > 2147483647LL) {
        set_error("%s: invalid E8P decode geometry", name);  // e8p_decode.py:52
        return ORX_ERR_BAD_VARIANT;
    }
    // 8 and 16 are steps of the tile list (the reference's decode kernels take 8-row tiles, e8p_decode.py:36-58, and
    // route_metadata builds such lists by default): integer_vq_grouped runs them on the MFMA tiles, e8p_decode_grouped on
    // the streaming kernel, whose workgroup takes the stretch of up to 32 rows that starts at a multiple of 32
    const bool small_list = f->block_m == 8 || f->block_m == 16;
    const bool small_tile = small_list && (vq || f->packed_k == 64);  // 64-wide blocks are read by the MFMA tiles only
    if (f->block_m != 32 && f->block_m != 64 && f->block_m != 128 && !small_list) {
        set_error("%s: block_m must be 8, 16, 32, 64 or 128 (row step of the routed tile list)", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (small_list && !small_tile && (f->flags2 != 0 || (f->algorithm != kAuto && f->algorithm != kStream))) {
        set_error("%s: tile lists in steps of 8 or 16 rows run on the streaming kernel (algorithm auto or stream, int8 rows, plain epilogue)",
                  name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->packed_k != 128 && f->packed_k != 64 && f->packed_k != 0) {  // e8p_decode.py:43, integer_vq.py:75
        set_error("%s: packed_k must be 128 or 64 (K-major blocks) or 0 (row-major per expert)", name);
        return ORX_ERR_BAD_VARIANT;
    }
    // Zero coordinates, per-expert tables, patches, 8- and 16-row tile lists and 64-wide blocks are served by
    // the MFMA tiles with the general decode.
    const bool general = patched || !shared_table || basis == "any" || small_tile || f->packed_k == 64 || book_form != kBookSelector;
    f->H = (general ? kGeneralDecode : 0) | (patched ? kPatched : 0) | (shared_table ? 0 : kExpertTables) | (vq ? kTakesPatch : 0) |
           (book_form << kBookFormShift);
    if (general && (f->flags2 != 0 || (f->algorithm != kAuto && f->algorithm != kMfma))) {
        set_error("%s: patched, shared_table=false, basis=any, block_m 8|16 and packed_k=64 run on the MFMA tiles "
                  "(algorithm auto or mfma, int8 rows, plain epilogue)", name);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->algorithm == kResident && !grouped_resident_eligible(f->N, f->K, f->block_m, f->tiles, 0, 0, f->capacity)) {
        set_error("%s: algorithm=resident needs block_m=32, at most 1024 tiles, N a multiple of 32 and K/128 even or a multiple of 3, K <= 2304",
                  name);
        return ORX_ERR_BAD_VARIANT;
    }
    // gather=true: A and AS are per token, SlotToken names every slot's token, and the kernel gathers the rows
    // while it stages a tile (no dispatch copy).  epilogue=swiglu: N = gate | up; Act (slots, N/2) receives
    // fp16(silu(gate) * up), RowMax (slots, zero before the launch) is raised to the fp32 bits of every slot's
    // largest |Act|, and C may be null.  input_dtype=float16: A holds such fp16 rows and RowMax their maxima; the
    // rows are quantised by the A8 rule while staged, and AS and Q (either may be null) receive scales and codes.
    // All three are forms of the resident kernel: served where `auto` picks it, or by name.
    if (f->flags2 != 0) {
        if ((f->algorithm != kAuto && f->algorithm != kResident) ||
            !grouped_resident_eligible(f->N, f->K, f->block_m, f->tiles, f->flags2 & 3, f->flags2 >> 2, f->capacity) ||
            (f->algorithm == kAuto && !grouped_resident_preferred(f->capacity, f->E, f->N))) {
            set_error("%s: gather, epilogue=swiglu and input_dtype=float16 are forms of the resident kernel (block_m=32, "
                      "gathered slots that fit LDS beside the staged rows, K <= 1024 for float16 rows) where the routed rows fill the chip", name);
            return ORX_ERR_BAD_VARIANT;
        }
    }
    {
        const uint32_t nullable = 0x80000000u;
        const bool rows16 = (f->flags2 & 3) == 2, gathered = (f->flags2 & 3) == 1, swiglu = (f->flags2 >> 2) == 1;
        f->args.clear();
        f->args.push_back({"A", ArgPointer, 16});
        f->args.push_back({"AS", ArgPointer, rows16 ? nullable | 2u : 2u});
        if (swiglu) f->args.push_back({"Act", ArgPointer, 8});
        f->args.push_back({"Book", ArgPointer, 4});
        f->args.push_back({"C", ArgPointer, swiglu ? nullable | 8u : 2u});
        f->args.push_back({"Counts", ArgPointer, 4});
        f->args.push_back({"Offsets", ArgPointer, 4});
        f->args.push_back({"P", ArgPointer, 16});
        // (E, K/128, N) u16 when patched; the reference binds a one-element dummy otherwise: never read, may be null
        if (vq) f->args.push_back({"Patch", ArgPointer, patched ? 2u : nullable | 2u});
        if (rows16) f->args.push_back({"Q", ArgPointer, nullable | 8u});
        if (rows16 || swiglu) f->args.push_back({"RowMax", ArgPointer, 4});
        if (gathered) f->args.push_back({"SlotToken", ArgPointer, 4});
        f->args.push_back({"TileCount", ArgPointer, 4});
        f->args.push_back({"TileExpert", ArgPointer, 4});
        f->args.push_back({"TileRow", ArgPointer, 4});
        f->args.push_back({"WS", ArgPointer, 2});
        if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    }
    f->geometry = grouped_geometry;
    f->launch = grouped_launch;
    // several kernels with different block sizes serve this symbol: report the device-wide limits
    f->device_function = nullptr;
    return ORX_OK;
}

// ---- integer_vq: every expert multiplies its own M rows (integer_vq.py:217-228, 262-300) -------------------
// A, AS, Book, C, P, Patch, WS.  A is (E*M, K); expert e owns rows [e*M, (e+1)*M).  Runs on the MFMA tiles with
// the general decode: any selector table, shared or per expert, patch words, blocks of 128 or 64 or row-major.
int vq_direct_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = ceil_div((uint32_t)f.N, 128u);
    g->grid[1] = ceil_div((uint32_t)f.M, (uint32_t)f.block_m);
    g->grid[2] = (uint32_t)f.E;
    g->block[0] = 256;
    return ORX_OK;
}

int vq_direct_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0), p.as = pointer_arg<const __half>(args, 1);
    p.book = pointer_arg<const uint32_t>(args, 2), p.out = pointer_arg<void>(args, 3), p.w = pointer_arg<const void>(args, 4);
    p.patch = (f.H & kPatched) ? pointer_arg<const uint16_t>(args, 5) : nullptr;
    p.ws = pointer_arg<const __half>(args, 6);
    p.n = f.N, p.k = f.K, p.stride = f.N, p.m = f.capacity, p.packed_k = f.packed_k, p.out_f32 = 0;
    p.expert_weight_stride = (int64_t)f.N * (f.K / 8) * 2;
    p.book_form = (f.H >> kBookFormShift) & 3;
    p.book_stride = (f.H & kExpertTables) ? book_words(p.book_form) : 0;
    p.direct_rows = f.M;
    return launch_mfma_general(f.block_m, p, g, stream);
}

int make_vq_direct(const Variant& v, orx_function* f) {
    bool bad = false;
    f->E = (int)v.integer("E", 0, &bad);
    f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    const int block_m = (int)v.integer("block_m", 16, &bad);  // integer_vq.py:275
    f->packed_k = (int)v.integer("packed_k", 128, &bad);
    const bool patched = v.boolean("patched", false, &bad);
    const bool shared_table = v.boolean("shared_table", false, &bad);  // integer_vq.py:271
    const std::string kind = v.string("kind", "e8p", &bad);
    // Book (integer_vq.py:93-107): raw basis values (256, 2), signed values (512, 4) with shortbook, selector words
    // (256, 1) with shortbook + selectorbook
    const bool shortbook = v.boolean("shortbook", false, &bad), selectorbook = v.boolean("selectorbook", false, &bad);
    const bool byte_permute = v.boolean("byte_permute", false, &bad);
    for (const char* hint : {"block_n", "num_stages"}) v.accept(hint);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (kind != "e8p" || ((selectorbook || byte_permute) && !shortbook)) {
        set_error("integer_vq: kind must be e8p; selectorbook and byte_permute need shortbook");
        return ORX_ERR_BAD_VARIANT;
    }
    const int book_form = selectorbook ? kBookSelector : shortbook ? kBookSigned : kBookRaw;
    if (f->E <= 0 || f->M <= 0 || f->N <= 0 || f->K <= 0 || f->K % 128 || (int64_t)f->K * 128 * 128 > 2147483647LL ||
        (int64_t)f->E * f->M > 2147483647LL) {
        set_error("integer_vq: invalid integer VQ geometry");  // integer_vq.py:86
        return ORX_ERR_BAD_VARIANT;
    }
    if (block_m != 8 && block_m != 16 && block_m != 32 && block_m != 64) {
        set_error("integer_vq: invalid VQ row tile (block_m 8, 16, 32 or 64)");  // integer_vq.py:89-90
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->packed_k != 128 && f->packed_k != 64 && f->packed_k != 0) {
        set_error("integer_vq: packed_k must be 128 or 64 (K-major) or 0 (row-major per expert)");
        return ORX_ERR_BAD_VARIANT;
    }
    f->capacity = f->E * f->M;
    f->block_m = block_m < 32 ? 32 : block_m;  // 8 and 16 rows ride in a 32-row tile: the row ranges are the same
    f->H = kGeneralDecode | (patched ? kPatched : 0) | (shared_table ? 0 : kExpertTables) | kTakesPatch | (book_form << kBookFormShift);
    const uint32_t nullable = 0x80000000u;
    f->args = {{"A", ArgPointer, 16}, {"AS", ArgPointer, 2}, {"Book", ArgPointer, 4}, {"C", ArgPointer, 2},
               {"P", ArgPointer, 16}, {"Patch", ArgPointer, patched ? 2u : nullable | 2u}, {"WS", ArgPointer, 2}};
    f->geometry = vq_direct_geometry;
    f->launch = vq_direct_launch;
    f->device_function = block_m <= 32 ? reinterpret_cast<const void*>(&gemm_kernel<kQ2, 32, 128, 1, true, false, true>)
                                       : reinterpret_cast<const void*>(&gemm_kernel<kQ2, 64, 128, 2, true, false, true>);
    return ORX_OK;
}

// ---- routed Q4 / W8 banks (kernels/cuda/model/moe.py:52-143) ---------------------------------
// A, AS, Book, Counts, Offsets, Out, TileCount, TileExpert, TileRow, W, WS[, m]: the buffers of
// moe.py:115-127 in generated-ABI order.  The tile list is the caller's (built with the variant's
// block_m); a tile runs on the smallest MFMA tile that holds block_m rows.
int experts_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = ceil_div((uint32_t)f.N, 128u);
    g->grid[1] = (uint32_t)f.tiles * (f.block_m == 256 ? 2u : 1u);  // a listed tile of 256 rows: two MFMA tiles of 128
    g->block[0] = 256;
    return ORX_OK;
}

int experts_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    GemmParams p = {};
    p.a = pointer_arg<const int8_t>(args, 0);
    p.as = pointer_arg<const __half>(args, 1);
    p.book = pointer_arg<const uint32_t>(args, 2);
    p.counts = pointer_arg<const int>(args, 3);
    p.offsets = pointer_arg<const int>(args, 4);
    p.out = pointer_arg<void>(args, 5);
    p.tile_count = pointer_arg<const int>(args, 6);
    p.tile_expert = pointer_arg<const int>(args, 7);
    p.tile_row = pointer_arg<const int>(args, 8);
    p.w = pointer_arg<const void>(args, 9);
    p.ws = pointer_arg<const __half>(args, 10);
    p.n = f.N, p.k = f.K, p.stride = f.N, p.m = f.capacity * f.top_k, p.out_f32 = 0;
    p.tile_rows = f.block_m;
    p.list_split = f.block_m == 256 ? 2 : 0;
    const int bm = f.block_m <= 32 ? 32 : f.block_m <= 64 ? 64 : 128;
    if (f.flags == kQ4) {
        p.packed_k = 128;
        p.expert_weight_stride = (int64_t)f.N * (f.K / 2);
        return launch_mfma<kQ4, true>(bm, p, g, stream);
    }
    p.packed_k = 0;
    p.expert_weight_stride = (int64_t)f.N * f.K;
    return launch_mfma<kW8, true>(bm, p, g, stream);
}

int make_integer_experts(const Variant& v, orx_function* f) {
    bool bad = false;
    f->capacity = f->M = (int)v.integer("M", 0, &bad);
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    f->top_k = (int)v.integer("top_k", 0, &bad);
    f->block_m = (int)v.integer("block_m", 16, &bad);
    f->dynamic_rows = v.boolean("dynamic_rows", false, &bad);
    const std::string codec = v.string("codec", "e8p_q4", &bad);
    if (!bad && codec == "e8p_q4" && !two_stage_coefficients_ok(v, "integer_experts")) return ORX_ERR_BAD_VARIANT;
    // the reference's tile hints: checked as it checks them (moe.py:72-88), otherwise not used
    const long long block_n = v.integer("block_n", 64, &bad), block_k = v.integer("block_k", 128, &bad);
    const long long stages = v.integer("stages", 2, &bad), minimum_blocks = v.integer("minimum_blocks", 1, &bad);
    (void)v.integer("tail_m", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    const bool w8 = codec == "w8";
    const bool block_m_ok = f->block_m == 8 || f->block_m == 16 || f->block_m == 32 || f->block_m == 64 || f->block_m == 128 ||
                            f->block_m == 256;  // moe.py:77
    if (f->M <= 0 || f->N <= 0 || f->K <= 0 || f->E <= 0 || f->top_k <= 0 || f->top_k > f->E || f->K % 128 || !block_m_ok ||
        (block_n != 32 && block_n != 64 && block_n != 128) || (!w8 && codec != "e8p_q4") ||
        (w8 && (f->block_m == 8 || block_n == 32)) || (block_k != 128 && block_k != 256) || f->K % block_k ||
        (stages != 1 && stages != 2) || minimum_blocks <= 0 || (int64_t)f->K * 128 * 128 > 2147483647LL) {
        set_error("integer_experts: invalid grouped integer projection geometry");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = w8 ? kW8 : kQ4;
    const int64_t assignments = (int64_t)f->M * f->top_k;
    f->tiles = (int)((assignments + f->block_m - 1) / f->block_m + std::min<int64_t>(f->E, assignments));  // moe.py:89
    f->args = {{"A", ArgPointer, 16},        {"AS", ArgPointer, 2},         {"Book", ArgPointer, 4},
               {"Counts", ArgPointer, 4},    {"Offsets", ArgPointer, 4},    {"Out", ArgPointer, 2},
               {"TileCount", ArgPointer, 4}, {"TileExpert", ArgPointer, 4}, {"TileRow", ArgPointer, 4},
               {"W", ArgPointer, 16},        {"WS", ArgPointer, 2}};
    if (f->dynamic_rows) f->args.push_back({"m", ArgI32, 4});
    f->geometry = experts_geometry;
    f->launch = experts_launch;
    f->device_function = nullptr;
    return ORX_OK;
}

// ---- unpack ----------------------------------------------------------------------------------
// Book, Output, W
int unpack_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = ceil_div((uint32_t)((int64_t)f.N * (f.K / 8)), 256u);
    g->block[0] = 256;
    return ORX_OK;
}

int unpack_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    const uint32_t* book = pointer_arg<const uint32_t>(args, 0);
    uint2* out = pointer_arg<uint2>(args, 1);
    const void* w = pointer_arg<const void>(args, 2);
    if (f.flags == kQ4)
        ORX_LAUNCH((unpack_kernel<kQ4>), dim3(g.grid[0]), dim3(256), 0, stream, w, book, out, f.N, f.K, f.packed_k, nullptr);
    else
        ORX_LAUNCH((unpack_kernel<kQ2>), dim3(g.grid[0]), dim3(256), 0, stream, w, book, out, f.N, f.K, f.packed_k, nullptr);
    return hip_check(hipGetLastError(), "launch unpack");
}

// expand_experts (kernels/cuda/model/moe.py:146-173): Book, Counts, Out, W.  slots used: N, K, E
int expand_geometry(const orx_function& f, int rows, Geometry* g) {
    (void)rows;
    g->grid[0] = ceil_div((uint32_t)((int64_t)f.N * (f.K / 8)), 256u);
    g->grid[1] = (uint32_t)f.E;
    g->block[0] = 256;
    return ORX_OK;
}
int expand_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, void** args) {
    (void)rows;
    ORX_LAUNCH((unpack_kernel<kQ4>), dim3(g.grid[0], g.grid[1]), dim3(256), 0, stream, pointer_arg<const void>(args, 3),
                       pointer_arg<const uint32_t>(args, 0), pointer_arg<uint2>(args, 2), f.N, f.K, 128,
                       pointer_arg<const int>(args, 1));
    return hip_check(hipGetLastError(), "launch expand_experts");
}
int make_expand_experts(const Variant& v, orx_function* f) {
    bool bad = false;
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->E = (int)v.integer("E", 0, &bad);
    const int block_n = (int)v.integer("block_n", 64, &bad), block_k = (int)v.integer("block_k", 256, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    // moe.py:152-153: whole tiles of the reference's kernel; the codes come in K-major blocks of 128
    if (f->N <= 0 || f->K <= 0 || f->E <= 0 || block_n <= 0 || block_k <= 0 || f->N % block_n || f->K % block_k || f->K % 128) {
        set_error("expand_experts: need N, K, E > 0, N a multiple of block_n, K a multiple of block_k and of 128");
        return ORX_ERR_BAD_VARIANT;
    }
    f->capacity = 1;
    f->args = {{"Book", ArgPointer, 4}, {"Counts", ArgPointer, 4}, {"Out", ArgPointer, 8}, {"W", ArgPointer, 4}};
    f->geometry = expand_geometry;
    f->launch = expand_launch;
    f->device_function = reinterpret_cast<const void*>(&unpack_kernel<kQ4>);
    return ORX_OK;
}

int make_unpack(const Variant& v, orx_function* f, int codec) {
    if (codec == kQ4 && !two_stage_coefficients_ok(v, "e8p_q4_unpack")) return ORX_ERR_BAD_VARIANT;
    bool bad = false;
    f->N = (int)v.integer("N", 0, &bad);
    f->K = (int)v.integer("K", 0, &bad);
    f->packed_k = (int)v.integer("packed_k", 0, &bad);
    if (bad) return ORX_ERR_BAD_VARIANT;
    if (f->N <= 0 || f->K <= 0 || f->K % 128 || (f->packed_k != 0 && f->packed_k != 64 && f->packed_k != 128)) {
        set_error("%s: need N,K > 0, K a multiple of 128, packed_k in {0,64,128}", f->symbol.c_str());
        return ORX_ERR_BAD_VARIANT;
    }
    f->capacity = 1;
    f->flags = codec;
    f->args = {{"Book", ArgPointer, 4}, {"Output", ArgPointer, 8}, {"W", ArgPointer, 4}};
    f->geometry = unpack_geometry;
    f->launch = unpack_launch;
    f->device_function = reinterpret_cast<const void*>(&unpack_kernel<kQ4>);
    return ORX_OK;
}
int make_q4_unpack(const Variant& v, orx_function* f) { return make_unpack(v, f, kQ4); }
int make_q2_unpack(const Variant& v, orx_function* f) { return make_unpack(v, f, kQ2); }

}  // namespace

const Registration* gemm_registrations(int* count) {
    static const Registration rows[] = {
    {"e8p_q4_projection", make_q4_projection,
     "M, N, K, dynamic_rows=false, algorithm=auto|gemv|stream|resident|wide|mfma, packed_k=0|64|128, output_dtype=float16|float32, "
     "input_dtype=int8|float16, rotate=false, workspace=false, split_k=true, "
     "output_stride=N, block_m=0|32|64|128|256, gemv_passes=0, decode_in_gemm=false",
     "A,AS,Book,Out,S[,Signs],W[,Workspace][,m]"},
    {"int8_projection", make_w8_projection,
     "M, N, K, dynamic_rows=false, algorithm=auto|gemv|stream|mfma, output_dtype=float16|float32, output_stride=N, "
     "block_m=0|32|64|128|256, workspace=false, split_k=true",
     "A,Output,TokenScale,Weight,WeightScale[,Workspace][,m]"},
    {"int8_small_projection", make_w8_small_projection,
     "M, N, K, dynamic_rows=false, output_dtype=float16|float32, output_stride=N, block_m=min(M,4) (1..8), block_n=4|8|16, workspace=false",
     "A,Output,TokenScale,Weight,WeightScale[,Workspace][,m]"},
    {"int8_swiglu", make_int8_swiglu, "M, N, K, dynamic_rows=false, algorithm=tensor_core|dp4a, block_m, block_n (checked, not used)",
     "A,Gate,GateScale,Output,TokenScale,Up,UpScale[,m]"},
    {"e8p_decode_grouped", make_q2_grouped,
     "rows, E, tiles, N, K, block_m=32|64|128|8|16 (row step of the tile list), packed_k=128|64|0, dynamic_rows=false, algorithm=auto|stream|resident|mfma, input_dtype=int8|float16, gather=false, epilogue=none|swiglu",
     "A,AS[,Act],Book,C,Counts,Offsets,P[,Q][,RowMax][,SlotToken],TileCount,TileExpert,TileRow,WS[,m]"},
    {"integer_vq", make_vq_direct,
     "E, M (rows of every expert), N, K, block_m=16|8|32|64, packed_k=128|64|0, patched=false, shared_table=false, shortbook=false, "
     "selectorbook=false (Book: raw basis (256,2) | signed values (512,4) with shortbook | selector words (256,1) with both)",
     "A,AS,Book,C,P,Patch,WS"},
    {"integer_vq_grouped", make_q2_grouped,
     "rows, E, tiles, N, K, block_m=16|8|32|64|128, packed_k=128|64|0, dynamic_rows=false, patched=false, shared_table=false, shortbook=false, "
     "selectorbook=false (Book as for integer_vq), basis=spread29|any, "
     "algorithm=auto|stream|resident|mfma, input_dtype=int8|float16, gather=false, epilogue=none|swiglu",
     "A,AS[,Act],Book,C,Counts,Offsets,P,Patch[,Q][,RowMax][,SlotToken],TileCount,TileExpert,TileRow,WS[,m]"},
    {"integer_experts", make_integer_experts,
     "M, N, K, E, top_k, codec=e8p_q4|w8, block_m=16 (8..256), dynamic_rows=false, block_n, block_k, stages, tail_m, minimum_blocks",
     "A,AS,Book,Counts,Offsets,Out,TileCount,TileExpert,TileRow,W,WS[,m]"},
    {"e8p_q4_unpack", make_q4_unpack, "N, K, packed_k=0|64|128", "Book,Output,W"},
    {"e8p_q2_unpack", make_q2_unpack, "N, K, packed_k=0|64|128", "Book,Output,W"},
    {"q4_projection", make_row_q4_projection,
     "M, N, K, BN=64, BK=128, output_dtype=float16|float32, magnitudes=[3,10,19,31,46,67,93,127], block_m=8, dynamic_rows=false, "
     "stages=2, output_stride=N, tail_m=0, group_m=0, workspace=false",
     "A,AS,Out,S,W[,Workspace][,m]"},
    {"q4_gemv", make_row_q4_gemv,
     "M, N, K, BN=16, output_dtype=float16|float32, magnitudes=[...], dynamic_rows=false, block_m=min(M,8), output_stride=N",
     "A,AS,Out,S,W[,m]"},
    {"unpack_q4", make_row_q4_unpack, "N, K, magnitudes=[3,10,19,31,46,67,93,127]", "Output,W"},
    {"expand_experts", make_expand_experts, "N, K, E, block_n=64, block_k=256", "Book,Counts,Out,W"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
