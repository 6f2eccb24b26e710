// Two-stage (Q4) projections for 3..32 token rows (batched decode): one resident workgroup per CU.
//
// Reference counterparts: the small-row Tensor Core schedules of kernels/cuda/model/integer_core.py
// (block_m 8..32) behind kernels/cuda/model/e8p_q4.py:143-264.  Arithmetic: exact int32 over the full
// K, (float(acc) * ws) * as.
//
// MI355X design.  With so few rows the projection is a weight stream (0.5 byte per weight):
//  * Output channels are dealt to CUs in equal contiguous runs (N / CUs each, 68 at N = 17408), cut
//    into blocks of 16 channels for v_mfma_i32_16x16x64_i8, so every CU has the same work.
//  * K is split over the decoding waves.  A wave keeps the token fragments of its K slice in
//    registers for the whole kernel (they are the same for every channel block), so activations are
//    read once per CU.
//  * Codes are decoded with two 8-byte lookups per stage in tables stored 16 times (one copy per
//    lane of an access group, so lanes never share a bank; the address is one v_perm_b32); the two
//    stages share one pair of tables (values v+8, shifted by the stage's weight when combined).
//  * The K-slice partial sums of a block are added with LDS integer atomics (exact in any order);
//    after a barrier 16 x M threads rescale and store the block while the others decode the next.
// Two kernels share this: dense_specialized_kernel (K up to 5120 in steps of 512: four loader waves
// stream the codes into LDS, eight decoder waves never touch memory) and dense_resident_kernel (K up
// to 8192 in steps of 1024: sixteen waves, each loading its own codes through a register ring).
#include <hip/hip_fp16.h>

#include "e8p_device.h"
#include "orx_internal.h"

namespace orx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Tables: entry i of the basis table ((h ^ 8) per coordinate) at byte i*256 + copy*8, entry u of the
// sign/parity mask table at u*256 + 128 + copy*8, 16 copies each.  With the entry index in the
// address's second byte, one v_perm_b32 builds a lookup address from a byte of the code.
constexpr uint32_t kMaskOffset = 128;
constexpr uint32_t kSumBase = 65536;      // two sets of kMaxHeld buffers of 16 channels x 33 ints
constexpr int kSumStride = 33;
constexpr int kSumBuffer = 16 * kSumStride;
constexpr int kMaxHeld = 3;               // channel blocks between two barriers (= ring depth)
constexpr uint32_t kScaleBase = kSumBase + 2 * kMaxHeld * kSumBuffer * 4;  // fp16 weight scales of this CU's channels

struct DenseParams {
    const int8_t* a;
    const uint8_t* w;
    const uint32_t* book;
    const __half* ws;
    const __half* as;
    void* out;
    int n, k, stride, m, out_f32, k_major;
};

// W: waves per workgroup (K is split over them); S: 64-wide K steps per wave (K = 64 W S); CB: token
// tiles of 16; P: channel blocks whose codes a lane holds at once.
template <int W, int S, int CB, int P>
__global__ __launch_bounds__(W * 64) void dense_resident_kernel(DenseParams p) {
    constexpr int kWaves = W, kThreads = W * 64;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int column = lane & 15, quarter = lane >> 4;  // MFMA operand row/column and 16-byte K group
    const int groups = (int)gridDim.x, group = (int)blockIdx.x;
    const int run = (p.n + groups - 1) / groups;        // channels per CU
    const int first_row = group * run;
    const int rows_here = min(run, p.n - first_row);
    if (rows_here <= 0) return;                         // same for the whole workgroup
    const int blocks = (rows_here + 15) / 16;
    int* sums = reinterpret_cast<int*>(lds + kSumBase);
    __half* scales = reinterpret_cast<__half*>(lds + kScaleBase);

    // ---- set-up reads ------------------------------------------------------------------------------
    // A lane's K positions inside its wave's slice: steps come in pairs, and in a pair the lane owns 32
    // consecutive weights (first 16 for the even step, next 16 for the odd one), so that its codes
    // of a pair are one 16-byte load; an odd last step is an 8-byte load.  Both operands follow the
    // same map, which is all the MFMA needs.
    uint32_t selector = 0;
    if (wave < 4) selector = p.book[tid];
    constexpr int kPairs = S / 2;
    constexpr bool kOdd = S % 2 != 0;
    const int k_slice = p.k / kWaves;
    auto step_offset = [&](int s) {  // first weight of step s for this lane, inside the slice
        return s < 2 * kPairs ? 128 * (s >> 1) + 32 * quarter + 16 * (s & 1) : 64 * s + 16 * quarter;
    };
    v4u tokens[CB][S];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
        const int8_t* row = p.a + (int64_t)min(16 * c + column, p.m - 1) * p.k + wave * k_slice;
#pragma unroll
        for (int s = 0; s < S; ++s) tokens[c][s] = *reinterpret_cast<const v4u*>(row + step_offset(s));
    }
    // codes of this lane: channel row `column` of a block (8 weights per 4-byte code)
    const int64_t row_bytes = p.k / 2;
    struct Codes {
        v4u pair[kPairs > 0 ? kPairs : 1];
        v2u last;
    };
    auto load_codes = [&](Codes& codes, int block) {
        const int row = first_row + min(16 * block + column, rows_here - 1);
        const uint8_t* src = p.w + row * row_bytes + wave * (k_slice / 2);
#pragma unroll
        for (int d = 0; d < kPairs; ++d) codes.pair[d] = *reinterpret_cast<const v4u*>(src + 64 * d + 16 * quarter);
        if (kOdd) codes.last = *reinterpret_cast<const v2u*>(src + 32 * (S - 1) + 8 * quarter);
    };
    // Only the first block's codes travel with the set-up reads; the rest of the ring is requested
    // after the barrier.  A wave cannot issue anything while one of its loads waits for a slot in
    // the CU's memory pipeline, so a whole stream requested up front would hold back the table
    // build and with it every wave's first MFMA.
    Codes ring[P];
    load_codes(ring[0], 0);
    // finalising threads: token tid/16, channel tid%16 of a block
    const int out_channel = tid & 15, out_token = tid >> 4;
    const bool finalises = out_token < p.m && out_token < 16 * CB;
    const float token_scale = __half2float(p.as[min(out_token, p.m - 1)]);
    for (int i = tid; i < rows_here; i += kThreads) scales[i] = p.ws[first_row + i];

    static_assert(W >= 8, "waves 0-3 build the basis table, waves 4-7 the mask table");
    if (wave < 8) {
        const int entry = tid & 255;
        const uint2 value = wave < 4 ? byte_basis_biased(selector, 0) : byte_mask_biased((uint32_t)entry, 0);
        const uint4 pair = make_uint4(value.x, value.y, value.x, value.y);
        uint8_t* dst = lds + entry * 256 + (wave < 4 ? 0 : kMaskOffset);
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(dst + 16 * i) = pair;
    }
    for (int i = tid; i < 2 * kMaxHeld * kSumBuffer; i += kThreads) sums[i] = 0;
    __syncthreads();
#pragma unroll
    for (int slot = 1; slot < P; ++slot) load_codes(ring[slot], min(slot, blocks - 1));

    // byte 0: this lane's copy in the basis half of an entry, byte 1: in the mask half
    const uint32_t copy = (uint32_t)(lane & 15) * 8;
    const uint32_t columns = copy | (kMaskOffset | copy) << 8;
    // selectors of v_perm_b32(code, columns): address byte 0 = a byte of `columns`, byte 1 = a byte of the code
    constexpr uint32_t kBasisLow = 0x0C0C0500u, kMaskLow = 0x0C0C0401u, kBasisHigh = 0x0C0C0700u, kMaskHigh = 0x0C0C0601u;
    auto lookup = [&](uint32_t code, uint32_t selector) {
        return *reinterpret_cast<const uint2*>(lds + __builtin_amdgcn_perm(code, columns, selector));
    };
    // one u32 two-stage code -> 8 int8 weights: w + 128 = 8 (v0 + 8) + 2 (v1 + 8) + 53 in every byte
    auto decode = [&](uint32_t code) {
        const uint2 b0 = lookup(code, kBasisLow), m0 = lookup(code, kMaskLow);
        const uint2 b1 = lookup(code, kBasisHigh), m1 = lookup(code, kMaskHigh);
        uint2 w;
        w.x = ((((b0.x ^ m0.x) << 3) + ((b1.x ^ m1.x) << 1)) + 0x35353535u) ^ 0x80808080u;
        w.y = ((((b0.y ^ m0.y) << 3) + ((b1.y ^ m1.y) << 1)) + 0x35353535u) ^ 0x80808080u;
        return w;
    };

    // One barrier per group of P blocks: the waves decode P blocks back to back, each into its own
    // sum buffer, meet once, and the finalising threads store the group while the others go on.
    // (Tried: no barrier at all, with an arrival counter per block and the last wave storing it.  The
    // waves then drift apart by up to 8 us, because a wave whose loads are accepted late by the CU's
    // memory pipeline never catches up, and the kernel gets slower.)
    static_assert(P <= kMaxHeld, "one sum buffer per held block");
    for (int first = 0, set = 0; first < blocks; first += P, set ^= 1) {
        int* group_sums = sums + set * (kMaxHeld * kSumBuffer);
#pragma unroll
        for (int slot = 0; slot < P; ++slot) {
            const int block = first + slot;
            if (block < blocks) {  // same for the whole workgroup
                v4i acc[CB];
#pragma unroll
                for (int c = 0; c < CB; ++c) acc[c] = v4i{0, 0, 0, 0};
#pragma unroll
                for (int s = 0; s < S; ++s) {
                    uint32_t first_code, second_code;  // the 16 weights of this step
                    if (s < 2 * kPairs) {
                        const v4u pair = ring[slot].pair[s >> 1];
                        first_code = (s & 1) ? pair.z : pair.x, second_code = (s & 1) ? pair.w : pair.y;
                    } else {
                        first_code = ring[slot].last.x, second_code = ring[slot].last.y;
                    }
                    const uint2 lo = decode(first_code), hi = decode(second_code);
                    const v4i weights = {(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
#pragma unroll
                    for (int c = 0; c < CB; ++c) {
                        const v4i token = {(int)tokens[c][s].x, (int)tokens[c][s].y, (int)tokens[c][s].z, (int)tokens[c][s].w};
                        acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(weights, token, acc[c], 0, 0, 0);
                    }
                }
                if (block + P < blocks) load_codes(ring[slot], block + P);
                // accumulator i of a lane: channel 4*quarter + i, token 16*c + column
                int* mine = group_sums + slot * kSumBuffer + 4 * quarter * kSumStride + column;
#pragma unroll
                for (int c = 0; c < CB; ++c)
#pragma unroll
                    for (int i = 0; i < 4; ++i) atomicAdd(mine + i * kSumStride + 16 * c, acc[c][i]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int slot = 0; slot < P; ++slot) {
            const int channel = 16 * (first + slot) + out_channel;
            if (finalises && channel < rows_here) {
                int* cell = group_sums + slot * kSumBuffer + out_channel * kSumStride + out_token;
                const float value = rescale(*cell, __half2float(scales[channel]), token_scale);
                *cell = 0;
                const int64_t index = (int64_t)out_token * p.stride + first_row + channel;
                if (p.out_f32)
                    reinterpret_cast<float*>(p.out)[index] = value;
                else
                    reinterpret_cast<__half*>(p.out)[index] = __float2half_rn(value);
            }
        }
    }
}

// ---- the same projection with loader waves -------------------------------------------------------------
// A wave cannot issue anything while one of its vector loads waits for a slot in the CU's memory
// pipeline, and in a bandwidth-bound kernel that is most of the time: in the kernel above the decode
// of a wave is serialised behind its own code loads (decode alone 12.9 us, loads alone 13.4 us,
// together 19.5 us at N=17408, K=5120, 8 rows).  Here four loader waves do nothing but request the
// CU's codes, whole rows at a time and straight into LDS (no registers, fully contiguous requests),
// while eight decoder waves (two per SIMD, K split eight ways) never touch memory after set-up: they
// read their codes from LDS.  Two code buffers of 16 channel rows each; one barrier per block.
constexpr int kDecoders = 8, kLoaders = 4;
constexpr int kSpecThreads = (kDecoders + kLoaders) * 64;
constexpr int kRowPad = 16;  // bytes between staged code rows: 16 rows read at the same K then hit 16 different bank groups

__device__ __forceinline__ void direct_load_16(const void* global, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// S: 64-wide K steps per decoder wave (K = 512 S); CB: token tiles of 16; KM: K-major codes (K/128
// blocks of N rows x 64 bytes; S is even then, so a decoder wave owns whole K blocks).
template <int S, int CB, bool KM>
__global__ __launch_bounds__(kSpecThreads) void dense_specialized_kernel(DenseParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int column = lane & 15, quarter = lane >> 4;
    const int groups = (int)gridDim.x, group = (int)blockIdx.x;
    const int run = (p.n + groups - 1) / groups;
    const int first_row = group * run;
    const int rows_here = min(run, p.n - first_row);
    if (rows_here <= 0) return;  // same for the whole workgroup
    const int blocks = (rows_here + 15) / 16;
    constexpr int kRowBytes = 256 * S;                       // codes of one channel row
    constexpr int kPitch = kRowBytes + kRowPad;
    constexpr int kPieces = (kRowBytes + 1023) / 1024;       // 1 KiB requests per row
    constexpr int kKBlocks = kDecoders * S / 2;              // K-major: one 1 KiB request per K block and channel block
    constexpr int kPerLoader = (KM ? kKBlocks : 16 * kPieces) / kLoaders;  // requests of one loader wave per block
    static_assert(16 * kPieces % kLoaders == 0, "every loader wave issues the same number of requests");
    static_assert(!KM || S % 2 == 0, "K-major: a decoder wave owns whole K blocks");
    int* sums = reinterpret_cast<int*>(lds + kSumBase);
    __half* scales = reinterpret_cast<__half*>(lds + kScaleBase);
    const uint32_t code_base = kScaleBase + (((uint32_t)run * 2 + 15) & ~15u);
    auto buffer = [&](int block) { return lds + code_base + (block & 1) * (16 * kPitch); };
    // The block that is not full (this CU's last rows) goes first: it lands quickly, while the tables
    // are still being built, and the kernel does not end with a block that is mostly padding.
    const int odd_rows = rows_here & 15;
    auto block_start = [&](int block) { return odd_rows == 0 ? 16 * block : block == 0 ? rows_here - odd_rows : 16 * (block - 1); };
    auto block_rows = [&](int block) { return odd_rows != 0 && block == 0 ? odd_rows : 16; };

    if (wave >= kDecoders) {
        // ---- loader waves ----
        // One block is in flight at a time, requested the moment its buffer is released.  One block
        // per CU (10 MB over the chip) already keeps HBM busy: it lands 2 us after the request,
        // which is the CU's share of the bandwidth.  Requesting more at once only delays the first
        // block, because everything in flight shares that bandwidth (two blocks at the start: first
        // MFMA at 5.2 us; a third block parked in the loaders' registers: 0.7 us slower overall).
        const int loader = wave - kDecoders;
        auto request = [&](int block) {
            const int rows_in_block = block_rows(block), start = block_start(block);
            uint8_t* dst = buffer(block);
            if constexpr (KM) {
                // One request is one K block of the 16 rows: 1 KiB contiguous in memory.  LDS position
                // i (16 bytes each) holds row i/4, piece (i%4) ^ ((i/8)&3): with that swizzle the
                // decoders' reads of one piece of 16 different rows fall into different bank groups.
                const int row = lane >> 2, piece = (lane & 3) ^ ((lane >> 3) & 3);
                // (blocks of 64: the K block's two halves lie N rows x 32 bytes apart, 512 contiguous bytes each)
                const uint8_t* src = p.k_major == 2 ? p.w + ((int64_t)first_row + start + row) * 32 + (piece & 1) * 16 +
                                                          (int64_t)(piece >> 1) * p.n * 32
                                                    : p.w + ((int64_t)first_row + start + row) * 64 + piece * 16;
#pragma unroll
                for (int i = 0; i < kPerLoader; ++i) {
                    const int kb = loader + kLoaders * i;
                    if (row < rows_in_block) direct_load_16(src + (int64_t)kb * p.n * 64, dst + kb * 1024);
                }
            } else {
                const uint8_t* src = p.w + (int64_t)(first_row + start) * kRowBytes;
#pragma unroll
                for (int i = 0; i < kPerLoader; ++i) {
                    const int piece = loader + kLoaders * i, row = piece / kPieces, part = piece - row * kPieces;
                    const int offset = part * 1024 + lane * 16;
                    if (row < rows_in_block && offset < kRowBytes)
                        direct_load_16(src + (int64_t)row * kRowBytes + offset, dst + row * kPitch + part * 1024);
                }
            }
        };
        request(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS requests are not waited for by a barrier
        __syncthreads();
        for (int block = 0; block < blocks; ++block) {
            if (block + 1 < blocks) request(block + 1);       // its buffer was released at the last barrier
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();                                   // block + 1 has landed, the decoders are done with `block`
        }
        return;
    }

    // ---- decoder waves ----
    uint32_t selector = 0;
    if (wave < 4) selector = p.book[tid];
    constexpr int kPairs = S / 2;
    constexpr bool kOdd = S % 2 != 0;
    constexpr int kSlice = 64 * S;  // K positions of one decoder wave
    auto step_offset = [&](int s) {  // same K map as above: pairs of steps share 32 consecutive weights per lane
        return s < 2 * kPairs ? 128 * (s >> 1) + 32 * quarter + 16 * (s & 1) : 64 * s + 16 * quarter;
    };
    v4u tokens[CB][S];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
        const int8_t* row = p.a + (int64_t)min(16 * c + column, p.m - 1) * p.k + wave * kSlice;
#pragma unroll
        for (int s = 0; s < S; ++s) tokens[c][s] = *reinterpret_cast<const v4u*>(row + step_offset(s));
    }
    const int out_channel = tid & 15, out_token = tid >> 4;  // 512 decoder threads: 32 tokens x 16 channels
    const bool finalises = out_token < p.m && out_token < 16 * CB;
    const float token_scale = __half2float(p.as[min(out_token, p.m - 1)]);
    for (int i = tid; i < rows_here; i += kDecoders * 64) scales[i] = p.ws[first_row + i];
    {
        const int entry = tid & 255;
        const uint2 value = wave < 4 ? byte_basis_biased(selector, 0) : byte_mask_biased((uint32_t)entry, 0);
        const uint4 pair = make_uint4(value.x, value.y, value.x, value.y);
        uint8_t* dst = lds + entry * 256 + (wave < 4 ? 0 : kMaskOffset);
#pragma unroll
        for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(dst + 16 * i) = pair;
    }
    for (int i = tid; i < 2 * kSumBuffer; i += kDecoders * 64) sums[i] = 0;
    __syncthreads();

    const uint32_t copy = (uint32_t)(lane & 15) * 8;
    const uint32_t columns = copy | (kMaskOffset | copy) << 8;
    constexpr uint32_t kBasisLow = 0x0C0C0500u, kMaskLow = 0x0C0C0401u, kBasisHigh = 0x0C0C0700u, kMaskHigh = 0x0C0C0601u;
    // The tables start at LDS address 0 (the kernel has no static LDS), so the permuted bytes are the
    // address itself.
    typedef const __attribute__((address_space(3))) v2u* TableEntry;
    auto lookup = [&](uint32_t code, uint32_t selector_bytes) {
        return *reinterpret_cast<TableEntry>((uintptr_t)__builtin_amdgcn_perm(code, columns, selector_bytes));
    };
    // All lookups of a group of codes are requested before the first is used: with two decoder waves
    // per SIMD there is little else to hide the LDS latency behind.
    struct Looked {
        v2u b0, m0, b1, m1;
    };
    auto request = [&](uint32_t code) {
        return Looked{lookup(code, kBasisLow), lookup(code, kMaskLow), lookup(code, kBasisHigh), lookup(code, kMaskHigh)};
    };
    // one u32 two-stage code -> 8 int8 weights: w + 128 = 8 (v0 + 8) + 2 (v1 + 8) + 53 in every byte
    auto combine = [&](const Looked& l) {
        v2u w;
        w.x = ((((l.b0.x ^ l.m0.x) << 3) + ((l.b1.x ^ l.m1.x) << 1)) + 0x35353535u) ^ 0x80808080u;
        w.y = ((((l.b0.y ^ l.m0.y) << 3) + ((l.b1.y ^ l.m1.y) << 1)) + 0x35353535u) ^ 0x80808080u;
        return w;
    };
    auto multiply = [&](v4i (&acc)[CB], const v2u& lo, const v2u& hi, int s) {
        const v4i weights = {(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const v4i token = {(int)tokens[c][s].x, (int)tokens[c][s].y, (int)tokens[c][s].z, (int)tokens[c][s].w};
            acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(weights, token, acc[c], 0, 0, 0);
        }
    };
    // this lane's codes in a buffer: row `column`, this wave's K slice, then 64 bytes per pair of steps
    const int lane_codes = KM ? wave * (S / 2) * 1024 + (column * 4 + (quarter ^ ((column >> 1) & 3))) * 16
                              : column * kPitch + wave * (kSlice / 2) + 16 * quarter;
    constexpr int kPairBytes = KM ? 1024 : 64;

    for (int block = 0; block < blocks; ++block) {
        const uint8_t* src = buffer(block) + lane_codes;
        v4i acc[CB];
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[c] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int d = 0; d < kPairs; ++d) {
            const v4u pair = *reinterpret_cast<const v4u*>(src + kPairBytes * d);
            const Looked l0 = request(pair.x), l1 = request(pair.y), l2 = request(pair.z), l3 = request(pair.w);
            multiply(acc, combine(l0), combine(l1), 2 * d);
            multiply(acc, combine(l2), combine(l3), 2 * d + 1);
        }
        if (kOdd) {
            const v2u last = *reinterpret_cast<const v2u*>(src + 32 * (S - 1) - 8 * quarter);  // lane_codes holds 16 * quarter
            const Looked l0 = request(last.x), l1 = request(last.y);
            multiply(acc, combine(l0), combine(l1), S - 1);
        }
        int* block_sums = sums + (block & 1) * kSumBuffer;
        int* mine = block_sums + 4 * quarter * kSumStride + column;
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) atomicAdd(mine + i * kSumStride + 16 * c, acc[c][i]);
        __syncthreads();
        const int channel = block_start(block) + out_channel;
        // every cell is cleared, also those of padding rows: the buffer serves another block next
        int* cell = block_sums + out_channel * kSumStride + out_token;
        const int total = out_token < 16 * CB ? *cell : 0;
        if (out_token < 16 * CB) *cell = 0;
        if (finalises && out_channel < block_rows(block)) {
            const float value = rescale(total, __half2float(scales[channel]), token_scale);
            const int64_t index = (int64_t)out_token * p.stride + first_row + channel;
            if (p.out_f32)
                reinterpret_cast<float*>(p.out)[index] = value;
            else
                reinterpret_cast<__half*>(p.out)[index] = __float2half_rn(value);
        }
    }
}


// Channel blocks whose codes a lane holds at once: 3 (2 where the token fragments of a long K leave
// less room); ring depths beyond that only delay the first MFMA.
constexpr int held_blocks(int steps, int tiles) { return 4 * steps * tiles + 6 * steps > 84 ? 2 : 3; }

// One workgroup of 16 waves per CU.  (Tried for up to 16 rows: two workgroups of 8 waves per CU, each
// wave owning K/8, so that one workgroup decodes while the other waits for memory: 20.6 against
// 19.2 us.)
int waves_for(int rows, int k) {
    (void)rows, (void)k;
    return 16;
}
int workgroups_for(int rows, int k) { return device_compute_units() * (waves_for(rows, k) == 8 ? 2 : 1); }

uint32_t lds_bytes(int n, int workgroups) {
    const int run = (n + workgroups - 1) / workgroups;
    return kScaleBase + (((uint32_t)run * 2 + 15) & ~15u);
}
constexpr uint32_t kLdsLimit = 160 * 1024;

template <int W, int S, int CB>
int launch_shape(const DenseParams& p, hipStream_t stream) {
    constexpr int P = held_blocks(S, CB);
    static DeviceOnce opted_in;  // dynamic LDS above 64 KiB needs an opt-in per kernel and device
    const int ready = opted_in.run([] {
        return hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&dense_resident_kernel<W, S, CB, P>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit),
                         "hipFuncSetAttribute");
    });
    if (ready != ORX_OK) return ready;
    const int workgroups = workgroups_for(p.m, p.k);
    ORX_LAUNCH((dense_resident_kernel<W, S, CB, P>), dim3(workgroups), dim3(W * 64), lds_bytes(p.n, workgroups),
                       stream, p);
    return hip_check(hipGetLastError(), "launch projection (resident)");
}

uint32_t specialized_lds_bytes(int n, int k) {
    const int run = (n + device_compute_units() - 1) / device_compute_units();
    return kScaleBase + (((uint32_t)run * 2 + 15) & ~15u) + 2u * 16u * (uint32_t)(k / 2 + kRowPad);
}

// Loader-wave kernel: K a multiple of 512 up to 5120 (a decoder wave holds the token fragments of K/8).
bool specialized_fits(int n, int k, int packed_k) {
    if (k % 512 != 0 || k / 512 > 10 || specialized_lds_bytes(n, k) > kLdsLimit) return false;
    return packed_k == 0 || ((packed_k == 128 || packed_k == 64) && k % 1024 == 0);
}

template <int S, int CB, bool KM>
int launch_specialized_shape(const DenseParams& p, hipStream_t stream) {
    static DeviceOnce opted_in;  // dynamic LDS above 64 KiB needs an opt-in per kernel and device
    const int ready = opted_in.run([] {
        return hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&dense_specialized_kernel<S, CB, KM>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit),
                         "hipFuncSetAttribute");
    });
    if (ready != ORX_OK) return ready;
    ORX_LAUNCH((dense_specialized_kernel<S, CB, KM>), dim3(device_compute_units()), dim3(kSpecThreads),
                       specialized_lds_bytes(p.n, p.k), stream, p);
    return hip_check(hipGetLastError(), "launch projection (resident, loader waves)");
}

template <int S>
int launch_specialized(const DenseParams& p, hipStream_t stream) {
    if constexpr (S % 2 == 0) {
        if (p.k_major)
            return p.m <= 16 ? launch_specialized_shape<S, 1, true>(p, stream) : launch_specialized_shape<S, 2, true>(p, stream);
    }
    return p.m <= 16 ? launch_specialized_shape<S, 1, false>(p, stream) : launch_specialized_shape<S, 2, false>(p, stream);
}

template <int S16>  // S16: steps per wave with 16 waves
int launch_steps(const DenseParams& p, hipStream_t stream) {
    return p.m <= 16 ? launch_shape<16, S16, 1>(p, stream) : launch_shape<16, S16, 2>(p, stream);
}

}  // namespace

// Row-major two-stage codes, K a multiple of 1024 up to 8192 (a wave's K slice is whole 64-wide
// steps and its token fragments fit in registers), at most 32 rows per launch.
bool dense_resident_eligible(int n, int k, int packed_k) {
    if (specialized_fits(n, k, packed_k)) return true;
    return packed_k == 0 && k % 1024 == 0 && k / 1024 <= 8 && lds_bytes(n, device_compute_units()) <= kLdsLimit;
}

void dense_resident_geometry(int rows, int n, int k, int packed_k, Geometry* g) {
    const int chunk = rows < 32 ? rows : 32;  // rows per launch
    g->grid[1] = g->grid[2] = 1;
    if (specialized_fits(n, k, packed_k)) {
        g->grid[0] = (uint32_t)device_compute_units();
        g->block[0] = kSpecThreads;
        g->shared = specialized_lds_bytes(n, k);
        return;
    }
    g->grid[0] = (uint32_t)workgroups_for(chunk, k);
    g->block[0] = (uint32_t)waves_for(chunk, k) * 64;
    g->shared = lds_bytes(n, (int)g->grid[0]);
}

int dense_resident_launch(const int8_t* a, const void* w, const uint32_t* book, const __half* ws, const __half* as,
                          void* out, int rows, int n, int k, int stride, int packed_k, bool out_f32, hipStream_t stream) {
    if (rows < 1 || rows > 32 || !dense_resident_eligible(n, k, packed_k)) {
        set_error("projection (resident): needs 1..32 rows and K a multiple of 512 up to 5120 or of 1024 up to 8192");
        return ORX_ERR_BAD_VARIANT;
    }
    DenseParams p = {};
    p.a = a, p.w = reinterpret_cast<const uint8_t*>(w), p.book = book, p.ws = ws, p.as = as, p.out = out;
    p.n = n, p.k = k, p.stride = stride, p.m = rows, p.out_f32 = out_f32, p.k_major = packed_k == 64 ? 2 : packed_k != 0;  // 1: blocks of 128, 2: blocks of 64
    if (specialized_fits(n, k, packed_k)) {
        switch (k / 512) {
            case 1: return launch_specialized<1>(p, stream);
            case 2: return launch_specialized<2>(p, stream);
            case 3: return launch_specialized<3>(p, stream);
            case 4: return launch_specialized<4>(p, stream);
            case 5: return launch_specialized<5>(p, stream);
            case 6: return launch_specialized<6>(p, stream);
            case 7: return launch_specialized<7>(p, stream);
            case 8: return launch_specialized<8>(p, stream);
            case 9: return launch_specialized<9>(p, stream);
            default: return launch_specialized<10>(p, stream);
        }
    }
    switch (k / 1024) {
        case 1: return launch_steps<1>(p, stream);
        case 2: return launch_steps<2>(p, stream);
        case 3: return launch_steps<3>(p, stream);
        case 4: return launch_steps<4>(p, stream);
        case 5: return launch_steps<5>(p, stream);
        case 6: return launch_steps<6>(p, stream);
        case 7: return launch_steps<7>(p, stream);
        default: return launch_steps<8>(p, stream);
    }
}

}  // namespace orx
