// Device-side E8P decode helpers shared by every kernel of liborx (gfx950 only).
//
// A u16 code is b = code>>8 (basis row), u = code&255 (sign bits + parity).
// With p = popcount(u)&1 and m = u^p, coordinate j decodes to
//     q_j = t[b][j] * (1 - 2*bit(m, SIGN_BITS[j])) + (1 - 2p),   SIGN_BITS = {0,4,1,5,2,6,3,7}
// (python/orinfer_build/quantization/vq.py:17,34-43).  Every basis value t is
// +-2, +-6 or +-10, i.e. t = 2h with h odd, and q = 2v+1 with
//     v_j = h_j XOR mask_j,   mask_j = (bit(m,..) ? 0xE : 0) ^ p          (4-bit two's complement)
// so one code decodes with two table reads and one XOR: a per-basis word and a
// per-low-byte word.  The same identity on whole bytes gives q_j = t_j ^ mask3_j with
// mask3 in {0x01, 0xFD, 0x03, 0xFF}.  The reference's nibble decoder rests on the same
// identity (quantization/vq.py:105-118); it needs a basis without zeros, which the E8P
// basis is (quantization/e8p.py:15-25).
//
// `Book` as bound by the engine is the (256,1) u32 selector table: nibble j =
// magnitude id {0:2, 1:6, 2:10, 3:0} | 4 when negative (vq.py:74-93).  The tables below
// are rebuilt from it in LDS by every workgroup, so swapping Book between graph replays
// is honoured.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace orx {

// Nibble position of coordinate j inside a packed 8-nibble word: coordinates 0..3 sit in
// the even nibbles (low nibble of bytes 0..3), coordinates 4..7 in the odd nibbles.
// (word & 0x0F0F0F0F) is then the byte vector of coordinates 0..3 and
// ((word >> 4) & 0x0F0F0F0F) that of coordinates 4..7.
__device__ __forceinline__ int nibble_slot(int j) { return j < 4 ? 2 * j : 2 * (j - 4) + 1; }

// h = t/2 of coordinate j from a selector word; 0 for the "zero" id (unsupported basis).
__device__ __forceinline__ int selector_half(uint32_t selector, int j) {
    const uint32_t id = (selector >> (4 * j)) & 7u;
    const int mag = (int)(id & 3u);
    const int h = mag == 3 ? 0 : 2 * mag + 1;
    return (id & 4u) ? -h : h;
}

// Sign bit of coordinate j in the parity-adjusted low byte m.
__device__ __forceinline__ uint32_t sign_bit(uint32_t m, int j) {
    const int bit = (j & 1) ? 4 + (j >> 1) : (j >> 1);
    return (m >> bit) & 1u;
}

// ---- nibble tables (GEMV path): v word = nib[b] ^ msk[u], signed 4-bit v per coordinate ----
__device__ __forceinline__ uint32_t nibble_basis_word(uint32_t selector, uint32_t bias) {
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        word |= (((uint32_t)selector_half(selector, j) ^ bias) & 15u) << (4 * nibble_slot(j));
    return word;
}

__device__ __forceinline__ uint32_t nibble_mask_word(uint32_t u) {
    const uint32_t p = __popc(u) & 1u;
    const uint32_t m = u ^ p;
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        word |= ((sign_bit(m, j) ? 0xEu : 0u) ^ p) << (4 * nibble_slot(j));
    return word;
}

// ---- byte tables: 8 bytes per entry in coordinate order ---------------------------------
// "biased nibble" form: byte j = ((h_j ^ 8) & 15) << shift and mask_j << shift.  XOR of a basis
// entry and a mask entry is (v_j + 8) << shift, an unsigned value that never carries out of
// its byte for shift <= 3.
__device__ __forceinline__ uint2 byte_basis_biased(uint32_t selector, int shift) {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        lo |= ((((uint32_t)selector_half(selector, j) ^ 8u) & 15u) << shift) << (8 * j);
        hi |= ((((uint32_t)selector_half(selector, j + 4) ^ 8u) & 15u) << shift) << (8 * j);
    }
    return make_uint2(lo, hi);
}

__device__ __forceinline__ uint2 byte_mask_biased(uint32_t u, int shift) {
    const uint32_t p = __popc(u) & 1u;
    const uint32_t m = u ^ p;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        lo |= (((sign_bit(m, j) ? 0xEu : 0u) ^ p) << shift) << (8 * j);
        hi |= (((sign_bit(m, j + 4) ? 0xEu : 0u) ^ p) << shift) << (8 * j);
    }
    return make_uint2(lo, hi);
}

// "signed byte" form (single-stage Q2): byte j = t_j and mask3_j; XOR is q_j itself.
__device__ __forceinline__ uint2 byte_basis_signed(uint32_t selector) {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        lo |= ((uint32_t)(2 * selector_half(selector, j)) & 255u) << (8 * j);
        hi |= ((uint32_t)(2 * selector_half(selector, j + 4)) & 255u) << (8 * j);
    }
    return make_uint2(lo, hi);
}

__device__ __forceinline__ uint2 byte_mask_signed(uint32_t u) {
    const uint32_t p = __popc(u) & 1u;
    const uint32_t m = u ^ p;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = sign_bit(m, j) ? (p ? 0xFFu : 0xFDu) : (p ? 0x03u : 0x01u);
        const uint32_t b = sign_bit(m, j + 4) ? (p ? 0xFFu : 0xFDu) : (p ? 0x03u : 0x01u);
        lo |= a << (8 * j);
        hi |= b << (8 * j);
    }
    return make_uint2(lo, hi);
}

// LDS tables for the byte decoders.
struct Q4ByteTables {   // w = 4*q0 + q1 = 8*(v0+8) + 2*(v1+8) - 75
    uint2 basis0[256];  // (h^8) << 3
    uint2 mask0[256];   // mask << 3
    uint2 basis1[256];  // (h^8) << 1
    uint2 mask1[256];   // mask << 1
};
struct Q2ByteTables {
    uint2 basis[256];   // t
    uint2 mask[256];    // mask3
};

__device__ __forceinline__ void build_tables(Q4ByteTables& t, const uint32_t* __restrict__ book, int tid, int threads) {
    for (int i = tid; i < 256; i += threads) {
        const uint32_t s = book[i];
        t.basis0[i] = byte_basis_biased(s, 3);
        t.basis1[i] = byte_basis_biased(s, 1);
        t.mask0[i] = byte_mask_biased((uint32_t)i, 3);
        t.mask1[i] = byte_mask_biased((uint32_t)i, 1);
    }
}

__device__ __forceinline__ void build_tables(Q2ByteTables& t, const uint32_t* __restrict__ book, int tid, int threads) {
    for (int i = tid; i < 256; i += threads) {
        t.basis[i] = byte_basis_signed(book[i]);
        t.mask[i] = byte_mask_signed((uint32_t)i);
    }
}

// The four table entries one two-stage code needs; split from the arithmetic so that a kernel can
// issue the LDS reads early and combine them later (software pipelining around MFMAs).
struct Q4Lookups {
    uint2 b0, m0, b1, m1;
};
__device__ __forceinline__ Q4Lookups lookup_q4(const Q4ByteTables& t, uint32_t code) {
    Q4Lookups l;
    l.b0 = t.basis0[(code >> 8) & 255u];
    l.m0 = t.mask0[code & 255u];
    l.b1 = t.basis1[code >> 24];
    l.m1 = t.mask1[(code >> 16) & 255u];
    return l;
}
__device__ __forceinline__ uint2 combine_q4(const Q4Lookups& l) {
    uint2 w;
    w.x = ((l.b0.x ^ l.m0.x) + (l.b1.x ^ l.m1.x) + 0x35353535u) ^ 0x80808080u;
    w.y = ((l.b0.y ^ l.m0.y) + (l.b1.y ^ l.m1.y) + 0x35353535u) ^ 0x80808080u;
    return w;
}

// One u32 two-stage code -> 8 int8 weights (two words: coordinates 0..3 and 4..7).
// (x0 + x1 + 53) is w+128 in every byte, in [73,183]: no carry between bytes; the XOR
// turns offset binary into two's complement.
__device__ __forceinline__ uint2 decode_q4(const Q4ByteTables& t, uint32_t code) {
    const uint2 b0 = t.basis0[(code >> 8) & 255u];
    const uint2 m0 = t.mask0[code & 255u];
    const uint2 b1 = t.basis1[code >> 24];
    const uint2 m1 = t.mask1[(code >> 16) & 255u];
    uint2 w;
    w.x = ((b0.x ^ m0.x) + (b1.x ^ m1.x) + 0x35353535u) ^ 0x80808080u;
    w.y = ((b0.y ^ m0.y) + (b1.y ^ m1.y) + 0x35353535u) ^ 0x80808080u;
    return w;
}

// One u16 single-stage code -> 8 int8 weights.
__device__ __forceinline__ uint2 decode_q2(const Q2ByteTables& t, uint32_t code) {
    const uint2 b = t.basis[(code >> 8) & 255u];
    const uint2 m = t.mask[code & 255u];
    return make_uint2(b.x ^ m.x, b.y ^ m.y);
}

// Single-stage decode for any basis and every form of Book the reference's decoder takes
// (kernels/cuda/model/integer_vq.py:26-53, 163-192): the (256, 2) table of raw int8 basis values (its default), the
// (512, 4) table of signed values at both parities (quantization/vq.py:44-69: shortbook) and the (256, 1) selector
// words (shortbook + selectorbook).  All three become the middle one in LDS: for basis row b at parity p the eight
// weights with every sign bit clear (+t + 1 - 2p) and with every sign bit set (-t + 1 - 2p), bytes wrapping as int8
// arithmetic does; a code then picks each byte from one or the other by its sign bits.  A zero coordinate is
// 1 - 2p either way, any even value decodes as the reference's word arithmetic does, nothing is assumed of the basis.
enum BookForm { kBookSelector = 0, kBookRaw = 1, kBookSigned = 2 };
__host__ __device__ constexpr int book_words(int form) { return form == kBookSelector ? 256 : form == kBookRaw ? 512 : 2048; }

struct Q2GeneralTables {
    uint4 value[512];  // [p * 256 + b]: .x/.y all signs clear (coordinates 0-3, 4-7), .z/.w all signs set
    uint2 pick[256];   // [m]: 0xFF in byte j where sign bit SIGN_BITS[j] of the parity-adjusted low byte m is set
};

// bytewise -t + d and t + d of four int8 values
__device__ __forceinline__ uint32_t bytes_plus(uint32_t t, int d, bool negate) {
    uint32_t out = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int v = (int)(int8_t)(t >> (8 * j));
        out |= (uint32_t)(uint8_t)((negate ? -v : v) + d) << (8 * j);
    }
    return out;
}

__device__ __forceinline__ void build_tables(Q2GeneralTables& t, const uint32_t* __restrict__ book, int form, int tid, int threads) {
    for (int i = tid; i < 512; i += threads) {
        const int row = i & 255, parity = i >> 8;
        if (form == kBookSigned) {  // columns: low half +, low half -, high half +, high half - (vq.py:62-69)
            const uint32_t* words = book + (int64_t)i * 4;
            t.value[i] = make_uint4(words[0], words[2], words[1], words[3]);
        } else {
            uint2 basis;
            if (form == kBookRaw)
                basis = make_uint2(book[row * 2], book[row * 2 + 1]);
            else
                basis = byte_basis_signed(book[row]);
            const int d = 1 - 2 * parity;
            t.value[i] = make_uint4(bytes_plus(basis.x, d, false), bytes_plus(basis.y, d, false), bytes_plus(basis.x, d, true),
                                    bytes_plus(basis.y, d, true));
        }
    }
    for (int m = tid; m < 256; m += threads) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (sign_bit((uint32_t)m, j)) lo |= 0xFFu << (8 * j);
            if (sign_bit((uint32_t)m, j + 4)) hi |= 0xFFu << (8 * j);
        }
        t.pick[m] = make_uint2(lo, hi);
    }
}

__device__ __forceinline__ uint2 decode_q2(const Q2GeneralTables& t, uint32_t code) {
    const uint32_t parity = __popc(code & 255u) & 1u;
    const uint4 v = t.value[parity * 256u + ((code >> 8) & 255u)];
    const uint2 m = t.pick[(code & 255u) ^ parity];
    return make_uint2((v.x & ~m.x) | (v.z & m.x), (v.y & ~m.y) | (v.w & m.y));
}

// Byte offset of the 16-byte chunk `q` (0..3: 32 weights each) of weight row `row` in the 128-wide
// K step `kt` of two-stage codes stored K-major, (K/packed_k, N, packed_k/8) u32 with packed_k = 128
// or 64 (kernels/cuda/model/e8p_q4.py:250).
__device__ __forceinline__ int64_t q4_k_major_chunk(int packed_k, int n, int row, int kt, int q) {
    if (packed_k == 128) return ((int64_t)kt * n + row) * 64 + q * 16;
    return ((int64_t)(kt * 2 + (q >> 1)) * n + row) * 32 + (q & 1) * 16;
}

// ---- y = (w - 1) / 2 as bytes, from the reference's nibble words (quantization/vq.py:105-118) ----------------
// sign-extends the four nibbles at bits 0-3 of every byte
__device__ __forceinline__ uint32_t extend_nibbles(uint32_t t) { return t | ((t & 0x08080808u) * 0x1Eu); }

// bytewise a + b of signed bytes whose sums fit a byte
__device__ __forceinline__ uint32_t add_bytes(uint32_t a, uint32_t b) {
    return ((a & 0x7F7F7F7Fu) + (b & 0x7F7F7F7Fu)) ^ ((a ^ b) & 0x80808080u);
}

// Tables of the INT4-exact expert kernels' decode (kernels/cuda/model/e8p_core.py:7-10, 45-60), one entry per thread
// for threads 0..255.  `value[b]`: y of basis row b at even parity without sign bits; `change[u]`: what a code's low byte
// u changes in it (a coordinate's sign bit negates its nibble: the stored values are odd, so xor 0xe; odd parity lowers
// every nibble by one, xor 1, and flips the first coordinate's sign too).  Both as sign-extended bytes, the even nibbles
// of the reference's word (coordinates 0, 1, 4, 5) in .x and the odd ones (2, 3, 6, 7) in .y: sign extension commutes
// with xor, so a code decodes with two 8-byte lookups and two xors.  `selector_form`: Book holds selector words.
__device__ __forceinline__ void build_half_tables(uint2* value, uint2* change, const uint32_t* book, bool selector_form, int entry) {
    uint32_t word = book[entry];
    if (selector_form) {
        uint32_t nibbles = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int coordinate = (i & 4) | ((i & 1) << 1) | ((i & 2) >> 1);
            nibbles |= ((uint32_t)selector_half(word, coordinate) & 15u) << (4 * i);
        }
        word = nibbles;
    }
    value[entry] = make_uint2(extend_nibbles(word & 0x0F0F0F0Fu), extend_nibbles((word >> 4) & 0x0F0F0F0Fu));
    const uint32_t u = (uint32_t)entry, parity = __popc(u) & 1u;
    const uint32_t bits = (u & 0x03u) | ((u & 0x30u) >> 2) | ((u & 0x0Cu) << 2) | (u & 0xC0u);  // nibble i <- sign bit
    uint32_t spread = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) spread |= ((bits >> i) & 1u) << (4 * i + 1);
    const uint32_t flip = (spread * 7u) ^ (parity * 0x1111111Fu);
    change[entry] = make_uint2(extend_nibbles(flip & 0x0F0F0F0Fu), extend_nibbles((flip >> 4) & 0x0F0F0F0Fu));
}

__device__ __forceinline__ uint2 decode_half(const uint2* value, const uint2* change, uint32_t code) {
    const uint2 v = value[(code >> 8) & 255u], c = change[code & 255u];
    return make_uint2(v.x ^ c.x, v.y ^ c.y);
}

// two-stage code: y = 4 y_coarse + y_fine (coarse in the low half)
__device__ __forceinline__ uint2 decode_half_q4(const uint2* value, const uint2* change, uint32_t code) {
    const uint2 coarse = decode_half(value, change, code & 0xFFFFu), fine = decode_half(value, change, code >> 16);
    return make_uint2(add_bytes((coarse.x & 0x3F3F3F3Fu) << 2, fine.x), add_bytes((coarse.y & 0x3F3F3F3Fu) << 2, fine.y));
}

// Eight activations from a low and a high plane word: byte = low nibble | high nibble << 4, even nibbles in .x
__device__ __forceinline__ uint2 plane_bytes(uint32_t low, uint32_t high) {
    return make_uint2((low & 0x0F0F0F0Fu) | ((high & 0x0F0F0F0Fu) << 4), ((low >> 4) & 0x0F0F0F0Fu) | (high & 0xF0F0F0F0u));
}

// fp32 epilogue shared by every projection: (float(acc) * ws) * as, two separate roundings
// (kernels/cuda/model/integer_core.py:19-22).
__device__ __forceinline__ float rescale(int acc, float weight_scale, float token_scale) {
    float value = ((float)acc * weight_scale) * token_scale;
    // Opaque to the optimiser: a following fp16 cast must not be merged with the multiply into a
    // mixed-precision fused op, which rounds once instead of fp32-then-fp16.
    asm volatile("" : "+v"(value));
    return value;
}

}  // namespace orx
