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

#include "e8p_device.h"
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
    constexpr int D = 4;  // register ring of 16-byte chunks per lane
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

// ---- host side -----------------------------------------------------------------------------
// slots: N, K, stride, capacity, block_m (= passes), flags (= codec), out_f32
int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess)
            cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

uint32_t gemv_lds_bytes(const orx_function& f, int mr) {
    const uint32_t planes = f.flags == kW8 ? (uint32_t)mr * f.K : (uint32_t)mr * (f.K / 8) * 8;
    return planes;
}

int mr_for(int rows) { return rows <= 1 ? 1 : rows <= 2 ? 2 : 4; }

int gemv_geometry(const orx_function& f, int rows, Geometry* g) {
    g->grid[0] = ceil_div((uint32_t)f.N, (uint32_t)(kRowsPerPass * f.block_m));
    g->block[0] = kThreads;
    g->shared = gemv_lds_bytes(f, mr_for(rows));
    return ORX_OK;
}

template <int CODEC>
int gemv_launch_codec(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                      const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out) {
    const dim3 grid(g.grid[0]), block(kThreads);
    const uint4* wp = reinterpret_cast<const uint4*>(w);
    switch (mr_for(rows)) {
        case 1:
            hipLaunchKernelGGL((gemv_rowmajor_kernel<CODEC, 1>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
        case 2:
            hipLaunchKernelGGL((gemv_rowmajor_kernel<CODEC, 2>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
        default:
            hipLaunchKernelGGL((gemv_rowmajor_kernel<CODEC, 4>), grid, block, g.shared, stream, a, wp, book, ws, as, out,
                               f.N, f.K, f.stride, rows, f.block_m, (int)f.out_f32);
            break;
    }
    return hip_check(hipGetLastError(), "launch projection (gemv)");
}

}  // namespace

int gemv_prepare_device();

// Launchers used by the projection factories.  Argument order is the caller's business:
// they pass already-unmarshalled pointers.
int gemv_launch(const orx_function& f, int rows, const Geometry& g, hipStream_t stream, const int8_t* a,
                const void* w, const uint32_t* book, const __half* ws, const __half* as, void* out) {
    // LDS opt-in needs a device, so it happens at the first launch rather than at resolve time
    const int ready = gemv_prepare_device();
    if (ready != ORX_OK) return ready;
    if (f.flags == kQ4) return gemv_launch_codec<kQ4>(f, rows, g, stream, a, w, book, ws, as, out);
    if (f.flags == kQ2) return gemv_launch_codec<kQ2>(f, rows, g, stream, a, w, book, ws, as, out);
    return gemv_launch_codec<kW8>(f, rows, g, stream, a, w, book, ws, as, out);
}

int gemv_geometry_for(const orx_function& f, int rows, Geometry* g) { return gemv_geometry(f, rows, g); }

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
    if (gemv_lds_bytes(*f, 4) > 160 * 1024 - 4096) {
        set_error("%s: K=%d does not fit the gemv activation planes in LDS", f->symbol.c_str(), f->K);
        return ORX_ERR_BAD_VARIANT;
    }
    f->device_function = reinterpret_cast<const void*>(&gemv_rowmajor_kernel<kQ4, 1>);
    return ORX_OK;
}

int gemv_prepare_device() {
    // Dynamic LDS above 64 KiB needs an opt-in per kernel (kernels.rs:171-190 does the same on CUDA).
    static bool done = false;
    if (done) return ORX_OK;
    const int limit = 160 * 1024 - 4096;  // the static tables take 2064 bytes of the 160 KiB
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
#undef ORX_OPT_IN
    done = true;
    return ORX_OK;
}

const Registration* gemv_registrations(int* count) {
    static const Registration rows[] = {{nullptr, nullptr, nullptr, nullptr}
    };
    *count = 0;
    return rows;
}

}  // namespace orx
