// Diagnostics, not part of the path: what the part sustains by itself, as the ceilings that the
// kernels' roofline fractions are read against.  `bench.py --mfma-probe` and `--read-probe` run them.
#include <hip/hip_runtime.h>

#include <string>

#include "orx_internal.h"

namespace orx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// ---- int8_mfma_probe: what the matrix pipe sustains by itself ---------------------------------
// A diagnostic, not part of the path: eight waves per CU issue v_mfma_i32_32x32x32_i8 back to back
// from registers (no memory, no LDS), with all-zero operands or with eight random fragments per
// operand rotated through the instructions.  The two rates differ by what the data costs in power:
// it is the ceiling that the projections' int8 fractions should be read against.
namespace {
template <bool RANDOM>
__global__ __launch_bounds__(512) void mfma_probe_kernel(int* out, int iterations) {
    v4i fa[8], fb[8];
    uint32_t x = (threadIdx.x + blockIdx.x * 512u) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x ^= x << 13, x ^= x >> 17, x ^= x << 5;
            fa[i][j] = RANDOM ? (int)x : 0;
            x ^= x << 13, x ^= x >> 17, x ^= x << 5;
            fb[i][j] = RANDOM ? (int)x : 0;
        }
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[(i + 3) & 7], acc[i], 0, 0, 0);
    }
    int folded = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) folded ^= acc[i][j];
    // one word per workgroup, so that the loop cannot be removed; the value carries no meaning
    if (threadIdx.x == 0) out[blockIdx.x] = folded;
}

int mfma_probe_geometry(const orx_function&, int, Geometry* g) {
    g->grid[0] = (uint32_t)device_compute_units();
    g->block[0] = 512;
    return ORX_OK;
}
int mfma_probe_launch(const orx_function& f, int, const Geometry& g, hipStream_t stream, void** args) {
    int* out = pointer_arg<int>(args, 0);
    if (f.flags)
        hipLaunchKernelGGL(mfma_probe_kernel<true>, dim3(g.grid[0]), dim3(512), 0, stream, out, f.K);
    else
        hipLaunchKernelGGL(mfma_probe_kernel<false>, dim3(g.grid[0]), dim3(512), 0, stream, out, f.K);
    return hip_check(hipGetLastError(), "launch int8_mfma_probe");
}
}  // namespace

// Out: one int32 per CU (at least 1024 of them).  Operations per launch: CUs * 8 waves * iterations * 8 * 65536.
int make_mfma_probe(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("iterations", 20000, &bad);
    const std::string operands = v.string("operands", "random", &bad);
    if (bad || f->K <= 0 || f->K > (1 << 24) || (operands != "random" && operands != "zero")) {
        set_error("int8_mfma_probe: iterations in 1..2^24, operands random|zero");
        return ORX_ERR_BAD_VARIANT;
    }
    f->flags = operands == "random";
    f->M = f->capacity = 1;
    f->args = {{"Out", ArgPointer, 4}};
    f->geometry = mfma_probe_geometry;
    f->launch = mfma_probe_launch;
    f->device_function = f->flags ? reinterpret_cast<const void*>(&mfma_probe_kernel<true>)
                                  : reinterpret_cast<const void*>(&mfma_probe_kernel<false>);
    return ORX_OK;
}

// ---- hbm_read_probe: a plain streaming read ---------------------------------------------------
// Every thread reads four 16-byte pieces per iteration, grid-stride, and folds them into one word
// that is never stored: the rate a read of `bytes` bytes reaches when nothing else is done with it,
// launch included.  The caller rotates more source buffers than the caches hold.
namespace {
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ source, size_t pieces, uint32_t* out) {
    constexpr int kUnroll = 4;
    size_t i = (size_t)blockIdx.x * 256 * kUnroll + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256 * kUnroll;
    uint32_t folded = 0;
    for (; i + 256 * (kUnroll - 1) < pieces; i += stride) {
        uint4 v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) v[u] = source[i + 256 * u];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) folded ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (folded == 0x12345678u) out[0] = folded;  // keeps the loads alive; practically never true
}
int read_probe_geometry(const orx_function& f, int, Geometry* g) {
    g->grid[0] = (uint32_t)(device_compute_units() * f.tiles);
    g->block[0] = 256;
    return ORX_OK;
}
// Out, Source
int read_probe_launch(const orx_function& f, int, const Geometry& g, hipStream_t stream, void** args) {
    hipLaunchKernelGGL(read_probe_kernel, dim3(g.grid[0]), dim3(256), 0, stream, pointer_arg<const uint4>(args, 1),
                       (size_t)f.slots * 64, pointer_arg<uint32_t>(args, 0));
    return hip_check(hipGetLastError(), "launch hbm_read_probe");
}
}  // namespace

int make_read_probe(const Variant& v, orx_function* f) {
    bool bad = false;
    const long long bytes = v.integer("bytes", 0, &bad);
    f->tiles = (int)v.integer("workgroups_per_cu", 8, &bad);
    // whole kilobytes: a workgroup's iteration is 256 threads x 4 pieces x 16 bytes
    if (bad || bytes <= 0 || bytes % 16384 || bytes > (1ll << 34) || f->tiles < 1 || f->tiles > 64) {
        set_error("hbm_read_probe: bytes a positive multiple of 16384 up to 2^34, workgroups_per_cu in 1..64");
        return ORX_ERR_BAD_VARIANT;
    }
    f->slots = (int)(bytes / 1024);  // 16-byte pieces / 64
    f->M = f->capacity = 1;
    f->args = {{"Out", ArgPointer, 4}, {"Source", ArgPointer, 16}};
    f->geometry = read_probe_geometry;
    f->launch = read_probe_launch;
    f->device_function = reinterpret_cast<const void*>(&read_probe_kernel);
    return ORX_OK;
}

// ---- lds_lookup_probe: random 4-byte reads of a 256-entry table in LDS -------------------------
// The decode of every E8P code is two such lookups per stage.  `copies` is how often the table is
// stored: entry e, copy c at word e * copies + c, and lane l reads copy l mod copies; 1 is a compact
// 1 KiB table (the lanes of a wave collide in the banks), 64 gives every lane its own bank.  Sixteen
// waves per CU issue eight independent lookups per iteration; nothing else competes for the LDS.
namespace {
typedef __attribute__((address_space(3))) const uint32_t lds_word;
template <int COPIES>
__global__ __launch_bounds__(1024) void lds_lookup_probe_kernel(uint32_t* out, int iterations) {
    extern __shared__ uint32_t probe_table[];
    for (int i = threadIdx.x; i < 256 * COPIES; i += 1024) probe_table[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const uint32_t column = ((threadIdx.x & 63u) % COPIES) * 4u;
    uint32_t x = threadIdx.x * 2654435761u + blockIdx.x + 1u, folded = 0;
    for (int it = 0; it < iterations; ++it) {
        x ^= x << 13, x ^= x >> 17, x ^= x << 5;
        const uint32_t y = x ^ (x >> 7) ^ 0x9E3779B9u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t a0 = ((x >> (8 * j)) & 255u) * (COPIES * 4u) + column;
            const uint32_t a1 = ((y >> (8 * j)) & 255u) * (COPIES * 4u) + column;
            folded ^= *reinterpret_cast<lds_word*>(a0);
            folded ^= *reinterpret_cast<lds_word*>(a1);
        }
    }
    if (folded == 0x1234567u) out[0] = folded;  // keeps the lookups alive; practically never true
}
int lds_probe_geometry(const orx_function& f, int, Geometry* g) {
    g->grid[0] = (uint32_t)device_compute_units();
    g->block[0] = 1024;
    g->shared = 256u * (uint32_t)f.tiles * 4u;
    return ORX_OK;
}
template <int COPIES>
int lds_probe_launch_as(const orx_function& f, const Geometry& g, hipStream_t stream, uint32_t* out) {
    static DeviceOnce opted_in;  // 64 copies are 64 KiB of dynamic LDS
    const int ready = opted_in.run([] {
        return hip_check(hipFuncSetAttribute(reinterpret_cast<const void*>(&lds_lookup_probe_kernel<COPIES>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024),
                         "hipFuncSetAttribute");
    });
    if (ready != ORX_OK) return ready;
    hipLaunchKernelGGL(lds_lookup_probe_kernel<COPIES>, dim3(g.grid[0]), dim3(1024), g.shared, stream, out, f.K);
    return hip_check(hipGetLastError(), "launch lds_lookup_probe");
}
int lds_probe_launch(const orx_function& f, int, const Geometry& g, hipStream_t stream, void** args) {
    uint32_t* out = pointer_arg<uint32_t>(args, 0);
    if (f.tiles == 1) return lds_probe_launch_as<1>(f, g, stream, out);
    if (f.tiles == 32) return lds_probe_launch_as<32>(f, g, stream, out);
    return lds_probe_launch_as<64>(f, g, stream, out);
}
}  // namespace

// Out: one word.  Lane lookups per launch: CUs * 1024 * iterations * 8 (wave instructions: a 64th of that).
int make_lds_probe(const Variant& v, orx_function* f) {
    bool bad = false;
    f->K = (int)v.integer("iterations", 2000, &bad);
    f->tiles = (int)v.integer("copies", 64, &bad);
    if (bad || f->K <= 0 || f->K > (1 << 24) || (f->tiles != 1 && f->tiles != 32 && f->tiles != 64)) {
        set_error("lds_lookup_probe: iterations in 1..2^24, copies 1|32|64");
        return ORX_ERR_BAD_VARIANT;
    }
    f->M = f->capacity = 1;
    f->args = {{"Out", ArgPointer, 4}};
    f->geometry = lds_probe_geometry;
    f->launch = lds_probe_launch;
    f->device_function = f->tiles == 1    ? reinterpret_cast<const void*>(&lds_lookup_probe_kernel<1>)
                         : f->tiles == 32 ? reinterpret_cast<const void*>(&lds_lookup_probe_kernel<32>)
                                          : reinterpret_cast<const void*>(&lds_lookup_probe_kernel<64>);
    return ORX_OK;
}

const Registration* probe_registrations(int* count) {
    static const Registration rows[] = {
    {"int8_mfma_probe", make_mfma_probe, "iterations=20000, operands=random|zero (diagnostic: the matrix pipe alone)", "Out"},
    {"hbm_read_probe", make_read_probe, "bytes, workgroups_per_cu=8 (diagnostic: a plain streaming read)", "Out,Source"},
    {"lds_lookup_probe", make_lds_probe, "iterations=2000, copies=64|32|1 (diagnostic: random table reads in LDS)", "Out"},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

}  // namespace orx
