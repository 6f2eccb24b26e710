// Host-side internals of liborx: the resolved-function record and the registration
// interface each kernel file implements.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../include/orx.h"

namespace orx {

// One value of the flat variant JSON object.
struct Value {
    enum Kind { Null, Bool, Number, String } kind = Null;
    double number = 0;
    std::string text;
};

struct Variant {
    std::map<std::string, Value> fields;
    // Keys a factory has looked at.  orx_resolve refuses a variant with a key nobody read: a misspelt or
    // unsupported option must not silently resolve to the default behaviour (the reference's factories raise
    // on an unknown keyword).  `accept` marks a key that is understood and deliberately not used.
    // (shared by the copies a factory hands to another factory)
    std::shared_ptr<std::map<std::string, bool>> read = std::make_shared<std::map<std::string, bool>>();
    void accept(const char* key) const { (*read)[key] = true; }
    bool has(const char* key) const {
        (*read)[key] = true;
        return fields.count(key) != 0;
    }
    // Integer field with a default; sets `bad` if the field exists but is not an integer.
    long long integer(const char* key, long long fallback, bool* bad) const;
    bool boolean(const char* key, bool fallback, bool* bad) const;
    std::string string(const char* key, const char* fallback, bool* bad) const;
};

bool parse_variant(const char* json, Variant* out, std::string* error);
// false (with the error set) unless the variant's `coefficients` are absent or (4, 1)
bool two_stage_coefficients_ok(const Variant& v, const char* symbol);

enum ArgKind { ArgPointer = 0, ArgI32 = 1 };
struct ArgSpec {
    const char* name;
    ArgKind kind;
    uint32_t alignment;  // bytes the pointer must be aligned to (dtype alignment only)
};

struct Geometry {
    uint32_t grid[3] = {1, 1, 1};
    uint32_t block[3] = {1, 1, 1};
    uint32_t shared = 0;
};

}  // namespace orx

// The handle behind orx_fn.  Shape parameters are generic integer slots so that one record
// type serves every kernel family; each family documents which slots it reads.
struct orx_function {
    std::string symbol;
    std::vector<orx::ArgSpec> args;
    // Optional buffers that the variant's `omit` key took out of the caller's argument list (indices into
    // `args`, ascending): the launch sees a null pointer there.  Empty for most handles.
    std::vector<int> omitted;
    bool dynamic_rows = false;  // last argument is `int32 m`
    int capacity = 0;           // largest row count (M of the variant)
    // shape / configuration
    int M = 0, N = 0, K = 0, E = 0, top_k = 0, H = 0, stride = 0, group = 0, tiles = 0, slots = 0;
    int block_m = 0, block_n = 0, packed_k = 0, algorithm = 0, flags = 0, flags2 = 0;
    int tile_hint = 0;  // projections: row tile preferred while the live rows fit one such tile (0 = none)
    bool out_f32 = false;
    bool input_f16 = false;  // single-row projection that quantises its fp16 activations itself
    bool rotate_input = false;  // ... after the signed block-128 rotation (takes a Signs buffer)
    const void* device_function = nullptr;  // for hipFuncGetAttributes
    // The handle owns no device memory.  A kernel that needs scratch beyond its inputs and outputs
    // (int32 partial tiles of split launches, int8 weights decoded once per launch) takes it from the
    // caller as a trailing `Workspace` buffer when the variant says `workspace=true`; without it the
    // handle keeps to the kernels that need none.  workspace_arg = index of that argument or -1.
    bool takes_workspace = false;
    int workspace_arg = -1;
    // bytes of Workspace a launch of `rows` rows reads and writes (0: none needed)
    uint64_t (*workspace_need)(const orx_function&, int rows) = nullptr;
    // rows -> geometry; returns ORX_OK or an error code
    int (*geometry)(const orx_function&, int rows, orx::Geometry*) = nullptr;
    // enqueue on stream; args already validated for count/alignment
    // (the launch reads its Workspace pointer, if it takes one, from args[workspace_arg])
    int (*launch)(const orx_function&, int rows, const orx::Geometry&, hipStream_t, void** args) = nullptr;
};

namespace orx {

void set_error(const char* format, ...);
int hip_check(hipError_t code, const char* operation);

// Every kernel launch of the library goes through ORX_LAUNCH.  While a thread records (orx_query_rows), a launch
// enqueues nothing and leaves its function, grid, block and dynamic LDS bytes in that thread's list instead: the
// query then reads the attributes of the very kernel a launch of that row count would start.
struct LaunchRecord {
    const void* function;
    uint32_t grid, block, shared;
};
bool recording_launches();
void record_launch(const void* function, dim3 grid, dim3 block, uint32_t shared);
#define ORX_LAUNCH(kernel, grid, block, shared, stream, ...)                                                          \
    do {                                                                                                              \
        if (::orx::recording_launches())                                                                              \
            ::orx::record_launch(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(block), (uint32_t)(shared)); \
        else                                                                                                          \
            hipLaunchKernelGGL(kernel, grid, block, shared, stream, __VA_ARGS__);                                     \
    } while (0)

// Each kernel file exports one factory per symbol: fills `f` from the variant or returns an
// error code after set_error().
typedef int (*Factory)(const Variant&, orx_function* f);
struct Registration {
    const char* symbol;
    Factory factory;
    const char* variant_keys;  // human-readable list for orx_catalog()
    const char* arguments;     // launch order, comma separated
};

// Implemented by the kernel translation units (host functions, so the tables never reach device code).
const Registration* quant_registrations(int* count);
const Registration* gemv_registrations(int* count);
const Registration* gemm_registrations(int* count);
const Registration* moe_registrations(int* count);
const Registration* plane_registrations(int* count);

template <typename T>
static inline T* pointer_arg(void** args, int index) {
    return *reinterpret_cast<T**>(args[index]);
}
static inline int int_arg(void** args, int index) { return *reinterpret_cast<int32_t*>(args[index]); }

static inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// The device current on the calling thread (0 if there is none, as on a build machine).
int current_device();
// Compute units of the current device (256 where no device answers).  Cached per device.
int device_compute_units();

// Buffers of a routed expert projection as the resident kernel takes them (null where a form has none).
struct GroupedBuffers {
    const void* a = nullptr;        // rows: int8 (slots, K); gathered: int8 (tokens, K); fp16 (slots, K) values to quantise
    const void* as = nullptr;       // row scales (per slot, or per token when gathered); an output for fp16 rows
    const void* w = nullptr;
    const uint32_t* book = nullptr;
    const void* ws = nullptr;       // fp16 channel scales (E, N)
    void* out = nullptr;            // fp16 (slots, N); optional with the SwiGLU epilogue
    const int* counts = nullptr;
    const int* offsets = nullptr;
    const int* tile_expert = nullptr;
    const int* tile_row = nullptr;
    const int* tile_count = nullptr;
    const int* slot_token = nullptr;  // gathered rows: token of every slot
    const int* row_max = nullptr;     // fp32 bits of every slot's largest magnitude: read with fp16 rows, raised by the SwiGLU epilogue
    void* act = nullptr;              // SwiGLU epilogue: fp16 (slots, N/2)
    void* q = nullptr;                // fp16 rows: the codes, optional
};

// One-time set-up that has to happen once per DEVICE (function attributes are per device), safe to
// reach from several session threads: the set-up itself is idempotent, the flag is atomic.
struct DeviceOnce {
    std::atomic<uint64_t> done{0};
    template <typename F>
    int run(F&& setup) {
        const uint64_t bit = 1ull << (current_device() & 63);
        if (done.load(std::memory_order_acquire) & bit) return ORX_OK;
        const int code = setup();
        if (code == ORX_OK) done.fetch_or(bit, std::memory_order_release);
        return code;
    }
};

}  // namespace orx
