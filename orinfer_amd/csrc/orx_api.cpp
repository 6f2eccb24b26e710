// liborx C ABI: resolve + launch, the HIP stand-in for orinfer's Catalog::resolve
// (crates/orinfer-engine/src/backend/cuda/kernels.rs:114-192) and launch_kernel
// (crates/orinfer-engine/src/backend/cuda/mod.rs:312-341).
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <memory>
#include <new>

#include "orx_internal.h"

namespace orx {

static thread_local char g_error[512] = "";

void set_error(const char* format, ...) {
    va_list ap;
    va_start(ap, format);
    vsnprintf(g_error, sizeof g_error, format, ap);
    va_end(ap);
}

int hip_check(hipError_t code, const char* operation) {
    if (code == hipSuccess) return ORX_OK;
    // Same text shape as the reference's check(): "<op>: CUDA error <code>" (mod.rs:48-55).
    set_error("%s: HIP error %d (%s)", operation, (int)code, hipGetErrorName(code));
    return (int)code;
}

namespace {
thread_local std::vector<LaunchRecord>* g_recording = nullptr;
}
bool recording_launches() { return g_recording != nullptr; }
void record_launch(const void* function, dim3 grid, dim3 block, uint32_t shared) {
    g_recording->push_back({function, grid.x, block.x * block.y * block.z, shared});
}

int current_device() {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return device;
}

int device_compute_units() {
    static std::atomic<int> cached[64];
    const int slot = current_device() & 63;
    int units = cached[slot].load(std::memory_order_relaxed);
    if (units == 0) {
        hipDeviceProp_t prop;
        int count = 0;
        if (hipGetDeviceCount(&count) == hipSuccess && count > 0 &&
            hipGetDeviceProperties(&prop, current_device()) == hipSuccess)
            units = prop.multiProcessorCount;
        else
            (void)hipGetLastError();
        if (units <= 0) units = 256;
        cached[slot].store(units, std::memory_order_relaxed);
    }
    return units;
}

// ---- flat JSON object parser -------------------------------------------------------------
namespace {
struct Cursor {
    const char* p;
    void skip() {
        while (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r') ++p;
    }
};

bool parse_string(Cursor& c, std::string* out) {
    if (*c.p != '"') return false;
    ++c.p;
    out->clear();
    while (*c.p && *c.p != '"') {
        if (*c.p == '\\') {
            ++c.p;
            if (!*c.p) return false;
        }
        out->push_back(*c.p++);
    }
    if (*c.p != '"') return false;
    ++c.p;
    return true;
}
}  // namespace

bool parse_variant(const char* json, Variant* out, std::string* error) {
    out->fields.clear();
    if (json == nullptr) return true;
    Cursor c{json};
    c.skip();
    if (*c.p == 0) return true;
    if (*c.p != '{') {
        *error = "variant must be a JSON object";
        return false;
    }
    ++c.p;
    c.skip();
    if (*c.p == '}') return true;
    for (;;) {
        c.skip();
        std::string key;
        if (!parse_string(c, &key)) {
            *error = "expected a string key";
            return false;
        }
        c.skip();
        if (*c.p != ':') {
            *error = "expected ':' after key " + key;
            return false;
        }
        ++c.p;
        c.skip();
        Value v;
        if (*c.p == '"') {
            v.kind = Value::String;
            if (!parse_string(c, &v.text)) {
                *error = "bad string value for " + key;
                return false;
            }
        } else if (!strncmp(c.p, "true", 4)) {
            v.kind = Value::Bool;
            v.number = 1;
            c.p += 4;
        } else if (!strncmp(c.p, "false", 5)) {
            v.kind = Value::Bool;
            v.number = 0;
            c.p += 5;
        } else if (!strncmp(c.p, "null", 4)) {
            v.kind = Value::Null;
            c.p += 4;
        } else if (*c.p == '[') {
            // a flat list of integers (the reference factories' tuples, e.g. coefficients=(4, 1)) is kept as the
            // string "4,1"
            ++c.p;
            v.kind = Value::String;
            for (;;) {
                c.skip();
                if (*c.p == ']') break;
                char* end = nullptr;
                const long long item = strtoll(c.p, &end, 10);
                if (end == c.p) {
                    *error = "list of " + key + " must hold integers";
                    return false;
                }
                c.p = end;
                if (!v.text.empty()) v.text += ",";
                v.text += std::to_string(item);
                c.skip();
                if (*c.p == ',') ++c.p;
                else if (*c.p != ']') {
                    *error = "bad list for " + key;
                    return false;
                }
            }
            ++c.p;
        } else {
            char* end = nullptr;
            v.number = strtod(c.p, &end);
            if (end == c.p) {
                *error = "bad value for " + key;
                return false;
            }
            v.kind = Value::Number;
            c.p = end;
        }
        if (out->fields.count(key)) {
            *error = "duplicate key " + key;
            return false;
        }
        out->fields[key] = v;
        c.skip();
        if (*c.p == ',') {
            ++c.p;
            continue;
        }
        if (*c.p == '}') {
            ++c.p;
            c.skip();
            if (*c.p != 0) {
                *error = "trailing text after the object";
                return false;
            }
            return true;
        }
        *error = "expected ',' or '}'";
        return false;
    }
}

long long Variant::integer(const char* key, long long fallback, bool* bad) const {
    (*read)[key] = true;
    auto it = fields.find(key);
    if (it == fields.end() || it->second.kind == Value::Null) return fallback;
    // every integer of a variant is a shape, a count or a tile size and is stored in an int: a value
    // outside the int range is refused here rather than wrapped by the casts of the factories
    if (it->second.kind != Value::Number || std::floor(it->second.number) != it->second.number ||
        !(std::fabs(it->second.number) <= 2147483647.0)) {
        *bad = true;
        set_error("variant field %s must be an integer of at most 31 bits", key);
        return fallback;
    }
    return (long long)it->second.number;
}

bool Variant::boolean(const char* key, bool fallback, bool* bad) const {
    (*read)[key] = true;
    auto it = fields.find(key);
    if (it == fields.end() || it->second.kind == Value::Null) return fallback;
    if (it->second.kind != Value::Bool) {
        *bad = true;
        set_error("variant field %s must be true or false", key);
        return fallback;
    }
    return it->second.number != 0;
}

std::string Variant::string(const char* key, const char* fallback, bool* bad) const {
    (*read)[key] = true;
    auto it = fields.find(key);
    if (it == fields.end() || it->second.kind == Value::Null) return fallback;
    if (it->second.kind != Value::String) {
        *bad = true;
        set_error("variant field %s must be a string", key);
        return fallback;
    }
    return it->second.text;
}

// The two-stage codec's weights are 4 * coarse + residual (quantization/e8p_q4.py:19-29 allows other coprime
// pairs; the model builder accepts [4, 1] only, models/qwen35/test_build.py:695-709, and so do the kernels here).
bool two_stage_coefficients_ok(const Variant& v, const char* symbol) {
    bool bad = false;
    std::string given = v.string("coefficients", "4,1", &bad);
    given.erase(std::remove(given.begin(), given.end(), ' '), given.end());
    if (bad || given != "4,1") {
        set_error("%s: coefficients must be (4, 1): the kernels decode 4 * coarse + residual", symbol);
        return false;
    }
    return true;
}

// ---- catalog -------------------------------------------------------------------------------
namespace {
struct Table {
    const Registration* rows;
    int count;
};
constexpr int kTables = 5;
void tables(Table out[kTables]) {
    out[0].rows = quant_registrations(&out[0].count);
    out[1].rows = gemv_registrations(&out[1].count);
    out[2].rows = gemm_registrations(&out[2].count);
    out[3].rows = moe_registrations(&out[3].count);
    out[4].rows = plane_registrations(&out[4].count);
}
const Registration* find(const char* symbol) {
    Table t[kTables];
    tables(t);
    for (auto& table : t)
        for (int i = 0; i < table.count; ++i)
            if (!strcmp(table.rows[i].symbol, symbol)) return &table.rows[i];
    return nullptr;
}
}  // namespace
}  // namespace orx

// ---- library-owned scratch for callers that cannot allocate ------------------------------------
// orx_launch_static_scratch() runs a launch on this array instead of a caller's Workspace.  The name
// `scratch` is a host-side stand-in for the symbol, not a device address: the address is asked for
// once per device (hipGetSymbolAddress, with that device current) and only that pointer is ever
// handed to a kernel.  Every device the library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[ORX_STATIC_SCRATCH_BYTES];

namespace orx {
namespace {
std::atomic<void*> g_scratch_address[64];

// Address of `scratch` on the current device; looked up on the first call per device (the calling thread's
// current device: a handle is resolved, and launched, with the launch device current).  The lookup is a runtime
// call that may not run while `stream` is capturing: orx_resolve of a workspace handle does it ahead of time
// for the device current then, and a first launch on another device under capture is refused.
int static_scratch_address(void** out, hipStream_t stream = nullptr, bool launching = false) {
    const int slot = current_device() & 63;
    void* address = g_scratch_address[slot].load(std::memory_order_acquire);
    if (address == nullptr && launching) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &status) != hipSuccess) (void)hipGetLastError();
        if (status != hipStreamCaptureStatusNone) {
            set_error("orx_launch_static_scratch: the scratch of device %d has not been looked up yet and the stream is "
                      "capturing: resolve the handle (or launch once) with this device current before the capture", slot);
            return ORX_ERR_BAD_ARGUMENT;
        }
    }
    if (address == nullptr) {
        const int code = hip_check(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
        if (code != ORX_OK) return code;
        if (address == nullptr || reinterpret_cast<uintptr_t>(address) % 256 != 0) {
            set_error("hipGetSymbolAddress(scratch): unusable address %p", address);
            return ORX_ERR_INTERNAL;
        }
        g_scratch_address[slot].store(address, std::memory_order_release);
    }
    *out = address;
    return ORX_OK;
}
}  // namespace
}  // namespace orx

using namespace orx;

namespace {

// No C++ exception crosses the C boundary: every entry point runs its body through guard().
template <typename F>
int guard(const char* entry, F&& body) {
    try {
        return body();
    } catch (const std::bad_alloc&) {
        set_error("%s: out of host memory", entry);
        return ORX_ERR_INTERNAL;
    } catch (const std::exception& e) {
        set_error("%s: %s", entry, e.what());
        return ORX_ERR_INTERNAL;
    } catch (...) {
        set_error("%s: unknown failure", entry);
        return ORX_ERR_INTERNAL;
    }
}

int resolve(const char* symbol, const char* variant_json, orx_fn* out) {
    // A package record has one `symbol` string and no place for a variant (artifact.rs:87-110), so
    // a symbol may carry it: "family?M=1&N=9728&K=2560&algorithm=gemv".  Values that are not
    // integers or true/false are taken as strings.
    std::string family(symbol), inline_variant;
    const size_t mark = family.find('?');
    if (mark != std::string::npos) {
        const std::string query = family.substr(mark + 1);
        family.resize(mark);
        inline_variant = "{";
        size_t at = 0;
        while (at < query.size()) {
            size_t end = query.find('&', at);
            if (end == std::string::npos) end = query.size();
            const std::string pair = query.substr(at, end - at);
            const size_t eq = pair.find('=');
            if (eq == std::string::npos || eq == 0) {
                set_error("orx_resolve %s: malformed variant in symbol", symbol);
                return ORX_ERR_BAD_VARIANT;
            }
            const std::string key = pair.substr(0, eq), value = pair.substr(eq + 1);
            bool number = !value.empty();
            for (size_t c = 0; c < value.size(); ++c)
                if (!(isdigit((unsigned char)value[c]) || (c == 0 && value[c] == '-' && value.size() > 1))) number = false;
            if (inline_variant.size() > 1) inline_variant += ",";
            inline_variant += "\"" + key + "\":";
            inline_variant += (number || value == "true" || value == "false") ? value : "\"" + value + "\"";
            at = end + 1;
        }
        inline_variant += "}";
        if (variant_json != nullptr && variant_json[0] != 0 && strcmp(variant_json, "{}") != 0) {
            set_error("orx_resolve %s: variant given both in the symbol and as JSON", symbol);
            return ORX_ERR_BAD_VARIANT;
        }
        variant_json = inline_variant.c_str();
    }
    const Registration* r = find(family.c_str());
    if (r == nullptr) {
        set_error("orx_resolve: unknown symbol %s", family.c_str());
        return ORX_ERR_UNKNOWN_SYMBOL;
    }
    Variant variant;
    std::string why;
    if (!parse_variant(variant_json, &variant, &why)) {
        set_error("orx_resolve %s: %s", family.c_str(), why.c_str());
        return ORX_ERR_BAD_VARIANT;
    }
    // the record owns host memory only, so every failure path is a plain delete
    std::unique_ptr<orx_function> f(new orx_function());
    f->symbol = family;
    const int code = r->factory(variant, f.get());
    if (code != ORX_OK) return code;
    // `omit`: optional buffers that the caller's program does not use leave the argument list (a package record has
    // no way to say "null", artifact.rs:184-194); the kernel sees a null pointer in their place
    bool bad_omit = false;
    const std::string omit = variant.string("omit", "", &bad_omit);
    if (bad_omit) return ORX_ERR_BAD_VARIANT;
    for (size_t at = 0; at < omit.size();) {
        size_t end = omit.find(',', at);
        if (end == std::string::npos) end = omit.size();
        const std::string name = omit.substr(at, end - at);
        at = end + 1;
        int index = -1;
        for (size_t i = 0; i < f->args.size(); ++i)
            if (name == f->args[i].name) index = (int)i;
        const bool optional = index >= 0 && f->args[index].kind == ArgPointer && (f->args[index].alignment & 0x80000000u) &&
                              name != "Workspace";
        if (!optional || std::count(f->omitted.begin(), f->omitted.end(), index)) {
            set_error("orx_resolve %s: omit names %s, which is not an optional buffer of this variant", family.c_str(),
                      name.c_str());
            return ORX_ERR_BAD_VARIANT;
        }
        f->omitted.push_back(index);
    }
    std::sort(f->omitted.begin(), f->omitted.end());
    if (!f->omitted.empty() && f->args.size() > 64) {
        set_error("orx_resolve %s: too many arguments for omit", family.c_str());
        return ORX_ERR_BAD_VARIANT;
    }
    for (const auto& field : variant.fields) {
        if (!variant.read->count(field.first)) {
            set_error("orx_resolve %s: unknown variant key %s (keys: %s)", family.c_str(), field.first.c_str(), r->variant_keys);
            return ORX_ERR_BAD_VARIANT;
        }
    }
    if (f->geometry == nullptr || f->launch == nullptr || f->args.empty()) {
        set_error("orx_resolve %s: incomplete kernel record", symbol);
        return ORX_ERR_BAD_VARIANT;
    }
    if (f->takes_workspace) {
        f->workspace_arg = -1;
        for (size_t i = 0; i < f->args.size(); ++i)
            if (!strcmp(f->args[i].name, "Workspace")) f->workspace_arg = (int)i;
        if (f->workspace_arg < 0 || f->workspace_need == nullptr) {
            set_error("orx_resolve %s: incomplete workspace record", symbol);
            return ORX_ERR_BAD_VARIANT;
        }
        // set-up for orx_launch_static_scratch on the device current now (resolve is never under graph
        // capture, the first launch may be); a machine without a device simply has nothing to look up
        int devices = 0;
        if (hipGetDeviceCount(&devices) == hipSuccess && devices > 0) {
            void* unused = nullptr;
            (void)static_scratch_address(&unused);
        } else {
            (void)hipGetLastError();
        }
    }
    *out = f.release();
    return ORX_OK;
}

// Validates a launch against the record and returns the row count and geometry it runs with.
int check_launch(const orx_function* f, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
                 void** args, bool workspace_from_caller, int* rows_out, Geometry* want) {
    if (f == nullptr || grid == nullptr || block == nullptr || args == nullptr) {
        set_error("orx_launch: null handle, geometry or argument list");
        return ORX_ERR_BAD_ARGUMENT;
    }
    const int count = (int)f->args.size();
    for (int i = 0; i < count; ++i) {
        if (i == f->workspace_arg && !workspace_from_caller) continue;  // replaced by the library's scratch
        if (args[i] == nullptr) {
            set_error("launch %s: argument %d (%s) is null", f->symbol.c_str(), i, f->args[i].name);
            return ORX_ERR_BAD_ARGUMENT;
        }
        if (f->args[i].kind == ArgPointer) {
            const uint64_t address = *reinterpret_cast<uint64_t*>(args[i]);
            if (address == 0 && !(f->args[i].alignment & 0x80000000u)) {
                set_error("launch %s: buffer %s is a null device pointer", f->symbol.c_str(), f->args[i].name);
                return ORX_ERR_BAD_ARGUMENT;
            }
            const uint32_t alignment = f->args[i].alignment & 0x7fffffffu;
            if (alignment > 1 && address % alignment) {
                set_error("launch %s: buffer %s is not %u-byte aligned", f->symbol.c_str(), f->args[i].name,
                          alignment);
                return ORX_ERR_BAD_ARGUMENT;
            }
        }
    }
    int rows = f->capacity;
    if (f->dynamic_rows) {
        rows = int_arg(args, count - 1);
        if (rows < 1 || rows > f->capacity) {
            set_error("launch %s: rows %d outside the kernel capacity %d", f->symbol.c_str(), rows, f->capacity);
            return ORX_ERR_ROWS;
        }
    }
    int code = f->geometry(*f, rows, want);
    if (code != ORX_OK) return code;
    for (int i = 0; i < 3; ++i) {
        if (grid[i] != want->grid[i] || block[i] != want->block[i]) {
            set_error("launch %s: geometry grid(%u,%u,%u) block(%u,%u,%u) does not fit the kernel, which needs "
                      "grid(%u,%u,%u) block(%u,%u,%u) for %d rows",
                      f->symbol.c_str(), grid[0], grid[1], grid[2], block[0], block[1], block[2], want->grid[0],
                      want->grid[1], want->grid[2], want->block[0], want->block[1], want->block[2], rows);
            return ORX_ERR_BAD_GEOMETRY;
        }
    }
    if (shared_bytes != want->shared) {
        set_error("launch %s: dynamic shared bytes %u, kernel needs %u", f->symbol.c_str(), shared_bytes, want->shared);
        return ORX_ERR_BAD_GEOMETRY;
    }
    *rows_out = rows;
    return ORX_OK;
}

// Index into f->args of the caller's argument `visible` (the list without the omitted buffers), or -1.
int full_index(const orx_function* f, int visible) {
    if (visible < 0) return -1;
    int seen = 0;
    for (int i = 0; i < (int)f->args.size(); ++i) {
        if (std::binary_search(f->omitted.begin(), f->omitted.end(), i)) continue;
        if (seen++ == visible) return i;
    }
    return -1;
}

// The caller's argument list with a null pointer at every omitted buffer.  `storage` must hold 64 entries.
void** expand_args(const orx_function* f, void** args, void** storage) {
    static uint64_t null_pointer = 0;  // never written
    if (f == nullptr || args == nullptr || f->omitted.empty() || f->args.size() > 64) return args;
    int next = 0;
    for (int i = 0; i < (int)f->args.size(); ++i)
        storage[i] = std::binary_search(f->omitted.begin(), f->omitted.end(), i) ? (void*)&null_pointer : args[next++];
    return storage;
}

uint64_t workspace_need(const orx_function* f, int rows) {
    return f->takes_workspace && f->workspace_need != nullptr ? f->workspace_need(*f, rows) : 0;
}

}  // namespace

extern "C" {

int orx_resolve(const char* symbol, const char* variant_json, orx_fn* out) {
    if (out == nullptr || symbol == nullptr) {
        set_error("orx_resolve: null symbol or output");
        return ORX_ERR_BAD_ARGUMENT;
    }
    *out = nullptr;
    return guard("orx_resolve", [&] { return resolve(symbol, variant_json, out); });
}

int orx_release(orx_fn f) {
    delete f;  // host memory only: a handle owns nothing on the device
    return ORX_OK;
}

int orx_query_rows(orx_fn f, int32_t rows, uint32_t* max_threads_per_block, uint32_t* static_lds_bytes) {
    if (f == nullptr) {
        set_error("orx_query: null handle");
        return ORX_ERR_BAD_ARGUMENT;
    }
    return guard("orx_query", [&] {
        const int live = rows <= 0 ? f->capacity : rows;
        if (live > f->capacity || (!f->dynamic_rows && live != f->capacity)) {
            set_error("%s: rows %d outside the kernel capacity %d", f->symbol.c_str(), live, f->capacity);
            return (int)ORX_ERR_ROWS;
        }
        const void* function = f->device_function;
        if (function == nullptr) {
            // a handle that starts one of several kernels depending on the live rows: run its launch for this row
            // count with recording on (nothing is enqueued, no argument is dereferenced) and take the kernel whose
            // grid, block and LDS bytes are the ones orx_geometry reports, i.e. the one a package records
            Geometry want;
            int code = f->geometry(*f, live, &want);
            if (code != ORX_OK) return code;
            uint64_t zero[64] = {};
            void* args[64];
            if (f->args.size() > 64) {
                set_error("orx_query %s: too many arguments", f->symbol.c_str());
                return (int)ORX_ERR_INTERNAL;
            }
            for (size_t i = 0; i < f->args.size(); ++i) args[i] = &zero[i];
            if (f->dynamic_rows) *reinterpret_cast<int32_t*>(&zero[f->args.size() - 1]) = live;
            std::vector<LaunchRecord> seen;
            g_recording = &seen;
            try {
                code = f->launch(*f, live, want, nullptr, args);
            } catch (...) {
                g_recording = nullptr;
                throw;
            }
            g_recording = nullptr;
            if (code != ORX_OK) return code;
            for (const LaunchRecord& r : seen)
                if (function == nullptr && r.grid == want.grid[0] && r.block == want.block[0] * want.block[1] * want.block[2] &&
                    r.shared == want.shared)
                    function = r.function;
            if (function == nullptr && !seen.empty()) function = seen.back().function;
            if (function == nullptr) {
                set_error("orx_query %s: the launch of %d rows starts no kernel", f->symbol.c_str(), live);
                return (int)ORX_ERR_INTERNAL;
            }
        }
        hipFuncAttributes attr;
        memset(&attr, 0, sizeof attr);
        const int code = hip_check(hipFuncGetAttributes(&attr, function), "hipFuncGetAttributes");
        if (code != ORX_OK) return code;
        if (max_threads_per_block) *max_threads_per_block = (uint32_t)attr.maxThreadsPerBlock;
        if (static_lds_bytes) *static_lds_bytes = (uint32_t)attr.sharedSizeBytes;
        return (int)ORX_OK;
    });
}

int orx_query(orx_fn f, uint32_t* max_threads_per_block, uint32_t* static_lds_bytes) {
    return orx_query_rows(f, 0, max_threads_per_block, static_lds_bytes);
}

int orx_geometry(orx_fn f, int32_t rows, uint32_t grid[3], uint32_t block[3], uint32_t* shared_bytes) {
    if (f == nullptr) {
        set_error("orx_geometry: null handle");
        return ORX_ERR_BAD_ARGUMENT;
    }
    return guard("orx_geometry", [&] {
        int live = rows <= 0 ? f->capacity : rows;
        if (live > f->capacity || (!f->dynamic_rows && live != f->capacity)) {
            // DynamicBatchKernel::launch rejects rows outside 1..capacity (operators/dynamic.rs:96-98).
            set_error("%s: rows %d outside the kernel capacity %d", f->symbol.c_str(), live, f->capacity);
            return (int)ORX_ERR_ROWS;
        }
        Geometry g;
        int code = f->geometry(*f, live, &g);
        if (code != ORX_OK) return code;
        for (int i = 0; i < 3; ++i) {
            if (grid) grid[i] = g.grid[i];
            if (block) block[i] = g.block[i];
        }
        if (shared_bytes) *shared_bytes = g.shared;
        return (int)ORX_OK;
    });
}

int orx_workspace_bytes(orx_fn f, int32_t rows, uint64_t* bytes) {
    if (f == nullptr || bytes == nullptr) {
        set_error("orx_workspace_bytes: null handle or output");
        return ORX_ERR_BAD_ARGUMENT;
    }
    return guard("orx_workspace_bytes", [&] {
        *bytes = 0;
        if (rows > f->capacity || (rows > 0 && !f->dynamic_rows && rows != f->capacity)) {
            set_error("%s: rows %d outside the kernel capacity %d", f->symbol.c_str(), rows, f->capacity);
            return (int)ORX_ERR_ROWS;
        }
        if (rows > 0 || !f->dynamic_rows) {
            *bytes = workspace_need(f, rows > 0 ? rows : f->capacity);
            return (int)ORX_OK;
        }
        // rows <= 0 on a dynamic kernel: what the engine allocates once, the largest need of any row count
        uint64_t most = 0;
        for (int r = 1; r <= f->capacity; ++r) most = std::max(most, workspace_need(f, r));
        *bytes = most;
        return (int)ORX_OK;
    });
}

int orx_arg_count(orx_fn f) { return f ? (int)(f->args.size() - f->omitted.size()) : 0; }

const char* orx_arg_name(orx_fn f, int index) {
    const int at = f ? full_index(f, index) : -1;
    return at < 0 ? "" : f->args[at].name;
}

int orx_arg_kind(orx_fn f, int index) {
    const int at = f ? full_index(f, index) : -1;
    return at < 0 ? -1 : (int)f->args[at].kind;
}

int orx_launch(orx_fn f, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
               void* hip_stream, void** args) {
    return guard("orx_launch", [&, args]() mutable {
        int rows = 0;
        Geometry want;
        void* full[64];
        args = expand_args(f, args, full);
        const int code = check_launch(f, grid, block, shared_bytes, args, true, &rows, &want);
        if (code != ORX_OK) return code;
        const uint64_t need = workspace_need(f, rows);
        if (need != 0 && *reinterpret_cast<uint64_t*>(args[f->workspace_arg]) == 0) {
            set_error("launch %s: %d rows need a Workspace of %llu bytes (orx_workspace_bytes), the buffer is null",
                      f->symbol.c_str(), rows, (unsigned long long)need);
            return (int)ORX_ERR_WORKSPACE;
        }
        return f->launch(*f, rows, want, reinterpret_cast<hipStream_t>(hip_stream), args);
    });
}

int orx_launch_static_scratch(orx_fn f, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
                              void* hip_stream, void** args) {
    return guard("orx_launch_static_scratch", [&, args]() mutable {
        int rows = 0;
        Geometry want;
        void* full[64];
        args = expand_args(f, args, full);
        const int code = check_launch(f, grid, block, shared_bytes, args, false, &rows, &want);
        if (code != ORX_OK) return code;
        if (!f->takes_workspace)  // nothing to replace: the plain launch
            return f->launch(*f, rows, want, reinterpret_cast<hipStream_t>(hip_stream), args);
        const uint64_t need = workspace_need(f, rows);
        if (need > (uint64_t)ORX_STATIC_SCRATCH_BYTES) {
            set_error("launch %s: %d rows need %llu bytes of scratch, the library's static scratch holds %llu "
                      "(ORX_STATIC_SCRATCH_BYTES): pass a Workspace to orx_launch instead",
                      f->symbol.c_str(), rows, (unsigned long long)need, (unsigned long long)ORX_STATIC_SCRATCH_BYTES);
            return (int)ORX_ERR_WORKSPACE;
        }
        void* address = nullptr;
        const int found = static_scratch_address(&address, reinterpret_cast<hipStream_t>(hip_stream), true);
        if (found != ORX_OK) return found;
        // the caller's argument list with the Workspace slot pointing at the library's scratch
        const size_t count = f->args.size();
        void* patched[64];
        if (count > 64) {
            set_error("launch %s: too many arguments", f->symbol.c_str());
            return (int)ORX_ERR_INTERNAL;
        }
        for (size_t i = 0; i < count; ++i) patched[i] = args[i];
        patched[f->workspace_arg] = &address;
        return f->launch(*f, rows, want, reinterpret_cast<hipStream_t>(hip_stream), patched);
    });
}

const char* orx_last_error(void) { return g_error; }

const char* orx_catalog(void) {
    // built once, also when two session threads ask at the same time
    static const std::string* text = [] {
        std::string* s = new (std::nothrow) std::string();
        if (s == nullptr) return (const std::string*)nullptr;
        try {
            *s = "{\"kernels\":[";
            Table t[kTables];
            tables(t);
            bool first = true;
            for (auto& table : t)
                for (int i = 0; i < table.count; ++i) {
                    if (!first) *s += ",";
                    first = false;
                    *s += "{\"symbol\":\"";
                    *s += table.rows[i].symbol;
                    *s += "\",\"variant_keys\":\"";
                    *s += table.rows[i].variant_keys;
                    *s += "\",\"arguments\":\"";
                    *s += table.rows[i].arguments;
                    *s += "\"}";
                }
            *s += "]}";
        } catch (...) {
            delete s;
            return (const std::string*)nullptr;
        }
        return (const std::string*)s;
    }();
    return text != nullptr ? text->c_str() : "{\"kernels\":[]}";
}

}  // extern "C"
