// orx_run_fixture -- runs one fixture (buffers + kernel records + a validation block) through the C
// ABI of liborx, the way the engine's own single-kernel harness proves a kernel package:
// `orinfer run-artifact MANIFEST` (crates/orinfer-cli/src/diag.rs:85,217-218 ->
// crates/orinfer-engine/src/backend/cuda/mod.rs:359-720, fixture schema in artifact.rs:16-37).
//
// Sequence (same order as the reference harness):
//   1. allocate and upload every buffer, check pointer alignment
//   2. per kernel record: orx_resolve, orx_query_rows limits, launch record checked against orx_geometry
//   3. launch all records on one stream; compare the named output with an fp32 reference file by
//      relative L2
//   4. capture the records in a graph; poison the output with 0xFF, replay, require byte-identical
//      output
//   5. zero the named input, replay, require an all-zero output; restore it, replay, require
//      byte-identical output again
//   6. time 3 x `repetitions` graph replays with events
// Prints one JSON report on stdout; exit code 0 only if every check passed.
//
// Manifest (JSON; paths relative to the manifest):
//   {"schema_version": 1, "target": "gfx950",
//    "buffers": [{"name": "A", "bytes": 1024, "file": "A.bin"}, {"name": "Out", "bytes": 512, "fill": 0}],
//    "kernels": [{"symbol": "e8p_q4_projection", "variant": {"M": 1, "N": 256, "K": 256},
//                 "grid": [..], "block": [..], "shared": 0,          (optional: default orx_geometry)
//                 "rows": 1,                                           (live rows for dynamic kernels)
//                 "args": [{"buffer": "A"}, {"buffer": "AS", "offset": 0}, {"i32": 1}]}],
//    "validation": {"output": "Out", "output_dtype": "f16", "reference": "Out.f32", "elements": 256,
//                   "relative_l2_tolerance": 1e-3, "zero_input": "A", "repetitions": 20}}
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/orx.h"

namespace {

// ---- a small JSON reader (objects, arrays, strings, numbers, booleans, null) ----------------
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    double number = 0;
    std::string text;                       // string value, or the raw text of an object
    std::vector<Json> items;                // array elements
    std::vector<std::pair<std::string, Json>> fields;
    const Json* get(const char* key) const {
        for (const auto& f : fields)
            if (f.first == key) return &f.second;
        return nullptr;
    }
};

struct Parser {
    const std::string& s;
    size_t i = 0;
    std::string error;
    explicit Parser(const std::string& source) : s(source) {}
    void skip() {
        while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i;
    }
    bool fail(const char* what) {
        if (error.empty()) error = std::string(what) + " at byte " + std::to_string(i);
        return false;
    }
    bool parse_string(std::string* out) {
        if (s[i] != '"') return fail("expected string");
        ++i;
        while (i < s.size() && s[i] != '"') {
            if (s[i] == '\\' && i + 1 < s.size()) {
                const char c = s[i + 1];
                out->push_back(c == 'n' ? '\n' : c == 't' ? '\t' : c);
                i += 2;
            } else {
                out->push_back(s[i++]);
            }
        }
        if (i >= s.size()) return fail("unterminated string");
        ++i;
        return true;
    }
    bool parse(Json* out) {
        skip();
        if (i >= s.size()) return fail("unexpected end");
        const char c = s[i];
        if (c == '{') {
            const size_t begin = i;
            out->kind = Json::Object;
            ++i;
            skip();
            if (i < s.size() && s[i] == '}') {
                ++i;
                out->text = s.substr(begin, i - begin);
                return true;
            }
            for (;;) {
                skip();
                std::string key;
                if (!parse_string(&key)) return false;
                skip();
                if (i >= s.size() || s[i] != ':') return fail("expected ':'");
                ++i;
                Json value;
                if (!parse(&value)) return false;
                out->fields.emplace_back(key, std::move(value));
                skip();
                if (i < s.size() && s[i] == ',') {
                    ++i;
                    continue;
                }
                if (i < s.size() && s[i] == '}') {
                    ++i;
                    break;
                }
                return fail("expected ',' or '}'");
            }
            out->text = s.substr(begin, i - begin);
            return true;
        }
        if (c == '[') {
            out->kind = Json::Array;
            ++i;
            skip();
            if (i < s.size() && s[i] == ']') {
                ++i;
                return true;
            }
            for (;;) {
                Json value;
                if (!parse(&value)) return false;
                out->items.push_back(std::move(value));
                skip();
                if (i < s.size() && s[i] == ',') {
                    ++i;
                    continue;
                }
                if (i < s.size() && s[i] == ']') {
                    ++i;
                    break;
                }
                return fail("expected ',' or ']'");
            }
            return true;
        }
        if (c == '"') {
            out->kind = Json::String;
            return parse_string(&out->text);
        }
        if (s.compare(i, 4, "true") == 0) {
            out->kind = Json::Bool, out->number = 1, i += 4;
            return true;
        }
        if (s.compare(i, 5, "false") == 0) {
            out->kind = Json::Bool, out->number = 0, i += 5;
            return true;
        }
        if (s.compare(i, 4, "null") == 0) {
            out->kind = Json::Null, i += 4;
            return true;
        }
        char* end = nullptr;
        out->number = std::strtod(s.c_str() + i, &end);
        if (end == s.c_str() + i) return fail("unexpected character");
        out->kind = Json::Number;
        i = (size_t)(end - s.c_str());
        return true;
    }
};

struct Failure {
    std::string what;
};
[[noreturn]] void die(const std::string& what) { throw Failure{what}; }
void hip(hipError_t code, const char* op) {
    if (code != hipSuccess) die(std::string(op) + ": HIP error " + std::to_string((int)code) + " (" + hipGetErrorName(code) + ")");
}
void orx(int code, const char* op) {
    if (code != ORX_OK) die(std::string(op) + ": error " + std::to_string(code) + ": " + orx_last_error());
}

std::vector<char> read_file(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) die("cannot read " + path);
    return std::vector<char>((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
}

struct Buffer {
    std::string name;
    size_t bytes = 0;
    void* device = nullptr;
    std::vector<char> host;  // initial contents
};

struct Record {
    orx_fn function = nullptr;
    uint32_t grid[3] = {1, 1, 1}, block[3] = {1, 1, 1}, shared = 0;
    std::vector<uint64_t> pointer_values;  // storage for args (8 bytes each, pointers and scalars alike)
    std::vector<void*> args;
};

double as_number(const Json* j, double fallback) { return j && j->kind == Json::Number ? j->number : fallback; }

int run(const std::string& manifest_path, std::ostringstream& report) {
    const std::vector<char> raw = read_file(manifest_path);
    const std::string source(raw.begin(), raw.end());
    Parser parser(source);
    Json root;
    if (!parser.parse(&root) || root.kind != Json::Object) die("manifest: " + (parser.error.empty() ? "not an object" : parser.error));
    if ((int)as_number(root.get("schema_version"), 0) != 1) die("manifest: schema_version must be 1");
    const std::string directory = manifest_path.find('/') == std::string::npos ? "." : manifest_path.substr(0, manifest_path.rfind('/'));

    hipStream_t stream;
    hip(hipStreamCreate(&stream), "hipStreamCreate");

    // 1. buffers
    std::map<std::string, Buffer> buffers;
    const Json* list = root.get("buffers");
    if (!list || list->kind != Json::Array) die("manifest: buffers[] missing");
    for (const Json& b : list->items) {
        Buffer buffer;
        const Json* name = b.get("name");
        if (!name || name->kind != Json::String) die("manifest: buffer without name");
        buffer.name = name->text;
        buffer.bytes = (size_t)as_number(b.get("bytes"), 0);
        if (const Json* file = b.get("file")) {
            buffer.host = read_file(directory + "/" + file->text);
            if (buffer.bytes == 0) buffer.bytes = buffer.host.size();
            if (buffer.host.size() != buffer.bytes) die("buffer " + buffer.name + ": file size differs from bytes");
        } else {
            buffer.host.assign(buffer.bytes, (char)(int)as_number(b.get("fill"), 0));
        }
        if (buffer.bytes == 0) die("buffer " + buffer.name + ": zero bytes");
        hip(hipMalloc(&buffer.device, buffer.bytes), "hipMalloc");
        if (reinterpret_cast<uintptr_t>(buffer.device) % 256 != 0) die("buffer " + buffer.name + ": allocation not 256-byte aligned");
        hip(hipMemcpy(buffer.device, buffer.host.data(), buffer.bytes, hipMemcpyHostToDevice), "hipMemcpy upload");
        buffers[buffer.name] = std::move(buffer);
    }

    // 2. kernel records
    std::vector<Record> records;
    const Json* kernels = root.get("kernels");
    if (!kernels || kernels->kind != Json::Array || kernels->items.empty()) die("manifest: kernels[] missing");
    int device = 0;
    hipDeviceProp_t prop;
    hip(hipGetDevice(&device), "hipGetDevice");
    hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    for (const Json& k : kernels->items) {
        Record record;
        const Json* symbol = k.get("symbol");
        const Json* variant = k.get("variant");
        if (!symbol || symbol->kind != Json::String) die("manifest: kernel without symbol");
        orx(orx_resolve(symbol->text.c_str(), variant && variant->kind == Json::Object ? variant->text.c_str() : "{}", &record.function),
            "orx_resolve");
        uint32_t max_threads = 0, static_lds = 0;
        const int rows = (int)as_number(k.get("rows"), 0);
        // the limits of the kernel that these rows start (a projection handle picks its kernel by the live rows)
        orx(orx_query_rows(record.function, rows, &max_threads, &static_lds), "orx_query_rows");
        uint32_t grid[3], block[3], shared = 0;
        orx(orx_geometry(record.function, rows, grid, block, &shared), "orx_geometry");
        for (int d = 0; d < 3; ++d) record.grid[d] = grid[d], record.block[d] = block[d];
        record.shared = shared;
        auto read_triple = [&](const char* key, uint32_t* dst) {
            if (const Json* v = k.get(key)) {
                if (v->kind != Json::Array || v->items.size() != 3) die(std::string("kernel ") + symbol->text + ": " + key + " must have 3 entries");
                for (int d = 0; d < 3; ++d) dst[d] = (uint32_t)v->items[d].number;
            }
        };
        read_triple("grid", record.grid);
        read_triple("block", record.block);
        if (const Json* v = k.get("shared")) record.shared = (uint32_t)v->number;
        // the limits the engine checks before it accepts a record (kernels.rs:47-61,150-190)
        const uint32_t threads = record.block[0] * record.block[1] * record.block[2];
        if (threads == 0 || threads > max_threads) die("kernel " + symbol->text + ": block exceeds the function's thread limit");
        if ((size_t)static_lds + record.shared > (size_t)prop.sharedMemPerMultiprocessor && prop.sharedMemPerMultiprocessor > 0)
            die("kernel " + symbol->text + ": LDS request exceeds the device");
        const Json* args = k.get("args");
        if (!args || args->kind != Json::Array) die("kernel " + symbol->text + ": args[] missing");
        if ((int)args->items.size() != orx_arg_count(record.function))
            die("kernel " + symbol->text + ": takes " + std::to_string(orx_arg_count(record.function)) + " arguments, manifest has " +
                std::to_string(args->items.size()));
        record.pointer_values.resize(args->items.size());
        for (size_t a = 0; a < args->items.size(); ++a) {
            const Json& arg = args->items[a];
            if (const Json* name = arg.get("buffer")) {
                if (orx_arg_kind(record.function, (int)a) != 0)
                    die("kernel " + symbol->text + ": argument " + orx_arg_name(record.function, (int)a) + " is a scalar");
                auto it = buffers.find(name->text);
                if (it == buffers.end()) die("kernel " + symbol->text + ": unknown buffer " + name->text);
                const size_t offset = (size_t)as_number(arg.get("offset"), 0);
                if (offset >= it->second.bytes) die("kernel " + symbol->text + ": offset beyond buffer " + name->text);
                // the engine sizes a Workspace buffer from orx_workspace_bytes before it accepts the record
                if (std::string(orx_arg_name(record.function, (int)a)) == "Workspace") {
                    uint64_t need = 0;
                    orx(orx_workspace_bytes(record.function, rows, &need), "orx_workspace_bytes");
                    if (it->second.bytes - offset < need)
                        die("kernel " + symbol->text + ": Workspace buffer " + name->text + " holds " +
                            std::to_string(it->second.bytes - offset) + " bytes, the launch needs " + std::to_string(need));
                }
                record.pointer_values[a] = reinterpret_cast<uint64_t>(static_cast<char*>(it->second.device) + offset);
            } else if (const Json* value = arg.get("i32")) {
                if (orx_arg_kind(record.function, (int)a) != 1)
                    die("kernel " + symbol->text + ": argument " + orx_arg_name(record.function, (int)a) + " is a pointer");
                const int32_t scalar = (int32_t)value->number;
                std::memcpy(&record.pointer_values[a], &scalar, sizeof scalar);
            } else {
                die("kernel " + symbol->text + ": argument must be a buffer or an i32 object");
            }
        }
        for (auto& v : record.pointer_values) record.args.push_back(&v);
        records.push_back(std::move(record));
    }
    auto launch_all = [&]() {
        for (Record& r : records) orx(orx_launch(r.function, r.grid, r.block, r.shared, stream, r.args.data()), "orx_launch");
    };

    // 3. eager run + relative L2 against the fp32 reference
    const Json* validation = root.get("validation");
    if (!validation || validation->kind != Json::Object) die("manifest: validation missing");
    const Json* output_name = validation->get("output");
    if (!output_name || buffers.find(output_name->text) == buffers.end()) die("validation: unknown output buffer");
    Buffer& output = buffers[output_name->text];
    launch_all();
    hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    std::vector<char> first(output.bytes);
    hip(hipMemcpy(first.data(), output.device, output.bytes, hipMemcpyDeviceToHost), "hipMemcpy download");
    double relative_l2 = -1;
    bool reference_ok = true;
    if (const Json* reference = validation->get("reference")) {
        const std::vector<char> ref_raw = read_file(directory + "/" + reference->text);
        const size_t elements = ref_raw.size() / 4;
        const float* ref = reinterpret_cast<const float*>(ref_raw.data());
        const Json* dtype = validation->get("output_dtype");
        const std::string kind = dtype ? dtype->text : "f16";
        const size_t width = kind == "f32" || kind == "i32" ? 4 : kind == "i8" ? 1 : 2;
        if (elements * width > output.bytes) die("validation: reference has more elements than the output buffer");
        double diff = 0, norm = 0;
        for (size_t e = 0; e < elements; ++e) {
            double got;
            if (kind == "f32")
                got = reinterpret_cast<const float*>(first.data())[e];
            else if (kind == "i32")
                got = reinterpret_cast<const int32_t*>(first.data())[e];
            else if (kind == "i8")
                got = reinterpret_cast<const int8_t*>(first.data())[e];
            else
                got = __half2float(reinterpret_cast<const __half*>(first.data())[e]);
            diff += (got - ref[e]) * (got - ref[e]);
            norm += (double)ref[e] * ref[e];
        }
        relative_l2 = std::sqrt(diff) / std::max(std::sqrt(norm), 1e-30);
        reference_ok = relative_l2 <= as_number(validation->get("relative_l2_tolerance"), 1e-3);
    }

    // 4. graph capture, poisoned output, replay
    hipGraph_t graph;
    hipGraphExec_t executable;
    hip(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal), "hipStreamBeginCapture");
    launch_all();
    hip(hipStreamEndCapture(stream, &graph), "hipStreamEndCapture");
    hip(hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    auto replay_and_fetch = [&](std::vector<char>* into) {
        hip(hipGraphLaunch(executable, stream), "hipGraphLaunch");
        hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
        into->resize(output.bytes);
        hip(hipMemcpy(into->data(), output.device, output.bytes, hipMemcpyDeviceToHost), "hipMemcpy download");
    };
    // bytes the kernels do not write (strides, rows beyond m) keep their initial contents, so the
    // comparison is on the bytes that differ from the poison after the eager run... the poison run
    // is compared on the positions the eager run wrote, i.e. where `first` differs from the initial image
    std::vector<char> poisoned, zeroed, restored;
    hip(hipMemset(output.device, 0xFF, output.bytes), "hipMemset poison");
    replay_and_fetch(&poisoned);
    size_t written = 0, poison_mismatch = 0;
    for (size_t b = 0; b < output.bytes; ++b) {
        const bool wrote = poisoned[b] != (char)0xFF || first[b] == (char)0xFF;
        if (poisoned[b] != (char)0xFF) ++written;
        if (wrote && poisoned[b] != first[b]) ++poison_mismatch;
    }
    const bool replay_ok = poison_mismatch == 0 && written > 0;

    // 5. zero input -> zero output; restored input -> identical output
    bool zero_ok = true, restore_ok = true;
    if (const Json* zero_name = validation->get("zero_input")) {
        auto it = buffers.find(zero_name->text);
        if (it == buffers.end()) die("validation: unknown zero_input buffer");
        hip(hipMemset(it->second.device, 0, it->second.bytes), "hipMemset zero input");
        hip(hipMemset(output.device, 0xFF, output.bytes), "hipMemset poison");
        replay_and_fetch(&zeroed);
        for (size_t b = 0; b < output.bytes; ++b)
            if (poisoned[b] != (char)0xFF && zeroed[b] != 0) zero_ok = false;
        hip(hipMemcpy(it->second.device, it->second.host.data(), it->second.bytes, hipMemcpyHostToDevice), "hipMemcpy restore");
        hip(hipMemset(output.device, 0xFF, output.bytes), "hipMemset poison");
        replay_and_fetch(&restored);
        restore_ok = restored == poisoned;
    }

    // 6. timing: 3 x repetitions replays
    const int repetitions = std::max(1, (int)as_number(validation->get("repetitions"), 20));
    hipEvent_t start, stop;
    hip(hipEventCreate(&start), "hipEventCreate");
    hip(hipEventCreate(&stop), "hipEventCreate");
    float best_ms = 1e30f, trial_ms[3];
    for (int trial = 0; trial < 3; ++trial) {
        hip(hipEventRecord(start, stream), "hipEventRecord");
        for (int r = 0; r < repetitions; ++r) hip(hipGraphLaunch(executable, stream), "hipGraphLaunch");
        hip(hipEventRecord(stop, stream), "hipEventRecord");
        hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
        hip(hipEventElapsedTime(&trial_ms[trial], start, stop), "hipEventElapsedTime");
        best_ms = std::min(best_ms, trial_ms[trial]);
    }
    std::sort(trial_ms, trial_ms + 3);

    const bool ok = reference_ok && replay_ok && zero_ok && restore_ok;
    report << "{\"ok\": " << (ok ? "true" : "false") << ", \"kernels\": " << records.size() << ", \"relative_l2\": " << relative_l2
           << ", \"reference_ok\": " << (reference_ok ? "true" : "false") << ", \"graph_replay_identical\": " << (replay_ok ? "true" : "false")
           << ", \"output_bytes_written\": " << written << ", \"zero_input_gives_zero\": " << (zero_ok ? "true" : "false")
           << ", \"restored_input_identical\": " << (restore_ok ? "true" : "false") << ", \"repetitions\": " << repetitions
           << ", \"median_us_per_replay\": " << trial_ms[1] * 1e3 / repetitions << ", \"best_us_per_replay\": " << best_ms * 1e3 / repetitions
           << "}";

    (void)hipGraphExecDestroy(executable);
    (void)hipGraphDestroy(graph);
    for (Record& r : records) orx_release(r.function);
    for (auto& b : buffers) (void)hipFree(b.second.device);
    (void)hipStreamDestroy(stream);
    return ok ? 0 : 1;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: orx_run_fixture MANIFEST.json\n");
        return 2;
    }
    std::ostringstream report;
    try {
        const int code = run(argv[1], report);
        std::printf("%s\n", report.str().c_str());
        return code;
    } catch (const Failure& failure) {
        std::printf("{\"ok\": false, \"error\": \"%s\"}\n", failure.what.c_str());
        std::fprintf(stderr, "orx_run_fixture: %s\n", failure.what.c_str());
        return 3;
    }
}
