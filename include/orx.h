/* orx.h -- C ABI of liborx.so: MI355X (gfx950) kernels for orinfer's quantized linear path.
 *
 * The orinfer engine launches every device kernel through one data-driven entry
 * point: a `Kernel` record (symbol, grid, block, shared bytes, ordered args) is
 * resolved to a function handle and launched with `cuLaunchKernel(f, grid, block,
 * shared, stream, void** args, NULL)`.  This header is that entry point for HIP.
 * Nothing here allocates device memory (not at resolve, not at launch: a handle is
 * host memory only), synchronises or touches the host after the launch is enqueued;
 * every kernel reads its tables, scales and routing metadata from device memory at
 * run time, so a launch can be captured in a hipGraph and replayed after the caller
 * changed buffer contents.  The engine owns every buffer (AGENTS.md:41), scratch
 * included: a kernel that wants scratch takes it as a `Workspace` buffer argument.
 *
 * Argument convention (crates/orinfer-engine/src/backend/cuda/mod.rs:282-299,319):
 * args[i] points at an 8-byte device pointer or at a 4-byte scalar.  The ORDER of
 * arguments per symbol is the generated host ABI of the reference (buffer names in
 * ASCII order, then scalars; dynamic-row kernels take `int32 m` last) and is
 * published by orx_arg_name() and orx_catalog().  The reference marshals
 * Pointer, I32, U32, I64, U64 and F32 values; every kernel of this path takes device
 * pointers and int32 row counts only, so those are the two kinds there are.
 *
 * Shapes: K is a multiple of 128 for codes and of 64 for int8 weights (int8_projection.py:29;
 * a K that ends in half a step of 128 is served by the MFMA tile kernel at every row count);
 * two-stage codes are
 * row-major (packed_k = 0) or K-major in blocks of 128 or 64 (packed_k = 128 | 64,
 * e8p_q4.py:78-80,250).  Blocks of 64 are read by the streaming and the MFMA tile
 * kernels at every row count; the one-row GEMV and the resident kernel read row-major
 * codes and blocks of 128 only (production stores 128, models/qwen35/build.py:212).
 * Single-stage (routed expert) codes are decoded by an XOR identity that needs a basis
 * without zero coordinates, which the E8P basis is (quantization/vq.py:96-118 has the
 * same contract); `integer_vq_grouped` also takes the reference decoder's other options
 * (integer_vq.py:93-258) with its defaults: Book as the (256,2) table of raw int8 basis values, as the (512,4)
 * table of signed values (shortbook=true) or as (256,1) selector words (shortbook=true, selectorbook=true);
 * basis=any (selector ids for zero coordinates), one
 * table per expert (shared_table=false, the reference's default: Book is (E, ...)), patch words (patched=true:
 * Patch is (E,K/128,N) u16), tile lists of 8 or 16 rows and K-major blocks of 64.  These
 * run on the MFMA tile kernel only.  The symbol always lists Patch, as the reference's
 * host ABI does; without patched=true it is never read and may be null.
 *
 * The reference's INT4-exact expert kernels (e8p_exact.py, e8p_prefill.py) take A8 rows as two planes
 * of nibble words, Low and High, with the rows' integer sums: split_a8, split_prefill_a8,
 * split_routed_prefill_a8, dispatch_prefill_a8, pack_expert_tokens, expand_expert_slots and
 * rotate_expert_a8 write them, e8p_exact_grouped and e8p_prefill_grouped multiply them (on int8
 * MFMA, the nibbles put back together on the way into LDS; Sum is added as given).  Same symbols,
 * variant keys and argument order as the reference (flash_next/experts.rs:207-215).
 *
 * Thread model: one thread per device session, one explicit stream
 * (backend/cuda/mod.rs:1-3).  Handles are immutable after orx_resolve: launches of one
 * handle, or of different handles, may run concurrently on distinct streams as long as
 * their buffers (the Workspace included) are distinct.  One-time set-up inside the
 * library is per device and safe to reach from several session threads.
 */
#ifndef ORX_H
#define ORX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes.  0 = success.  Values 1..9999 are hipError_t values passed through
 * unchanged (the reference returns the driver's numeric code, mod.rs:48-55);
 * values >= 10000 are raised by the catalog itself before anything is enqueued. */
#define ORX_OK 0
#define ORX_ERR_UNKNOWN_SYMBOL 10001   /* no kernel of that name in the catalog            */
#define ORX_ERR_BAD_VARIANT 10002      /* variant JSON unparsable or geometry not supported */
#define ORX_ERR_BAD_GEOMETRY 10003     /* grid/block/shared do not fit the resolved kernel   */
#define ORX_ERR_BAD_ARGUMENT 10004     /* null handle, null args, misaligned pointer         */
#define ORX_ERR_ROWS 10005             /* dynamic rows outside 1..capacity                   */
#define ORX_ERR_WORKSPACE 10006        /* the launch needs a Workspace and got none / too small a one */
#define ORX_ERR_INTERNAL 10007         /* a C++ exception (out of host memory ...) stopped at the boundary */

typedef struct orx_function* orx_fn;

/* Replaces Catalog::resolve = cuModuleLoadData + cuModuleGetFunction + attribute checks
 * (crates/orinfer-engine/src/backend/cuda/kernels.rs:114-192).  `symbol` is a kernel
 * family of the catalog; `variant_json` is a flat JSON object carrying what the
 * reference bakes into a cubin at compile time (shape, tile, layout, dtype), the way
 * package `Definition`s do (crates/orinfer-model-sdk/src/catalog.rs:32-50).
 * Example: orx_resolve("e8p_q4_projection",
 *                      "{\"M\":1,\"N\":9728,\"K\":2560,\"algorithm\":\"gemv\"}", &f).
 * Values are integers, strings, booleans or flat lists of integers.  A key the family does
 * not know is refused (ORX_ERR_BAD_VARIANT, the message lists the family's keys), as the
 * reference's factories raise on an unknown keyword: no option is ever ignored silently. */
int orx_resolve(const char* symbol, const char* variant_json, orx_fn* out);

/* Drops a handle (cuModuleUnload in Session::cleanup).  Host memory only. */
int orx_release(orx_fn f);

/* Replaces cuFuncGetAttribute(MAX_THREADS_PER_BLOCK / SHARED_SIZE_BYTES)
 * (kernels.rs:150-170): limits the caller validates its launch record against. */
int orx_query(orx_fn f, uint32_t* max_threads_per_block, uint32_t* static_lds_bytes);

/* The same for the kernel that a launch of `rows` live rows starts (rows <= 0: the variant's own M,
 * which is what orx_query reports).  A projection handle picks its kernel by the live rows (one-row
 * GEMV, batched-decode kernels, MFMA tiles): the attributes are read from that kernel, the one whose
 * grid, block and LDS bytes orx_geometry returns for the same rows, so a record per row range
 * (crates/orinfer-model-sdk/src/operators/rows.rs:14-58) is validated against its own function as
 * kernels.rs:150-170 validates a cubin's.  Enqueues nothing. */
int orx_query_rows(orx_fn f, int32_t rows, uint32_t* max_threads_per_block, uint32_t* static_lds_bytes);

/* The launch geometry a package would record for this kernel: the static grid of a
 * fixed-row kernel, or the RowExpression result of a dynamic one for `rows` live rows
 * (crates/orinfer-model-sdk/src/operators/dynamic.rs:93-118).  rows <= 0 means the
 * variant's own M.  Fails with ORX_ERR_ROWS when rows exceeds the capacity. */
int orx_geometry(orx_fn f, int32_t rows, uint32_t grid[3], uint32_t block[3], uint32_t* shared_bytes);

/* Scratch the engine provides (AGENTS.md:41 "the engine owns every buffer"; the reference's
 * kernels have none, so this has no counterpart there beyond the buffer table of
 * crates/orinfer-model-sdk/src/artifact.rs:60-72 in which the engine would list it).  A
 * projection resolved with `"workspace": true` takes one more buffer, `Workspace`, after its
 * weights (256-byte aligned; contents need not be kept between launches; launches that overlap
 * in time need distinct ones).  *bytes = what a launch of `rows` rows reads and writes there;
 * rows <= 0 asks for the largest need of any row count up to the capacity, which is what an
 * engine allocates once.  0 means the launch uses none and the pointer may be null.  Handles
 * resolved without the key never use scratch (whole tiles, decode inside the GEMM). */
int orx_workspace_bytes(orx_fn f, int32_t rows, uint64_t* bytes);

/* Argument list of the resolved kernel, in launch order (contracts/abi.py:26-80 parses
 * the same from the generated host.txt).  kind: 0 = device pointer, 1 = int32 scalar. */
int orx_arg_count(orx_fn f);
const char* orx_arg_name(orx_fn f, int index);
int orx_arg_kind(orx_fn f, int index);

/* Replaces launch_kernel = cuLaunchKernel (backend/cuda/mod.rs:312-341).  Enqueues the
 * kernel on `hip_stream` (a hipStream_t, may be 0).  grid/block/shared must equal what
 * orx_geometry() returns for the row count passed in `m` (validated; the reference
 * validates records in kernels.rs:47-61).  Never blocks, never allocates.  A launch may
 * enqueue more than one kernel (weight expansion + GEMM, split tiles + their sum, row slices
 * of a batched-decode kernel): the recorded grid/block/shared are those of its main kernel and
 * the whole launch is one node sequence under graph capture. */
int orx_launch(orx_fn f, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
               void* hip_stream, void** args);

/* Size of the library's own scratch, one copy per device for the life of the process. */
#define ORX_STATIC_SCRATCH_BYTES (64u << 20)

/* No counterpart in the reference.  For callers that cannot allocate device memory at all -- code
 * that is already under hipGraph capture when it learns its shapes, tight serving loops and
 * harnesses that forbid hipMalloc: orx_launch for a handle resolved with `"workspace": true`, with
 * the Workspace argument ignored (its slot in `args` may be null) and the library's static device
 * array of ORX_STATIC_SCRATCH_BYTES used in its place.  Everything else -- geometry check,
 * arguments, results -- is orx_launch's.  A launch that needs more than ORX_STATIC_SCRATCH_BYTES
 * (orx_workspace_bytes tells) fails with ORX_ERR_WORKSPACE and enqueues nothing.  Calls no
 * allocator.  All calls on one device share that device's array: calls that overlap in time on
 * one device (two streams) race; calls in stream order do not (nothing in the array has to
 * survive from one launch to the next, and nothing has to be zero when a launch starts).
 * The array's address is looked up once per device, for the calling thread's current device:
 * orx_resolve of a workspace handle does it for the device current then, so resolve (or launch
 * once) with the launch device current before a capture begins; a first launch on a device whose
 * address is not known yet, on a stream that is capturing, fails with ORX_ERR_BAD_ARGUMENT. */
int orx_launch_static_scratch(orx_fn f, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
                              void* hip_stream, void** args);

/* Thread-local text of the last failure on this thread (mod.rs:48-55 formats
 * "<op>: CUDA error <code>").  Never NULL. */
const char* orx_last_error(void);

/* JSON text listing every symbol, its variant keys and its argument order. Static storage. */
const char* orx_catalog(void);

#ifdef __cplusplus
}
#endif
#endif /* ORX_H */
