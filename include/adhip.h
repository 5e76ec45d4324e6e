/*
 * adhip -- C ABI of the MI355X (gfx950) execution backend for the autodiff-ir-rust `Device` interface.
 *
 * Every entry point is what a Rust `HipDevice` (an `impl Device`, reference src/core/ir.rs:126-143) binds
 * over FFI.  Plain pointers and sizes only; no exceptions or panics cross this boundary: functions return
 * 0 on success and a non-zero code on failure, with the message available from adhip_last_error().
 *
 * A context is used by one thread at a time (the reference holds its DEVICE mutex around every call,
 * src/core/ir.rs:180-198, src/core/value.rs:83-91).
 */
#ifndef ADHIP_H
#define ADHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct adhip_ctx adhip_ctx;
typedef struct adhip_program adhip_program;

/* Library version string. */
const char* adhip_version(void);

/* Open HIP device `device_ordinal` and create a context (one stream).
 * Replaces OpenCL::new(CLDeviceType) -- reference src/devices/opencl/device.rs:41-58. */
int adhip_create(int device_ordinal, adhip_ctx** out);

/* Release the context, its compiled kernels, the programs it kept and its result buffers. */
void adhip_destroy(adhip_ctx* ctx);

/* Message of the last failure on this context (empty string if none).  ctx may be NULL for failures of
 * adhip_create / adhip_lower_describe (a thread-local message is returned). */
const char* adhip_last_error(adhip_ctx* ctx);

/* Device::execute -- reference src/core/ir.rs:128, src/devices/opencl/device.rs:62-88.
 * `program` is the serialised nested IR procedure (wire format: autodiff-ir-rust_amd/adhip/ir.py and
 * csrc/ir.cpp), ending in EX; `dep_ids` is the keep list (reference src/core/dependency.rs).  Starts from
 * fresh device state, uploads every CreateMat payload (host pointers inside `program` are borrowed until
 * the call returns), runs until the first EX and copies every kept id back to host memory owned by ctx.
 * The context keeps the plans and device buffers of the last few distinct programs (same command stream and
 * keep list; payload contents may differ), so executing a program again costs upload + run + read-back only;
 * ADHIP_EXEC_CACHE=0 in the environment turns that off. */
int adhip_execute(adhip_ctx* ctx, const uint8_t* program, size_t program_len, const char* const* dep_ids,
                  size_t n_dep_ids);

/* Device::get_tensor -- reference src/core/ir.rs:131, src/devices/opencl/device.rs:90-102.
 * Returns 0 and sets data/dims/ndim (memory owned by ctx, valid until the next execute/readback/destroy),
 * 1 if `id` was not kept or never defined (the reference's ValueData::none()), another code on error. */
int adhip_get_tensor(adhip_ctx* ctx, const char* id, const float** data, const uint64_t** dims, size_t* ndim);

/* Device::dot_prod_shape default -- reference src/core/ir.rs:140-142: out = {a[0], b[last]}. */
int adhip_dot_prod_shape(const uint64_t* a_dims, size_t a_ndim, const uint64_t* b_dims, size_t b_ndim, uint64_t out[2]);

/* ---- adhip_execute in stages, for callers that keep a program resident on the GPU -------------------
 * adhip_execute(ctx, ...) == program_create + program_upload + program_run + program_readback + destroy.
 * These have no separate counterpart in the reference, whose execute() does all of it in one call
 * (src/devices/opencl/device.rs:62-88). */

/* Parse, lower to kernels, compile them (hipRTC, cached per context) and allocate device buffers. */
int adhip_program_create(adhip_ctx* ctx, const uint8_t* program, size_t program_len, const char* const* dep_ids,
                         size_t n_dep_ids, adhip_program** out);
/* Copy every CreateMat payload to the device (host pointers given at create time must still be valid). */
int adhip_program_upload(adhip_program* p);
/* Run from the current device state to the first EX; returns after the stream has drained. */
int adhip_program_run(adhip_program* p);
/* The same without the final wait: the kernels are queued on the context's stream and the call returns (a loop or
 * branch that the host has to decide still waits for its predicate).  Several runs can be queued back to back;
 * adhip_program_sync waits for all of them and must be called before upload, read-back or destroy. */
int adhip_program_enqueue(adhip_program* p);
int adhip_program_sync(adhip_program* p);

/* adhip_program_enqueue for callers that cannot allocate device memory while they run (tight serving loops, harnesses
 * that forbid it; a straight-line program also under HIP stream capture).  No counterpart in the reference.
 * Every temporary of the program (partial sums of reductions, slices of split matrix products, intermediate tensors)
 * and its control-flow flags are placed in a static device array of ADHIP_STATIC_SCRATCH_BYTES that the library holds
 * on every GPU it runs on, instead of in the program's own allocations; inputs, kept tensors and ids that live across
 * control flow stay in the buffers the program got at create time.  The call makes no hipMalloc / hipFree and no
 * allocating library call, on the device or on the host, and launches every kernel directly (no graph capture or
 * instantiation, no profiling events).  A straight-line program is queued and the call returns without waiting, like
 * adhip_program_enqueue.  A program with loops or branches behaves as it does there too: the host reads predicates
 * back (a 4-byte asynchronous copy into pinned memory the context holds since adhip_create, then a wait on the
 * stream) -- once for a counted loop, once per batch of iterations for a data-dependent one, once per If -- which
 * allocates nothing but blocks, and is not legal while the caller captures the stream.  A program whose temporaries
 * and flags need more than ADHIP_STATIC_SCRATCH_BYTES is refused with an error that names both sizes.  All programs
 * of all contexts on one GPU share that GPU's array and find the last call's contents in it (every kernel writes
 * what it later reads from there, so nothing needs clearing).  Runs queued on one context follow one another on its
 * stream; runs of different contexts on the same GPU that overlap in time race on the array -- wait for one
 * (adhip_program_sync) before a run of another context starts. */
#define ADHIP_STATIC_SCRATCH_BYTES (32u << 20)
int adhip_program_enqueue_noalloc(adhip_program* p);
/* Copy kept ids to host memory owned by the context (then served by adhip_get_tensor). */
int adhip_program_readback(adhip_program* p);
void adhip_program_destroy(adhip_program* p);

/* Per-kernel timing with HIP events on the context's stream (off by default). */
int adhip_program_set_profiling(adhip_program* p, int enabled);
int adhip_program_kernel_count(adhip_program* p);
/* Launch site i: label, launches so far, total milliseconds, algorithmic bytes and flops of one launch. */
int adhip_program_kernel_stat(adhip_program* p, int i, char* label, size_t label_cap, uint64_t* launches,
                              double* total_ms, double* bytes_per_launch, double* flops_per_launch);
/* Generated HIP source of launch site i (owned by the program). */
const char* adhip_program_kernel_source(adhip_program* p, int i);
/* Text description of buffers, kernels and control structure (owned by the program). */
const char* adhip_program_describe(adhip_program* p);

/* Lower only (no GPU needed): writes the same description into `out`.  Returns non-zero and writes the
 * message into `out` on failure. */
int adhip_lower_describe(const uint8_t* program, size_t program_len, const char* const* dep_ids, size_t n_dep_ids,
                         char* out, size_t out_cap);

/* Lower and compile every generated kernel with hipRTC for `arch` (default "gfx950") without touching a
 * GPU: the build-time check that the device code is valid.  Writes a one-line summary or the error; the
 * summary ends with "; spilling kernels: <name> (<n> scalar, <n> vector registers spilled, <n> bytes of scratch
 * per lane); ..." when the compiler's metadata of a code object records any. */
int adhip_compile_check(const uint8_t* program, size_t program_len, const char* const* dep_ids, size_t n_dep_ids,
                        const char* arch, char* out, size_t out_cap);

#ifdef __cplusplus
}
#endif
#endif /* ADHIP_H */
