/*
 * emmy_hip.h — C ABI of libemmy_hip.so, the gfx950 kernel launcher.
 *
 * This is the whole device boundary of the backend: HIP source text goes in,
 * code objects come out (hipRTC), code objects become launchable functions,
 * and launches / events / graphs run on a caller-supplied HIP stream.  The
 * library never allocates device memory: every pointer in a launch's argument
 * list is borrowed from the caller (PyTorch-ROCm tensors' data_ptr()).
 *
 * It replaces, for AMD GPUs, what the reference obtains from the nvcc binary
 * plus cupy's driver bindings:
 *   - emmy/compiler/backend/cuda/nvcc.py:118-177   (compile_to_cubin / load_function)
 *   - emmy/compiler/backend/cuda/program.py:48     (_ensure_dynamic_smem_attr)
 *   - emmy/compiler/backend/cuda/program.py:394-424 (_launch)
 *   - emmy/compiler/backend/cuda/program.py:574-611 (_wait_for_event watchdog)
 *   - emmy/compiler/backend/cuda/program.py:1152-1325 (benchmark_program: events, graphs)
 *
 * Conventions
 *   - Every function returns 0 on success, otherwise the hipError_t (positive)
 *     or, for emh_compile, the hiprtcResult offset by EMH_RTC_ERROR_BASE.
 *     Nothing throws.  emh_last_error() returns a thread-local message for the
 *     most recent failure on the calling thread.
 *   - Handles are opaque pointers.  A handle is owned by the caller from the
 *     call that returns it until the matching destroy/unload/free call.
 *   - Buffers returned through `void**` / `char**` out-parameters are
 *     malloc'd by the library and released with emh_free().
 *   - `stream` is a hipStream_t passed as void*; NULL is the legacy default
 *     stream.  The library creates no threads and keeps no global device
 *     state; it is re-entrant per handle.
 */
#ifndef EMMY_HIP_H
#define EMMY_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EMH_RTC_ERROR_BASE 100000
#define EMH_ABI_VERSION 1

/* Library / device discovery -------------------------------------------- */

/* ABI version of the loaded library (EMH_ABI_VERSION it was built with). */
int emh_abi_version(void);

/* Number of visible HIP devices; 0 (not an error) when there is none.
 * Replaces cupy.cuda.runtime.getDeviceCount as used by
 * emmy/compiler/backend/cuda/program.py:1382-1533 (device fan-out). */
int emh_device_count(int* count);

/* Static properties of `device` the schedule heuristics read: gcnArchName
 * (e.g. "gfx950:sramecc+:xnack-") copied into arch[arch_len], compute-unit
 * count, LDS bytes per workgroup, wavefront size, engine clock in kHz and
 * total global memory in bytes.  Replaces the cupy device-attribute reads in
 * emmy/compiler/context.py:69-260 (Context.from_device). */
int emh_device_props(int device, char* arch, size_t arch_len, int* compute_units,
                     int* lds_bytes_per_block, int* wavefront_size, int* clock_khz,
                     size_t* global_mem_bytes);

/* Compilation ------------------------------------------------------------ */

/* Compile HIP source `src` (one or more extern "C" __global__ functions) for
 * `arch` ("gfx950") with hipRTC.  `name` labels the translation unit in
 * diagnostics.  `opts` are extra compiler options appended after
 * --offload-arch.  On success *code / *code_len receive the code object.
 * *log (may be NULL) always receives the compiler log when one exists, also
 * on failure.  Needs no GPU.  Replaces compile_to_cubin,
 * emmy/compiler/backend/cuda/nvcc.py:118-152. */
int emh_compile(const char* src, const char* name, const char* arch, const char* const* opts,
                int nopts, void** code, size_t* code_len, char** log);

/* Release a buffer handed out by emh_compile. NULL is allowed. */
void emh_free(void* p);

/* Modules and functions --------------------------------------------------- */

/* Load a code object onto the current device.  Replaces cp.RawModule(path=…),
 * emmy/compiler/backend/cuda/nvcc.py:177. */
int emh_module_load(const void* code, size_t code_len, void** module);
int emh_module_unload(void* module);

/* Look up an extern "C" kernel by name.  Replaces RawModule.get_function,
 * emmy/compiler/backend/cuda/nvcc.py:177. */
int emh_get_function(void* module, const char* name, void** fn);

/* Allow `fn` to be launched with up to `bytes` of dynamic LDS (needed above
 * the 64 KiB default).  Replaces _ensure_dynamic_smem_attr,
 * emmy/compiler/backend/cuda/program.py:48. */
int emh_func_set_dynamic_lds(void* fn, int bytes);

/* Static resource usage of `fn`: vector registers per lane, static LDS bytes,
 * private (spill) bytes per lane and the launch-bounds thread cap.  Any out
 * pointer may be NULL.  Replaces the cupy kernel-attribute reads of
 * emmy/commands/run.py:606-667 (_print_kernel_stats). */
int emh_func_attributes(void* fn, int* num_regs, int* static_lds_bytes, int* private_bytes,
                        int* max_threads);

/* Launch ------------------------------------------------------------------- */

/* Launch `fn` on `stream`.  `args` holds `nargs` pointers, each to the storage
 * of one kernel parameter, in signature order: device pointers first, then
 * `int` runtime values.  Geometry is validated (non-zero, block <= 1024
 * threads) before the driver is called.  Replaces _launch,
 * emmy/compiler/backend/cuda/program.py:394-424. */
int emh_launch(void* fn, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
               void* stream, void** args, int nargs);

/* Largest workspace (bytes) emh_launch_scratch can lend a kernel. */
#define EMH_SCRATCH_MAX_BYTES (16u * 1024u * 1024u)

/* emh_launch with the kernel's workspace lent by the library — an entry point
 * that allocates nothing.  It has no counterpart in the reference (whose
 * runtime allocates every buffer through cupy); it is for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Kernels that need device memory beyond
 * their inputs and outputs — the fp32 partial planes of a split contraction
 * (partial kernel writes them, combine kernel folds them) — take that
 * workspace as one pointer parameter; here parameter number `scratch_arg`
 * (0-based, a device-pointer slot of `args`) is pointed at byte
 * `scratch_offset` of a file-scope device array of EMH_SCRATCH_MAX_BYTES that
 * every GPU the library runs on holds until the process ends; the value the
 * caller stored in that slot is ignored and `args` is not modified.  With
 * `zero_first` the `scratch_bytes` bytes from the offset are cleared on
 * `stream` by a fill kernel first (never hipMemsetAsync: the call may be
 * under capture).  Everything else is emh_launch.  Fails, launching nothing,
 * when scratch_offset + scratch_bytes exceeds EMH_SCRATCH_MAX_BYTES, when
 * the offset is not a multiple of 256 or the size not a multiple of 4, or
 * when scratch_arg is not a slot of `args`.  Calls no hipMalloc / hipFree.
 * All calls on one GPU share that GPU's array and it keeps the last call's
 * contents: calls that overlap in time on one GPU (two streams, two threads)
 * race on it, and a kernel that accumulates must ask for zero_first.
 * The array used is the one of the calling thread's *current* device
 * (hipGetDevice), not of the device `stream` was created on: make the
 * stream's device current before the call, as for emh_launch itself. */
int emh_launch_scratch(void* fn, const unsigned grid[3], const unsigned block[3],
                       unsigned lds_bytes, void* stream, void** args, int nargs, int scratch_arg,
                       size_t scratch_offset, size_t scratch_bytes, int zero_first);

/* Asynchronous byte fill of device memory on `stream`.  Replaces the
 * zero_outputs fill of emmy/compiler/backend/cuda/program.py:403-404.  Must
 * not be called while `stream` is being captured into a graph (use a fill
 * kernel there). */
int emh_memset_async(void* dptr, int value, size_t bytes, void* stream);

/* Streams ------------------------------------------------------------------- */

/* A non-blocking stream of default priority (graph capture cannot run on the
 * legacy default stream).  Replaces cp.cuda.Stream(non_blocking=True),
 * emmy/compiler/backend/cuda/program.py:1152-1325. */
int emh_stream_create(void** stream);
int emh_stream_destroy(void* stream);
int emh_stream_synchronize(void* stream);

/* Events ------------------------------------------------------------------- */

/* Timing events.  Replace cp.cuda.Event / get_elapsed_time,
 * emmy/compiler/backend/cuda/program.py:574-611 and :960-1036. */
int emh_event_create(void** event);
int emh_event_record(void* event, void* stream);
int emh_event_synchronize(void* event);
/* *done = 1 when the event has completed, 0 while it is pending (the watchdog
 * polls this instead of blocking). */
int emh_event_query(void* event, int* done);
int emh_event_elapsed_ms(void* start, void* stop, float* ms);
int emh_event_destroy(void* event);

/* Graphs ------------------------------------------------------------------- */

/* Capture every launch issued on `stream` between begin and end into an
 * executable graph, and replay it.  Replace the stream-capture / graph-launch
 * use of emmy/compiler/backend/cuda/program.py:843-907 and :1152-1325. */
int emh_graph_begin_capture(void* stream);
int emh_graph_end_capture(void* stream, void** graph_exec);
int emh_graph_launch(void* graph_exec, void* stream);
int emh_graph_destroy(void* graph_exec);

/* Errors ------------------------------------------------------------------- */

/* Message for the calling thread's most recent failing call ("" if none).
 * The pointer stays valid until the next failing call on this thread. */
const char* emh_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* EMMY_HIP_H */
