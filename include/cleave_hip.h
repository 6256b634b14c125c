/*
 * cleave_hip.h - C ABI of libcleave_hip.so, the MI355X (gfx950) back end's
 * compile / load / launch / time boundary.
 *
 * The reference has no C FFI on this path: its runtime hands generated source
 * text to a third-party JIT and gets a Python callable back
 * (python/cleave/runtime/compile.py:30-58, `_compile` and
 * `_load_main_kernel_from_code`), times it with CUDA events and graph replay
 * through torch (python/cleave/runtime/timer.py:14-108) and reads device
 * limits through a ctypes binding of the CUDA runtime
 * (python/cleave/arch/driver/cuda_driver.py:80-218).  Each entry point below
 * names the reference interface it stands in for.
 *
 * Conventions
 *   - every function returns 0 on success, otherwise a non-zero code; the
 *     text of the failure is available from chip_last_error() on the calling
 *     thread until that thread's next call into the library;
 *   - nothing here throws, allocates device memory for the caller's tensors,
 *     or touches torch: buffers are plain device pointers owned by the caller;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - handles (`chip_module`, `chip_function`) are opaque pointers owned by
 *     the library until chip_module_unload().
 */
#ifndef CLEAVE_HIP_H
#define CLEAVE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CHIP_ABI_VERSION 1

/* Error classes returned by every entry point (0 = success). */
enum chip_status {
  CHIP_OK = 0,
  CHIP_ERR_INVALID = 1,   /* bad argument (null pointer, bad size) */
  CHIP_ERR_COMPILE = 2,   /* hiprtc rejected the source; see the log */
  CHIP_ERR_RUNTIME = 3,   /* a HIP runtime call failed */
  CHIP_ERR_LDS = 4        /* requested LDS exceeds the device limit */
};

/* Device limits the schedule search is derived from.  Replaces the
 * cudaDeviceProp fields read at python/cleave/arch/driver/cuda_driver.py:80-218
 * and the constants at python/cleave/arch/cuda.py:121-183. */
typedef struct chip_device_info {
  int32_t abi_version;
  int32_t device;
  int32_t compute_units;          /* 256 on MI355X */
  int32_t wavefront_size;         /* 64 */
  int32_t max_threads_per_block;  /* 1024 */
  int32_t lds_bytes_per_block;    /* opt-in maximum, 160 KiB on gfx950 */
  int32_t regs_per_block;
  int32_t clock_khz;
  int32_t memory_clock_khz;
  int32_t memory_bus_bits;
  int32_t l2_bytes;
  int32_t reserved0;
  uint64_t total_memory_bytes;
  char arch_name[64];             /* e.g. "gfx950:sramecc+:xnack-" */
  char name[128];
  char uuid[40];                  /* hex of hipUUID; keys the per-GPU lock file
                                     (python/cleave/runtime/gpu.py:15-38) */
} chip_device_info;

/* ABI version of the loaded library.  Has no counterpart in the reference
 * (its boundary is Python objects, never a versioned binary interface). */
int chip_abi_version(void);

/* Last failure text on this thread ("" if none). Never NULL.  Carries what
 * the reference gets as a Python exception out of its JIT and classifies at
 * python/cleave/runtime/evaluate.py:107-133. */
const char* chip_last_error(void);

/* Number of visible HIP devices, or a negative chip_status.  Stands in for
 * the device enumeration behind python/cleave/runtime/gpu.py:15-38. */
int chip_device_count(void);

/* Fill `info` for device `dev`.  Stands in for get_cuda_device_properties and
 * the attribute getters at python/cleave/arch/driver/cuda_driver.py:80-218. */
int chip_device_info_get(int dev, chip_device_info* info);

/* Compile HIP source text for `arch` (e.g. "gfx950") with hiprtc.
 * Stands in for `tl.compile` at python/cleave/runtime/compile.py:30-34.
 *   opts/nopts : extra compiler options (may be NULL/0)
 *   code/size  : receives a malloc'd code object; free with chip_free
 *   log        : receives a malloc'd NUL-terminated compiler log (may be
 *                empty); free with chip_free.  Filled on failure too.
 * Needs no GPU: the code object can be built on a host without one. */
int chip_compile(const char* source, const char* name, const char* arch,
                 const char* const* opts, int nopts,
                 void** code, size_t* size, char** log);

/* Release memory returned by chip_compile.  Has no counterpart in the
 * reference (the JIT's kernel object owns its binary there). */
void chip_free(void* p);

/* Load a code object on the current device.  Second half of what `tl.compile`
 * returns at python/cleave/runtime/compile.py:30-34 (a loaded, callable
 * kernel); kept separate so compile can run on a GPU-less host. */
int chip_module_load(const void* code, size_t size, void** module);

/* Unload a module and every function handle obtained from it.  Stands in
 * for dropping the JIT kernel in the worker's per-task cleanup
 * (python/cleave/runtime/workers.py:93-101). */
int chip_module_unload(void* module);

/* Look up an `extern "C" __global__` entry by name: `main_kernel`, the entry
 * the reference loads at python/cleave/runtime/compile.py:37-58. */
int chip_get_function(void* module, const char* name, void** fn);

/* Static resource usage of a kernel (for occupancy-aware ranking and spill
 * detection).  Has no counterpart in the reference, which learns of register
 * or shared-memory overflow only from the launch failure markers at
 * python/cleave/runtime/evaluate.py:96-104. */
typedef struct chip_func_attr {
  int32_t num_regs;           /* VGPRs per lane */
  int32_t static_lds_bytes;
  int32_t scratch_bytes;      /* private (spill) bytes per lane */
  int32_t max_threads_per_block;
} chip_func_attr;
int chip_function_attributes(void* fn, chip_func_attr* out);

/* Launch `fn`.  `args` is an array of `nargs` pointers to the argument
 * values, exactly as hipModuleLaunchKernel takes them.  `lds_bytes` is the
 * dynamic LDS size; values above 64 KiB are opted into here, and a request
 * beyond the device limit returns CHIP_ERR_LDS (the counterpart of the
 * reference's "Failed to set the allowed dynamic shared memory size" marker,
 * python/cleave/runtime/evaluate.py:96). */
int chip_launch(void* fn, const uint32_t grid[3], const uint32_t block[3],
                uint32_t lds_bytes, void* stream, void** args, int nargs);

/* One launch of a multi-kernel sequence (a split partial + its combine). */
typedef struct chip_launch_desc {
  void* fn;
  uint32_t grid[3];
  uint32_t block[3];
  uint32_t lds_bytes;
  int32_t nargs;
  void** args;
} chip_launch_desc;

/* Enqueue `n` launches back to back on `stream`.  Stands in for the kernel
 * call inside the reference's fused partial+combine `main_kernel`
 * (python/cleave/codegen/split.py:78-125) and for `kernel(*args)` at
 * python/cleave/runtime/timer.py:66-73. */
int chip_launch_seq(const chip_launch_desc* seq, int n, void* stream);

/* Bytes of the fixed scratch array each GPU holds for chip_launch_seq_fixed_scratch. */
#define CHIP_FIXED_SCRATCH_BYTES (64ull << 20)

/* Names one pointer argument of a launch sequence that is to point into the
 * fixed scratch array: argument `arg` of launch `launch`, at byte `offset`
 * (a multiple of 256) from the array's start. */
typedef struct chip_scratch_arg {
  int32_t launch;
  int32_t arg;
  uint64_t offset;
} chip_scratch_arg;

/* chip_launch_seq for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * Has no counterpart in the reference, whose callers always allocate the
 * split partials (python/cleave/runtime/autotune.py:164-227).  The scratch
 * buffers of the sequence -- the split partials a partial kernel writes and
 * its combine reads -- live in a fixed array of CHIP_FIXED_SCRATCH_BYTES that
 * is part of the library and is held by every GPU the library runs on until
 * the process ends; inputs and outputs are still the caller's.  For each of
 * the `nrefs` entries of `refs` the named argument is launched with the
 * address `array + offset` (whatever the caller's slot holds is ignored and
 * left untouched); `scratch_bytes` is the extent the caller's layout uses.
 *   - scratch_bytes above CHIP_FIXED_SCRATCH_BYTES, an offset that is not a
 *     multiple of 256 or lies outside scratch_bytes, more than 8 launches,
 *     64 arguments per launch or 64 entries in `refs`, or two entries that
 *     name the same argument: CHIP_ERR_INVALID, nothing is launched (every
 *     check runs before the fill kernel and the first launch);
 *   - the call makes no hipMalloc / hipFree and no other allocating call;
 *   - all calls on one GPU share that GPU's array and it keeps the previous
 *     call's contents: `clear` != 0 zeroes the first scratch_bytes with a fill
 *     kernel on `stream` before the first launch (for kernels that accumulate
 *     into scratch; kernels that write every element they later read need no
 *     clear); calls that overlap in time on one GPU race on the array. */
int chip_launch_seq_fixed_scratch(const chip_launch_desc* seq, int n, void* stream,
                                  const chip_scratch_arg* refs, int nrefs,
                                  uint64_t scratch_bytes, int clear);

/* Time the sequence: `warmup` untimed passes, then `iters` passes between two
 * hipEvents recorded on `stream`; *ms_per_iter = elapsed / iters.  When
 * `nsets` > 1, `arg_sets` holds nsets*n alternative `args` arrays (set-major)
 * and pass i uses set i % nsets, so a working set larger than the last-level
 * cache can be rotated through.  `arg_sets` may be NULL when nsets <= 1.
 * Stands in for `mean_launch_ms` / `replay_rounds`
 * (python/cleave/runtime/timer.py:51-108): the loop runs inside the library,
 * so no host-language dispatch sits in the timed region. */
int chip_time_launches(const chip_launch_desc* seq, int n, void* stream,
                       int warmup, int iters, int nsets, void*** arg_sets,
                       float* ms_per_iter);

/* The same measurement taken the way the reference takes it
 * (`capture_launch_graph` / `replay_rounds`, python/cleave/runtime/timer.py:14-73):
 * `warmup` eager passes, then `batch` passes of the sequence are captured into
 * one HIP graph (kernel nodes only) and the graph is replayed `rounds` times
 * between two hipEvents; *ms_per_iter = elapsed / (rounds * batch).  Capture and
 * replay run on a stream this call creates (default priority) after draining
 * `stream`, because the legacy default stream cannot be captured; the call
 * returns with that stream drained and destroyed.  Argument rotation as in
 * chip_time_launches (pass i of the batch uses set i % nsets). */
int chip_time_graph(const chip_launch_desc* seq, int n, void* stream,
                    int warmup, int batch, int rounds, int nsets,
                    void*** arg_sets, float* ms_per_iter);

#ifdef __cplusplus
}
#endif
#endif /* CLEAVE_HIP_H */
