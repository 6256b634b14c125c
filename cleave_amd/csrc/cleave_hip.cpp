// libcleave_hip.so: hiprtc compile, module load, launch and event timing behind a C ABI.
// The operators' kernels are generated source text compiled at run time; the only device code in
// this file is the fixed scratch array of chip_launch_seq_fixed_scratch and its fill kernel.
#include "cleave_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(int status, const std::string& text) {
  g_error = text;
  return status;
}

int hip_fail(const char* what, hipError_t e) {
  return fail(CHIP_ERR_RUNTIME, std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")");
}

#define HIP_TRY(call)                                  \
  do {                                                 \
    hipError_t e_ = (call);                            \
    if (e_ != hipSuccess) return hip_fail(#call, e_);  \
  } while (0)

struct Module {
  hipModule_t handle = nullptr;
};

// The largest dynamic LDS a kernel may ask for on `dev` (cached per device).
int lds_limit(int dev, int* out) {
  static std::mutex mu;
  static int cached[64];
  static bool known[64];
  std::lock_guard<std::mutex> lock(mu);
  if (dev >= 0 && dev < 64 && known[dev]) {
    *out = cached[dev];
    return CHIP_OK;
  }
  int optin = 0, plain = 0;
  hipError_t e = hipDeviceGetAttribute(&plain, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
  if (e != hipSuccess) return hip_fail("hipDeviceGetAttribute(MaxSharedMemoryPerBlock)", e);
  e = hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, dev);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    optin = 0;
  }
  int lim = optin > plain ? optin : plain;
  if (dev >= 0 && dev < 64) {
    cached[dev] = lim;
    known[dev] = true;
  }
  *out = lim;
  return CHIP_OK;
}

int launch_one(const chip_launch_desc& d, void** args, hipStream_t stream) {
  if (!d.fn) return fail(CHIP_ERR_INVALID, "chip_launch: null function");
  for (int i = 0; i < 3; ++i) {
    if (d.grid[i] == 0 || d.block[i] == 0)
      return fail(CHIP_ERR_INVALID, "chip_launch: zero grid or block extent");
  }
  if ((uint64_t)d.block[0] * d.block[1] * d.block[2] > 1024)
    return fail(CHIP_ERR_INVALID, "chip_launch: more than 1024 threads per block");
  hipFunction_t f = reinterpret_cast<hipFunction_t>(d.fn);
  if (d.lds_bytes > 64 * 1024) {
    int dev = 0, lim = 0;
    HIP_TRY(hipGetDevice(&dev));
    int rc = lds_limit(dev, &lim);
    if (rc) return rc;
    if ((int)d.lds_bytes > lim) {
      char buf[160];
      snprintf(buf, sizeof buf, "LDS limit exceeded: kernel asks for %u bytes, device allows %d", d.lds_bytes, lim);
      return fail(CHIP_ERR_LDS, buf);
    }
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(f),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)d.lds_bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      char buf[160];
      snprintf(buf, sizeof buf, "LDS limit exceeded: could not opt in to %u bytes of dynamic LDS (%s)",
               d.lds_bytes, hipGetErrorName(e));
      return fail(CHIP_ERR_LDS, buf);
    }
  }
  HIP_TRY(hipModuleLaunchKernel(f, d.grid[0], d.grid[1], d.grid[2], d.block[0], d.block[1], d.block[2],
                                d.lds_bytes, stream, args, nullptr));
  return CHIP_OK;
}

}  // namespace

// ---- fixed scratch: device memory for callers that cannot allocate ---------------------------
// One array per GPU, part of this library's code object, held until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress: the device address it resolves
// to (one per GPU) is what kernels, and the fill below, are given.
static __device__ __align__(256) unsigned char scratch[CHIP_FIXED_SCRATCH_BYTES];

static __global__ void __launch_bounds__(256) chip_scratch_fill_zero(uint4* p, unsigned long long n16) {
  unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x;
  const unsigned long long stride = (unsigned long long)gridDim.x * 256;
  for (; i < n16; i += stride) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

namespace {

constexpr int kMaxDevices = 64;
constexpr int kMaxSeq = 8;          // launches per call of the fixed-scratch entry point
constexpr int kMaxArgs = 64;        // arguments per launch there
constexpr int kMaxScratchRefs = 64; // scratch arguments per call there

// Device address of `scratch` on the current device, resolved once per device with that device
// current (every GPU holds its own copy of the array at its own address).
int fixed_scratch_ptr(unsigned char** out) {
  static std::mutex mu;
  static unsigned char* ptrs[kMaxDevices];
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(CHIP_ERR_INVALID, "fixed scratch: device index out of range");
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    unsigned char* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
    if (!p) return fail(CHIP_ERR_RUNTIME, "fixed scratch: hipGetSymbolAddress returned a null address");
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return CHIP_OK;
}

}  // namespace

extern "C" {

int chip_abi_version(void) { return CHIP_ABI_VERSION; }

const char* chip_last_error(void) { return g_error.c_str(); }

int chip_device_count(void) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    hip_fail("hipGetDeviceCount", e);
    return -CHIP_ERR_RUNTIME;
  }
  return n;
}

int chip_device_info_get(int dev, chip_device_info* info) {
  if (!info) return fail(CHIP_ERR_INVALID, "chip_device_info_get: null info");
  hipDeviceProp_t p;
  HIP_TRY(hipGetDeviceProperties(&p, dev));
  std::memset(info, 0, sizeof *info);
  info->abi_version = CHIP_ABI_VERSION;
  info->device = dev;
  info->compute_units = p.multiProcessorCount;
  info->wavefront_size = p.warpSize;
  info->max_threads_per_block = p.maxThreadsPerBlock;
  int lim = 0;
  int rc = lds_limit(dev, &lim);
  if (rc) return rc;
  info->lds_bytes_per_block = lim;
  info->regs_per_block = p.regsPerBlock;
  info->clock_khz = p.clockRate;
  info->memory_clock_khz = p.memoryClockRate;
  info->memory_bus_bits = p.memoryBusWidth;
  info->l2_bytes = p.l2CacheSize;
  info->total_memory_bytes = p.totalGlobalMem;
  snprintf(info->arch_name, sizeof info->arch_name, "%s", p.gcnArchName);
  snprintf(info->name, sizeof info->name, "%s", p.name);
  hipUUID id;
  if (hipDeviceGetUuid(&id, dev) == hipSuccess) {
    static const char* hex = "0123456789abcdef";
    for (int i = 0; i < 16; ++i) {
      unsigned char c = (unsigned char)id.bytes[i];
      info->uuid[2 * i] = hex[c >> 4];
      info->uuid[2 * i + 1] = hex[c & 15];
    }
    info->uuid[32] = 0;
  } else {
    (void)hipGetLastError();
  }
  return CHIP_OK;
}

int chip_compile(const char* source, const char* name, const char* arch, const char* const* opts, int nopts,
                 void** code, size_t* size, char** log) {
  if (log) *log = nullptr;
  if (!source || !code || !size) return fail(CHIP_ERR_INVALID, "chip_compile: null source/code/size");
  *code = nullptr;
  *size = 0;
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail(CHIP_ERR_COMPILE, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
  std::string archopt = std::string("--offload-arch=") + (arch && *arch ? arch : "gfx950");
  std::vector<const char*> all;
  all.push_back(archopt.c_str());
  for (int i = 0; i < nopts; ++i)
    if (opts && opts[i]) all.push_back(opts[i]);
  r = hiprtcCompileProgram(prog, (int)all.size(), all.data());
  size_t log_size = 0;
  hiprtcGetProgramLogSize(prog, &log_size);
  std::string text(log_size, '\0');
  if (log_size) hiprtcGetProgramLog(prog, &text[0]);
  while (!text.empty() && text.back() == '\0') text.pop_back();
  if (log) {
    *log = (char*)std::malloc(text.size() + 1);
    if (*log) std::memcpy(*log, text.c_str(), text.size() + 1);
  }
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return fail(CHIP_ERR_COMPILE, std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + text);
  }
  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r != HIPRTC_SUCCESS || n == 0) {
    hiprtcDestroyProgram(&prog);
    return fail(CHIP_ERR_COMPILE, "hiprtcGetCodeSize: no code object produced");
  }
  void* buf = std::malloc(n);
  if (!buf) {
    hiprtcDestroyProgram(&prog);
    return fail(CHIP_ERR_INVALID, "chip_compile: out of host memory");
  }
  r = hiprtcGetCode(prog, (char*)buf);
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    std::free(buf);
    return fail(CHIP_ERR_COMPILE, std::string("hiprtcGetCode: ") + hiprtcGetErrorString(r));
  }
  *code = buf;
  *size = n;
  return CHIP_OK;
}

void chip_free(void* p) { std::free(p); }

int chip_module_load(const void* code, size_t size, void** module) {
  if (!code || !size || !module) return fail(CHIP_ERR_INVALID, "chip_module_load: null code/module");
  *module = nullptr;
  Module* m = new Module();
  hipError_t e = hipModuleLoadData(&m->handle, code);
  if (e != hipSuccess) {
    delete m;
    return hip_fail("hipModuleLoadData", e);
  }
  *module = m;
  // Set-up of the fixed scratch array for this device happens here, with the device current: every
  // function handle a caller can launch comes out of a module loaded on its device, so the
  // fixed-scratch entry point finds the address resolved.  (It resolves it itself otherwise.)
  unsigned char* unused = nullptr;
  std::string kept = g_error;
  if (fixed_scratch_ptr(&unused) != CHIP_OK) {
    (void)hipGetLastError();
    g_error = kept;
  }
  return CHIP_OK;
}

int chip_module_unload(void* module) {
  if (!module) return CHIP_OK;
  Module* m = static_cast<Module*>(module);
  hipError_t e = hipModuleUnload(m->handle);
  delete m;
  if (e != hipSuccess) return hip_fail("hipModuleUnload", e);
  return CHIP_OK;
}

int chip_get_function(void* module, const char* name, void** fn) {
  if (!module || !name || !fn) return fail(CHIP_ERR_INVALID, "chip_get_function: null argument");
  *fn = nullptr;
  hipFunction_t f = nullptr;
  hipError_t e = hipModuleGetFunction(&f, static_cast<Module*>(module)->handle, name);
  if (e != hipSuccess) return hip_fail((std::string("hipModuleGetFunction(") + name + ")").c_str(), e);
  *fn = f;
  return CHIP_OK;
}

int chip_function_attributes(void* fn, chip_func_attr* out) {
  if (!fn || !out) return fail(CHIP_ERR_INVALID, "chip_function_attributes: null argument");
  hipFunction_t f = reinterpret_cast<hipFunction_t>(fn);
  int v = 0;
  HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, f));
  out->num_regs = v;
  HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f));
  out->static_lds_bytes = v;
  HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f));
  out->scratch_bytes = v;
  HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f));
  out->max_threads_per_block = v;
  return CHIP_OK;
}

int chip_launch(void* fn, const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes, void* stream,
                void** args, int nargs) {
  if (!grid || !block) return fail(CHIP_ERR_INVALID, "chip_launch: null grid/block");
  if (nargs > 0 && !args) return fail(CHIP_ERR_INVALID, "chip_launch: null args");
  chip_launch_desc d;
  d.fn = fn;
  for (int i = 0; i < 3; ++i) {
    d.grid[i] = grid[i];
    d.block[i] = block[i];
  }
  d.lds_bytes = lds_bytes;
  d.nargs = nargs;
  d.args = args;
  return launch_one(d, args, static_cast<hipStream_t>(stream));
}

int chip_launch_seq(const chip_launch_desc* seq, int n, void* stream) {
  if (!seq || n <= 0) return fail(CHIP_ERR_INVALID, "chip_launch_seq: empty sequence");
  for (int i = 0; i < n; ++i) {
    int rc = launch_one(seq[i], seq[i].args, static_cast<hipStream_t>(stream));
    if (rc) return rc;
  }
  return CHIP_OK;
}

int chip_launch_seq_fixed_scratch(const chip_launch_desc* seq, int n, void* stream, const chip_scratch_arg* refs,
                                  int nrefs, uint64_t scratch_bytes, int clear) {
  if (!seq || n <= 0) return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: empty sequence");
  if (n > kMaxSeq) return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: more than 8 launches in one call");
  if (nrefs < 0 || (nrefs > 0 && !refs)) return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: bad scratch argument list");
  if (nrefs > kMaxScratchRefs) return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: more than 64 scratch arguments");
  if (scratch_bytes > CHIP_FIXED_SCRATCH_BYTES) {
    char buf[200];
    snprintf(buf, sizeof buf, "chip_launch_seq_fixed_scratch: %llu bytes of scratch asked for, the fixed array holds %llu",
             (unsigned long long)scratch_bytes, (unsigned long long)CHIP_FIXED_SCRATCH_BYTES);
    return fail(CHIP_ERR_INVALID, buf);
  }
  for (int i = 0; i < n; ++i)
    if (seq[i].nargs < 0 || seq[i].nargs > kMaxArgs || (seq[i].nargs > 0 && !seq[i].args))
      return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: a launch has no argument array or more than 64 arguments");
  for (int r = 0; r < nrefs; ++r) {
    const chip_scratch_arg& a = refs[r];
    if (a.launch < 0 || a.launch >= n || a.arg < 0 || a.arg >= seq[a.launch].nargs)
      return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: scratch argument names no argument of the sequence");
    if (a.offset % 256 || a.offset >= scratch_bytes)
      return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: scratch offset not a multiple of 256 or outside scratch_bytes");
    for (int q = 0; q < r; ++q)
      if (refs[q].launch == a.launch && refs[q].arg == a.arg)
        return fail(CHIP_ERR_INVALID, "chip_launch_seq_fixed_scratch: one argument is named by two scratch entries");
  }
  unsigned char* base = nullptr;
  int rc = fixed_scratch_ptr(&base);
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (clear && scratch_bytes) {
    // a fill kernel, not hipMemsetAsync: callers may be recording this stream into a graph
    const unsigned long long n16 = (scratch_bytes + 15) / 16;
    unsigned blocks = (unsigned)((n16 + 255) / 256);
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(chip_scratch_fill_zero, dim3(blocks), dim3(256), 0, s, reinterpret_cast<uint4*>(base), n16);
    HIP_TRY(hipGetLastError());
  }
  // the caller's argument arrays are left as they are: each launch gets a copy of its pointer
  // array (on this stack) whose scratch slots point at addresses inside the fixed array
  void* values[kMaxScratchRefs];
  int used = 0;
  for (int i = 0; i < n; ++i) {
    void* args[kMaxArgs];
    for (int j = 0; j < seq[i].nargs; ++j) args[j] = seq[i].args[j];
    for (int r = 0; r < nrefs; ++r) {
      if (refs[r].launch != i) continue;
      values[used] = base + refs[r].offset;
      args[refs[r].arg] = &values[used++];
    }
    rc = launch_one(seq[i], args, s);
    if (rc) return rc;
  }
  return CHIP_OK;
}

int chip_time_launches(const chip_launch_desc* seq, int n, void* stream, int warmup, int iters, int nsets,
                       void*** arg_sets, float* ms_per_iter) {
  if (!seq || n <= 0 || !ms_per_iter) return fail(CHIP_ERR_INVALID, "chip_time_launches: bad sequence or output");
  if (iters <= 0 || warmup < 0) return fail(CHIP_ERR_INVALID, "chip_time_launches: iters must be > 0 and warmup >= 0");
  if (nsets > 1 && !arg_sets) return fail(CHIP_ERR_INVALID, "chip_time_launches: nsets > 1 needs arg_sets");
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto pass = [&](int it) -> int {
    for (int i = 0; i < n; ++i) {
      void** args = seq[i].args;
      if (nsets > 1) args = arg_sets[(size_t)(it % nsets) * n + i];
      int rc = launch_one(seq[i], args, s);
      if (rc) return rc;
    }
    return CHIP_OK;
  };
  for (int it = 0; it < warmup; ++it) {
    int rc = pass(it);
    if (rc) return rc;
  }
  hipEvent_t t0, t1;
  HIP_TRY(hipEventCreate(&t0));
  hipError_t e = hipEventCreate(&t1);
  if (e != hipSuccess) {
    (void)hipEventDestroy(t0);
    return hip_fail("hipEventCreate", e);
  }
  int rc = CHIP_OK;
  e = hipEventRecord(t0, s);
  if (e != hipSuccess) rc = hip_fail("hipEventRecord", e);
  for (int it = 0; rc == CHIP_OK && it < iters; ++it) rc = pass(warmup + it);
  if (rc == CHIP_OK) {
    e = hipEventRecord(t1, s);
    if (e != hipSuccess) rc = hip_fail("hipEventRecord", e);
  }
  if (rc == CHIP_OK) {
    e = hipEventSynchronize(t1);
    if (e != hipSuccess) rc = hip_fail("hipEventSynchronize", e);
  }
  float ms = 0.f;
  if (rc == CHIP_OK) {
    e = hipEventElapsedTime(&ms, t0, t1);
    if (e != hipSuccess) rc = hip_fail("hipEventElapsedTime", e);
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc == CHIP_OK) *ms_per_iter = ms / (float)iters;
  return rc;
}

int chip_time_graph(const chip_launch_desc* seq, int n, void* stream, int warmup, int batch, int rounds, int nsets,
                    void*** arg_sets, float* ms_per_iter) {
  if (!seq || n <= 0 || !ms_per_iter) return fail(CHIP_ERR_INVALID, "chip_time_graph: bad sequence or output");
  if (batch <= 0 || rounds <= 0 || warmup < 0)
    return fail(CHIP_ERR_INVALID, "chip_time_graph: batch and rounds must be > 0 and warmup >= 0");
  if (nsets > 1 && !arg_sets) return fail(CHIP_ERR_INVALID, "chip_time_graph: nsets > 1 needs arg_sets");
  hipStream_t caller = static_cast<hipStream_t>(stream);
  // Work queued on the caller's stream comes first; capture and replay then run on a stream of
  // this call's own (the legacy default stream cannot be captured), at the default priority.
  HIP_TRY(hipStreamSynchronize(caller));
  hipStream_t s = nullptr;
  HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  hipEvent_t t0 = nullptr, t1 = nullptr;
  int rc = CHIP_OK;
  auto pass = [&](int it) -> int {
    for (int i = 0; i < n; ++i) {
      void** args = seq[i].args;
      if (nsets > 1) args = arg_sets[(size_t)(it % nsets) * n + i];
      int r = launch_one(seq[i], args, s);
      if (r) return r;
    }
    return CHIP_OK;
  };
  auto step = [&](const char* what, hipError_t e) {
    if (rc == CHIP_OK && e != hipSuccess) rc = hip_fail(what, e);
  };
  for (int it = 0; rc == CHIP_OK && it < warmup; ++it) rc = pass(it);
  step("hipStreamSynchronize", hipStreamSynchronize(s));
  if (rc == CHIP_OK) {
    // only kernel launches are recorded: no memset or copy nodes
    step("hipStreamBeginCapture", hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    if (rc == CHIP_OK) {
      int prc = CHIP_OK;
      for (int it = 0; prc == CHIP_OK && it < batch; ++it) prc = pass(warmup + it);
      hipError_t e = hipStreamEndCapture(s, &graph);   // always end the capture, also after a failed launch
      if (prc != CHIP_OK) rc = prc;
      step("hipStreamEndCapture", e);
    }
  }
  if (rc == CHIP_OK) step("hipGraphInstantiate", hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  if (rc == CHIP_OK) step("hipGraphLaunch", hipGraphLaunch(exec, s));          // one untimed replay
  step("hipStreamSynchronize", hipStreamSynchronize(s));
  if (rc == CHIP_OK) step("hipEventCreate", hipEventCreate(&t0));
  if (rc == CHIP_OK) step("hipEventCreate", hipEventCreate(&t1));
  if (rc == CHIP_OK) step("hipEventRecord", hipEventRecord(t0, s));
  for (int r = 0; rc == CHIP_OK && r < rounds; ++r) step("hipGraphLaunch", hipGraphLaunch(exec, s));
  if (rc == CHIP_OK) step("hipEventRecord", hipEventRecord(t1, s));
  if (rc == CHIP_OK) step("hipEventSynchronize", hipEventSynchronize(t1));
  float ms = 0.f;
  if (rc == CHIP_OK) step("hipEventElapsedTime", hipEventElapsedTime(&ms, t0, t1));
  (void)hipStreamSynchronize(s);
  if (t0) (void)hipEventDestroy(t0);
  if (t1) (void)hipEventDestroy(t1);
  if (exec) (void)hipGraphExecDestroy(exec);
  if (graph) (void)hipGraphDestroy(graph);
  (void)hipStreamDestroy(s);
  if (rc == CHIP_OK) *ms_per_iter = ms / ((float)rounds * (float)batch);
  return rc;
}

}  // extern "C"
