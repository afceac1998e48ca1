// libemmy_hip.so — C-ABI kernel launcher for gfx950 (see include/emmy_hip.h).
//
// C++ over hipRTC and the HIP module API, built with hipcc for gfx950.  Kernels
// arrive as source text from the Python emitter; the only device code here is
// the scratch array emh_launch_scratch lends to kernels and the kernel that
// clears it.  The library allocates no device memory and starts no threads.
#include "emmy_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

// Workspace lent to kernels by emh_launch_scratch.  In host code this name is a
// stand-in, not a device address: the per-device address comes from
// hipGetSymbolAddress (scratch_base below) and only that is ever handed on.
static __device__ __align__(256) unsigned char emh_scratch[EMH_SCRATCH_MAX_BYTES];

__global__ void __launch_bounds__(256) emh_scratch_zero_words(unsigned int* __restrict__ p, size_t words) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += (size_t)gridDim.x * 256) p[i] = 0u;
}

namespace {

thread_local std::string g_last_error;

int fail_hip(hipError_t e, const char* what) {
  g_last_error = std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")";
  // Clear the sticky per-thread error so the next unrelated call is not blamed.
  (void)hipGetLastError();
  return static_cast<int>(e) == 0 ? -1 : static_cast<int>(e);
}

int fail_rtc(hiprtcResult r, const char* what) {
  g_last_error = std::string(what) + ": " + hiprtcGetErrorString(r);
  return EMH_RTC_ERROR_BASE + static_cast<int>(r);
}

int fail_arg(const char* what) {
  g_last_error = what;
  return static_cast<int>(hipErrorInvalidValue);
}

#define EMH_HIP(call)                               \
  do {                                              \
    hipError_t e_ = (call);                         \
    if (e_ != hipSuccess) return fail_hip(e_, #call); \
  } while (0)

// Address of emh_scratch on the current device, looked up once per device (each GPU holds its
// own copy of the array at its own address).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char* g_scratch_base[kMaxDevices] = {};

int scratch_base(unsigned char** out) {
  int dev = -1;
  EMH_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail_arg("emh_launch_scratch: device index out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_base[dev]) {
    void* p = nullptr;
    EMH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(emh_scratch)));
    if (!p) return fail_arg("emh_launch_scratch: the scratch array has no address on this device");
    g_scratch_base[dev] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_base[dev];
  return 0;
}

}  // namespace

extern "C" {

int emh_abi_version(void) { return EMH_ABI_VERSION; }

int emh_device_count(int* count) {
  if (!count) return fail_arg("emh_device_count: count is NULL");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e == hipErrorNoDevice || e == hipErrorInsufficientDriver) {
    (void)hipGetLastError();
    *count = 0;
    return 0;
  }
  if (e != hipSuccess) return fail_hip(e, "hipGetDeviceCount");
  *count = n;
  return 0;
}

int emh_device_props(int device, char* arch, size_t arch_len, int* compute_units,
                     int* lds_bytes_per_block, int* wavefront_size, int* clock_khz,
                     size_t* global_mem_bytes) {
  hipDeviceProp_t p;
  EMH_HIP(hipGetDeviceProperties(&p, device));
  if (arch && arch_len) {
    std::snprintf(arch, arch_len, "%s", p.gcnArchName);
  }
  if (compute_units) *compute_units = p.multiProcessorCount;
  if (lds_bytes_per_block) *lds_bytes_per_block = static_cast<int>(p.sharedMemPerBlock);
  if (wavefront_size) *wavefront_size = p.warpSize;
  if (clock_khz) *clock_khz = p.clockRate;
  if (global_mem_bytes) *global_mem_bytes = p.totalGlobalMem;
  return 0;
}

int emh_compile(const char* src, const char* name, const char* arch, const char* const* opts,
                int nopts, void** code, size_t* code_len, char** log) {
  if (log) *log = nullptr;
  if (!src || !arch || !code || !code_len) return fail_arg("emh_compile: NULL argument");
  if (nopts < 0 || (nopts > 0 && !opts)) return fail_arg("emh_compile: bad option list");
  *code = nullptr;
  *code_len = 0;

  hiprtcProgram prog = nullptr;
  std::string unit = std::string(name && *name ? name : "kernel") + ".hip";
  hiprtcResult r = hiprtcCreateProgram(&prog, src, unit.c_str(), 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcCreateProgram");

  std::string arch_opt = std::string("--offload-arch=") + arch;
  std::vector<const char*> all;
  all.push_back(arch_opt.c_str());
  for (int i = 0; i < nopts; ++i) all.push_back(opts[i]);

  hiprtcResult cr = hiprtcCompileProgram(prog, static_cast<int>(all.size()), all.data());

  size_t log_size = 0;
  std::string log_text;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    log_text.resize(log_size);
    if (hiprtcGetProgramLog(prog, &log_text[0]) != HIPRTC_SUCCESS) log_text.clear();
  }
  if (log && !log_text.empty()) {
    *log = static_cast<char*>(std::malloc(log_text.size() + 1));
    if (*log) std::memcpy(*log, log_text.c_str(), log_text.size() + 1);
  }
  if (cr != HIPRTC_SUCCESS) {
    int rc = fail_rtc(cr, "hiprtcCompileProgram");
    if (!log_text.empty()) {
      // Keep the tail: the first error usually sits near the end of a long log.
      const size_t keep = 4000;
      g_last_error += "\n" + (log_text.size() > keep ? log_text.substr(log_text.size() - keep) : log_text);
    }
    (void)hiprtcDestroyProgram(&prog);
    return rc;
  }

  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r != HIPRTC_SUCCESS || n == 0) {
    (void)hiprtcDestroyProgram(&prog);
    return fail_rtc(r == HIPRTC_SUCCESS ? HIPRTC_ERROR_INTERNAL_ERROR : r, "hiprtcGetCodeSize");
  }
  void* buf = std::malloc(n);
  if (!buf) {
    (void)hiprtcDestroyProgram(&prog);
    return fail_arg("emh_compile: out of host memory");
  }
  r = hiprtcGetCode(prog, static_cast<char*>(buf));
  (void)hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    std::free(buf);
    return fail_rtc(r, "hiprtcGetCode");
  }
  *code = buf;
  *code_len = n;
  return 0;
}

void emh_free(void* p) { std::free(p); }

int emh_module_load(const void* code, size_t code_len, void** module) {
  if (!code || code_len == 0 || !module) return fail_arg("emh_module_load: NULL argument");
  hipModule_t m = nullptr;
  EMH_HIP(hipModuleLoadData(&m, code));
  *module = m;
  return 0;
}

int emh_module_unload(void* module) {
  if (!module) return 0;
  EMH_HIP(hipModuleUnload(static_cast<hipModule_t>(module)));
  return 0;
}

int emh_get_function(void* module, const char* name, void** fn) {
  if (!module || !name || !fn) return fail_arg("emh_get_function: NULL argument");
  hipFunction_t f = nullptr;
  EMH_HIP(hipModuleGetFunction(&f, static_cast<hipModule_t>(module), name));
  *fn = f;
  return 0;
}

int emh_func_set_dynamic_lds(void* fn, int bytes) {
  if (!fn || bytes < 0) return fail_arg("emh_func_set_dynamic_lds: bad argument");
  EMH_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  return 0;
}

int emh_func_attributes(void* fn, int* num_regs, int* static_lds_bytes, int* private_bytes,
                        int* max_threads) {
  if (!fn) return fail_arg("emh_func_attributes: fn is NULL");
  hipFunction_t f = static_cast<hipFunction_t>(fn);
  if (num_regs) EMH_HIP(hipFuncGetAttribute(num_regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, f));
  if (static_lds_bytes)
    EMH_HIP(hipFuncGetAttribute(static_lds_bytes, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f));
  if (private_bytes)
    EMH_HIP(hipFuncGetAttribute(private_bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f));
  if (max_threads)
    EMH_HIP(hipFuncGetAttribute(max_threads, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f));
  return 0;
}

int emh_launch(void* fn, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
               void* stream, void** args, int nargs) {
  if (!fn || !grid || !block) return fail_arg("emh_launch: NULL argument");
  if (nargs < 0 || (nargs > 0 && !args)) return fail_arg("emh_launch: bad argument list");
  for (int i = 0; i < nargs; ++i)
    if (!args[i]) return fail_arg("emh_launch: NULL kernel-parameter slot");
  for (int i = 0; i < 3; ++i)
    if (grid[i] == 0 || block[i] == 0) return fail_arg("emh_launch: zero-sized grid or block");
  unsigned long long threads = 1ull * block[0] * block[1] * block[2];
  if (threads > 1024) return fail_arg("emh_launch: block exceeds 1024 threads");
  if (lds_bytes > 160u * 1024u) return fail_arg("emh_launch: LDS request exceeds 160 KiB");
  EMH_HIP(hipModuleLaunchKernel(static_cast<hipFunction_t>(fn), grid[0], grid[1], grid[2], block[0],
                                block[1], block[2], lds_bytes, static_cast<hipStream_t>(stream),
                                args, nullptr));
  return 0;
}

int emh_launch_scratch(void* fn, const unsigned grid[3], const unsigned block[3],
                       unsigned lds_bytes, void* stream, void** args, int nargs, int scratch_arg,
                       size_t scratch_offset, size_t scratch_bytes, int zero_first) {
  constexpr int kMaxArgs = 64;
  if (!fn || !grid || !block) return fail_arg("emh_launch_scratch: NULL argument");
  if (nargs <= 0 || nargs > kMaxArgs || !args) return fail_arg("emh_launch_scratch: bad argument list (1..64 parameters)");
  if (scratch_arg < 0 || scratch_arg >= nargs) return fail_arg("emh_launch_scratch: scratch_arg is not a parameter of the kernel");
  if (scratch_offset % 256 != 0 || scratch_bytes % 4 != 0)
    return fail_arg("emh_launch_scratch: scratch_offset must be a multiple of 256 and scratch_bytes of 4");
  if (scratch_bytes == 0 || scratch_offset > EMH_SCRATCH_MAX_BYTES || scratch_bytes > EMH_SCRATCH_MAX_BYTES - scratch_offset) {
    g_last_error = "emh_launch_scratch: workspace of " + std::to_string(scratch_bytes) + " bytes at offset " +
                   std::to_string(scratch_offset) + " does not fit the library's " + std::to_string(EMH_SCRATCH_MAX_BYTES) +
                   "-byte scratch array (EMH_SCRATCH_MAX_BYTES)";
    return static_cast<int>(hipErrorInvalidValue);
  }
  unsigned char* base = nullptr;
  if (int rc = scratch_base(&base)) return rc;
  void* ws = base + scratch_offset;  // the device address, never the array's name
  void* local[kMaxArgs];
  for (int i = 0; i < nargs; ++i) local[i] = args[i];
  local[scratch_arg] = &ws;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (zero_first) {
    const size_t words = scratch_bytes / 4;
    const unsigned blocks = static_cast<unsigned>(std::min<size_t>(1024, (words + 255) / 256));
    hipLaunchKernelGGL(emh_scratch_zero_words, dim3(blocks), dim3(256), 0, s, reinterpret_cast<unsigned int*>(ws), words);
    EMH_HIP(hipGetLastError());
  }
  return emh_launch(fn, grid, block, lds_bytes, stream, local, nargs);
}

int emh_memset_async(void* dptr, int value, size_t bytes, void* stream) {
  if (bytes == 0) return 0;
  if (!dptr) return fail_arg("emh_memset_async: dptr is NULL");
  EMH_HIP(hipMemsetAsync(dptr, value, bytes, static_cast<hipStream_t>(stream)));
  return 0;
}

int emh_stream_create(void** stream) {
  if (!stream) return fail_arg("emh_stream_create: stream is NULL");
  hipStream_t s = nullptr;
  EMH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return 0;
}

int emh_stream_destroy(void* stream) {
  if (!stream) return 0;
  EMH_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return 0;
}

int emh_stream_synchronize(void* stream) {
  EMH_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}

int emh_event_create(void** event) {
  if (!event) return fail_arg("emh_event_create: event is NULL");
  hipEvent_t e = nullptr;
  EMH_HIP(hipEventCreate(&e));
  *event = e;
  return 0;
}

int emh_event_record(void* event, void* stream) {
  if (!event) return fail_arg("emh_event_record: event is NULL");
  EMH_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return 0;
}

int emh_event_synchronize(void* event) {
  if (!event) return fail_arg("emh_event_synchronize: event is NULL");
  EMH_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return 0;
}

int emh_event_query(void* event, int* done) {
  if (!event || !done) return fail_arg("emh_event_query: NULL argument");
  hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipSuccess) {
    *done = 1;
    return 0;
  }
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *done = 0;
    return 0;
  }
  return fail_hip(e, "hipEventQuery");
}

int emh_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return fail_arg("emh_event_elapsed_ms: NULL argument");
  EMH_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return 0;
}

int emh_event_destroy(void* event) {
  if (!event) return 0;
  EMH_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return 0;
}

int emh_graph_begin_capture(void* stream) {
  if (!stream) return fail_arg("emh_graph_begin_capture: the legacy default stream cannot be captured");
  EMH_HIP(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeThreadLocal));
  return 0;
}

int emh_graph_end_capture(void* stream, void** graph_exec) {
  if (!stream || !graph_exec) return fail_arg("emh_graph_end_capture: NULL argument");
  hipGraph_t g = nullptr;
  EMH_HIP(hipStreamEndCapture(static_cast<hipStream_t>(stream), &g));
  hipGraphExec_t ex = nullptr;
  hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) return fail_hip(e, "hipGraphInstantiate");
  *graph_exec = ex;
  return 0;
}

int emh_graph_launch(void* graph_exec, void* stream) {
  if (!graph_exec) return fail_arg("emh_graph_launch: graph_exec is NULL");
  EMH_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
  return 0;
}

int emh_graph_destroy(void* graph_exec) {
  if (!graph_exec) return 0;
  EMH_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
  return 0;
}

const char* emh_last_error(void) { return g_last_error.c_str(); }

}  // extern "C"
