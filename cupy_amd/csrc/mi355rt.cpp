// mi355rt: HIP / hiprtc part of the C-ABI shim declared in include/mi355rt.h.
//
// Thin, re-entrant wrappers: no global state besides the thread-local text of
// the last failure.  Every function returns a status instead of throwing.
#include "mi355rt.h"

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

// Device memory owned by the library itself, for rt_launch_packed_scratch: the
// place where a kernel keeps data beyond its inputs and outputs (the partial
// results of a reduction split over workgroups) when the caller may not
// allocate.  Every GPU the library runs on holds its own copy until the
// process ends.  In host code this name is a stand-in, not an address: the
// address on a device comes from hipGetSymbolAddress (scratch_address below)
// and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[RT_SCRATCH_MAX_BYTES];

namespace {

thread_local std::string g_last_error;

int fail_hip(hipError_t e, const char* what) {
  // HIP keeps a sticky per-thread error; drain it so that an unrelated later
  // call does not report this failure again.
  (void)hipGetLastError();
  g_last_error = std::string(what) + ": " + hipGetErrorName(e) + ": " + hipGetErrorString(e);
  return static_cast<int>(e);
}

int fail_rtc(hiprtcResult r, const char* what) {
  g_last_error = std::string(what) + ": " + hiprtcGetErrorString(r);
  return RT_ERR_RTC_BASE + static_cast<int>(r);
}

int fail_invalid(const char* what) {
  g_last_error = what;
  return RT_ERR_INVALID;
}

#define RT_HIP(call)                               \
  do {                                             \
    hipError_t e_ = (call);                        \
    if (e_ != hipSuccess) return fail_hip(e_, #call); \
  } while (0)

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Address of `scratch` on the CURRENT device, looked up once per device.
int scratch_address(void** out) {
  int dev = 0;
  RT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail_invalid("scratch: device number out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    RT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail_invalid("scratch: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

char* dup_string(const std::string& s) {
  char* p = static_cast<char*>(std::malloc(s.size() + 1));
  if (p) std::memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

}  // namespace

// Used by pool.cpp to report failures through the same thread-local slot.
void rt_set_last_error_(const char* text) { g_last_error = text ? text : ""; }

extern "C" {

const char* rt_error_string(int status) {
  if (status == 0) return "success";
  if (status == RT_ERR_POOL_OOM) return "out of memory (pool limit or allocator failure)";
  if (status == RT_ERR_INVALID) return "invalid argument";
  if (status >= RT_ERR_RTC_BASE && status < RT_ERR_POOL_OOM)
    return hiprtcGetErrorString(static_cast<hiprtcResult>(status - RT_ERR_RTC_BASE));
  return hipGetErrorString(static_cast<hipError_t>(status));
}

const char* rt_error_name(int status) {
  if (status == 0) return "hipSuccess";
  if (status == RT_ERR_POOL_OOM) return "RT_ERR_POOL_OOM";
  if (status == RT_ERR_INVALID) return "RT_ERR_INVALID";
  if (status >= RT_ERR_RTC_BASE && status < RT_ERR_POOL_OOM) return "HIPRTC_ERROR";
  return hipGetErrorName(static_cast<hipError_t>(status));
}

const char* rt_last_error_string(void) { return g_last_error.c_str(); }

// ---- device -----------------------------------------------------------------

int rt_init(void) {
  RT_HIP(hipInit(0));
  // the library's scratch array on the device that is current now; other
  // devices are looked up by the first rt_launch_packed_scratch on them
  void* p = nullptr;
  return scratch_address(&p);
}

int rt_device_count(int* count) {
  if (!count) return fail_invalid("rt_device_count: null output");
  *count = 0;
  RT_HIP(hipGetDeviceCount(count));
  return 0;
}

int rt_get_device(int* device) {
  if (!device) return fail_invalid("rt_get_device: null output");
  RT_HIP(hipGetDevice(device));
  return 0;
}

int rt_set_device(int device) {
  RT_HIP(hipSetDevice(device));
  return 0;
}

int rt_device_get_props(int device, rt_device_props* out) {
  if (!out) return fail_invalid("rt_device_get_props: null output");
  hipDeviceProp_t p;
  RT_HIP(hipGetDeviceProperties(&p, device));
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->name, sizeof(out->name), "%s", p.name);
  std::snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
  out->compute_units = p.multiProcessorCount;
  out->warp_size = p.warpSize;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->max_threads_per_cu = p.maxThreadsPerMultiProcessor;
  out->clock_khz = p.clockRate;
  out->memory_clock_khz = p.memoryClockRate;
  out->memory_bus_width = p.memoryBusWidth;
  out->l2_cache_bytes = p.l2CacheSize;
  out->shared_mem_per_block = static_cast<int64_t>(p.sharedMemPerBlock);
  out->total_global_mem = static_cast<int64_t>(p.totalGlobalMem);
  return 0;
}

int rt_device_synchronize(void) {
  RT_HIP(hipDeviceSynchronize());
  return 0;
}

int rt_driver_version(int* version) {
  if (!version) return fail_invalid("rt_driver_version: null output");
  RT_HIP(hipDriverGetVersion(version));
  return 0;
}

int rt_runtime_version(int* version) {
  if (!version) return fail_invalid("rt_runtime_version: null output");
  RT_HIP(hipRuntimeGetVersion(version));
  return 0;
}

int rt_mem_info(size_t* free_bytes, size_t* total_bytes) {
  size_t f = 0, t = 0;
  RT_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return 0;
}

// ---- compile ----------------------------------------------------------------

int rt_rtc_version(int* major, int* minor) {
  int ma = 0, mi = 0;
  hiprtcResult r = hiprtcVersion(&ma, &mi);
  if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcVersion");
  if (major) *major = ma;
  if (minor) *minor = mi;
  return 0;
}

static int compile_impl(const char* source, const char* name,
                        int n_options, const char* const* options,
                        int n_headers, const char* const* headers,
                        const char* const* header_names,
                        int n_names, const char* const* name_expressions, char** lowered,
                        void** code, size_t* code_len, char** log) {
  if (!source || !code || !code_len || !log) return fail_invalid("rt_compile: null argument");
  if (n_names < 0 || (n_names > 0 && (!name_expressions || !lowered)))
    return fail_invalid("rt_compile_named: bad name expression arguments");
  *code = nullptr;
  *code_len = 0;
  *log = nullptr;
  for (int i = 0; i < n_names; ++i) lowered[i] = nullptr;
  hiprtcProgram prog = nullptr;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kernel.hip", n_headers,
                                       const_cast<const char**>(headers),
                                       const_cast<const char**>(header_names));
  if (r != HIPRTC_SUCCESS) {
    *log = dup_string("");
    return fail_rtc(r, "hiprtcCreateProgram");
  }
  for (int i = 0; i < n_names; ++i) {
    r = hiprtcAddNameExpression(prog, name_expressions[i]);
    if (r != HIPRTC_SUCCESS) {
      *log = dup_string("");
      hiprtcDestroyProgram(&prog);
      return fail_rtc(r, "hiprtcAddNameExpression");
    }
  }
  hiprtcResult rc = hiprtcCompileProgram(prog, n_options, const_cast<const char**>(options));
  size_t log_size = 0;
  std::string log_text;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    log_text.resize(log_size);
    if (hiprtcGetProgramLog(prog, &log_text[0]) != HIPRTC_SUCCESS) log_text.clear();
    while (!log_text.empty() && log_text.back() == '\0') log_text.pop_back();
  }
  *log = dup_string(log_text);
  if (rc != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return fail_rtc(rc, "hiprtcCompileProgram");
  }
  // lowered names live inside the program object: copy them before it goes
  for (int i = 0; i < n_names; ++i) {
    const char* low = nullptr;
    r = hiprtcGetLoweredName(prog, name_expressions[i], &low);
    if (r != HIPRTC_SUCCESS || !low) {
      for (int k = 0; k < i; ++k) { std::free(lowered[k]); lowered[k] = nullptr; }
      hiprtcDestroyProgram(&prog);
      return fail_rtc(r != HIPRTC_SUCCESS ? r : HIPRTC_ERROR_NAME_EXPRESSION_NOT_VALID,
                      "hiprtcGetLoweredName");
    }
    lowered[i] = dup_string(low);
  }
  size_t size = 0;
  r = hiprtcGetCodeSize(prog, &size);
  void* buf = nullptr;
  if (r == HIPRTC_SUCCESS) {
    buf = std::malloc(size ? size : 1);
    if (buf) r = hiprtcGetCode(prog, static_cast<char*>(buf));
  }
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS || !buf) {
    std::free(buf);
    for (int k = 0; k < n_names; ++k) { std::free(lowered[k]); lowered[k] = nullptr; }
    if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcGetCode");
    return fail_invalid("rt_compile: out of host memory");
  }
  *code = buf;
  *code_len = size;
  return 0;
}

int rt_compile(const char* source, const char* name,
               int n_options, const char* const* options,
               int n_headers, const char* const* headers,
               const char* const* header_names,
               void** code, size_t* code_len, char** log) {
  return compile_impl(source, name, n_options, options, n_headers, headers, header_names,
                      0, nullptr, nullptr, code, code_len, log);
}

int rt_compile_named(const char* source, const char* name,
                     int n_options, const char* const* options,
                     int n_headers, const char* const* headers,
                     const char* const* header_names,
                     int n_names, const char* const* name_expressions, char** lowered_names,
                     void** code, size_t* code_len, char** log) {
  return compile_impl(source, name, n_options, options, n_headers, headers, header_names,
                      n_names, name_expressions, lowered_names, code, code_len, log);
}

void rt_free_buffer(void* p) { std::free(p); }

// ---- module / function / launch ------------------------------------------------

int rt_module_load(const void* image, void** module) {
  if (!image || !module) return fail_invalid("rt_module_load: null argument");
  hipModule_t m = nullptr;
  RT_HIP(hipModuleLoadData(&m, image));
  *module = m;
  return 0;
}

int rt_module_unload(void* module) {
  RT_HIP(hipModuleUnload(static_cast<hipModule_t>(module)));
  return 0;
}

int rt_module_get_function(void* module, const char* name, void** function) {
  if (!module || !name || !function) return fail_invalid("rt_module_get_function: null argument");
  hipFunction_t f = nullptr;
  RT_HIP(hipModuleGetFunction(&f, static_cast<hipModule_t>(module), name));
  *function = f;
  return 0;
}

int rt_module_get_global(void* module, const char* name, void** dptr, size_t* bytes) {
  if (!module || !name) return fail_invalid("rt_module_get_global: null argument");
  hipDeviceptr_t p = nullptr;
  size_t n = 0;
  RT_HIP(hipModuleGetGlobal(&p, &n, static_cast<hipModule_t>(module), name));
  if (dptr) *dptr = p;
  if (bytes) *bytes = n;
  return 0;
}

int rt_func_get_attribute(int attribute, void* function, int* value) {
  if (!function || !value) return fail_invalid("rt_func_get_attribute: null argument");
  RT_HIP(hipFuncGetAttribute(value, static_cast<hipFunction_attribute>(attribute),
                             static_cast<hipFunction_t>(function)));
  return 0;
}

int rt_func_set_attribute(void* function, int attribute, int value) {
  if (!function) return fail_invalid("rt_func_set_attribute: null function");
  hipFuncAttribute attr;
  switch (attribute) {
    case HIP_FUNC_ATTRIBUTE_MAX_DYNAMIC_SHARED_SIZE_BYTES:
      attr = hipFuncAttributeMaxDynamicSharedMemorySize;
      break;
    case HIP_FUNC_ATTRIBUTE_PREFERRED_SHARED_MEMORY_CARVEOUT:
      attr = hipFuncAttributePreferredSharedMemoryCarveout;
      break;
    default:
      return fail_invalid("rt_func_set_attribute: this attribute cannot be set");
  }
  RT_HIP(hipFuncSetAttribute(function, attr, value));
  return 0;
}

int rt_occupancy_max_active_blocks(void* function, int block_size, size_t dynamic_smem,
                                   int* num_blocks) {
  if (!function || !num_blocks) return fail_invalid("rt_occupancy_max_active_blocks: null argument");
  RT_HIP(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(
      num_blocks, static_cast<hipFunction_t>(function), block_size, dynamic_smem));
  return 0;
}

int rt_launch(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
              unsigned bz, unsigned shared_mem, void* stream, void** params) {
  if (!function) return fail_invalid("rt_launch: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail_invalid("rt_launch: zero-sized grid or block");
  RT_HIP(hipModuleLaunchKernel(static_cast<hipFunction_t>(function), gx, gy, gz, bx, by, bz,
                               shared_mem, static_cast<hipStream_t>(stream), params, nullptr));
  return 0;
}

int rt_launch_cooperative(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                          unsigned by, unsigned bz, unsigned shared_mem, void* stream,
                          void** params) {
  if (!function) return fail_invalid("rt_launch_cooperative: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail_invalid("rt_launch_cooperative: zero-sized grid or block");
  RT_HIP(hipModuleLaunchCooperativeKernel(static_cast<hipFunction_t>(function), gx, gy, gz, bx,
                                          by, bz, shared_mem, static_cast<hipStream_t>(stream),
                                          params));
  return 0;
}

int rt_launch_packed(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                     unsigned by, unsigned bz, unsigned shared_mem, void* stream,
                     const void* arg_block, size_t arg_block_size) {
  if (!function) return fail_invalid("rt_launch_packed: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail_invalid("rt_launch_packed: zero-sized grid or block");
  size_t size = arg_block_size;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(arg_block),
                   HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  RT_HIP(hipModuleLaunchKernel(static_cast<hipFunction_t>(function), gx, gy, gz, bx, by, bz,
                               shared_mem, static_cast<hipStream_t>(stream), nullptr, extra));
  return 0;
}

int rt_launch_packed_timed(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                           unsigned by, unsigned bz, unsigned shared_mem, void* stream,
                           const void* arg_block, size_t arg_block_size, void* start_event,
                           void* stop_event) {
  if (!function) return fail_invalid("rt_launch_packed_timed: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail_invalid("rt_launch_packed_timed: zero-sized grid or block");
  // (this launch takes its grid in work-items, 32 bits per dimension)
  if (static_cast<uint64_t>(gx) * bx > 0xffffffffull ||
      static_cast<uint64_t>(gy) * by > 0xffffffffull ||
      static_cast<uint64_t>(gz) * bz > 0xffffffffull)
    return fail_invalid("rt_launch_packed_timed: more than 2^32 - 1 work-items in one dimension");
  size_t size = arg_block_size;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(arg_block),
                   HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  RT_HIP(hipExtModuleLaunchKernel(static_cast<hipFunction_t>(function), gx * bx, gy * by, gz * bz,
                                  bx, by, bz, shared_mem, static_cast<hipStream_t>(stream),
                                  nullptr, extra, static_cast<hipEvent_t>(start_event),
                                  static_cast<hipEvent_t>(stop_event), 0));
  return 0;
}

int rt_launch_packed_scratch(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                             unsigned by, unsigned bz, unsigned shared_mem, void* stream,
                             const void* arg_block, size_t arg_block_size,
                             size_t scratch_arg_offset, size_t scratch_bytes) {
  if (!function) return fail_invalid("rt_launch_packed_scratch: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail_invalid("rt_launch_packed_scratch: zero-sized grid or block");
  if (scratch_bytes > RT_SCRATCH_MAX_BYTES) {
    char msg[160];
    std::snprintf(msg, sizeof(msg),
                  "rt_launch_packed_scratch: %zu bytes of scratch requested, the library holds %zu",
                  scratch_bytes, static_cast<size_t>(RT_SCRATCH_MAX_BYTES));
    return fail_invalid(msg);
  }
  unsigned char block[RT_SCRATCH_MAX_ARG_BLOCK];
  if (!arg_block || arg_block_size > sizeof(block))
    return fail_invalid("rt_launch_packed_scratch: argument block missing or larger than "
                        "RT_SCRATCH_MAX_ARG_BLOCK bytes");
  // (compared without adding to the offset: an offset near SIZE_MAX must not wrap)
  if (scratch_arg_offset % sizeof(void*) != 0 || arg_block_size < sizeof(void*) ||
      scratch_arg_offset > arg_block_size - sizeof(void*))
    return fail_invalid("rt_launch_packed_scratch: the pointer slot lies outside the argument "
                        "block or is not 8-byte aligned");
  void* ptr = nullptr;
  int status = scratch_address(&ptr);
  if (status != 0) return status;
  std::memcpy(block, arg_block, arg_block_size);
  std::memcpy(block + scratch_arg_offset, &ptr, sizeof(ptr));
  size_t size = arg_block_size;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, block, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                   HIP_LAUNCH_PARAM_END};
  RT_HIP(hipModuleLaunchKernel(static_cast<hipFunction_t>(function), gx, gy, gz, bx, by, bz,
                               shared_mem, static_cast<hipStream_t>(stream), nullptr, extra));
  return 0;
}

// ---- memory ---------------------------------------------------------------------

int rt_malloc(void** dptr, size_t size) {
  if (!dptr) return fail_invalid("rt_malloc: null output");
  *dptr = nullptr;
  RT_HIP(hipMalloc(dptr, size));
  return 0;
}

int rt_free(void* dptr) {
  RT_HIP(hipFree(dptr));
  return 0;
}

int rt_host_alloc(void** hptr, size_t size) {
  if (!hptr) return fail_invalid("rt_host_alloc: null output");
  *hptr = nullptr;
  RT_HIP(hipHostMalloc(hptr, size, hipHostMallocDefault));
  return 0;
}

int rt_host_free(void* hptr) {
  RT_HIP(hipHostFree(hptr));
  return 0;
}

int rt_memcpy(void* dst, const void* src, size_t size, int kind) {
  if (size == 0) return 0;
  RT_HIP(hipMemcpy(dst, src, size, static_cast<hipMemcpyKind>(kind)));
  return 0;
}

int rt_memcpy_async(void* dst, const void* src, size_t size, int kind, void* stream) {
  if (size == 0) return 0;
  RT_HIP(hipMemcpyAsync(dst, src, size, static_cast<hipMemcpyKind>(kind),
                        static_cast<hipStream_t>(stream)));
  return 0;
}

int rt_memset(void* dptr, int value, size_t size) {
  if (size == 0) return 0;
  RT_HIP(hipMemset(dptr, value, size));
  return 0;
}

int rt_memset_async(void* dptr, int value, size_t size, void* stream) {
  if (size == 0) return 0;
  RT_HIP(hipMemsetAsync(dptr, value, size, static_cast<hipStream_t>(stream)));
  return 0;
}

// ---- streams / events ---------------------------------------------------------------

int rt_stream_create(void** stream, int non_blocking) {
  if (!stream) return fail_invalid("rt_stream_create: null output");
  hipStream_t s = nullptr;
  RT_HIP(hipStreamCreateWithFlags(&s, non_blocking ? hipStreamNonBlocking : hipStreamDefault));
  *stream = s;
  return 0;
}

int rt_stream_destroy(void* stream) {
  RT_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return 0;
}

int rt_stream_synchronize(void* stream) {
  RT_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}

int rt_stream_query(void* stream, int* done) {
  hipError_t e = hipStreamQuery(static_cast<hipStream_t>(stream));
  if (e == hipSuccess) {
    if (done) *done = 1;
    return 0;
  }
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    if (done) *done = 0;
    return 0;
  }
  return fail_hip(e, "hipStreamQuery");
}

int rt_stream_wait_event(void* stream, void* event) {
  RT_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return 0;
}

int rt_event_create(void** event, int disable_timing) {
  if (!event) return fail_invalid("rt_event_create: null output");
  hipEvent_t e = nullptr;
  RT_HIP(hipEventCreateWithFlags(&e, disable_timing ? hipEventDisableTiming : hipEventDefault));
  *event = e;
  return 0;
}

int rt_event_destroy(void* event) {
  RT_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return 0;
}

int rt_event_record(void* event, void* stream) {
  RT_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return 0;
}

int rt_event_synchronize(void* event) {
  RT_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return 0;
}

int rt_event_query(void* event, int* done) {
  hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipSuccess) {
    if (done) *done = 1;
    return 0;
  }
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    if (done) *done = 0;
    return 0;
  }
  return fail_hip(e, "hipEventQuery");
}

int rt_event_elapsed_ms(float* ms, void* start, void* end) {
  if (!ms) return fail_invalid("rt_event_elapsed_ms: null output");
  RT_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(end)));
  return 0;
}

}  // extern "C"
