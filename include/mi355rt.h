/*
 * mi355rt -- C ABI of the MI355X (gfx950) runtime shim used by the generated-kernel
 * hot path (ElementwiseKernel / ReductionKernel / ufunc / fuse / memory pool).
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, returns an
 * `int` status (0 = success, a hipError_t value, or RT_ERR_RTC_BASE + hiprtcResult)
 * and never throws across the boundary.  Handles (module, function, stream, event,
 * pool) are opaque `void*`.  Buffers handed back through `void** / char**` out
 * parameters are malloc'ed by the library and released with rt_free_buffer().
 *
 * Each declaration names the interface of the reference (cupy/cupy, paths relative
 * to the reference tree) that it takes the place of.
 */
#ifndef MI355RT_H_
#define MI355RT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RT_ERR_RTC_BASE 10000 /* status = RT_ERR_RTC_BASE + hiprtcResult */
#define RT_ERR_POOL_OOM 20001 /* pool limit reached / allocator out of memory */
#define RT_ERR_INVALID 20002  /* bad argument caught by the shim itself       */

/* memcpy kinds, numerically equal to hipMemcpyKind */
#define RT_MEMCPY_H2H 0
#define RT_MEMCPY_H2D 1
#define RT_MEMCPY_D2H 2
#define RT_MEMCPY_D2D 3
#define RT_MEMCPY_DEFAULT 4

typedef struct rt_device_props {
  char name[256];
  char arch[64];              /* e.g. "gfx950:sramecc+:xnack-" */
  int32_t compute_units;      /* multiProcessorCount */
  int32_t warp_size;
  int32_t max_threads_per_block;
  int32_t max_threads_per_cu;
  int32_t clock_khz;
  int32_t memory_clock_khz;
  int32_t memory_bus_width;
  int32_t l2_cache_bytes;
  int64_t shared_mem_per_block;
  int64_t total_global_mem;
} rt_device_props;

/* ---- status / errors ---------------------------------------------------- */

/* replaces check_status + error-name lookup: cupy_backends/cuda/api/driver.pyx:48-73,
 * cupy_backends/cuda/api/runtime.pyx:128-146, cupy_backends/cuda/libs/nvrtc.pyx:37-53 */
const char* rt_error_string(int status);
const char* rt_error_name(int status);
/* text of the last failure on the calling thread (never NULL) */
const char* rt_last_error_string(void);

/* ---- device -------------------------------------------------------------- */

/* hipInit(0); safe to call repeatedly.  runtime.pyx has no counterpart: the
 * reference initialises lazily inside the first runtime call. */
int rt_init(void);
/* runtime.pyx:411 getDeviceCount */
int rt_device_count(int* count);
/* runtime.pyx:191 getDevice / :417 setDevice */
int rt_get_device(int* device);
int rt_set_device(int device);
/* runtime.pyx:203 getDeviceProperties */
int rt_device_get_props(int device, rt_device_props* out);
/* runtime.pyx:421 deviceSynchronize */
int rt_device_synchronize(void);
/* runtime.pyx:153 driverGetVersion / :159 runtimeGetVersion */
int rt_driver_version(int* version);
int rt_runtime_version(int* version);
/* runtime.pyx:610 memGetInfo */
int rt_mem_info(size_t* free_bytes, size_t* total_bytes);

/* ---- compile (hiprtc) ----------------------------------------------------- */

/* nvrtc.pyx:56 getVersion */
int rt_rtc_version(int* major, int* minor);
/*
 * One call for createProgram + compileProgram + getPTX(→hiprtcGetCode) +
 * getProgramLog + destroyProgram (nvrtc.pyx:84-230; driver of those calls:
 * cupy/cuda/compiler.py:832-880 `_NVRTCProgram.compile`).
 * `headers`/`header_names` are in-memory include files (may be 0 / NULL).
 * On success `*code` and `*code_len` hold the gfx950 code object.  `*log` is always set
 * (possibly to an empty string) unless allocation fails; free both with
 * rt_free_buffer().
 */
int rt_compile(const char* source, const char* name,
               int n_options, const char* const* options,
               int n_headers, const char* const* headers,
               const char* const* header_names,
               void** code, size_t* code_len, char** log);
/* The same with C++ name expressions (nvrtc.pyx:232-250 addNameExpression /
 * getLoweredName; used by cupy/_core/raw.pyx:439-499 `RawModule.get_function`
 * for template kernels): `lowered_names[i]` receives the mangled symbol of
 * `name_expressions[i]` as a malloc'd string (free each with rt_free_buffer). */
int rt_compile_named(const char* source, const char* name,
                     int n_options, const char* const* options,
                     int n_headers, const char* const* headers,
                     const char* const* header_names,
                     int n_names, const char* const* name_expressions,
                     char** lowered_names,
                     void** code, size_t* code_len, char** log);
void rt_free_buffer(void* p);

/* ---- module / function / launch ------------------------------------------- */

/* driver.pyx:233 moduleLoadData, :243 moduleUnload, :250 moduleGetFunction,
 * :261 moduleGetGlobal (cupy/cuda/function.pyx:174-208 `Module`) */
int rt_module_load(const void* image, void** module);
int rt_module_unload(void* module);
int rt_module_get_function(void* module, const char* name, void** function);
int rt_module_get_global(void* module, const char* name, void** dptr, size_t* bytes);
/* driver.pyx:309 funcGetAttribute; `attribute` is a hipFunction_attribute value */
int rt_func_get_attribute(int attribute, void* function, int* value);
/* driver.pyx:322-330 funcSetAttribute (a stub returning hipErrorUnknown in
 * cupy_backends/hip/cupy_hip.h:130-132; real here).  `attribute` is a
 * hipFunction_attribute value as for rt_func_get_attribute; the two settable
 * ones are MAX_DYNAMIC_SHARED_SIZE_BYTES and PREFERRED_SHARED_MEMORY_CARVEOUT
 * (cupy/_core/raw.pyx:226-287). */
int rt_func_set_attribute(void* function, int attribute, int value);
/* driver.pyx:335 occupancyMaxActiveBlocksPerMultiprocessor (a stub returning
 * hipErrorUnknown in cupy_backends/hip/cupy_hip.h:125-137; real here) */
int rt_occupancy_max_active_blocks(void* function, int block_size,
                                   size_t dynamic_smem, int* num_blocks);
/* driver.pyx:273 launchKernel (cupy/cuda/function.pyx:92-131 `_launch`):
 * `params[i]` points at the i-th kernel argument. */
int rt_launch(void* function,
              unsigned gx, unsigned gy, unsigned gz,
              unsigned bx, unsigned by, unsigned bz,
              unsigned shared_mem, void* stream, void** params);
/* driver.pyx:289-301 launchCooperativeKernel (a stub returning hipErrorUnknown
 * in cupy_backends/hip/cupy_hip.h:121-123; real here): all workgroups of the
 * grid are resident at once, so the kernel may synchronise the whole grid
 * (cooperative_groups::this_grid().sync()).  A grid larger than the device can
 * hold at once is refused with hipErrorCooperativeLaunchTooLarge.  Used by
 * RawKernel(enable_cooperative_groups=True) (cupy/cuda/function.pyx:113-131). */
int rt_launch_cooperative(void* function,
                          unsigned gx, unsigned gy, unsigned gz,
                          unsigned bx, unsigned by, unsigned bz,
                          unsigned shared_mem, void* stream, void** params);
/* Same launch with the arguments already laid out as the kernel's argument
 * block (each argument at its natural alignment); saves building the pointer
 * array that function.pyx:104-127 builds per call. */
int rt_launch_packed(void* function,
                     unsigned gx, unsigned gy, unsigned gz,
                     unsigned bx, unsigned by, unsigned bz,
                     unsigned shared_mem, void* stream,
                     const void* arg_block, size_t arg_block_size);

/* No counterpart in the reference (its profiler brackets host calls with
 * events, cupyx/profiler/_time.py:164-234).  For measurement: rt_launch_packed
 * with two events that receive the start and the end of THIS kernel's execution
 * on the device, so that rt_event_elapsed_ms(start, stop) is the duration a
 * profiler's kernel trace reports for the dispatch, with nothing of the
 * neighbouring launches in it.  Both events must exist; either may be null. */
int rt_launch_packed_timed(void* function,
                           unsigned gx, unsigned gy, unsigned gz,
                           unsigned bx, unsigned by, unsigned bz,
                           unsigned shared_mem, void* stream,
                           const void* arg_block, size_t arg_block_size,
                           void* start_event, void* stop_event);

/*
 * No counterpart in the reference.  For callers that cannot allocate device
 * memory -- code under HIP graph capture, serving loops, harnesses that forbid
 * hipMalloc: rt_launch_packed for a kernel that needs a scratch buffer (the
 * partial results of a reduction split over workgroups, which the Python layer
 * otherwise takes from the memory pool), with that buffer inside the library:
 * a static device array of RT_SCRATCH_MAX_BYTES per GPU.  The 8 bytes at
 * `scratch_arg_offset` of the argument block (the kernel's pointer parameter
 * for the buffer) are replaced by the array's address on the current device;
 * `scratch_bytes` is what the kernel will use of it and is refused with
 * RT_ERR_INVALID beyond RT_SCRATCH_MAX_BYTES, as is an argument block of more
 * than RT_SCRATCH_MAX_ARG_BLOCK bytes.  Allocates nothing, on the host or the
 * device.  All calls on one GPU share the one array: it keeps what the last
 * call left (the reduction kernels write every partial before they read it, so
 * nothing needs clearing), and two calls that overlap in time on one GPU --
 * different streams or threads -- race on it.
 */
#define RT_SCRATCH_MAX_BYTES (8u << 20)
#define RT_SCRATCH_MAX_ARG_BLOCK 4096
int rt_launch_packed_scratch(void* function,
                             unsigned gx, unsigned gy, unsigned gz,
                             unsigned bx, unsigned by, unsigned bz,
                             unsigned shared_mem, void* stream,
                             const void* arg_block, size_t arg_block_size,
                             size_t scratch_arg_offset, size_t scratch_bytes);

/* ---- raw device / pinned host memory --------------------------------------- */

/* runtime.pyx:515 malloc, :588 free */
int rt_malloc(void** dptr, size_t size);
int rt_free(void* dptr);
/* runtime.pyx:571 hostAlloc, :593 freeHost */
int rt_host_alloc(void** hptr, size_t size);
int rt_host_free(void* hptr);
/* runtime.pyx:616 memcpy, :621 memcpyAsync */
int rt_memcpy(void* dst, const void* src, size_t size, int kind);
int rt_memcpy_async(void* dst, const void* src, size_t size, int kind, void* stream);
/* runtime.pyx:706 memset, :711 memsetAsync */
int rt_memset(void* dptr, int value, size_t size);
int rt_memset_async(void* dptr, int value, size_t size, void* stream);

/* ---- streams / events ------------------------------------------------------ */

/* runtime.pyx:893 streamCreate, :901 streamCreateWithFlags (non_blocking != 0),
 * :932 streamDestroy, :938 streamSynchronize, :1008 streamQuery,
 * :1012 streamWaitEvent.  Streams are always created at default priority. */
int rt_stream_create(void** stream, int non_blocking);
int rt_stream_destroy(void* stream);
int rt_stream_synchronize(void* stream);
int rt_stream_query(void* stream, int* done);
int rt_stream_wait_event(void* stream, void* event);
/* runtime.pyx:1047 eventCreate / :1054 eventCreateWithFlags (disable_timing),
 * :1062 eventDestroy, :1081 eventRecord, :1087 eventSynchronize,
 * :1077 eventQuery, :1068 eventElapsedTime */
int rt_event_create(void** event, int disable_timing);
int rt_event_destroy(void* event);
int rt_event_record(void* event, void* stream);
int rt_event_synchronize(void* event);
int rt_event_query(void* event, int* done);
int rt_event_elapsed_ms(float* ms, void* start, void* end);

/* ---- device memory pool ------------------------------------------------------
 * Native core of cupy/cuda/memory.pyx:359-446 (_Chunk), :1055-1199 (_Arena),
 * :1218-1563 (SingleDeviceMemoryPool).  One pool serves one device.  Blocks are
 * cached per stream: a block freed on stream S is handed out again only to
 * requests made on S (stream order makes that reuse safe without a sync).
 * Sizes are rounded up to RT_POOL_UNIT bytes.
 */
#define RT_POOL_UNIT 512

/* Allocator callbacks let a host-side test drive the pool with fake addresses
 * (the reference does the same with a mock allocator,
 * tests/cupy_tests/cuda_tests/test_memory.py:20-36).  alloc returns 0 on
 * success and stores the address; any other value is treated as out-of-memory. */
typedef int (*rt_pool_alloc_fn)(void* ctx, size_t size, uint64_t* address);
typedef void (*rt_pool_free_fn)(void* ctx, uint64_t address, size_t size);

/* memory.pyx:1258 SingleDeviceMemoryPool.__init__ (allocator = hipMalloc/hipFree) */
int rt_pool_create(void** pool);
int rt_pool_create_with_allocator(void** pool, rt_pool_alloc_fn alloc_fn,
                                  rt_pool_free_fn free_fn, void* ctx);
/* Releases every cached block; blocks still in use are leaked to the driver. */
int rt_pool_destroy(void* pool);
/* memory.pyx:1323-1386 malloc/_malloc: best fit in the arena of `stream_ident`,
 * split the remainder, else allocate (honouring the limit, releasing cached
 * blocks before giving up, :1518-1563).  size 0 is rejected with RT_ERR_INVALID:
 * the caller hands out a plain zero-size allocation itself (:1358-1359). */
int rt_pool_malloc(void* pool, size_t size, uint64_t stream_ident, uint64_t* address);
/* memory.pyx:1388-1398 free: return the block to its arena and merge with free
 * neighbours of the same underlying allocation. */
int rt_pool_free(void* pool, uint64_t address);
/* memory.pyx:1400-1428 free_all_blocks: release unsplit cached blocks of one
 * arena (all_streams == 0) or of every arena. */
int rt_pool_free_all_blocks(void* pool, int all_streams, uint64_t stream_ident);
/* memory.pyx:1436-1462 n_free_blocks / used_bytes / free_bytes / total_bytes */
int rt_pool_stats(void* pool, size_t* used_bytes, size_t* free_bytes,
                  size_t* total_bytes, size_t* n_free_blocks);
/* memory.pyx:1492-1516 set_limit / get_limit (0 = unlimited) */
int rt_pool_set_limit(void* pool, size_t limit_bytes);
int rt_pool_get_limit(void* pool, size_t* limit_bytes);
/* memory.pyx:1041-1046 _round_size */
size_t rt_pool_round_size(size_t size);

#ifdef __cplusplus
}
#endif
#endif /* MI355RT_H_ */
