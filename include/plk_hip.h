/* Thin C ABI over the HIP runtime: device memory, streams, events, code-object loading and
 * launch of a linked pipeline kernel.  No torch types, plain pointers and sizes.
 *
 * Replaces, for gfx950, the driver-API backend the reference binds through ctypes:
 * class CudaBackend in pipec/src/pipec2/host/cuda.py:35-356 (allocate/free/zero/upload/
 * readback/synchronize :118-176, event_* :177-215, launch :257-265, module load :219-243).
 * Every function returns PLK_OK or one of the PLK_E_* codes of the provider ABI
 * (pipec/src/pipec2/host/include/pipelink_host_abi_v2.h:21-28); the text of the last
 * failure on the calling thread is available from plk_hip_last_error(). */
#ifndef PLK_HIP_H
#define PLK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef PLK_STATUS_CODES_DEFINED
#define PLK_STATUS_CODES_DEFINED
enum {
  PLK_OK = 0,
  PLK_E_VERSION = 1,
  PLK_E_CAPACITY = 2,
  PLK_E_ARGUMENT = 3,
  PLK_E_CONTRACT = 4,
  PLK_E_RESOURCE = 5,
  PLK_E_BUILD = 6,
  PLK_E_RELEASE = 7
};
#endif

typedef struct plk_hip_module plk_hip_module;     /* one loaded code object */
typedef struct plk_hip_function plk_hip_function; /* one kernel of it */

/* device properties the resource solver's gfx950 profile is checked against */
typedef struct plk_hip_device_info {
  int32_t compute_units;
  int32_t wavefront_size;
  int32_t max_lds_per_workgroup;
  int32_t max_threads_per_workgroup;
  int32_t clock_khz;
  int32_t memory_clock_khz;
  int32_t l2_bytes;
  int32_t reserved;
  int64_t total_memory;
  char arch[64];
} plk_hip_device_info;

const char* plk_hip_last_error(void);
int plk_hip_device_count(int32_t* count);
int plk_hip_set_device(int32_t device);                              /* CudaBackend.current() */
int plk_hip_device_info_get(int32_t device, plk_hip_device_info* out);

int plk_hip_alloc(size_t bytes, uint64_t* addr);                     /* CudaBackend.allocate */
int plk_hip_free(uint64_t addr);                                     /* CudaBackend.free */
int plk_hip_zero(uint64_t addr, size_t bytes, void* stream);         /* CudaBackend.zero */
int plk_hip_fill_u8(uint64_t addr, int value, size_t bytes, void* stream);
int plk_hip_upload(uint64_t dst, const void* src, size_t bytes, void* stream);   /* CudaBackend.upload */
int plk_hip_readback(void* dst, uint64_t src, size_t bytes, void* stream);       /* CudaBackend.readback */
int plk_hip_synchronize(void* stream);                               /* CudaBackend.synchronize */

int plk_hip_stream_create(void** stream);
int plk_hip_stream_destroy(void* stream);
/* Graph capture of one stream (CudaBackend.capture, host/cuda.py:267-286; Graph.launch / close, :358-382).  The stream
 * must be one made by plk_hip_stream_create.  While a stream is captured plk_hip_zero / plk_hip_fill_u8 record a
 * fill kernel, not a memset node; uploads and readbacks synchronise and cannot be captured. */
int plk_hip_graph_begin(void* stream);
int plk_hip_graph_end(void* stream, void** graph, void** executable);   /* ends the capture and instantiates it */
int plk_hip_graph_abort(void* stream);                                  /* ends a capture whose body failed; keeps nothing */
int plk_hip_graph_launch(void* executable, void* stream);
int plk_hip_graph_destroy(void* graph, void* executable);
int plk_hip_event_create(void** event);                              /* CudaBackend.event_create */
int plk_hip_event_record(void* event, void* stream);
int plk_hip_event_synchronize(void* event);
int plk_hip_event_elapsed_ms(void* start, void* stop, float* ms);
int plk_hip_event_destroy(void* event);

/* CudaBackend module load + cuModuleGetFunction; dyn_lds_bytes raises the kernel's dynamic
 * LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize). */
int plk_hip_module_load(const void* image, size_t bytes, plk_hip_module** out);
int plk_hip_module_unload(plk_hip_module* module);
int plk_hip_module_function(plk_hip_module* module, const char* name, uint32_t dyn_lds_bytes, plk_hip_function** out);

/* CudaBackend.launch: the kernel's sole argument is one pointer to the params image
 * (params_addr, device memory).  grid and block are in workgroups / threads. */
int plk_hip_launch(plk_hip_function* fn, const uint32_t grid[3], const uint32_t block[3], uint32_t dyn_lds_bytes,
                   void* stream, uint64_t params_addr);

#ifdef __cplusplus
}
#endif
#endif
