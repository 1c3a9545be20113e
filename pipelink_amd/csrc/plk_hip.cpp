// Implementation of include/plk_hip.h: the launch layer between the Python host code and
// the HIP runtime.  Errors never cross as exceptions; the failing call's text is kept per
// thread for plk_hip_last_error().
#include "plk_hip.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

struct plk_hip_function {
  hipFunction_t handle;
};
struct plk_hip_module {
  hipModule_t handle;
  std::vector<plk_hip_function*> functions;  // handed out by plk_hip_module_function, freed on unload
};

namespace {
thread_local std::string g_error;

int fail(int code, const char* what, hipError_t err) {
  char buf[512];
  std::snprintf(buf, sizeof buf, "%s: %s (%d)", what, hipGetErrorString(err), (int)err);
  g_error = buf;
  return code;
}
int fail_msg(int code, const char* what) {
  g_error = what;
  return code;
}
}  // namespace

// Fill for a stream that is being captured into a graph: a memset node recorded there is not replayed
// reliably on this stack, a kernel node is.
__global__ void plk_fill_kernel(unsigned char* dst, unsigned char value, size_t bytes) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < bytes; i += (size_t)gridDim.x * blockDim.x) dst[i] = value;
}

#define PLK_HIP_TRY(code, expr)                        \
  do {                                                 \
    hipError_t e_ = (expr);                            \
    if (e_ != hipSuccess) return fail(code, #expr, e_); \
  } while (0)

extern "C" {

const char* plk_hip_last_error(void) { return g_error.c_str(); }

// used by the other translation units of this library
int plk_hip_set_error(int code, const char* what) { return fail_msg(code, what); }

int plk_hip_device_count(int32_t* count) {
  if (!count) return fail_msg(PLK_E_ARGUMENT, "plk_hip_device_count: null output");
  int n = 0;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipGetDeviceCount(&n));
  *count = n;
  return PLK_OK;
}

int plk_hip_set_device(int32_t device) {
  PLK_HIP_TRY(PLK_E_RESOURCE, hipSetDevice(device));
  return PLK_OK;
}

int plk_hip_device_info_get(int32_t device, plk_hip_device_info* out) {
  if (!out) return fail_msg(PLK_E_ARGUMENT, "plk_hip_device_info_get: null output");
  hipDeviceProp_t prop;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipGetDeviceProperties(&prop, device));
  std::memset(out, 0, sizeof *out);
  out->compute_units = prop.multiProcessorCount;
  out->wavefront_size = prop.warpSize;
  out->max_lds_per_workgroup = (int32_t)prop.sharedMemPerBlock;
  out->max_threads_per_workgroup = prop.maxThreadsPerBlock;
  out->clock_khz = prop.clockRate;
  out->memory_clock_khz = prop.memoryClockRate;
  out->l2_bytes = prop.l2CacheSize;
  out->total_memory = (int64_t)prop.totalGlobalMem;
  std::snprintf(out->arch, sizeof out->arch, "%s", prop.gcnArchName);
  return PLK_OK;
}

int plk_hip_alloc(size_t bytes, uint64_t* addr) {
  if (!addr) return fail_msg(PLK_E_ARGUMENT, "plk_hip_alloc: null output");
  void* p = nullptr;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipMalloc(&p, bytes ? bytes : 1));
  *addr = (uint64_t)(uintptr_t)p;
  return PLK_OK;
}

int plk_hip_free(uint64_t addr) {
  PLK_HIP_TRY(PLK_E_RELEASE, hipFree((void*)(uintptr_t)addr));
  return PLK_OK;
}

int plk_hip_zero(uint64_t addr, size_t bytes, void* stream) { return plk_hip_fill_u8(addr, 0, bytes, stream); }

int plk_hip_fill_u8(uint64_t addr, int value, size_t bytes, void* stream) {
  if (!bytes) return PLK_OK;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (stream) PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamIsCapturing((hipStream_t)stream, &capturing));
  if (capturing == hipStreamCaptureStatusActive) {
    const unsigned blocks = (unsigned)((bytes + 256 * 64 - 1) / (256 * 64) < 4096 ? (bytes + 256 * 64 - 1) / (256 * 64) : 4096);
    hipLaunchKernelGGL(plk_fill_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (unsigned char*)(uintptr_t)addr,
                       (unsigned char)value, bytes);
    PLK_HIP_TRY(PLK_E_RESOURCE, hipGetLastError());
    return PLK_OK;
  }
  PLK_HIP_TRY(PLK_E_RESOURCE, hipMemsetAsync((void*)(uintptr_t)addr, value, bytes, (hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_graph_begin(void* stream) {
  if (!stream) return fail_msg(PLK_E_ARGUMENT, "plk_hip_graph_begin: the default stream cannot be captured; create one");
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return PLK_OK;
}

int plk_hip_graph_end(void* stream, void** graph, void** executable) {
  if (!graph || !executable) return fail_msg(PLK_E_ARGUMENT, "plk_hip_graph_end: null output");
  hipGraph_t g = nullptr;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamEndCapture((hipStream_t)stream, &g));
  hipGraphExec_t e = nullptr;
  const hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
  if (err != hipSuccess) {
    (void)hipGraphDestroy(g);
    return fail(PLK_E_RESOURCE, "hipGraphInstantiate", err);
  }
  *graph = (void*)g;
  *executable = (void*)e;
  return PLK_OK;
}

int plk_hip_graph_abort(void* stream) {
  hipGraph_t g = nullptr;
  const hipError_t err = hipStreamEndCapture((hipStream_t)stream, &g);
  if (g) (void)hipGraphDestroy(g);
  if (err != hipSuccess && err != hipErrorStreamCaptureInvalidated) return fail(PLK_E_RELEASE, "hipStreamEndCapture", err);
  return PLK_OK;
}

int plk_hip_graph_launch(void* executable, void* stream) {
  PLK_HIP_TRY(PLK_E_RESOURCE, hipGraphLaunch((hipGraphExec_t)executable, (hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_graph_destroy(void* graph, void* executable) {
  if (executable) PLK_HIP_TRY(PLK_E_RELEASE, hipGraphExecDestroy((hipGraphExec_t)executable));
  if (graph) PLK_HIP_TRY(PLK_E_RELEASE, hipGraphDestroy((hipGraph_t)graph));
  return PLK_OK;
}

int plk_hip_upload(uint64_t dst, const void* src, size_t bytes, void* stream) {
  if (!bytes) return PLK_OK;
  if (!src) return fail_msg(PLK_E_ARGUMENT, "plk_hip_upload: null source");
  PLK_HIP_TRY(PLK_E_RESOURCE,
              hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamSynchronize((hipStream_t)stream));  // src may be pageable and reused
  return PLK_OK;
}

int plk_hip_readback(void* dst, uint64_t src, size_t bytes, void* stream) {
  if (!bytes) return PLK_OK;
  if (!dst) return fail_msg(PLK_E_ARGUMENT, "plk_hip_readback: null destination");
  PLK_HIP_TRY(PLK_E_RESOURCE,
              hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamSynchronize((hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_synchronize(void* stream) {
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamSynchronize((hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_stream_create(void** stream) {
  if (!stream) return fail_msg(PLK_E_ARGUMENT, "plk_hip_stream_create: null output");
  hipStream_t s;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipStreamCreate(&s));  // default priority
  *stream = (void*)s;
  return PLK_OK;
}

int plk_hip_stream_destroy(void* stream) {
  PLK_HIP_TRY(PLK_E_RELEASE, hipStreamDestroy((hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_event_create(void** event) {
  if (!event) return fail_msg(PLK_E_ARGUMENT, "plk_hip_event_create: null output");
  hipEvent_t e;
  PLK_HIP_TRY(PLK_E_RESOURCE, hipEventCreate(&e));
  *event = (void*)e;
  return PLK_OK;
}

int plk_hip_event_record(void* event, void* stream) {
  PLK_HIP_TRY(PLK_E_RESOURCE, hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return PLK_OK;
}

int plk_hip_event_synchronize(void* event) {
  PLK_HIP_TRY(PLK_E_RESOURCE, hipEventSynchronize((hipEvent_t)event));
  return PLK_OK;
}

int plk_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!ms) return fail_msg(PLK_E_ARGUMENT, "plk_hip_event_elapsed_ms: null output");
  PLK_HIP_TRY(PLK_E_RESOURCE, hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return PLK_OK;
}

int plk_hip_event_destroy(void* event) {
  PLK_HIP_TRY(PLK_E_RELEASE, hipEventDestroy((hipEvent_t)event));
  return PLK_OK;
}

int plk_hip_module_load(const void* image, size_t bytes, plk_hip_module** out) {
  if (!image || !bytes || !out) return fail_msg(PLK_E_ARGUMENT, "plk_hip_module_load: null image or output");
  hipModule_t m;
  PLK_HIP_TRY(PLK_E_BUILD, hipModuleLoadData(&m, image));
  *out = new plk_hip_module{m, {}};
  return PLK_OK;
}

int plk_hip_module_unload(plk_hip_module* module) {
  if (!module) return PLK_OK;
  hipError_t e = hipModuleUnload(module->handle);
  for (plk_hip_function* f : module->functions) delete f;
  delete module;
  if (e != hipSuccess) return fail(PLK_E_RELEASE, "hipModuleUnload", e);
  return PLK_OK;
}

int plk_hip_module_function(plk_hip_module* module, const char* name, uint32_t dyn_lds_bytes,
                            plk_hip_function** out) {
  if (!module || !name || !out) return fail_msg(PLK_E_ARGUMENT, "plk_hip_module_function: null argument");
  hipFunction_t f;
  PLK_HIP_TRY(PLK_E_CONTRACT, hipModuleGetFunction(&f, module->handle, name));
  if (dyn_lds_bytes > 64 * 1024) {
    // Raising the limit is only needed (and only accepted) on runtimes that gate large dynamic LDS
    // behind the attribute; a refusal here is not an error, an oversized launch still reports one.
    if (hipFuncSetAttribute((const void*)f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn_lds_bytes) !=
        hipSuccess)
      (void)hipGetLastError();
  }
  module->functions.push_back(new plk_hip_function{f});
  *out = module->functions.back();
  return PLK_OK;
}

int plk_hip_launch(plk_hip_function* fn, const uint32_t grid[3], const uint32_t block[3], uint32_t dyn_lds_bytes,
                   void* stream, uint64_t params_addr) {
  if (!fn || !grid || !block) return fail_msg(PLK_E_ARGUMENT, "plk_hip_launch: null argument");
  if (!grid[0] || !grid[1] || !grid[2] || !block[0] || !block[1] || !block[2])
    return fail_msg(PLK_E_ARGUMENT, "plk_hip_launch: empty grid or block");
  if ((uint64_t)block[0] * block[1] * block[2] > 1024)
    return fail_msg(PLK_E_CAPACITY, "plk_hip_launch: more than 1024 threads per workgroup");
  if (dyn_lds_bytes > 160 * 1024) return fail_msg(PLK_E_CAPACITY, "plk_hip_launch: more than 160 KiB of LDS");
  void* arg = (void*)(uintptr_t)params_addr;
  size_t arg_bytes = sizeof arg;
  void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &arg, HIP_LAUNCH_PARAM_BUFFER_SIZE, &arg_bytes,
                    HIP_LAUNCH_PARAM_END};
  PLK_HIP_TRY(PLK_E_RESOURCE, hipModuleLaunchKernel(fn->handle, grid[0], grid[1], grid[2], block[0], block[1],
                                                    block[2], dyn_lds_bytes, (hipStream_t)stream, nullptr, config));
  return PLK_OK;
}

}  // extern "C"
