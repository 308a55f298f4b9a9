// Thin C-ABI layer over the HIP runtime and hipRTC.  It is the only
// translation unit that includes HIP headers; host code above it calls these
// functions with plain C types.  It stands in for what upstream does with
// system("./make_template.sh") + system("./a.out") (executor.cc:6-104) and for
// the cudaMalloc / cudaMemcpy / kernel-launch text it generates
// (code_builder.cc:1471-1575).
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstring>
#include <chrono>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/alphasparse_amd.h"

static thread_local std::string g_hip_err;
static int fail(const std::string &what, const char *detail) {
  g_hip_err = what + ": " + (detail ? detail : "?");
  return -1;
}
#define HIP_TRY(expr)                                            \
  do {                                                           \
    hipError_t e_ = (expr);                                      \
    if (e_ != hipSuccess) return fail(#expr, hipGetErrorString(e_)); \
  } while (0)

// Device memory that the library holds from its first upload on a GPU until the process ends, for the one entry
// point that must not allocate (as_builder_spmv_device_no_alloc): the kernels' scratch arrays are carved out of
// it instead of out of allocations of the builder.  Host code never uses the array's name as an address (on the
// host it is only a stand-in for the symbol): as_hip_static_scratch asks the runtime for the address the array has
// on the current GPU and hands that pointer out.  Every GPU has its own copy at its own address.
// (No `used` attribute on it: with that attribute the compiler keeps the device-side symbol local to the code
// object instead of exporting it for the host's lookup, and hipGetSymbolAddress cannot find it.)
static __device__ __align__(256) unsigned char scratch[AS_STATIC_SCRATCH_BYTES];
static const int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

extern "C" {

const char *as_hip_last_error(void) { return g_hip_err.c_str(); }

// Address and size of the static scratch array on `device` (looked up once per device, with that device
// current; later calls return the kept pointer and touch no HIP state).
int as_hip_static_scratch(int device, void **ptr, uint64_t *bytes) {
  if (device < 0 || device >= kMaxDevices || !ptr) return fail("as_hip_static_scratch", "bad device");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    int current = -1;
    HIP_TRY(hipGetDevice(&current));
    if (current != device) HIP_TRY(hipSetDevice(device));
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (current != device) (void)hipSetDevice(current);
    if (e != hipSuccess || !p) return fail("hipGetSymbolAddress(scratch)", hipGetErrorString(e));
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  if (bytes) *bytes = AS_STATIC_SCRATCH_BYTES;
  return 0;
}

int as_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int as_hip_init(int device) {
  HIP_TRY(hipSetDevice(device));
  HIP_TRY(hipFree(nullptr));
  return 0;
}

int as_hip_device_info(int device, char *name, int name_cap, int *cu_count, int *wave_size, uint64_t *lds_per_block,
                       uint64_t *global_mem) {
  hipDeviceProp_t p;
  HIP_TRY(hipGetDeviceProperties(&p, device));
  if (name && name_cap > 0) snprintf(name, name_cap, "%s (%s)", p.name, p.gcnArchName);
  if (cu_count) *cu_count = p.multiProcessorCount;
  if (wave_size) *wave_size = p.warpSize;
  if (lds_per_block) *lds_per_block = p.sharedMemPerBlock;
  if (global_mem) *global_mem = p.totalGlobalMem;
  return 0;
}

// hipRTC: source -> gfx950 code object.  Needs no GPU.  *code is malloc'ed.
int as_hip_compile(const char *src, const char *arch, const char *const *opts, int n_opts, void **code,
                   uint64_t *code_size, char **log) {
  if (log) *log = nullptr;
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, src, "spmv_module.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail("hiprtcCreateProgram", hiprtcGetErrorString(r));
  std::vector<const char *> o;
  std::string a = std::string("--offload-arch=") + (arch ? arch : "gfx950");
  o.push_back(a.c_str());
  o.push_back("-O3");
  o.push_back("-munsafe-fp-atomics");
  // packed-FP32 instructions are kept out of every code object
  o.push_back("-Xclang"); o.push_back("-target-feature"); o.push_back("-Xclang"); o.push_back("-packed-fp32-ops");
  for (int i = 0; i < n_opts; i++) o.push_back(opts[i]);
  r = hiprtcCompileProgram(prog, (int)o.size(), o.data());
  size_t ls = 0;
  hiprtcGetProgramLogSize(prog, &ls);
  if (log && ls > 1) {
    *log = (char *)malloc(ls + 1);
    hiprtcGetProgramLog(prog, *log);
    (*log)[ls] = 0;
  }
  if (r != HIPRTC_SUCCESS) {
    std::string l = (log && *log) ? *log : "";
    hiprtcDestroyProgram(&prog);
    return fail("hiprtcCompileProgram", (std::string(hiprtcGetErrorString(r)) + "\n" + l).c_str());
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  *code = malloc(cs);
  hiprtcGetCode(prog, (char *)*code);
  *code_size = cs;
  hiprtcDestroyProgram(&prog);
  return 0;
}

void as_hip_free_host(void *p) { free(p); }

int as_hip_module_load(const void *code, void **module) {
  hipModule_t m;
  HIP_TRY(hipModuleLoadData(&m, code));
  *module = (void *)m;
  return 0;
}
int as_hip_module_unload(void *module) {
  HIP_TRY(hipModuleUnload((hipModule_t)module));
  return 0;
}
int as_hip_get_kernel(void *module, const char *name, void **fn) {
  hipFunction_t f;
  HIP_TRY(hipModuleGetFunction(&f, (hipModule_t)module, name));
  *fn = (void *)f;
  return 0;
}

int as_hip_alloc(void **p, uint64_t bytes) {
  HIP_TRY(hipMalloc(p, bytes ? bytes : 4));
  return 0;
}
int as_hip_free(void *p) {
  HIP_TRY(hipFree(p));
  return 0;
}
int as_hip_h2d(void *dst, const void *src, uint64_t bytes) {
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return 0;
}
int as_hip_d2h(void *dst, const void *src, uint64_t bytes) {
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return 0;
}
int as_hip_memset_async(void *dst, int value, uint64_t bytes, void *stream) {
  HIP_TRY(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
  return 0;
}
int as_hip_stream_create(void **stream) {
  hipStream_t s;
  HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void *)s;
  return 0;
}
int as_hip_stream_destroy(void *stream) {
  HIP_TRY(hipStreamDestroy((hipStream_t)stream));
  return 0;
}
int as_hip_stream_sync(void *stream) {
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}
int as_hip_device_sync(void) {
  HIP_TRY(hipDeviceSynchronize());
  return 0;
}
int as_hip_event_create(void **ev) {
  hipEvent_t e;
  HIP_TRY(hipEventCreate(&e));
  *ev = (void *)e;
  return 0;
}
int as_hip_event_destroy(void *ev) {
  HIP_TRY(hipEventDestroy((hipEvent_t)ev));
  return 0;
}
int as_hip_event_record(void *ev, void *stream) {
  HIP_TRY(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
  return 0;
}
// Waits for an event.  The first half millisecond by polling: a blocked host thread is woken tens of microseconds
// after the event, which is a fifth of a timed region of twenty 17-us launches; after that it blocks.
int as_hip_event_sync(void *ev) {
  const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(500);
  for (;;) {
    const hipError_t e = hipEventQuery((hipEvent_t)ev);
    if (e == hipSuccess) return 0;
    if (e != hipErrorNotReady) HIP_TRY(e);
    if (std::chrono::steady_clock::now() >= until) break;
  }
  HIP_TRY(hipEventSynchronize((hipEvent_t)ev));
  return 0;
}
int as_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
  HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}
// make `stream` wait for `ev`
// Stream capture into a graph, for callers that replay a fixed sequence of launches (and for the test that the
// enqueue-only SpMV calls can be captured).  Capture mode "thread local": only this thread's calls are checked.
int as_hip_graph_capture_begin(void *stream) {
  HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return 0;
}
int as_hip_graph_capture_end(void *stream, void **graph_exec) {
  hipGraph_t g = nullptr;
  HIP_TRY(hipStreamEndCapture((hipStream_t)stream, &g));
  hipGraphExec_t e = nullptr;
  hipError_t r = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (r != hipSuccess) return fail("hipGraphInstantiate", hipGetErrorString(r));
  *graph_exec = e;
  return 0;
}
int as_hip_graph_launch(void *graph_exec, void *stream) {
  HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return 0;
}
int as_hip_graph_destroy(void *graph_exec) {
  HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return 0;
}
int as_hip_mem_info(uint64_t *free_bytes, uint64_t *total_bytes) {
  size_t f = 0, t = 0;
  HIP_TRY(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return 0;
}

int as_hip_stream_wait_event(void *stream, void *ev) {
  HIP_TRY(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)ev, 0));
  return 0;
}

int as_hip_launch(void *fn, unsigned grid, unsigned block, unsigned lds_bytes, void *stream, void **args) {
  if (grid == 0 || block == 0 || block > 1024) return fail("as_hip_launch", "bad launch shape");
  HIP_TRY(hipModuleLaunchKernel((hipFunction_t)fn, grid, 1, 1, block, 1, 1, lds_bytes, (hipStream_t)stream, args,
                                nullptr));
  return 0;
}

}  // extern "C"
