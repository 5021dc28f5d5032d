// HIP side of the C-ABI layer: device, memory, streams/events, runtime compilation.
#include "hip_abi.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {
thread_local std::string g_err;

int fail(hipError_t e, const char* what) {
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return (int)e;
}
#define HIPCHK(call)                        \
  do {                                      \
    hipError_t e_ = (call);                 \
    if (e_ != hipSuccess) return fail(e_, #call); \
  } while (0)
}  // namespace

extern "C" {

const char* mi355_last_error(void) { return g_err.c_str(); }

int mi355_device_count(int* count) {
  *count = 0;
  HIPCHK(hipGetDeviceCount(count));
  return 0;
}

int mi355_device_init(int device, char* name, size_t name_len, char* arch, size_t arch_len, int* compute_units,
                      size_t* total_mem) {
  HIPCHK(hipSetDevice(device));
  hipDeviceProp_t p;
  HIPCHK(hipGetDeviceProperties(&p, device));
  snprintf(name, name_len, "%s", p.name);
  snprintf(arch, arch_len, "%s", p.gcnArchName);
  *compute_units = p.multiProcessorCount;
  *total_mem = p.totalGlobalMem;
  return 0;
}

int mi355_mem_info(size_t* free_bytes, size_t* total_bytes) {
  HIPCHK(hipMemGetInfo(free_bytes, total_bytes));
  return 0;
}

int mi355_malloc(void** ptr, size_t bytes) {
  HIPCHK(hipMalloc(ptr, bytes));
  return 0;
}
int mi355_free(void* ptr) {
  HIPCHK(hipFree(ptr));
  return 0;
}
int mi355_host_alloc(void** ptr, size_t bytes) {
  HIPCHK(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return 0;
}
int mi355_host_free(void* ptr) {
  HIPCHK(hipHostFree(ptr));
  return 0;
}
int mi355_memcpy_h2d(void* dst, const void* src, size_t bytes, mi355_stream_t s) {
  HIPCHK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)s));
  return 0;
}
int mi355_memcpy_d2h(void* dst, const void* src, size_t bytes, mi355_stream_t s) {
  HIPCHK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)s));
  return 0;
}
int mi355_memcpy_d2d(void* dst, const void* src, size_t bytes, mi355_stream_t s) {
  HIPCHK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)s));
  return 0;
}

int mi355_stream_create(mi355_stream_t* s) {
  hipStream_t st;
  HIPCHK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  *s = (mi355_stream_t)st;
  return 0;
}
int mi355_stream_destroy(mi355_stream_t s) {
  HIPCHK(hipStreamDestroy((hipStream_t)s));
  return 0;
}
int mi355_stream_sync(mi355_stream_t s) {
  HIPCHK(hipStreamSynchronize((hipStream_t)s));
  return 0;
}
int mi355_capture_begin(mi355_stream_t s) {
  HIPCHK(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal));
  return 0;
}
int mi355_capture_end(mi355_stream_t s, mi355_graph_t* exec, int* num_nodes) {
  hipGraph_t graph = nullptr;
  HIPCHK(hipStreamEndCapture((hipStream_t)s, &graph));
  if (!graph) return 1;
  size_t n = 0;
  if (hipGraphGetNodes(graph, nullptr, &n) != hipSuccess) n = 0;
  if (num_nodes) *num_nodes = (int)n;
  hipGraphExec_t ge = nullptr;
  hipError_t e = hipGraphInstantiate(&ge, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return fail(e, "hipGraphInstantiate");
  *exec = (mi355_graph_t)ge;
  return 0;
}
int mi355_graph_launch(mi355_graph_t exec, mi355_stream_t s) {
  HIPCHK(hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)s));
  return 0;
}
int mi355_graph_destroy(mi355_graph_t exec) {
  HIPCHK(hipGraphExecDestroy((hipGraphExec_t)exec));
  return 0;
}

int mi355_event_create(mi355_event_t* e, int timing) {
  hipEvent_t ev;
  HIPCHK(hipEventCreateWithFlags(&ev, timing ? hipEventDefault : hipEventDisableTiming));
  *e = (mi355_event_t)ev;
  return 0;
}
int mi355_event_destroy(mi355_event_t e) {
  HIPCHK(hipEventDestroy((hipEvent_t)e));
  return 0;
}
int mi355_event_record(mi355_event_t e, mi355_stream_t s) {
  HIPCHK(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
  return 0;
}
int mi355_stream_wait_event(mi355_stream_t s, mi355_event_t e) {
  HIPCHK(hipStreamWaitEvent((hipStream_t)s, (hipEvent_t)e, 0));
  return 0;
}
int mi355_event_sync(mi355_event_t e) {
  HIPCHK(hipEventSynchronize((hipEvent_t)e));
  return 0;
}
int mi355_event_query(mi355_event_t e, int* ready) {
  hipError_t r = hipEventQuery((hipEvent_t)e);
  if (r == hipSuccess) { *ready = 1; return 0; }
  if (r == hipErrorNotReady) { *ready = 0; (void)hipGetLastError(); return 0; }
  return fail(r, "hipEventQuery");
}
int mi355_event_elapsed_ms(mi355_event_t a, mi355_event_t b, float* ms) {
  HIPCHK(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b));
  return 0;
}

const char* mi355_rtc_fingerprint(void) {
  static char buf[96];
  if (!buf[0]) {
    int major = 0, minor = 0;
    if (hiprtcVersion(&major, &minor) != HIPRTC_SUCCESS) major = minor = -1;
    snprintf(buf, sizeof buf, "hiprtc-%d.%d -O3 -ffp-contract=off -packed-fp32-ops wrapping-ints", major, minor);
  }
  return buf;
}

int mi355_rtc_compile(const char* source, const char* arch, char** code, size_t* code_size, char* log, size_t log_len) {
  hiprtcProgram prog;
  if (log && log_len) log[0] = 0;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, "fused.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) { g_err = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r); return 1; }
  std::string archOpt = std::string("--offload-arch=") + arch;
  // packed-fp32 instructions are switched off for every kernel of this library
  const char* opts[] = {archOpt.c_str(), "-O3", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, 7, opts);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string l(n, 0);
    if (n) hiprtcGetProgramLog(prog, &l[0]);
    if (log && log_len) snprintf(log, log_len, "%s", l.c_str());
    g_err = std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + l;
    hiprtcDestroyProgram(&prog);
    return 2;
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  char* buf = (char*)malloc(cs);
  hiprtcGetCode(prog, buf);
  hiprtcDestroyProgram(&prog);
  *code = buf;
  *code_size = cs;
  return 0;
}

int mi355_module_load(const char* code, mi355_function_t* fn) {
  hipModule_t mod;
  HIPCHK(hipModuleLoadData(&mod, code));
  hipFunction_t f;
  HIPCHK(hipModuleGetFunction(&f, mod, "k"));
  *fn = (mi355_function_t)f;
  return 0;
}

int mi355_launch(mi355_function_t fn, const unsigned grid[3], const unsigned block[3], void** arg_ptrs, int num_args,
                 mi355_stream_t s) {
  (void)num_args;
  HIPCHK(hipModuleLaunchKernel((hipFunction_t)fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                               (hipStream_t)s, arg_ptrs, nullptr));
  return 0;
}

}  // extern "C"
