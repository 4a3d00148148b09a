// Error text, version, and thin wrappers for stream capture into HIP graphs.
#include "common.h"

#include <stdarg.h>
#include <string.h>

static thread_local char g_error[512] = "";

void lq_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* lq_last_error() { return g_error; }

extern "C" int lq_abi_version() { return 5; }

// Compute units of the current device (256 if the runtime will not say).
int lq_compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}

// ---- HIP graphs: capture what a step launches on `stream`, replay it later ----
// Captured steps must not allocate and must not record memsets; the library's
// kernels obey both (buffers are cleared by fill kernels).

extern "C" int lq_graph_begin(hipStream_t stream) {
  hipError_t e = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal);
  LQ_REQUIRE(e == hipSuccess, "graph_begin: %s", hipGetErrorString(e));
  return 0;
}

extern "C" int lq_graph_end(hipStream_t stream, void** exec_out) {
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(stream, &graph);
  LQ_REQUIRE(e == hipSuccess && graph != nullptr, "graph_end: %s", hipGetErrorString(e));
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  LQ_REQUIRE(e == hipSuccess, "graph_instantiate: %s", hipGetErrorString(e));
  *exec_out = (void*)exec;
  return 0;
}

extern "C" int lq_graph_launch(void* exec, hipStream_t stream) {
  hipError_t e = hipGraphLaunch((hipGraphExec_t)exec, stream);
  LQ_REQUIRE(e == hipSuccess, "graph_launch: %s", hipGetErrorString(e));
  return 0;
}

extern "C" int lq_graph_destroy(void* exec) {
  hipError_t e = hipGraphExecDestroy((hipGraphExec_t)exec);
  LQ_REQUIRE(e == hipSuccess, "graph_destroy: %s", hipGetErrorString(e));
  return 0;
}
