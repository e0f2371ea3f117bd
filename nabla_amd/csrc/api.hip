// Library lifecycle, error channel, timing helpers and the custom-kernel loader.
#include "nbk_common.h"
#include <dlfcn.h>
#include <string.h>
#include <mutex>
#include <map>
#include <string>

static thread_local char g_err[512] = "";

void nbk_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static int g_num_cus = 0;  // written once with the same value by whoever gets there first
int nbk_num_cus(void) {
  if (g_num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_num_cus = n;
    else
      g_num_cus = 256;
  }
  return g_num_cus;
}

extern "C" const char* nbk_last_error(void) { return g_err; }
extern "C" int nbk_abi_version(void) { return NBK_ABI_VERSION; }

extern "C" int nbk_init(int device) {
  int n = 0;
  NBK_HIP(hipGetDeviceCount(&n));
  NBK_REQUIRE(device >= 0 && device < n, "nbk_init: device %d not in [0, %d)", device, n);
  NBK_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  NBK_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    nbk_set_error("nbk_init: device %d is %s; this library only carries gfx950 code", device,
                  prop.gcnArchName);
    return NBK_ERR_UNSUPPORTED;
  }
  return nbk_attention_static_setup();
}

// ---- events / stream sync ---------------------------------------------------
extern "C" int nbk_event_create(void** ev) {
  NBK_REQUIRE(ev != nullptr, "nbk_event_create: null out pointer");
  hipEvent_t e;
  NBK_HIP(hipEventCreate(&e));
  *ev = (void*)e;
  return NBK_OK;
}
extern "C" int nbk_event_record(void* ev, void* stream) {
  NBK_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
  return NBK_OK;
}
extern "C" int nbk_event_elapsed_ms(void* start, void* stop, float* ms) {
  NBK_REQUIRE(ms != nullptr, "nbk_event_elapsed_ms: null out pointer");
  NBK_HIP(hipEventSynchronize((hipEvent_t)stop));
  NBK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return NBK_OK;
}
extern "C" int nbk_event_destroy(void* ev) {
  NBK_HIP(hipEventDestroy((hipEvent_t)ev));
  return NBK_OK;
}
extern "C" int nbk_stream_sync(void* stream) {
  NBK_HIP(hipStreamSynchronize((hipStream_t)stream));
  return NBK_OK;
}

// ---- plan replay as a HIP graph -------------------------------------------------
extern "C" int nbk_stream_create(void** stream) {
  NBK_REQUIRE(stream != nullptr, "nbk_stream_create: null out pointer");
  hipStream_t s;
  NBK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void*)s;
  return NBK_OK;
}
extern "C" int nbk_stream_destroy(void* stream) {
  NBK_HIP(hipStreamDestroy((hipStream_t)stream));
  return NBK_OK;
}
extern "C" int nbk_graph_begin_capture(void* stream) {
  NBK_REQUIRE(stream != nullptr, "nbk_graph_begin_capture: the default stream cannot record");
  NBK_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return NBK_OK;
}
extern "C" int nbk_graph_end_capture(void* stream, void** graph_exec) {
  NBK_REQUIRE(graph_exec != nullptr, "nbk_graph_end_capture: null out pointer");
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  NBK_HIP(hipStreamEndCapture((hipStream_t)stream, &graph));
  NBK_REQUIRE(graph != nullptr, "nbk_graph_end_capture: the capture was invalidated");
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    nbk_set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
    return NBK_ERR_LAUNCH;
  }
  *graph_exec = (void*)exec;
  return NBK_OK;
}
extern "C" int nbk_graph_launch(void* graph_exec, void* stream) {
  NBK_REQUIRE(graph_exec != nullptr, "nbk_graph_launch: null graph");
  NBK_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return NBK_OK;
}
extern "C" int nbk_graph_destroy(void* graph_exec) {
  if (graph_exec) NBK_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return NBK_OK;
}

// ---- custom kernels -----------------------------------------------------------
// Libraries stay loaded for the life of the process; the handle table is the
// only mutable global and is guarded by a mutex.
static std::mutex g_lib_mu;
static std::map<std::string, void*> g_libs;

extern "C" int nbk_custom(const char* library_path, const char* name, const nbk_tensor* in,
                          int n_in, nbk_tensor* out, int n_out, void* stream) {
  NBK_REQUIRE(library_path && name, "nbk_custom: null library path or kernel name");
  NBK_REQUIRE(n_in >= 0 && n_out >= 1, "nbk_custom: needs at least one output");
  void* h = nullptr;
  {
    std::lock_guard<std::mutex> lk(g_lib_mu);
    auto it = g_libs.find(library_path);
    if (it == g_libs.end()) {
      h = dlopen(library_path, RTLD_NOW | RTLD_LOCAL);
      if (!h) {
        nbk_set_error("nbk_custom: cannot load '%s': %s", library_path, dlerror());
        return NBK_ERR_INVALID;
      }
      g_libs[library_path] = h;
    } else {
      h = it->second;
    }
  }
  nbk_custom_fn fn = (nbk_custom_fn)dlsym(h, name);
  if (!fn) {
    nbk_set_error("nbk_custom: kernel '%s' is not exported by '%s'", name, library_path);
    return NBK_ERR_INVALID;
  }
  int rc = fn(in, n_in, out, n_out, stream);
  if (rc != 0) {
    nbk_set_error("nbk_custom: kernel '%s' returned %d", name, rc);
    return NBK_ERR_LAUNCH;
  }
  return nbk_check_launch(name);
}
