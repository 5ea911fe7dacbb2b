// Runtime half of the C ABI: device, stream, memory, events, error text and the
// per-launch profiler.  Replaces the CUDA-driver binding of src/ttir.ts:225-417.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "../../include/bunker_hip.h"
#include "ops.h"

namespace bk {

static thread_local char g_err[1024] = "";
static bool g_inited = false;
static int g_device = -1;
static hipStream_t g_stream = nullptr;         // the stream launches and copies go to (bk_stream_use)
static hipStream_t g_main_stream = nullptr;    // the one bk_init made
static std::vector<hipStream_t> g_extra_streams;
static int g_cus = 256;

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
hipStream_t stream() { return g_stream; }
// the host waits for every stream of the library
static int sync_all() {
  BK_HIP(hipStreamSynchronize(g_main_stream));
  for (hipStream_t st : g_extra_streams) BK_HIP(hipStreamSynchronize(st));
  return BK_OK;
}
int num_cus() { return g_cus; }
bool inited() { return g_inited; }
int current_device() { return g_device; }

// ---- profiler: an event pair around every bk_launch, summed per kernel label
struct ProfPending { hipEvent_t a, b; int kernel; };
static bool g_prof = false;
static std::vector<ProfPending> g_pending;
static std::vector<hipEvent_t> g_pool;
static std::map<std::string, std::pair<double, long>> g_totals;   // label -> (ms, count)

bool prof_on() { return g_prof; }
int prof_begin(int kernel) {
  hipEvent_t a, b;
  if (g_pool.size() >= 2) { a = g_pool.back(); g_pool.pop_back(); b = g_pool.back(); g_pool.pop_back(); }
  else { BK_HIP(hipEventCreate(&a)); BK_HIP(hipEventCreate(&b)); }
  BK_HIP(hipEventRecord(a, g_stream));
  g_pending.push_back({a, b, kernel});
  return BK_OK;
}
int prof_end() {
  BK_HIP(hipEventRecord(g_pending.back().b, g_stream));
  return BK_OK;
}
std::string kernel_label(int kernel);   // api.hip
void kernels_release_all();             // api.hip
static std::map<uint64_t, int> g_graph_nodes;     // executable graph (bk_capture_end) -> kernel nodes it holds
static void graphs_release_all() {
  for (auto& kv : g_graph_nodes) (void)hipGraphExecDestroy((hipGraphExec_t)(uintptr_t)kv.first);
  g_graph_nodes.clear();
}
static int prof_collect() {
  if (int rc = sync_all()) return rc;
  for (auto& p : g_pending) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
      auto& t = g_totals[kernel_label(p.kernel)];
      t.first += ms; t.second += 1;
    }
    g_pool.push_back(p.a); g_pool.push_back(p.b);
  }
  g_pending.clear();
  return BK_OK;
}

}  // namespace bk

using namespace bk;

#define BK_NEED_INIT() \
  do { if (!g_inited) return set_error(BK_ERR_STATE, "bk_init has not been called"); } while (0)

// Between bk_capture_begin and bk_capture_end only launches are recorded; anything else would either end the capture with
// an error of the runtime's or, for a memset, put a node into the graph that replays wrongly on this platform.
static bool g_capturing = false;
bool bk::capturing() { return g_capturing; }
#define BK_NOT_CAPTURING(name) \
  do { if (g_capturing) return set_error(BK_ERR_STATE, name ": not legal between bk_capture_begin and bk_capture_end"); } while (0)

extern "C" {

int bk_init(int device) {
  if (g_inited) {
    if (device == g_device) return BK_OK;
    return set_error(BK_ERR_STATE, "already initialised on device %d", g_device);
  }
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0)
    return set_error(BK_ERR_HIP, "no HIP device available (%s): the gfx950 kernels need an MI355X",
                     e != hipSuccess ? hipGetErrorString(e) : "device count 0");
  if (device < 0 || device >= n) return set_error(BK_ERR_ARG, "device %d out of range (0..%d)", device, n - 1);
  BK_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  BK_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(BK_ERR_UNSUPPORTED, "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
  g_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  if (int rc = attn_noalloc_setup(device)) return rc;      // with `device` current: the address of its built-in scratch array
  BK_HIP(hipStreamCreateWithFlags(&g_main_stream, hipStreamNonBlocking));
  g_stream = g_main_stream;
  g_device = device;
  g_inited = true;
  return BK_OK;
}

int bk_shutdown(void) {
  if (!g_inited) return BK_OK;
  (void)sync_all();
  graphs_release_all();                   // executable graphs of bk_capture_end that were never destroyed
  kernels_release_all();
  for (auto& p : g_pending) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  for (auto& ev : g_pool) (void)hipEventDestroy(ev);
  g_pending.clear(); g_pool.clear(); g_totals.clear();
  for (hipStream_t st : g_extra_streams) (void)hipStreamDestroy(st);
  g_extra_streams.clear();
  (void)hipStreamDestroy(g_main_stream);
  attn_noalloc_teardown(g_device);
  g_stream = g_main_stream = nullptr; g_inited = false; g_device = -1;
  return BK_OK;
}

const char* bk_last_error(void) { return g_err; }

int bk_device_info(char* buf, int cap) {
  BK_NEED_INIT();
  BK_REQUIRE(buf && cap > 0, "bk_device_info: bad buffer");
  hipDeviceProp_t prop;
  BK_HIP(hipGetDeviceProperties(&prop, g_device));
  // some driver stacks leave the marketing name empty: fall back to the architecture name
  snprintf(buf, cap, "%s|%s|%d|%zu", prop.name[0] ? prop.name : prop.gcnArchName, prop.gcnArchName, prop.multiProcessorCount,
           prop.totalGlobalMem);
  return BK_OK;
}

int bk_alloc(uint64_t bytes, uint64_t* out) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_alloc");
  BK_REQUIRE(out, "bk_alloc: null out");
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
  if (e != hipSuccess) return set_error(BK_ERR_HIP, "hipMalloc(%llu bytes) failed: %s", (unsigned long long)bytes, hipGetErrorString(e));
  *out = (uint64_t)(uintptr_t)p;
  return BK_OK;
}
int bk_free(uint64_t ptr) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_free");
  if (!ptr) return BK_OK;
  if (int rc = sync_all()) return rc;
  BK_HIP(hipFree((void*)(uintptr_t)ptr));
  return BK_OK;
}
// Copies are ordered with the kernels: they go through the library's stream and
// the call returns when the copy is complete, as cuMemcpyHtoD/DtoH do.
int bk_htod(uint64_t dst, const void* src, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_htod");
  BK_REQUIRE(dst && src, "bk_htod: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, g_stream));
  BK_HIP(hipStreamSynchronize(g_stream));
  return BK_OK;
}
int bk_dtoh(void* dst, uint64_t src, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_dtoh");
  BK_REQUIRE(dst && src, "bk_dtoh: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, g_stream));
  BK_HIP(hipStreamSynchronize(g_stream));
  return BK_OK;
}
int bk_dtod(uint64_t dst, uint64_t src, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_dtod");
  BK_REQUIRE(dst && src, "bk_dtod: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemcpyAsync((void*)(uintptr_t)dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToDevice, g_stream));
  return BK_OK;
}
// Pinned staging memory and copies that return before the data has moved (cuMemAllocHost /
// cuMemcpyHtoDAsync of the reference's loaders); the caller orders them with bk_sync or events.
int bk_host_alloc(uint64_t bytes, uint64_t* out) {
  BK_NEED_INIT();
  BK_REQUIRE(out && bytes, "bk_host_alloc: null pointer or zero size");
  void* p = nullptr;
  BK_HIP(hipHostMalloc(&p, bytes, hipHostMallocDefault));
  *out = (uint64_t)(uintptr_t)p;
  return BK_OK;
}
int bk_host_free(uint64_t ptr) {
  BK_NEED_INIT();
  if (!ptr) return BK_OK;
  BK_HIP(hipHostFree((void*)(uintptr_t)ptr));
  return BK_OK;
}
int bk_htod_async(uint64_t dst, const void* src, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_htod_async");
  BK_REQUIRE(dst && src, "bk_htod_async: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, g_stream));
  return BK_OK;
}
int bk_dtoh_async(void* dst, uint64_t src, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_dtoh_async");
  BK_REQUIRE(dst && src, "bk_dtoh_async: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, g_stream));
  return BK_OK;
}
int bk_event_sync(uint64_t ev) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_event_sync");
  BK_REQUIRE(ev, "bk_event_sync: null event");
  BK_HIP(hipEventSynchronize((hipEvent_t)(uintptr_t)ev));
  return BK_OK;
}
int bk_memset(uint64_t dst, int value, uint64_t bytes) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_memset");
  BK_REQUIRE(dst, "bk_memset: null pointer");
  if (!bytes) return BK_OK;
  BK_HIP(hipMemsetAsync((void*)(uintptr_t)dst, value, bytes, g_stream));
  return BK_OK;
}
int bk_sync(void) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_sync");
  return sync_all();
}

// Further streams (default priority) for work that may overlap: launches, copies and event records go to the stream
// selected last; the order between streams is the caller's, through events.
int bk_stream_create(uint64_t* out) {
  BK_NEED_INIT();
  BK_REQUIRE(out, "bk_stream_create: null out");
  hipStream_t st;
  BK_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  g_extra_streams.push_back(st);
  *out = (uint64_t)(uintptr_t)st;
  return BK_OK;
}
static int find_stream(uint64_t s) {
  for (size_t i = 0; i < g_extra_streams.size(); i++)
    if ((uint64_t)(uintptr_t)g_extra_streams[i] == s) return (int)i;
  return -1;
}
int bk_stream_use(uint64_t s) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_stream_use");
  if (!s) { g_stream = g_main_stream; return BK_OK; }
  const int i = find_stream(s);
  BK_REQUIRE(i >= 0, "bk_stream_use: not a stream of bk_stream_create");
  g_stream = g_extra_streams[i];
  return BK_OK;
}
int bk_stream_wait_event(uint64_t ev) {
  BK_NEED_INIT();
  BK_REQUIRE(ev, "bk_stream_wait_event: null event");
  BK_HIP(hipStreamWaitEvent(g_stream, (hipEvent_t)(uintptr_t)ev, 0));
  return BK_OK;
}
int bk_stream_destroy(uint64_t s) {
  BK_NEED_INIT();
  const int i = find_stream(s);
  BK_REQUIRE(i >= 0, "bk_stream_destroy: not a stream of bk_stream_create");
  BK_HIP(hipStreamSynchronize(g_extra_streams[i]));
  if (g_stream == g_extra_streams[i]) g_stream = g_main_stream;
  BK_HIP(hipStreamDestroy(g_extra_streams[i]));
  g_extra_streams.erase(g_extra_streams.begin() + i);
  return BK_OK;
}

int bk_event_create(uint64_t* out) {
  BK_NEED_INIT();
  BK_REQUIRE(out, "bk_event_create: null out");
  hipEvent_t ev;
  BK_HIP(hipEventCreate(&ev));
  *out = (uint64_t)(uintptr_t)ev;
  return BK_OK;
}
int bk_event_record(uint64_t ev) {
  BK_NEED_INIT();
  BK_REQUIRE(ev, "bk_event_record: null event");
  BK_HIP(hipEventRecord((hipEvent_t)(uintptr_t)ev, g_stream));
  return BK_OK;
}
int bk_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms) {
  BK_NEED_INIT();
  BK_REQUIRE(start && stop && ms, "bk_event_elapsed_ms: null argument");
  BK_HIP(hipEventSynchronize((hipEvent_t)(uintptr_t)stop));
  BK_HIP(hipEventElapsedTime(ms, (hipEvent_t)(uintptr_t)start, (hipEvent_t)(uintptr_t)stop));
  return BK_OK;
}
int bk_event_destroy(uint64_t ev) {
  BK_NEED_INIT();
  if (ev) BK_HIP(hipEventDestroy((hipEvent_t)(uintptr_t)ev));
  return BK_OK;
}


int bk_capture_begin(void) {
  BK_NEED_INIT();
  if (g_capturing) return set_error(BK_ERR_STATE, "bk_capture_begin: a capture is already open");
  if (g_prof) return set_error(BK_ERR_STATE, "bk_capture_begin: switch the per-launch profiler off first");
  BK_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
  g_capturing = true;
  return BK_OK;
}
int bk_capture_end(uint64_t* graph) {
  BK_NEED_INIT();
  BK_REQUIRE(graph, "bk_capture_end: null out");
  if (!g_capturing) return set_error(BK_ERR_STATE, "bk_capture_end: no capture is open");
  g_capturing = false;
  hipGraph_t g = nullptr;
  BK_HIP(hipStreamEndCapture(g_stream, &g));
  size_t n_nodes = 0;
  (void)hipGraphGetNodes(g, nullptr, &n_nodes);
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) return set_error(BK_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  *graph = (uint64_t)(uintptr_t)exec;
  g_graph_nodes[*graph] = (int)n_nodes;
  return BK_OK;
}
int bk_graph_node_count(uint64_t graph, int* count) {
  BK_NEED_INIT();
  BK_REQUIRE(count, "bk_graph_node_count: null out");
  const auto it = g_graph_nodes.find(graph);
  if (it == g_graph_nodes.end()) return set_error(BK_ERR_ARG, "bk_graph_node_count: not a graph of bk_capture_end");
  *count = it->second;
  return BK_OK;
}
int bk_graph_launch(uint64_t graph) {
  BK_NEED_INIT();
  BK_NOT_CAPTURING("bk_graph_launch");
  BK_REQUIRE(graph, "bk_graph_launch: null graph");
  BK_HIP(hipGraphLaunch((hipGraphExec_t)(uintptr_t)graph, g_stream));
  return BK_OK;
}
int bk_graph_destroy(uint64_t graph) {
  BK_NEED_INIT();
  if (graph) BK_HIP(hipGraphExecDestroy((hipGraphExec_t)(uintptr_t)graph));
  g_graph_nodes.erase(graph);
  return BK_OK;
}

int bk_prof_enable(int on) { g_prof = on != 0; return BK_OK; }
int bk_prof_reset(void) {
  BK_NEED_INIT();
  int rc = prof_collect();
  g_totals.clear();
  return rc;
}
int bk_prof_report(char* buf, int cap) {
  BK_NEED_INIT();
  BK_REQUIRE(buf && cap > 0, "bk_prof_report: bad buffer");
  int rc = prof_collect();
  if (rc) return rc;
  std::vector<std::pair<std::string, std::pair<double, long>>> rows(g_totals.begin(), g_totals.end());
  for (size_t i = 0; i < rows.size(); i++)
    for (size_t j = i + 1; j < rows.size(); j++)
      if (rows[j].second.first > rows[i].second.first) std::swap(rows[i], rows[j]);
  double total = 0;
  for (auto& r : rows) total += r.second.first;
  int off = snprintf(buf, cap, "kernel elapsed (library stream), total %.3f ms\n", total);
  for (auto& r : rows) {
    if (off >= cap - 1) break;
    off += snprintf(buf + off, cap - off, "%10.3f ms %5.1f%% x%-6ld avg %8.2f us  %s\n", r.second.first,
                    total > 0 ? 100.0 * r.second.first / total : 0.0, r.second.second,
                    1000.0 * r.second.first / (double)r.second.second, r.first.c_str());
  }
  return BK_OK;
}

}  // extern "C"
