// Device, memory and stream entry points of the C ABI.
#include <cstring>
#include <mutex>

#include "dh_common.h"

namespace {
std::mutex g_mu;
thread_local char g_err[1024] = "";
bool g_ready = false;
int g_device = -1;
hipStream_t g_own_stream = nullptr;
hipStream_t g_stream = nullptr;
int g_num_cus = 0;
dh::Graph* g_capturing = nullptr;     // graph being captured on g_stream
float* g_splitk_ws = nullptr;        // partial products of the split-K prefill GEMM
constexpr size_t kSplitKWsBytes = (size_t)32 << 20;
float* g_row_scale = nullptr;        // [kRowScaleRows][2] activation row factors of the prefill GEMM
constexpr int kRowScaleRows = 65536;
void* g_packed_a = nullptr;          // packed f16 activations of the prefill GEMM
constexpr size_t kPackedABytes = (size_t)64 << 20;
float* g_widened_a = nullptr;        // f16 activations of dh_q4k_matmul widened to f32
constexpr size_t kWidenedABytes = (size_t)64 << 20;
uint32_t* g_kstatus = nullptr;       // kernel status word: pinned host memory, device-writable
thread_local int t_plan_cus = 0;      // > 0: a plan is being made on this thread for a device of that many compute units
thread_local int t_plan_family = 0;
thread_local int64_t t_plan_layout[16] = {};
}  // namespace

namespace dh {
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
hipStream_t stream() { return g_stream; }
bool ready() { return g_ready || t_plan_cus > 0; }
int num_cus() { return t_plan_cus > 0 ? t_plan_cus : g_num_cus; }
void plan_begin(int cus) {
  t_plan_cus = cus;
  t_plan_family = 0;
  for (auto& v : t_plan_layout) v = 0;
}
void plan_layout(int i, int64_t value) {
  // the first launch of a call describes it (further passes repeat it)
  if (t_plan_cus > 0 && t_plan_family == 0 && i >= 0 && i < 16) t_plan_layout[i] = value;
}
const int64_t* plan_layout_record() { return t_plan_layout; }
int plan_end() {
  t_plan_cus = 0;
  return t_plan_family;
}
bool plan_note(int family) {
  if (t_plan_cus <= 0) return false;
  if (t_plan_family == 0) t_plan_family = family;
  return true;
}
Graph* capturing_graph() { return g_capturing; }
void graph_note_attention(const GraphAttnCall& call) {
  Graph* g = g_capturing;
  if (!g) return;
  if (g->n_attn == g->cap_attn) {
    const int cap = g->cap_attn ? 2 * g->cap_attn : 64;
    GraphAttnCall* grown = new GraphAttnCall[cap];
    for (int i = 0; i < g->n_attn; i++) grown[i] = g->attn[i];
    delete[] g->attn;
    g->attn = grown;
    g->cap_attn = cap;
  }
  g->attn[g->n_attn++] = call;
}
void graph_note_finiteness(const GraphFiniteCall& call) {
  Graph* g = g_capturing;
  if (!g) return;
  if (g->n_fin == g->cap_fin) {
    const int cap = g->cap_fin ? 2 * g->cap_fin : 64;
    GraphFiniteCall* grown = new GraphFiniteCall[cap];
    for (int i = 0; i < g->n_fin; i++) grown[i] = g->fin[i];
    delete[] g->fin;
    g->fin = grown;
    g->cap_fin = cap;
  }
  g->fin[g->n_fin++] = call;
}
float* splitk_workspace(size_t* bytes) {
  *bytes = g_splitk_ws ? kSplitKWsBytes : 0;
  return g_splitk_ws;
}
float* gemm_row_scale() { return g_row_scale; }
void* gemm_packed_a(size_t* bytes) {
  *bytes = g_packed_a ? kPackedABytes : 0;
  return g_packed_a;
}
int gemm_row_scale_capacity() { return kRowScaleRows; }
float* widened_activations(size_t* bytes) {
  *bytes = g_widened_a ? kWidenedABytes : 0;
  return g_widened_a;
}
uint32_t* kernel_status_word() { return g_kstatus; }
int check_kernel_status(const char* op) {
  if (!g_kstatus) return 0;
  const uint32_t code = *static_cast<volatile uint32_t*>(g_kstatus);
  if (code == 0u) return 0;
  *static_cast<volatile uint32_t*>(g_kstatus) = 0u;
  gemv_chain_reset();
  const uint32_t kind = code >> 28, phase = (code >> 24) & 0xFu, block = code & 0xFFFFFFu;
  const char* what = kind == DH_KSTATUS_COLUMN_WAIT ? "a column's activation operands did not arrive (Q4_K GEMV)"
                     : kind == DH_KSTATUS_SLOT_WAIT ? "a tile slot was not released (Q4_K GEMV)"
                     : kind == DH_KSTATUS_EXCHANGE_WAIT ? "the previous product's outputs did not arrive from the other workgroups (chained Q4_K GEMV)"
                                                        : "unknown wait";
  return fail(3, "[%s] a kernel launched earlier gave up a bounded wait: %s; phase %u, workgroup %u; its outputs are "
              "undefined", op, what, phase, block);
}
}  // namespace dh

extern "C" {

const char* dh_last_error(void) { return g_err; }

// Frees whatever dh_init has allocated so far and returns the runtime to its unset state; the
// first failing call is the one reported.
static int release_all(const char* op) {
  hipError_t first = hipSuccess;
  auto note = [&](hipError_t e) {
    if (first == hipSuccess) first = e;
  };
  if (g_capturing) {
    // a capture left open: end it so the stream can be destroyed, and drop what it recorded
    hipGraph_t abandoned = nullptr;
    if (g_stream) (void)hipStreamEndCapture(g_stream, &abandoned);
    if (abandoned) (void)hipGraphDestroy(abandoned);
    delete[] g_capturing->attn;
    delete[] g_capturing->fin;
    delete g_capturing;
    g_capturing = nullptr;
  }
  if (g_own_stream) note(hipStreamDestroy(g_own_stream));
  if (g_splitk_ws) note(hipFree(g_splitk_ws));
  if (g_row_scale) note(hipFree(g_row_scale));
  if (g_packed_a) note(hipFree(g_packed_a));
  if (g_widened_a) note(hipFree(g_widened_a));
  if (g_kstatus) note(hipHostFree(g_kstatus));
  dh::gemv_chain_release();
  g_own_stream = nullptr;
  g_stream = nullptr;
  g_splitk_ws = nullptr;
  g_row_scale = nullptr;
  g_packed_a = nullptr;
  g_widened_a = nullptr;
  g_kstatus = nullptr;
  g_num_cus = 0;
  g_ready = false;
  g_device = -1;
  if (first != hipSuccess) return dh::fail(2, "[%s] releasing the runtime failed: %s", op, hipGetErrorString(first));
  return 0;
}

static int init_locked(int device_ordinal) {
  int count = 0;
  DH_CHECK_HIP("dh_init", hipGetDeviceCount(&count));
  if (device_ordinal < 0 || device_ordinal >= count)
    return dh::fail(1, "[dh_init] device %d not present (%d visible)", device_ordinal, count);
  DH_CHECK_HIP("dh_init", hipSetDevice(device_ordinal));
  hipDeviceProp_t prop;
  DH_CHECK_HIP("dh_init", hipGetDeviceProperties(&prop, device_ordinal));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return dh::fail(1, "[dh_init] this library is built for gfx950 only, device is %s",
                    prop.gcnArchName);
  DH_CHECK_HIP("dh_init", hipStreamCreateWithFlags(&g_own_stream, hipStreamDefault));
  g_stream = g_own_stream;
  g_num_cus = prop.multiProcessorCount;
  DH_CHECK_HIP("dh_init", hipMalloc(reinterpret_cast<void**>(&g_splitk_ws), kSplitKWsBytes));
  DH_CHECK_HIP("dh_init", hipMalloc(reinterpret_cast<void**>(&g_row_scale), (size_t)kRowScaleRows * 2 * sizeof(float)));
  DH_CHECK_HIP("dh_init", hipMalloc(&g_packed_a, kPackedABytes));
  DH_CHECK_HIP("dh_init", hipMalloc(reinterpret_cast<void**>(&g_widened_a), kWidenedABytes));
  DH_CHECK_HIP("dh_init", hipHostMalloc(reinterpret_cast<void**>(&g_kstatus), 64, hipHostMallocMapped));
  *g_kstatus = 0u;
  if (int rc = dh::attn_static_scratch_init(device_ordinal)) return rc;
  if (int rc = dh::gemv_chain_init(device_ordinal)) return rc;
  g_device = device_ordinal;
  g_ready = true;
  return 0;
}

int dh_init(int device_ordinal) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_ready) {
    if (device_ordinal != g_device)
      return dh::fail(1, "[dh_init] already initialised on device %d", g_device);
    return 0;
  }
  const int rc = init_locked(device_ordinal);
  if (rc != 0) {
    // keep the message of the step that failed; a second attempt starts from nothing
    char msg[sizeof(g_err)];
    memcpy(msg, g_err, sizeof(msg));
    release_all("dh_init");
    memcpy(g_err, msg, sizeof(msg));
  }
  return rc;
}

int dh_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_ready) return 0;
  DH_CHECK_HIP("dh_shutdown", hipStreamSynchronize(g_stream));
  return release_all("dh_shutdown");
}

int dh_set_stream(void* hip_stream) {
  DH_REQUIRE_INIT("dh_set_stream");
  if (g_capturing) return dh::fail(1, "[dh_set_stream] not possible while a graph is being captured (the capture belongs to the current stream)");
  g_stream = hip_stream ? static_cast<hipStream_t>(hip_stream) : g_own_stream;
  return 0;
}

void* dh_get_stream(void) { return g_stream; }

int dh_malloc(size_t bytes, void** d_out) {
  DH_REQUIRE_INIT("dh_malloc");
  if (!d_out) return dh::fail(1, "[dh_malloc] output pointer is null");
  *d_out = nullptr;
  if (g_capturing) return dh::fail(1, "[dh_malloc] not possible while a graph is being captured (allocate the step's buffers before dh_graph_begin)");
  if (bytes == 0) return dh::fail(1, "[dh_malloc] size must be positive");
  DH_CHECK_HIP("dh_malloc", hipMalloc(d_out, bytes));
  return 0;
}

int dh_free(void* d_ptr) {
  DH_REQUIRE_INIT("dh_free");
  if (g_capturing) return dh::fail(1, "[dh_free] not possible while a graph is being captured (it waits for the stream)");
  if (!d_ptr) return 0;
  DH_CHECK_HIP("dh_free", hipStreamSynchronize(g_stream));
  DH_CHECK_HIP("dh_free", hipFree(d_ptr));
  return dh::check_kernel_status("dh_free");
}

int dh_upload(void* d_dst, size_t dst_offset, const void* host_src, size_t bytes) {
  DH_REQUIRE_INIT("dh_upload");
  if (g_capturing) return dh::fail(1, "[dh_upload] not possible while a graph is being captured (it waits for the stream)");
  if (bytes == 0) return 0;
  if (!d_dst || !host_src) return dh::fail(1, "[dh_upload] null pointer");
  // Pageable host memory: hipMemcpyAsync stages it before returning, so the caller may
  // reuse host_src at once; ordering with earlier ops comes from the stream.
  DH_CHECK_HIP("dh_upload", hipMemcpyAsync(static_cast<char*>(d_dst) + dst_offset, host_src, bytes,
                                           hipMemcpyHostToDevice, g_stream));
  DH_CHECK_HIP("dh_upload", hipStreamSynchronize(g_stream));
  return dh::check_kernel_status("dh_upload");
}

int dh_download(void* host_dst, const void* d_src, size_t src_offset, size_t bytes) {
  DH_REQUIRE_INIT("dh_download");
  if (g_capturing) return dh::fail(1, "[dh_download] not possible while a graph is being captured (it waits for the stream)");
  if (bytes == 0) return 0;
  if (!host_dst || !d_src) return dh::fail(1, "[dh_download] null pointer");
  DH_CHECK_HIP("dh_download", hipMemcpyAsync(host_dst, static_cast<const char*>(d_src) + src_offset,
                                             bytes, hipMemcpyDeviceToHost, g_stream));
  DH_CHECK_HIP("dh_download", hipStreamSynchronize(g_stream));
  return dh::check_kernel_status("dh_download");
}

// ---- readback that does not wait: pinned host memory, an enqueued copy, an event to wait for -----
int dh_host_alloc(size_t bytes, void** out) {
  DH_REQUIRE_INIT("dh_host_alloc");
  if (!out || bytes == 0) return dh::fail(1, "[dh_host_alloc] need a size and a place for the pointer");
  DH_CHECK_HIP("dh_host_alloc", hipHostMalloc(out, bytes, hipHostMallocDefault));
  return 0;
}

int dh_host_free(void* p) {
  DH_REQUIRE_INIT("dh_host_free");
  if (!p) return 0;
  DH_CHECK_HIP("dh_host_free", hipHostFree(p));
  return 0;
}

int dh_download_async(void* host_dst, const void* d_src, size_t src_offset, size_t bytes) {
  DH_REQUIRE_INIT("dh_download_async");
  if (g_capturing) return dh::fail(1, "[dh_download_async] not possible while a graph is being captured");
  if (bytes == 0) return 0;
  if (!host_dst || !d_src) return dh::fail(1, "[dh_download_async] null pointer");
  DH_CHECK_HIP("dh_download_async", hipMemcpyAsync(host_dst, static_cast<const char*>(d_src) + src_offset, bytes,
                                                   hipMemcpyDeviceToHost, g_stream));
  return 0;
}

int dh_event_synchronize(void* ev) {
  DH_REQUIRE_INIT("dh_event_synchronize");
  if (!ev) return dh::fail(1, "[dh_event_synchronize] null event");
  DH_CHECK_HIP("dh_event_synchronize", hipEventSynchronize(static_cast<hipEvent_t>(ev)));
  // everything enqueued before the event has run: a kernel among it may have given up a bounded wait
  return dh::check_kernel_status("dh_event_synchronize");
}

int dh_copy(void* d_dst, size_t dst_offset, const void* d_src, size_t src_offset, size_t bytes) {
  DH_REQUIRE_INIT("dh_copy");
  if (bytes == 0) return 0;
  if (!d_dst || !d_src) return dh::fail(1, "[dh_copy] null pointer");
  DH_CHECK_HIP("dh_copy", hipMemcpyAsync(static_cast<char*>(d_dst) + dst_offset,
                                         static_cast<const char*>(d_src) + src_offset, bytes,
                                         hipMemcpyDeviceToDevice, g_stream));
  return 0;
}

__global__ void dh_fill_zero_kernel(uint32_t* p, int64_t words) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < words; i += stride) p[i] = 0u;
}

int dh_fill_zero(void* d_dst, size_t offset, size_t bytes) {
  DH_REQUIRE_INIT("dh_fill_zero");
  if (bytes == 0) return 0;
  if (!d_dst) return dh::fail(1, "[dh_fill_zero] null pointer");
  if ((offset | bytes) & 3) return dh::fail(1, "[dh_fill_zero] offset and size must be multiples of 4");
  // A fill kernel rather than hipMemsetAsync so the call can sit inside a captured graph.
  const int64_t words = (int64_t)(bytes / 4);
  const int grid = (int)std::min<int64_t>(dh::ceil_div(words, 256), 2048);
  hipLaunchKernelGGL(dh_fill_zero_kernel, dim3(grid), dim3(256), 0, g_stream,
                     reinterpret_cast<uint32_t*>(static_cast<char*>(d_dst) + offset), words);
  DH_CHECK_LAUNCH("dh_fill_zero");
  return 0;
}

int dh_event_create(void** ev_out) {
  DH_REQUIRE_INIT("dh_event_create");
  if (!ev_out) return dh::fail(1, "[dh_event_create] null pointer");
  hipEvent_t ev;
  DH_CHECK_HIP("dh_event_create", hipEventCreate(&ev));
  *ev_out = ev;
  return 0;
}

int dh_event_record(void* ev) {
  DH_REQUIRE_INIT("dh_event_record");
  DH_CHECK_HIP("dh_event_record", hipEventRecord(static_cast<hipEvent_t>(ev), g_stream));
  return 0;
}

int dh_event_elapsed_ms(void* start, void* stop, float* ms_out) {
  DH_REQUIRE_INIT("dh_event_elapsed_ms");
  DH_CHECK_HIP("dh_event_elapsed_ms", hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  DH_CHECK_HIP("dh_event_elapsed_ms", hipEventElapsedTime(ms_out, static_cast<hipEvent_t>(start),
                                                          static_cast<hipEvent_t>(stop)));
  return 0;
}

int dh_event_destroy(void* ev) {
  DH_REQUIRE_INIT("dh_event_destroy");
  DH_CHECK_HIP("dh_event_destroy", hipEventDestroy(static_cast<hipEvent_t>(ev)));
  return 0;
}

// ---- captured decode steps -------------------------------------------------------------------
int dh_graph_begin(void) {
  DH_REQUIRE_INIT("dh_graph_begin");
  if (g_capturing) return dh::fail(1, "[dh_graph_begin] a capture is already in progress");
  DH_CHECK_HIP("dh_graph_begin", hipStreamSynchronize(g_stream));
  g_capturing = new dh::Graph();
  const hipError_t e = hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal);
  if (e != hipSuccess) {
    delete g_capturing;
    g_capturing = nullptr;
    return dh::fail(2, "[dh_graph_begin] hipStreamBeginCapture failed: %s", hipGetErrorString(e));
  }
  return 0;
}

static void graph_free(dh::Graph* g) {
  if (!g) return;
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph) (void)hipGraphDestroy(g->graph);
  delete[] g->attn;
  delete[] g->fin;
  delete g;
}

int dh_graph_end(int position, void** graph_out) {
  DH_REQUIRE_INIT("dh_graph_end");
  if (!graph_out) return dh::fail(1, "[dh_graph_end] output pointer is null");
  *graph_out = nullptr;
  if (!g_capturing) return dh::fail(1, "[dh_graph_end] no capture in progress");
  dh::Graph* g = g_capturing;
  g_capturing = nullptr;
  hipError_t e = hipStreamEndCapture(g_stream, &g->graph);
  if (e != hipSuccess || !g->graph) {
    graph_free(g);
    return dh::fail(2, "[dh_graph_end] hipStreamEndCapture failed: %s", hipGetErrorString(e));
  }
  e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    graph_free(g);
    return dh::fail(2, "[dh_graph_end] hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  g->position = g->captured_position = position;
  if (int rc = dh::attn_graph_bind(g)) {
    graph_free(g);
    return rc;
  }
  if (int rc = dh::finite_graph_bind(g)) {
    graph_free(g);
    return rc;
  }
  *graph_out = g;
  return 0;
}

int dh_graph_set_max_position(void* graph, int max_position) {
  DH_REQUIRE_INIT("dh_graph_set_max_position");
  dh::Graph* g = static_cast<dh::Graph*>(graph);
  if (!g || !g->exec) return dh::fail(1, "[dh_graph_set_max_position] null graph");
  if (max_position < g->captured_position)
    return dh::fail(1, "[dh_graph_set_max_position] %d is below the captured position %d", max_position, g->captured_position);
  g->max_position = max_position;
  return 0;
}

int dh_graph_launch(void* graph, int position) {
  DH_REQUIRE_INIT("dh_graph_launch");
  dh::Graph* g = static_cast<dh::Graph*>(graph);
  if (!g || !g->exec) return dh::fail(1, "[dh_graph_launch] null graph");
  if (g_capturing) return dh::fail(1, "[dh_graph_launch] a capture is in progress");
  if (position < 0) return dh::fail(1, "[dh_graph_launch] position must be non-negative");
  if (g->max_position >= 0 && position > g->max_position)
    return dh::fail(1, "[dh_graph_launch] position %d is beyond the largest one the step's buffers were declared for (%d)",
                    position, g->max_position);
  if (position != g->position) {
    if (int rc = dh::attn_graph_set_position(g, position)) return rc;
    if (int rc = dh::finite_graph_set_position(g, position)) return rc;
    g->position = position;
  }
  DH_CHECK_HIP("dh_graph_launch", hipGraphLaunch(g->exec, g_stream));
  return 0;
}

int dh_graph_prepare(void* graph, int position) {
  DH_REQUIRE_INIT("dh_graph_prepare");
  dh::Graph* g = static_cast<dh::Graph*>(graph);
  if (!g || !g->exec) return dh::fail(1, "[dh_graph_prepare] null graph");
  if (g_capturing) return dh::fail(1, "[dh_graph_prepare] a capture is in progress");
  if (position < 0) return dh::fail(1, "[dh_graph_prepare] position must be non-negative");
  if (g->max_position >= 0 && position > g->max_position)
    return dh::fail(1, "[dh_graph_prepare] position %d is beyond the largest one the step's buffers were declared for (%d)",
                    position, g->max_position);
  if (position != g->position) {
    if (int rc = dh::attn_graph_set_position(g, position)) return rc;
    if (int rc = dh::finite_graph_set_position(g, position)) return rc;
    g->position = position;
  }
  return 0;
}

int dh_graph_destroy(void* graph) {
  DH_REQUIRE_INIT("dh_graph_destroy");
  if (!graph) return 0;
  DH_CHECK_HIP("dh_graph_destroy", hipStreamSynchronize(g_stream));
  graph_free(static_cast<dh::Graph*>(graph));
  return 0;
}

int dh_sync(void) {
  DH_REQUIRE_INIT("dh_sync");
  if (g_capturing) return dh::fail(1, "[dh_sync] not possible while a graph is being captured (it waits for the stream)");
  DH_CHECK_HIP("dh_sync", hipStreamSynchronize(g_stream));
  return dh::check_kernel_status("dh_sync");
}

}  // extern "C"
