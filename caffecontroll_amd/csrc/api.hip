// Process state, memory management and timing entry points of the driver library.
#include <cstdarg>
#include <cstring>
#include <cmath>
#include <mutex>
#include <random>
#include <vector>

#include "cct_common.h"

namespace cct {

static Context g_ctx;
static Tuning g_tuning;
static std::once_flag g_tuning_once;
static bool g_counters_dirty = false;
static std::mutex g_mu;
static thread_local char g_err[512] = "";

Context &ctx() { return g_ctx; }
Tuning &tuning() { return g_tuning; }

static void read_tuning_from_env() {
  auto geti = [](const char *name, int dflt) {
    const char *e = getenv(name);
    return e && *e ? atoi(e) : dflt;
  };
  g_tuning.direct_tile = geti("CCT_HIP_DIRECT_TILE", 0);
  g_tuning.direct_waves = geti("CCT_HIP_DIRECT_WAVES", 0);
  g_tuning.direct_tb = geti("CCT_HIP_DIRECT_TB", 0);
  g_tuning.direct_nospec = geti("CCT_HIP_DIRECT_NOSPEC", 0);
  g_tuning.direct_splits = geti("CCT_HIP_DIRECT_SPLITS", 0);
  g_tuning.direct_alds = geti("CCT_HIP_DIRECT_ALDS", 0);
  g_tuning.direct_wgrad_rows = geti("CCT_HIP_DIRECT_WGRAD_ROWS", 0);
  g_tuning.conv1x1_per_image = geti("CCT_HIP_CONV1X1_PER_IMAGE", 0);
  g_tuning.strided_wgrad = geti("CCT_HIP_STRIDED_WGRAD", 0);
  g_tuning.pool_plane = geti("CCT_HIP_POOL_PLANE", 0);
  g_tuning.gemm_nt = geti("CCT_HIP_GEMM_NT", 0);
  g_tuning.gemm_tile = geti("CCT_HIP_GEMM_TILE", -1);
  g_tuning.gemm_nodma = geti("CCT_HIP_GEMM_NODMA", 0);
}

// per host thread, like the error text: a launch on one thread never rewrites what another thread reads
static thread_local char g_last_kernel[192] = "";

void note_kernel(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_kernel, sizeof(g_last_kernel), fmt, ap);
  va_end(ap);
}

void mark_counters_dirty() {
  std::lock_guard<std::mutex> lk(g_mu);
  g_counters_dirty = true;
}

int grant_dynamic_lds(const void *kernel, size_t bytes, LdsGrant &st) {
  if (bytes <= 64 * 1024) return 0;
  std::lock_guard<std::mutex> lk(g_mu);  // `st` is shared by every host thread that launches this instance
  if (st.device == g_ctx.device && st.bytes >= bytes) return 0;
  CCT_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  st.device = g_ctx.device;
  st.bytes = bytes;
  return 0;
}

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static int init_locked(int device_id) {
  std::call_once(g_tuning_once, read_tuning_from_env);
  int count = 0;
  CCT_HIP_CHECK(hipGetDeviceCount(&count));
  CCT_REQUIRE(device_id >= 0 && device_id < count, "device %d not present (%d devices)", device_id,
              count);
  CCT_HIP_CHECK(hipSetDevice(device_id));
  if (g_ctx.device != device_id) {
    hipDeviceProp_t prop;
    CCT_HIP_CHECK(hipGetDeviceProperties(&prop, device_id));
    CCT_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
                "this library holds gfx950 code only; device %d is %s", device_id, prop.gcnArchName);
    g_ctx.device = device_id;
    g_ctx.compute_units = prop.multiProcessorCount;
    g_ctx.workspace = nullptr;
    g_ctx.workspace_bytes = 0;
    g_ctx.counters = nullptr;
  }
  return 0;
}

// Called at the top of every entry point: the reference creates a fresh std::thread per
// forward/backward call (src/bridges/PhysicalStratum.h:52-64), so the device must be
// re-selected on whichever thread arrives.
int ensure_init() {
  if (g_ctx.device < 0) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_ctx.device < 0) return init_locked(0);
    return 0;
  }
  CCT_HIP_CHECK(hipSetDevice(g_ctx.device));
  return 0;
}

int get_workspace(size_t bytes, void **out) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (bytes > g_ctx.workspace_bytes) {
    if (g_ctx.workspace) {
      CCT_HIP_CHECK(hipStreamSynchronize(g_ctx.stream));
      CCT_HIP_CHECK(hipFree(g_ctx.workspace));
      g_ctx.workspace = nullptr;
      g_ctx.workspace_bytes = 0;
    }
    const size_t want = (bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
    CCT_HIP_CHECK(hipMalloc(&g_ctx.workspace, want));
    g_ctx.workspace_bytes = want;
  }
  *out = g_ctx.workspace;
  return 0;
}

// The arrival counters must read zero when a launch starts; the workgroup that finishes a reduction
// puts its counter back to zero.  They are cleared here when they are created, after
// cct_hip_init() and after a launch that used them was refused (mark_counters_dirty).  All users
// run on the library's one stream, so a clear ordered on that stream is ordered before them.
int get_counters(unsigned int **out) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_ctx.counters) {
    CCT_HIP_CHECK(hipMalloc((void **)&g_ctx.counters, kMaxCounters * sizeof(unsigned int)));
    g_counters_dirty = true;
  }
  if (g_counters_dirty) {
    CCT_HIP_CHECK(hipStreamSynchronize(g_ctx.stream));
    CCT_HIP_CHECK(hipMemset(g_ctx.counters, 0, kMaxCounters * sizeof(unsigned int)));
    CCT_HIP_CHECK(hipDeviceSynchronize());
    g_counters_dirty = false;
  }
  *out = g_ctx.counters;
  return 0;
}

struct Timer {
  hipEvent_t start, stop;
};

}  // namespace cct

using namespace cct;

extern "C" {

int cct_hip_init(int device_id) {
  std::lock_guard<std::mutex> lk(g_mu);
  const int rc = init_locked(device_id);
  // an explicit (re-)initialisation also puts the reduction counters back to a known state
  if (!rc && g_ctx.counters) g_counters_dirty = true;
  return rc;
}

int cct_hip_set_tuning(const char *name, int value) {
  CCT_REQUIRE(name != nullptr, "set_tuning: null name");
  std::call_once(g_tuning_once, read_tuning_from_env);
  Tuning &t = tuning();
  struct { const char *name; int *field; } const table[] = {
      {"direct_tile", &t.direct_tile}, {"direct_waves", &t.direct_waves}, {"direct_tb", &t.direct_tb},
      {"direct_nospec", &t.direct_nospec}, {"direct_splits", &t.direct_splits}, {"direct_alds", &t.direct_alds},
      {"direct_wgrad_rows", &t.direct_wgrad_rows}, {"conv1x1_per_image", &t.conv1x1_per_image}, {"strided_wgrad", &t.strided_wgrad}, {"pool_plane", &t.pool_plane}, {"gemm_nt", &t.gemm_nt},
      {"gemm_tile", &t.gemm_tile}, {"gemm_nodma", &t.gemm_nodma}};
  for (const auto &e : table)
    if (!strcmp(e.name, name)) {
      *e.field = value;
      return 0;
    }
  return set_error(CCT_HIP_EINVAL, "set_tuning: unknown knob \"%s\"", name);
}

int cct_hip_set_stream(void *hip_stream) {
  CCT_ENSURE_INIT();
  ctx().stream = (hipStream_t)hip_stream;
  return 0;
}

int cct_hip_device_sync(void) {
  CCT_ENSURE_INIT();
  CCT_HIP_CHECK(hipStreamSynchronize(ctx().stream));
  return 0;
}

const char *cct_hip_last_error(void) { return g_err; }

const char *cct_hip_last_kernel(void) { return g_last_kernel; }

int cct_hip_compute_units(void) { return ctx().compute_units; }

int cct_hip_malloc(void **dev_ptr, size_t size_in_byte) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(dev_ptr != nullptr, "malloc: null result pointer");
  *dev_ptr = nullptr;
  if (size_in_byte == 0) return 0;
  CCT_HIP_CHECK(hipMalloc(dev_ptr, size_in_byte));
  return 0;
}

int cct_hip_free(void *dev_ptr) {
  CCT_ENSURE_INIT();
  if (dev_ptr) CCT_HIP_CHECK(hipFree(dev_ptr));
  return 0;
}

int cct_hip_memcpy(void *dst, const void *src, size_t size_in_byte, int kind) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(kind >= 0 && kind <= 2, "memcpy: kind %d not in {0,1,2}", kind);
  if (size_in_byte == 0) return 0;
  const hipMemcpyKind k =
      kind == 0 ? hipMemcpyHostToDevice : kind == 1 ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
  CCT_HIP_CHECK(hipMemcpyAsync(dst, src, size_in_byte, k, ctx().stream));
  if (kind != 2) CCT_HIP_CHECK(hipStreamSynchronize(ctx().stream));
  return 0;
}

// ---- overlapped host <-> device staging ------------------------------------------------------------
// Two side streams at the default priority, one per direction (the link is full duplex), and a pool of
// events that order them against the library's compute stream.
struct cct_hip_pipe {
  hipStream_t up = nullptr, down = nullptr;
  std::vector<hipEvent_t> events;
  size_t next_event = 0;
  int take(hipEvent_t *ev) {
    if (next_event == events.size()) {
      hipEvent_t e;
      CCT_HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
      events.push_back(e);
    }
    *ev = events[next_event++];
    return 0;
  }
};

int cct_hip_pipe_create(cct_hip_pipe **out) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out != nullptr, "pipe_create: null result pointer");
  cct_hip_pipe *p = new cct_hip_pipe;
  hipError_t e = hipStreamCreateWithFlags(&p->up, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&p->down, hipStreamNonBlocking);
  if (e != hipSuccess) {
    if (p->up) (void)hipStreamDestroy(p->up);
    delete p;
    return set_error((int)e, "pipe_create: %s", hipGetErrorString(e));
  }
  *out = p;
  return 0;
}

int cct_hip_pipe_destroy(cct_hip_pipe *p) {
  if (!p) return 0;
  (void)hipStreamSynchronize(p->up);
  (void)hipStreamSynchronize(p->down);
  for (hipEvent_t e : p->events) (void)hipEventDestroy(e);
  (void)hipStreamDestroy(p->up);
  (void)hipStreamDestroy(p->down);
  delete p;
  return 0;
}

int cct_hip_pipe_begin(cct_hip_pipe *p) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(p != nullptr, "pipe_begin: null pipe");
  // uploads must not overtake kernels already enqueued that still read the buffers they will overwrite
  hipEvent_t ev;
  if (int rc = p->take(&ev)) return rc;
  CCT_HIP_CHECK(hipEventRecord(ev, ctx().stream));
  CCT_HIP_CHECK(hipStreamWaitEvent(p->up, ev, 0));
  return 0;
}

int cct_hip_pipe_upload(cct_hip_pipe *p, void *dst_device, const void *src_host, size_t bytes, int *ticket) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(p && ticket && (bytes == 0 || (dst_device && src_host)), "pipe_upload: null argument");
  if (bytes) CCT_HIP_CHECK(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, p->up));
  hipEvent_t ev;
  if (int rc = p->take(&ev)) return rc;
  CCT_HIP_CHECK(hipEventRecord(ev, p->up));
  *ticket = (int)(p->next_event - 1);
  return 0;
}

int cct_hip_pipe_wait_upload(cct_hip_pipe *p, int ticket) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(p && ticket >= 0 && (size_t)ticket < p->next_event, "pipe_wait_upload: no such upload");
  CCT_HIP_CHECK(hipStreamWaitEvent(ctx().stream, p->events[ticket], 0));
  return 0;
}

int cct_hip_pipe_download(cct_hip_pipe *p, void *dst_host, const void *src_device, size_t bytes) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(p && (bytes == 0 || (dst_host && src_device)), "pipe_download: null argument");
  hipEvent_t ev;
  if (int rc = p->take(&ev)) return rc;
  CCT_HIP_CHECK(hipEventRecord(ev, ctx().stream));
  CCT_HIP_CHECK(hipStreamWaitEvent(p->down, ev, 0));
  if (bytes) CCT_HIP_CHECK(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, p->down));
  return 0;
}

int cct_hip_pipe_finish(cct_hip_pipe *p) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(p != nullptr, "pipe_finish: null pipe");
  CCT_HIP_CHECK(hipStreamSynchronize(p->up));
  CCT_HIP_CHECK(hipStreamSynchronize(ctx().stream));
  CCT_HIP_CHECK(hipStreamSynchronize(p->down));
  p->next_event = 0;
  return 0;
}

// ---- random fillers: drawn on the host exactly as CPUDriver does, then copied to the device ------
// std::mt19937 seeded with random_seed (std::random_device when -1) and the standard library's
// distribution objects, one draw per element in index order (src/sched/DeviceDriver_CPU.cpp:661-699).

static unsigned filler_seed(int random_seed) {
  if (random_seed != -1) return (unsigned)random_seed;
  std::random_device rd;
  return rd();
}

int cct_filler_draw_xavier(float *host, size_t n, size_t n_batch, int random_seed) {
  CCT_REQUIRE(host || n == 0, "filler_draw_xavier: null array");
  CCT_REQUIRE(n_batch > 0 && n / n_batch > 0, "filler_draw_xavier: fan-in must be positive");
  const size_t fan_in = n / n_batch;
  const float scale = std::sqrt(3.0 / fan_in);
  std::mt19937 gen(filler_seed(random_seed));
  std::uniform_real_distribution<float> uni(-scale, scale);
  for (size_t i = 0; i < n; ++i) host[i] = uni(gen);
  return 0;
}

int cct_filler_draw_bernoulli(float *host, size_t n, float p, int random_seed) {
  CCT_REQUIRE(host || n == 0, "filler_draw_bernoulli: null array");
  CCT_REQUIRE(p >= 0.0f && p <= 1.0f, "filler_draw_bernoulli: p must be in [0, 1]");
  std::mt19937 gen(filler_seed(random_seed));
  std::bernoulli_distribution bern(p);
  for (size_t i = 0; i < n; ++i) host[i] = bern(gen);
  return 0;
}

int cct_filler_draw_gaussian(float *host, size_t n, float mean, float std_dev, int random_seed) {
  CCT_REQUIRE(host || n == 0, "filler_draw_gaussian: null array");
  CCT_REQUIRE(std_dev >= 0.0f && std::isfinite(std_dev) && std::isfinite(mean),
              "filler_draw_gaussian: std must be finite and not negative");
  if (std_dev == 0.0f) {  // what the reference's normal_distribution(mean, 0) yields: the mean everywhere
    for (size_t i = 0; i < n; ++i) host[i] = mean;
    return 0;
  }
  std::mt19937 gen(filler_seed(random_seed));
  std::normal_distribution<float> gaussian(mean, std_dev);
  for (size_t i = 0; i < n; ++i) host[i] = gaussian(gen);
  return 0;
}

static int upload_filler(float *arr, const std::vector<float> &host) {
  CCT_REQUIRE(arr || host.empty(), "fill: null device array");
  return cct_hip_memcpy(arr, host.data(), host.size() * sizeof(float), 0);
}

int cct_hip_fill_xavier(float *arr, size_t n, size_t n_batch, int random_seed) {
  CCT_ENSURE_INIT();
  std::vector<float> host(n);
  int rc = cct_filler_draw_xavier(host.data(), n, n_batch, random_seed);
  return rc ? rc : upload_filler(arr, host);
}

int cct_hip_fill_bernoulli(float *arr, size_t n, float p, int random_seed) {
  CCT_ENSURE_INIT();
  std::vector<float> host(n);
  int rc = cct_filler_draw_bernoulli(host.data(), n, p, random_seed);
  return rc ? rc : upload_filler(arr, host);
}

int cct_hip_fill_gaussian(float *arr, size_t n, float mean, float std_dev, int random_seed) {
  CCT_ENSURE_INIT();
  std::vector<float> host(n);
  int rc = cct_filler_draw_gaussian(host.data(), n, mean, std_dev, random_seed);
  return rc ? rc : upload_filler(arr, host);
}

int cct_hip_timer_create(void **timer) {
  CCT_ENSURE_INIT();
  Timer *t = new Timer;
  CCT_HIP_CHECK(hipEventCreate(&t->start));
  CCT_HIP_CHECK(hipEventCreate(&t->stop));
  *timer = t;
  return 0;
}

int cct_hip_timer_destroy(void *timer) {
  Timer *t = (Timer *)timer;
  if (!t) return 0;
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
  return 0;
}

int cct_hip_timer_start(void *timer) {
  CCT_ENSURE_INIT();
  CCT_HIP_CHECK(hipEventRecord(((Timer *)timer)->start, ctx().stream));
  return 0;
}

int cct_hip_timer_stop(void *timer) {
  CCT_ENSURE_INIT();
  CCT_HIP_CHECK(hipEventRecord(((Timer *)timer)->stop, ctx().stream));
  return 0;
}

int cct_hip_timer_elapsed_ms(void *timer, float *ms) {
  CCT_ENSURE_INIT();
  Timer *t = (Timer *)timer;
  CCT_HIP_CHECK(hipEventSynchronize(t->stop));
  CCT_HIP_CHECK(hipEventElapsedTime(ms, t->start, t->stop));
  return 0;
}

}  // extern "C"
