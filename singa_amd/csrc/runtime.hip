// Device runtime behind the C ABI: one stream + one caching memory pool per opened device.
// Mirrors what SINGA's CudaGPU + DeviceMemPool give the Tensor layer
// (reference: src/core/device/cuda_gpu.cc:56-209, src/core/memory/memory.cc:32-118).
#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <new>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include <string.h>

#include "common.h"

// The auxiliary streams of all open devices: a kernel entry point that is handed one of them knows that its
// launch shares the chip with the main stream's work (sgh_stream_is_aux).
static std::mutex g_aux_mu;
static std::vector<hipStream_t> g_aux_streams;

bool sgh_stream_is_aux(hipStream_t s) {
  if (!s) return false;
  std::lock_guard<std::mutex> lock(g_aux_mu);
  for (hipStream_t a : g_aux_streams)
    if (a == s) return true;
  return false;
}


struct sgh_device {
  int id = 0;
  hipStream_t stream = nullptr;
  hipStream_t side = nullptr;  // uploads that must happen while `stream` is recording
  hipStream_t aux = nullptr;   // second compute stream (sgh_device_aux_stream), created on first use
  hipEvent_t fork_ev = nullptr, join_ev = nullptr;
  // blocks that work on the auxiliary stream uses (sgh_block_used_on): when freed they wait in
  // `pending` until the main stream has been ordered behind the auxiliary one (join / sync)
  std::unordered_set<void *> on_aux;
  std::vector<std::pair<void *, size_t>> pending;
  std::mutex mu;
  // free blocks keyed by their (rounded) size; blocks in use keyed by address
  std::multimap<size_t, void *> free_blocks;
  std::unordered_map<void *, size_t> live;
  size_t in_use = 0, cached = 0, driver_allocs = 0;
  // stream capture (sgh_graph_begin .. sgh_graph_end): blocks freed meanwhile are kept out of the
  // pool, because the captured kernels will write to them on every replay
  std::atomic<bool> capturing{false};   // (read by entry points that do not take the lock)
  std::vector<std::pair<void *, size_t>> held;
  std::unordered_set<void *> born;        // blocks handed out while recording
  std::vector<struct sgh_graph *> graphs;  // instantiated recordings of this device
  // sgh_upload_async: ring of pinned staging slots; a slot is reused once its copy has run
  static constexpr int kUploadSlots = 8;
  static constexpr size_t kUploadSlotBytes = 64 * 1024;
  char *upload_host = nullptr;   // kUploadSlots * kUploadSlotBytes of pinned memory, allocated on first use
  hipEvent_t upload_done[kUploadSlots] = {};
  int upload_next = 0;
};

struct sgh_graph {
  sgh_device *dev = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<std::pair<void *, size_t>> held;
  // blocks handed out during the recording and still in use when it ended: when their owner
  // frees them they join `held` instead of the pool, for the recorded kernels still write there
  std::unordered_set<void *> born;
};

struct sgh_event {
  hipEvent_t ev;
};

static int g_num_cus = 0;

int sgh_num_cus() {
  if (g_num_cus > 0) return g_num_cus;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
    g_num_cus = n;
  else
    g_num_cus = 256;
  return g_num_cus;
}

const sgh_env_switches &sgh_env() {
  static const sgh_env_switches e = [] {
    auto on = [](const char *n) { return getenv(n) != nullptr; };
    auto num = [](const char *n, int lo, int hi) {
      const char *v = getenv(n);
      if (!v) return -1;
      const int x = atoi(v);
      return x >= lo && x <= hi ? x : -1;
    };
    sgh_env_switches s{};
    s.dgrad3x3_off = on("SGH_DGRAD3X3_OFF"), s.wgrad3x3_off = on("SGH_WGRAD3X3_OFF");
    s.dgrad_fewc_off = on("SGH_DGRAD_FEWC_OFF"), s.wgrad_fewc_off = on("SGH_WGRAD_FEWC_OFF");
    s.dgrad_pointwise_off = on("SGH_DGRAD_POINTWISE_OFF"), s.conv16_off = on("SGH_CONV16_OFF");
    s.bn_ragged_off = on("SGH_BN_RAGGED_OFF"), s.fwd_fewc_off = on("SGH_FWD_FEWC_OFF"), s.bn_fwd_onchip_off = on("SGH_BN_FWD_ONCHIP_OFF"), s.bn_onchip_off = on("SGH_BN_ONCHIP_OFF"), s.pw_dgrad_off = on("SGH_PW_DGRAD_OFF");
    s.pw_wgrad_off = on("SGH_PW_WGRAD_OFF"), s.dgrad_fewc16_off = on("SGH_DGRAD_FEWC16_OFF");
    s.slab16_off = on("SGH_SLAB16_OFF");
    s.dgrad_tile = num("SGH_DGRAD_TILE", 0, 3), s.wgrad_tile = num("SGH_WGRAD_TILE", 0, 5);
    s.pw_tile = num("SGH_PW_TILE", 1, 2);
    s.conv_xcd_off = on("SGH_CONV_XCD_OFF");
    const char *bm = getenv("SGH_DGRAD3X3_BM");
    s.dgrad3x3_bm = bm ? (atoi(bm) == 64 ? 64 : 128) : 0;
    return s;
  }();
  return e;
}

// ---- weight epoch and the prepared-weights note of a convolution geometry
static std::atomic<unsigned long long> g_weights_epoch{1};

// Weight tensors whose re-laid copies are waiting in a workspace (sgh_conv_dgrad_prepare_multi), as address
// ranges.  Entry points that are known to update parameters advance the epoch outright; the elementwise ones,
// which a backward pass also calls on activations between the prepare and the data gradients, advance it only
// when their output lies inside one of these ranges (Tensor `*=`, `+=`, `-=` on a weight).
static std::mutex g_prepared_mu;
static std::vector<std::pair<const char *, size_t>> g_prepared;
static std::atomic<int> g_prepared_count{0};

unsigned long long sgh_weights_epoch() { return g_weights_epoch.load(std::memory_order_relaxed); }
void sgh_weights_epoch_bump() {
  g_weights_epoch.fetch_add(1, std::memory_order_relaxed);
  if (g_prepared_count.load(std::memory_order_relaxed) != 0) {   // every note is void now
    std::lock_guard<std::mutex> lk(g_prepared_mu);
    g_prepared.clear();
    g_prepared_count.store(0, std::memory_order_relaxed);
  }
}

void sgh_prepared_weights_add(const void *W, size_t bytes) {
  std::lock_guard<std::mutex> lk(g_prepared_mu);
  if (g_prepared.size() >= 4096) g_prepared.clear();   // (notes of earlier epochs that nobody used up)
  g_prepared.emplace_back(static_cast<const char *>(W), bytes);
  g_prepared_count.store(int(g_prepared.size()), std::memory_order_relaxed);
}

void sgh_note_write(const void *out, size_t bytes) {
  if (g_prepared_count.load(std::memory_order_relaxed) == 0 || !out) return;
  bool hit = false;
  {
    std::lock_guard<std::mutex> lk(g_prepared_mu);
    const char *o = static_cast<const char *>(out);
    for (const auto &r : g_prepared)
      if (o < r.first + r.second && r.first < o + bytes) {
        hit = true;
        break;
      }
  }
  if (hit) sgh_weights_epoch_bump();
}

bool sgh_prelaid_valid(const sgh_conv_geom *g, int dtype, const void *W, const void *workspace) {
  return g->prelaid_W != nullptr && g->prelaid_W == W && g->prelaid_ws == workspace && g->prelaid_dtype == dtype &&
         g->prelaid_epoch == sgh_weights_epoch();
}

void sgh_prelaid_clear(sgh_conv_geom *g) {
  g->prelaid_dtype = 0;
  g->prelaid_W = g->prelaid_ws = nullptr;
  g->prelaid_ws_bytes = 0;
  g->prelaid_epoch = 0;
}

void sgh_prelaid_clear_if_overlap(sgh_conv_geom *g, const void *workspace, size_t ws_bytes) {
  if (!g->prelaid_W || !workspace) return;
  const char *a = static_cast<const char *>(workspace), *b = static_cast<const char *>(g->prelaid_ws);
  if (a < b + g->prelaid_ws_bytes && b < a + ws_bytes) sgh_prelaid_clear(g);
}

// ---- kernel-level profiling records
struct ProfRec {
  const char *tag;
  double work;
  hipEvent_t a, b;
};
static std::vector<ProfRec> g_prof;
static std::vector<size_t> g_prof_open;  // indices of records whose stop event is not recorded yet (nesting)
static bool g_prof_on = false;
static std::atomic<int> g_recording{0};   // devices whose stream is recording a graph: no profiling records meanwhile

bool sgh_prof_on() { return g_prof_on && g_recording.load(std::memory_order_relaxed) == 0; }

void sgh_prof_start(const char *tag, double work, hipStream_t s) {
  if (!sgh_prof_on()) return;
  ProfRec r{tag, work, nullptr, nullptr};
  if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) return;
  (void)hipEventRecord(r.a, s);
  g_prof_open.push_back(g_prof.size());
  g_prof.push_back(r);
}

void sgh_prof_stop(hipStream_t s) {
  if (!sgh_prof_on() || g_prof_open.empty()) return;
  (void)hipEventRecord(g_prof[g_prof_open.back()].b, s);
  g_prof_open.pop_back();
}

// record whose events wait for the one launch of a sgh_prof_kernel_scope (-1: none); a record that turned
// into a marker pair sits in g_prof_open like any other
static long g_prof_kernel = -1;
static bool g_prof_kernel_spanned = false;

void sgh_prof_kernel_begin(const char *tag, double work) {
  g_prof_kernel = -1;
  g_prof_kernel_spanned = false;
  if (!sgh_prof_on()) return;
  ProfRec r{tag, work, nullptr, nullptr};
  if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) return;
  g_prof_kernel = long(g_prof.size());
  g_prof.push_back(r);
}

bool sgh_prof_kernel_take(hipEvent_t *start, hipEvent_t *stop) {
  if (g_prof_kernel < 0) return false;
  *start = g_prof[size_t(g_prof_kernel)].a;
  *stop = g_prof[size_t(g_prof_kernel)].b;
  g_prof_kernel = -1;
  return true;
}

void sgh_prof_kernel_span(hipStream_t s) {
  if (g_prof_kernel < 0) return;
  (void)hipEventRecord(g_prof[size_t(g_prof_kernel)].a, s);
  g_prof_open.push_back(size_t(g_prof_kernel));
  g_prof_kernel = -1;
  g_prof_kernel_spanned = true;
}

void sgh_prof_kernel_end(hipStream_t s) {
  if (g_prof_kernel_spanned) {
    g_prof_kernel_spanned = false;
    sgh_prof_stop(s);
  } else if (g_prof_kernel >= 0) {   // nothing was launched
    (void)hipEventRecord(g_prof[size_t(g_prof_kernel)].a, s);
    (void)hipEventRecord(g_prof[size_t(g_prof_kernel)].b, s);
    g_prof_kernel = -1;
  }
}

static void prof_clear() {
  g_prof_kernel = -1;
  g_prof_kernel_spanned = false;
  for (auto &r : g_prof) {
    if (r.a) (void)hipEventDestroy(r.a);
    if (r.b) (void)hipEventDestroy(r.b);
  }
  g_prof.clear();
  g_prof_open.clear();
}

// Pool granularity: 256 B up to 4 KiB, then power-of-two classes with four steps per octave
// (worst-case slack 19 %), so a training loop that frees and re-allocates the same tensor
// shapes every iteration always hits the cache.
static size_t round_block(size_t bytes) {
  if (bytes <= 4096) return (bytes + 255) & ~size_t(255);
  size_t p = 4096;
  while (p < bytes) p <<= 1;  // p >= bytes > p/2
  const size_t step = p >> 3;  // eighth of the upper power = quarter of the lower one
  size_t r = p >> 1;
  while (r < bytes) r += step;
  return r;
}

extern "C" {

const char *sgh_error_string(int rc) {
  switch (rc) {
    case SGH_OK: return "ok";
    case SGH_EINVAL: return "invalid argument";
    case SGH_EWORKSPACE: return "workspace missing or too small";
    case SGH_EUNSUPPORTED: return "unsupported configuration";
    case SGH_ELABEL: return "class label out of range";
    case SGH_ENOMEM: return "out of device memory";
    case SGH_ELIMIT: return "size beyond the fixed scratch buffer of a non-allocating entry point";
    case SGH_EEXCHANGE:
      return "workgroups of a one-pass BatchNorm kernel gave up waiting for each other: the outputs of that call are NaN";
    default: break;
  }
  if (rc > 0) return hipGetErrorString(static_cast<hipError_t>(rc));
  return "unknown error";
}

const char *sgh_version(void) { return "0.1.0"; }
const char *sgh_arch(void) { return "gfx950"; }

int sgh_device_count(int *count) {
  if (!count) return SGH_EINVAL;
  SGH_HIP_TRY(hipGetDeviceCount(count));
  return SGH_OK;
}

int sgh_device_open(int gpu_id, sgh_device **out) {
  if (!out || gpu_id < 0) return SGH_EINVAL;
  int n = 0;
  SGH_HIP_TRY(hipGetDeviceCount(&n));
  if (gpu_id >= n) return SGH_EINVAL;
  SGH_HIP_TRY(hipSetDevice(gpu_id));
  sgh_device *d = new (std::nothrow) sgh_device();
  if (!d) return SGH_ENOMEM;
  d->id = gpu_id;
  hipError_t e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&d->side, hipStreamNonBlocking);
  if (e != hipSuccess) {
    if (d->stream) (void)hipStreamDestroy(d->stream);
    delete d;
    return (int)e;
  }
  const int rc = sgh_bn_noalloc_setup();
  if (rc != SGH_OK) {
    (void)hipStreamDestroy(d->stream);
    (void)hipStreamDestroy(d->side);
    delete d;
    return rc;
  }
  *out = d;
  return SGH_OK;
}

// (dev->mu held) the main stream is ordered behind everything enqueued on the auxiliary stream so far:
// blocks that waited for that may be handed out again
static void release_pending(sgh_device *dev) {
  for (auto &b : dev->pending) {
    dev->free_blocks.emplace(b.second, b.first);
    dev->cached += b.second;
  }
  dev->pending.clear();
}

// (dev->mu held) nothing is running on either stream afterwards
static hipError_t quiesce(sgh_device *dev) {
  hipError_t e = hipStreamSynchronize(dev->stream);
  if (e == hipSuccess && dev->aux) e = hipStreamSynchronize(dev->aux);
  if (e == hipSuccess) release_pending(dev);
  return e;
}

int sgh_pool_trim(sgh_device *dev) {
  if (!dev) return SGH_EINVAL;
  std::lock_guard<std::mutex> lk(dev->mu);
  SGH_HIP_TRY(quiesce(dev));
  for (auto &kv : dev->free_blocks) (void)hipFree(kv.second);
  dev->free_blocks.clear();
  dev->cached = 0;
  return SGH_OK;
}

int sgh_device_close(sgh_device *dev) {
  if (!dev) return SGH_EINVAL;
  (void)hipSetDevice(dev->id);
  (void)quiesce(dev);   // both streams idle before any memory or stream goes away
  for (auto &kv : dev->free_blocks) (void)hipFree(kv.second);
  for (auto &kv : dev->live) (void)hipFree(kv.first);
  for (auto &b : dev->pending) (void)hipFree(b.first);
  (void)hipStreamDestroy(dev->stream);
  (void)hipStreamDestroy(dev->side);
  if (dev->aux) {
    {
      std::lock_guard<std::mutex> lock(g_aux_mu);
      for (size_t i = 0; i < g_aux_streams.size(); ++i)
        if (g_aux_streams[i] == dev->aux) {
          g_aux_streams.erase(g_aux_streams.begin() + long(i));
          break;
        }
    }
    (void)hipStreamDestroy(dev->aux);
  }
  if (dev->fork_ev) (void)hipEventDestroy(dev->fork_ev);
  if (dev->join_ev) (void)hipEventDestroy(dev->join_ev);
  for (hipEvent_t e : dev->upload_done)
    if (e) (void)hipEventDestroy(e);
  if (dev->upload_host) (void)hipHostFree(dev->upload_host);
  delete dev;
  return SGH_OK;
}

void *sgh_device_stream(sgh_device *dev) { return dev ? reinterpret_cast<void *>(dev->stream) : nullptr; }

void *sgh_device_aux_stream(sgh_device *dev) {
  if (!dev) return nullptr;
  if (!dev->aux) {
    (void)hipSetDevice(dev->id);
    if (hipStreamCreateWithFlags(&dev->aux, hipStreamNonBlocking) != hipSuccess) {   // (default priority)
      (void)hipGetLastError();
      dev->aux = nullptr;
    } else {
      std::lock_guard<std::mutex> lock(g_aux_mu);
      g_aux_streams.push_back(dev->aux);
    }
  }
  return reinterpret_cast<void *>(dev->aux);
}

int sgh_device_fork(sgh_device *dev, void **aux_stream) {
  if (!dev || !aux_stream) return SGH_EINVAL;
  // (while the main stream records, the event pair below pulls the auxiliary stream into the same recording: what
  // is enqueued there afterwards becomes a branch of the graph, which sgh_device_join closes)
  std::lock_guard<std::mutex> lk(dev->mu);   // (stream and event creation, and the record / wait pair, as one step)
  void *aux = sgh_device_aux_stream(dev);
  if (!aux) return SGH_ENOMEM;
  if (!dev->fork_ev) SGH_HIP_TRY(hipEventCreateWithFlags(&dev->fork_ev, hipEventDisableTiming));
  if (!dev->join_ev) SGH_HIP_TRY(hipEventCreateWithFlags(&dev->join_ev, hipEventDisableTiming));
  SGH_HIP_TRY(hipEventRecord(dev->fork_ev, dev->stream));
  SGH_HIP_TRY(hipStreamWaitEvent(dev->aux, dev->fork_ev, 0));
  *aux_stream = aux;
  return SGH_OK;
}

int sgh_device_join(sgh_device *dev) {
  if (!dev) return SGH_EINVAL;
  std::lock_guard<std::mutex> lk(dev->mu);
  if (!dev->aux || !dev->join_ev) return SGH_OK;   // never forked
  SGH_HIP_TRY(hipEventRecord(dev->join_ev, dev->aux));
  SGH_HIP_TRY(hipStreamWaitEvent(dev->stream, dev->join_ev, 0));
  if (!dev->capturing) release_pending(dev);   // (blocks freed during a recording stay with the graph)
  return SGH_OK;
}

int sgh_block_used_on(sgh_device *dev, void *ptr, void *stream) {
  if (!dev || !ptr) return SGH_EINVAL;
  std::lock_guard<std::mutex> lk(dev->mu);
  if (dev->live.find(ptr) == dev->live.end()) return SGH_EINVAL;
  if (dev->aux && stream == reinterpret_cast<void *>(dev->aux)) dev->on_aux.insert(ptr);
  else if (stream != reinterpret_cast<void *>(dev->stream)) return SGH_EINVAL;   // not a stream of this device
  return SGH_OK;
}

int sgh_stream_wait_event(void *stream, sgh_event *ev) {
  if (!ev) return SGH_EINVAL;
  SGH_HIP_TRY(hipStreamWaitEvent(sgh_stream_of(stream), ev->ev, 0));
  return SGH_OK;
}

int sgh_device_sync(sgh_device *dev) {
  if (!dev) return SGH_EINVAL;
  if (dev->capturing) return SGH_EUNSUPPORTED;  // nothing runs while the stream records
  std::lock_guard<std::mutex> lk(dev->mu);
  SGH_HIP_TRY(quiesce(dev));
  // workgroups of a one-pass BatchNorm kernel that gave up waiting for their channel's other slices left NaN
  // behind: the first wait after such a launch says so
  int gave_up = 0;
  const int rc = sgh_bn_take_exchange_failures(&gave_up);
  if (rc != SGH_OK) return rc;
  return gave_up ? SGH_EEXCHANGE : SGH_OK;
}

int sgh_graph_begin(sgh_device *dev) {
  if (!dev || dev->capturing) return SGH_EINVAL;
  // relaxed mode: the pool may still call hipMalloc while the stream records
  SGH_HIP_TRY(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeRelaxed));
  dev->capturing = true;
  g_recording.fetch_add(1, std::memory_order_relaxed);
  return SGH_OK;
}

int sgh_graph_end(sgh_device *dev, sgh_graph **out) {
  if (!dev || !out || !dev->capturing) return SGH_EINVAL;
  dev->capturing = false;
  g_recording.fetch_sub(1, std::memory_order_relaxed);
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(dev->stream, &g);
  sgh_graph *gr = new (std::nothrow) sgh_graph();
  if (e == hipSuccess && gr) e = hipGraphInstantiate(&gr->exec, g, nullptr, nullptr, 0);
  if (g) (void)hipGraphDestroy(g);
  std::lock_guard<std::mutex> lk(dev->mu);
  if (e != hipSuccess || !gr) {  // the blocks go back to the pool: nothing will replay
    for (auto &b : dev->held) {
      dev->free_blocks.emplace(b.second, b.first);
      dev->cached += b.second;
    }
    dev->held.clear();
    dev->born.clear();
    delete gr;
    (void)hipGetLastError();
    return e != hipSuccess ? (int)e : SGH_ENOMEM;
  }
  gr->dev = dev;
  gr->held.swap(dev->held);
  gr->born.swap(dev->born);
  dev->graphs.push_back(gr);
  *out = gr;
  return SGH_OK;
}

int sgh_graph_launch(sgh_graph *g) {
  if (!g || !g->exec || g->dev->capturing) return SGH_EINVAL;
  // what the recording holds is not known here: it may update weights (prepared data-gradient weights must not
  // outlive it) and it may run one-pass BatchNorm kernels (the next wait looks at their give-up counter)
  sgh_weights_epoch_bump();
  sgh_bn_mark_exchange_ran();
  SGH_HIP_TRY(hipGraphLaunch(g->exec, g->dev->stream));
  return SGH_OK;
}

int sgh_graph_destroy(sgh_graph *g) {
  if (!g) return SGH_EINVAL;
  sgh_device *dev = g->dev;
  (void)hipStreamSynchronize(dev->stream);
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  {
    std::lock_guard<std::mutex> lk(dev->mu);
    for (auto &b : g->held) {
      dev->free_blocks.emplace(b.second, b.first);
      dev->cached += b.second;
    }
    for (size_t i = 0; i < dev->graphs.size(); ++i)
      if (dev->graphs[i] == g) {
        dev->graphs.erase(dev->graphs.begin() + i);
        break;
      }
  }
  delete g;
  return SGH_OK;
}

int sgh_malloc(sgh_device *dev, void **ptr, size_t bytes) {
  if (!dev || !ptr) return SGH_EINVAL;
  if (bytes == 0) bytes = 1;
  const size_t r = round_block(bytes);
  std::lock_guard<std::mutex> lk(dev->mu);
  auto it = dev->free_blocks.find(r);
  void *p = nullptr;
  if (it != dev->free_blocks.end()) {
    p = it->second;
    dev->free_blocks.erase(it);
    dev->cached -= r;
  } else {
    hipError_t e = hipMalloc(&p, r);
    if (e == hipErrorOutOfMemory && !(dev->free_blocks.empty() && dev->pending.empty())) {
      // give the cache back to the driver once and retry
      (void)hipGetLastError();
      (void)quiesce(dev);
      for (auto &kv : dev->free_blocks) (void)hipFree(kv.second);
      dev->free_blocks.clear();
      dev->cached = 0;
      e = hipMalloc(&p, r);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return e == hipErrorOutOfMemory ? SGH_ENOMEM : (int)e;
    }
    dev->driver_allocs++;
  }
  dev->live.emplace(p, r);
  dev->in_use += r;
  if (dev->capturing) dev->born.insert(p);
  *ptr = p;
  return SGH_OK;
}

int sgh_free(sgh_device *dev, void *ptr) {
  if (!dev) return SGH_EINVAL;
  if (!ptr) return SGH_OK;
  std::lock_guard<std::mutex> lk(dev->mu);
  auto it = dev->live.find(ptr);
  if (it == dev->live.end()) return SGH_EINVAL;
  const size_t r = it->second;
  dev->live.erase(it);
  dev->in_use -= r;
  const bool aux_use = dev->on_aux.erase(ptr) != 0;
  if (dev->capturing) {  // part of the graph being recorded: reserved until the graph is destroyed
    dev->held.emplace_back(ptr, r);
    dev->born.erase(ptr);
    return SGH_OK;
  }
  for (sgh_graph *g : dev->graphs) {
    auto b = g->born.find(ptr);
    if (b != g->born.end()) {
      g->born.erase(b);
      g->held.emplace_back(ptr, r);
      return SGH_OK;
    }
  }
  if (aux_use) {
    // work on the auxiliary stream may still touch the block: it waits for the next join / sync
    dev->pending.emplace_back(ptr, r);
    return SGH_OK;
  }
  // Work already enqueued on the device stream may still read the block; the next owner's
  // work is enqueued behind it on the same stream, so immediate reuse is ordered correctly.
  dev->free_blocks.emplace(r, ptr);
  dev->cached += r;
  return SGH_OK;
}

int sgh_pool_stats(sgh_device *dev, size_t *in_use, size_t *cached, size_t *driver_allocs) {
  if (!dev) return SGH_EINVAL;
  std::lock_guard<std::mutex> lk(dev->mu);
  if (in_use) *in_use = dev->in_use;
  if (cached) *cached = dev->cached;
  if (driver_allocs) *driver_allocs = dev->driver_allocs;
  return SGH_OK;
}

int sgh_upload_async(sgh_device *dev, void *dst, const void *src, size_t bytes) {
  if (!dev) return SGH_EINVAL;
  if (bytes == 0) return SGH_OK;
  if (!dst || !src) return SGH_EINVAL;
  if (dev->capturing || bytes > sgh_device::kUploadSlotBytes) return sgh_memcpy(dev, dst, src, bytes, 1);
  sgh_weights_epoch_bump();   // the destination may be a weight tensor
  std::lock_guard<std::mutex> lk(dev->mu);
  if (!dev->upload_host) {
    void *h = nullptr;
    SGH_HIP_TRY(hipHostMalloc(&h, sgh_device::kUploadSlots * sgh_device::kUploadSlotBytes, hipHostMallocDefault));
    dev->upload_host = static_cast<char *>(h);
  }
  const int slot = dev->upload_next;
  dev->upload_next = (slot + 1) % sgh_device::kUploadSlots;
  if (!dev->upload_done[slot]) SGH_HIP_TRY(hipEventCreateWithFlags(&dev->upload_done[slot], hipEventDisableTiming));
  else SGH_HIP_TRY(hipEventSynchronize(dev->upload_done[slot]));   // the copy issued kUploadSlots uploads ago
  char *stage = dev->upload_host + size_t(slot) * sgh_device::kUploadSlotBytes;
  memcpy(stage, src, bytes);
  SGH_HIP_TRY(hipMemcpyAsync(dst, stage, bytes, hipMemcpyHostToDevice, dev->stream));
  SGH_HIP_TRY(hipEventRecord(dev->upload_done[slot], dev->stream));
  return SGH_OK;
}

int sgh_memcpy(sgh_device *dev, void *dst, const void *src, size_t bytes, int kind) {
  if (!dev || kind < 0 || kind > 3) return SGH_EINVAL;
  if (bytes == 0) return SGH_OK;
  if (!dst || !src) return SGH_EINVAL;
  if (kind == 1 || kind == 3) sgh_weights_epoch_bump();   // the destination may be a weight tensor
  static const hipMemcpyKind kinds[4] = {hipMemcpyHostToHost, hipMemcpyHostToDevice,
                                         hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice};
  if (dev->capturing && kind != 3) {
    // a host copy cannot wait on a recording stream: an upload happens now, outside the graph
    // (small tables the recorded kernels read); a download has nothing to read yet
    if (kind == 2) return SGH_EUNSUPPORTED;
    SGH_HIP_TRY(hipMemcpyAsync(dst, src, bytes, kinds[kind], dev->side));
    SGH_HIP_TRY(hipStreamSynchronize(dev->side));
    return SGH_OK;
  }
  SGH_HIP_TRY(hipMemcpyAsync(dst, src, bytes, kinds[kind], dev->stream));
  if (kind != 3) SGH_HIP_TRY(hipStreamSynchronize(dev->stream));
  return SGH_OK;
}

int sgh_prof_enable(int on) {
  if (on) prof_clear();
  g_prof_on = on != 0;
  return SGH_OK;
}

int sgh_prof_clear(void) {
  if (g_prof_on) return SGH_EINVAL;   // (records are still being taken)
  prof_clear();
  return SGH_OK;
}

int sgh_prof_count(int *n) {
  if (!n) return SGH_EINVAL;
  *n = int(g_prof.size());
  return SGH_OK;
}

int sgh_prof_get(int i, char *tag, size_t tag_len, float *ms, double *work) {
  if (i < 0 || size_t(i) >= g_prof.size() || !ms) return SGH_EINVAL;
  const ProfRec &r = g_prof[i];
  SGH_HIP_TRY(hipEventSynchronize(r.b));
  SGH_HIP_TRY(hipEventElapsedTime(ms, r.a, r.b));
  if (work) *work = r.work;
  if (tag && tag_len) {
    size_t k = 0;
    for (; r.tag[k] && k + 1 < tag_len; ++k) tag[k] = r.tag[k];
    tag[k] = 0;
  }
  return SGH_OK;
}

int sgh_event_create(sgh_event **ev) {
  if (!ev) return SGH_EINVAL;
  sgh_event *e = new (std::nothrow) sgh_event();
  if (!e) return SGH_ENOMEM;
  hipError_t rc = hipEventCreate(&e->ev);
  if (rc != hipSuccess) {
    delete e;
    return (int)rc;
  }
  *ev = e;
  return SGH_OK;
}

int sgh_event_destroy(sgh_event *ev) {
  if (!ev) return SGH_EINVAL;
  (void)hipEventDestroy(ev->ev);
  delete ev;
  return SGH_OK;
}

int sgh_event_record(sgh_event *ev, void *stream) {
  if (!ev) return SGH_EINVAL;
  SGH_HIP_TRY(hipEventRecord(ev->ev, sgh_stream_of(stream)));
  return SGH_OK;
}

int sgh_event_elapsed_ms(sgh_event *start, sgh_event *stop, float *ms) {
  if (!start || !stop || !ms) return SGH_EINVAL;
  SGH_HIP_TRY(hipEventSynchronize(stop->ev));
  SGH_HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
  return SGH_OK;
}

}  // extern "C"
