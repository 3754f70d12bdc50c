// Device context, pooled ref-counted allocations, copies and timers.
// Replaces the storage/device half of rai's candle backend:
// rai-core/src/backend/candle.rs:18-68 (TensorLike), :133-195 (device cache).
#include <map>
#include <mutex>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "common.h"

namespace rai {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

struct Block {
  int dev;
  size_t bytes;  // rounded size class
  int refs;
};

struct DeviceCtx {
  int dev = -1;
  bool ready = false;
  hipStream_t stream = nullptr;
  std::mutex mu;
  std::map<size_t, std::vector<void *>> pool;  // size class -> free blocks
  uint64_t in_use = 0, pooled = 0, n_mallocs = 0;
  // Blocks of up to kCarveMax bytes are cut from slabs of kSlabBytes (one hipMalloc per slab instead of one per first
  // use of a size: a 32-layer prefill through the graph evaluator asks for ~80 sizes it has not seen, at ~0.2 ms per
  // hipMalloc).  A cut block lives in the pool like any other once released; only whole hipMalloc blocks go back to
  // the driver in rai_hip_trim.
  char *slab = nullptr;
  size_t slab_left = 0;
  std::unordered_set<void *> carved;
  void *ws = nullptr;
  size_t ws_bytes = 0;
  unsigned long long *index_errors = nullptr;
  int num_cu = 0;                      // compute units of this GPU, asked of the device once
  int *fault_host = nullptr;           // pinned, device-visible word a kernel sets when a bounded wait of its own expires
  int *fault_dev = nullptr;            // the same word's device address
};

static constexpr int kMaxDev = 16;
static DeviceCtx g_ctx[kMaxDev];
static std::mutex g_mu;
static std::unordered_map<void *, Block> g_blocks;  // live (handed out) blocks

static constexpr size_t kSlabBytes = size_t(256) << 20, kCarveMax = size_t(32) << 20;

static size_t size_class(size_t bytes) {
  if (bytes == 0) bytes = 1;
  if (bytes <= (1u << 20)) return (bytes + 511) & ~size_t(511);
  const size_t two_mb = size_t(2) << 20;
  return (bytes + two_mb - 1) / two_mb * two_mb;
}

DeviceCtx *ctx(int dev) {
  if (dev < 0 || dev >= kMaxDev) {
    set_error("device index %d out of range", dev);
    return nullptr;
  }
  DeviceCtx *c = &g_ctx[dev];
  if (c->ready) return c;
  std::lock_guard<std::mutex> lk(g_mu);
  if (c->ready) return c;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || dev >= n) {
    set_error("no HIP device %d (count=%d, %s)", dev, n, hipGetErrorString(e));
    return nullptr;
  }
  // a failed set-up leaves nothing behind: the next call starts from scratch instead of leaking a stream and a buffer
  auto undo = [&]() {
    if (c->stream) (void)hipStreamDestroy(c->stream);
    if (c->index_errors) (void)hipFree(c->index_errors);
    if (c->fault_host) (void)hipHostFree(c->fault_host);
    c->stream = nullptr;
    c->index_errors = nullptr;
    c->fault_host = c->fault_dev = nullptr;
  };
  if ((e = hipSetDevice(dev)) != hipSuccess || (e = hipStreamCreate(&c->stream)) != hipSuccess ||
      (e = hipMalloc((void **)&c->index_errors, sizeof(unsigned long long))) != hipSuccess ||
      (e = hipMemset(c->index_errors, 0, sizeof(unsigned long long))) != hipSuccess ||
      (e = hipDeviceGetAttribute(&c->num_cu, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess ||
      (e = hipHostMalloc((void **)&c->fault_host, 64, hipHostMallocMapped)) != hipSuccess ||
      (e = hipHostGetDevicePointer((void **)&c->fault_dev, c->fault_host, 0)) != hipSuccess) {
    set_error("device %d init failed: %s", dev, hipGetErrorString(e));
    undo();
    return nullptr;
  }
  // per-device addresses of the library's fixed device arrays (this device is current here); the callee has set the
  // error text, device number included
  if (arg_static_scratch_init(dev) != RAI_OK) {
    undo();
    return nullptr;
  }
  *c->fault_host = 0;
  c->dev = dev;
  c->ready = true;
  return c;
}

hipStream_t stream_if_ready(int dev) {
  if (dev < 0 || dev >= kMaxDev || !g_ctx[dev].ready) {
    set_error("device %d is not initialised: call rai_hip_init(%d) first", dev, dev);
    return nullptr;
  }
  return g_ctx[dev].stream;
}

hipStream_t stream_of(int dev) {
  DeviceCtx *c = ctx(dev);
  return c ? c->stream : nullptr;
}

int device_cu_count(int dev) {
  DeviceCtx *c = ctx(dev);
  return c ? c->num_cu : 0;
}

int *kernel_fault_word(int dev) {
  DeviceCtx *c = ctx(dev);
  return c ? c->fault_dev : nullptr;
}

int check_kernel_fault(int dev) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  const int code = *(volatile int *)c->fault_host;
  if (code == 0) return RAI_OK;
  *(volatile int *)c->fault_host = 0;
  // whatever the kernels of that launch left behind is not to be trusted: start the next one from clean counters
  (void)streamk_counters_reset(dev, c->stream);
  (void)hipStreamSynchronize(c->stream);
  return fail(RAI_ERR_HIP, "device %d: a kernel gave up a bounded wait (code %d: %s); results since the last synchronisation are invalid",
              dev, code, code == RAI_FAULT_STREAMK ? "stream-K share never arrived"
              : code == RAI_FAULT_CHAIN ? "a block never reached a barrier of the decode chain kernel" : "unknown");
}

unsigned long long *index_error_counter(int dev) {
  DeviceCtx *c = ctx(dev);
  return c ? c->index_errors : nullptr;
}

int workspace(int dev, size_t bytes, void **out) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  std::lock_guard<std::mutex> lk(c->mu);
  if (bytes > c->ws_bytes) {
    // The old block may still be read by enqueued kernels: drain first.
    RAI_HIP_TRY(hipSetDevice(dev));
    RAI_HIP_TRY(hipStreamSynchronize(c->stream));
    if (c->ws) RAI_HIP_TRY(hipFree(c->ws));
    c->ws = nullptr;
    c->ws_bytes = 0;
    size_t want = size_class(bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes);
    hipError_t e = hipMalloc(&c->ws, want);
    if (e != hipSuccess) return fail(RAI_ERR_OOM, "workspace of %zu bytes: %s", want, hipGetErrorString(e));
    c->ws_bytes = want;
    c->n_mallocs++;
  }
  *out = c->ws;
  return RAI_OK;
}

int launch_check(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RAI_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
  return RAI_OK;
}

int validate(const rai_hip_tensor *t, const char *name) {
  if (!t) return fail(RAI_ERR_BAD_ARG, "%s: null tensor", name);
  if (t->rank < 0 || t->rank > RAI_HIP_MAX_RANK) return fail(RAI_ERR_BAD_SHAPE, "%s: rank %d", name, t->rank);
  if (dtype_size(t->dtype) == 0) return fail(RAI_ERR_BAD_DTYPE, "%s: dtype %d", name, t->dtype);
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) {
    if (t->shape[i] < 0) return fail(RAI_ERR_BAD_SHAPE, "%s: shape[%d]=%lld", name, i, (long long)t->shape[i]);
    if (t->stride[i] < 0) return fail(RAI_ERR_BAD_STRIDE, "%s: stride[%d]=%lld", name, i, (long long)t->stride[i]);
    n *= t->shape[i];
  }
  if (t->offset < 0) return fail(RAI_ERR_BAD_STRIDE, "%s: negative offset", name);
  if (n > 0 && !t->data) return fail(RAI_ERR_BAD_ARG, "%s: null data pointer", name);
  return RAI_OK;
}

void coalesce(int n, const rai_hip_tensor *const *ts, StridedArgs *out) {
  const rai_hip_tensor *t0 = ts[0];
  int r = 0;
  // Drop size-1 dims, then merge dim i into i+1 when every operand satisfies
  // stride[i] == stride[i+1] * shape[i+1].
  int64_t shp[RAI_HIP_MAX_RANK];
  int64_t str[3][RAI_HIP_MAX_RANK];
  for (int i = 0; i < t0->rank; ++i) {
    if (t0->shape[i] == 1) continue;
    shp[r] = t0->shape[i];
    for (int k = 0; k < n; ++k) str[k][r] = ts[k]->stride[i];
    ++r;
  }
  int w = 0;
  for (int i = 0; i < r; ++i) {
    if (w > 0) {
      bool merge = true;
      for (int k = 0; k < n; ++k)
        if (str[k][w - 1] != str[k][i] * shp[i]) merge = false;
      if (merge) {
        shp[w - 1] *= shp[i];
        for (int k = 0; k < n; ++k) str[k][w - 1] = str[k][i];
        continue;
      }
    }
    shp[w] = shp[i];
    for (int k = 0; k < n; ++k) str[k][w] = str[k][i];
    ++w;
  }
  if (w == 0) {
    w = 1;
    shp[0] = 1;
    for (int k = 0; k < n; ++k) str[k][0] = 1;
  }
  out->rank = w;
  for (int i = 0; i < RAI_HIP_MAX_RANK; ++i) {
    out->shape[i] = i < w ? shp[i] : 1;
    for (int k = 0; k < 3; ++k) out->stride[k][i] = (k < n && i < w) ? str[k][i] : 0;
  }
}

}  // namespace rai

using namespace rai;

extern "C" {

const char *rai_hip_last_error(void) { return g_err; }

int rai_hip_device_count(int *count) {
  RAI_REQUIRE(count, RAI_ERR_BAD_ARG, "count is null");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    *count = 0;
    return fail(RAI_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
  }
  *count = n;
  return RAI_OK;
}

int rai_hip_init(int dev) { return ctx(dev) ? RAI_OK : RAI_ERR_HIP; }

int rai_hip_sync(int dev) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  return check_kernel_fault(dev);
}

int rai_hip_alloc(int dev, size_t bytes, void **out) {
  RAI_REQUIRE(out, RAI_ERR_BAD_ARG, "out is null");
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  size_t cls = size_class(bytes);
  void *p = nullptr;
  {
    std::lock_guard<std::mutex> lk(c->mu);
    auto it = c->pool.find(cls);
    if (it != c->pool.end() && !it->second.empty()) {
      p = it->second.back();
      it->second.pop_back();
      c->pooled -= cls;
    }
  }
  if (!p && cls <= kCarveMax) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (c->slab_left < cls) {   // the rest of the old slab stays unused (at most one block's worth)
      void *fresh = nullptr;
      if (hipSetDevice(dev) == hipSuccess && hipMalloc(&fresh, kSlabBytes) == hipSuccess) {
        c->slab = (char *)fresh;
        c->slab_left = kSlabBytes;
        c->n_mallocs++;
      } else {
        (void)hipGetLastError();   // no room for a slab: a block of its own below
      }
    }
    if (c->slab_left >= cls) {
      p = c->slab;
      c->slab += cls;
      c->slab_left -= cls;
      c->carved.insert(p);
    }
  }
  if (!p) {
    RAI_HIP_TRY(hipSetDevice(dev));
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
      // Give pooled memory back and retry once.
      rai_hip_trim(dev);
      e = hipMalloc(&p, cls);
    }
    if (e != hipSuccess) return fail(RAI_ERR_OOM, "hipMalloc(%zu): %s", cls, hipGetErrorString(e));
    std::lock_guard<std::mutex> lk(c->mu);
    c->n_mallocs++;
  }
  {
    std::lock_guard<std::mutex> lk(g_mu);
    g_blocks[p] = Block{dev, cls, 1};
  }
  {
    std::lock_guard<std::mutex> lk(c->mu);
    c->in_use += cls;
  }
  *out = p;
  return RAI_OK;
}

int rai_hip_retain(void *ptr) {
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_blocks.find(ptr);
  if (it == g_blocks.end()) return fail(RAI_ERR_BAD_ARG, "retain of unknown pointer %p", ptr);
  it->second.refs++;
  return RAI_OK;
}

int rai_hip_release(void *ptr) {
  if (!ptr) return RAI_OK;
  Block b;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_blocks.find(ptr);
    if (it == g_blocks.end()) return fail(RAI_ERR_BAD_ARG, "release of unknown pointer %p", ptr);
    if (--it->second.refs > 0) return RAI_OK;
    b = it->second;
    g_blocks.erase(it);
  }
  // All work is ordered on the device's single stream, so a block returned to
  // the pool can be handed out again immediately: later kernels run after the
  // ones still reading it.
  DeviceCtx *c = &g_ctx[b.dev];
  std::lock_guard<std::mutex> lk(c->mu);
  c->pool[b.bytes].push_back(ptr);
  c->in_use -= b.bytes;
  c->pooled += b.bytes;
  return RAI_OK;
}

int rai_hip_mem_stats(int dev, uint64_t *in_use, uint64_t *pooled, uint64_t *n_device_mallocs) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  std::lock_guard<std::mutex> lk(c->mu);
  if (in_use) *in_use = c->in_use;
  if (pooled) *pooled = c->pooled;
  if (n_device_mallocs) *n_device_mallocs = c->n_mallocs;
  return RAI_OK;
}

int rai_hip_trim(int dev) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  RAI_HIP_TRY(hipSetDevice(dev));
  RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  std::lock_guard<std::mutex> lk(c->mu);
  for (auto &kv : c->pool) {
    std::vector<void *> kept;
    for (void *p : kv.second) {
      if (c->carved.count(p)) { kept.push_back(p); continue; }   // part of a slab: stays pooled
      (void)hipFree(p);
      c->pooled -= kv.first;
    }
    kv.second.swap(kept);
  }
  return RAI_OK;
}

int rai_hip_h2d(int dev, void *dst_dev, const void *src_host, size_t bytes) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  if (bytes == 0) return RAI_OK;
  RAI_REQUIRE(dst_dev && src_host, RAI_ERR_BAD_ARG, "h2d: null pointer");
  // Pageable source: hipMemcpyAsync stages it before returning, so the host
  // buffer may be reused by the caller right away.
  RAI_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, c->stream));
  RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  return RAI_OK;
}

int rai_hip_d2h(int dev, void *dst_host, const void *src_dev, size_t bytes) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  if (bytes == 0) return RAI_OK;
  RAI_REQUIRE(dst_host && src_dev, RAI_ERR_BAD_ARG, "d2h: null pointer");
  RAI_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, c->stream));
  RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  return check_kernel_fault(dev);   // what was copied came from kernels that may have given up a wait
}

int rai_hip_d2d(int dev, void *dst_dev, const void *src_dev, size_t bytes) {
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  if (bytes == 0) return RAI_OK;
  RAI_REQUIRE(dst_dev && src_dev, RAI_ERR_BAD_ARG, "d2d: null pointer");
  RAI_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, c->stream));
  return RAI_OK;
}

int rai_hip_to_device(int src_dev, const rai_hip_tensor *in, int dst_dev, const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "to_device: dtype %s vs %s", dtype_name(in->dtype),
              dtype_name(out->dtype));
  RAI_REQUIRE(same_shape(in, out), RAI_ERR_BAD_SHAPE, "to_device: shapes differ");
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "to_device: output must be contiguous");
  if (src_dev == dst_dev) return rai_hip_copy(dst_dev, in, out);
  DeviceCtx *cs = ctx(src_dev), *cd = ctx(dst_dev);
  if (!cs || !cd) return RAI_ERR_HIP;
  const size_t bytes = (size_t)numel(in) * dtype_size(in->dtype);
  if (bytes == 0) return RAI_OK;
  // a contiguous image of the source on its own device (the tensor itself when it already is one)
  void *tmp = nullptr;
  const void *src = (const char *)in->data + in->offset * (int64_t)dtype_size(in->dtype);
  if (!is_contiguous(in)) {
    RAI_TRY(rai_hip_alloc(src_dev, bytes, &tmp));
    rai_hip_tensor t = *out;
    t.data = tmp;
    t.offset = 0;
    int rc = rai_hip_copy(src_dev, in, &t);
    if (rc != RAI_OK) { (void)rai_hip_release(tmp); return rc; }
    src = tmp;
  }
  // the peer copy runs on the destination's stream, after everything queued on the source's stream so far
  hipError_t e = hipStreamSynchronize(cs->stream);
  if (e == hipSuccess) e = hipSetDevice(dst_dev);
  if (e == hipSuccess)
    e = hipMemcpyPeerAsync((char *)out->data + out->offset * (int64_t)dtype_size(out->dtype), dst_dev, src, src_dev, bytes,
                           cd->stream);
  if (e == hipSuccess && tmp) e = hipStreamSynchronize(cd->stream);   // tmp goes back to the source's pool below
  if (tmp) (void)rai_hip_release(tmp);
  if (e != hipSuccess) return fail(RAI_ERR_HIP, "to_device %d -> %d: %s", src_dev, dst_dev, hipGetErrorString(e));
  return RAI_OK;
}

struct Timer {
  int dev;
  hipEvent_t a, b;
};

int rai_hip_timer_create(int dev, void **timer) {
  RAI_REQUIRE(timer, RAI_ERR_BAD_ARG, "timer is null");
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  Timer *t = new Timer{dev, nullptr, nullptr};
  RAI_HIP_TRY(hipEventCreate(&t->a));
  RAI_HIP_TRY(hipEventCreate(&t->b));
  *timer = t;
  return RAI_OK;
}
int rai_hip_timer_start(void *timer) {
  Timer *t = static_cast<Timer *>(timer);
  RAI_REQUIRE(t, RAI_ERR_BAD_ARG, "timer is null");
  RAI_HIP_TRY(hipEventRecord(t->a, stream_of(t->dev)));
  return RAI_OK;
}
int rai_hip_timer_stop(void *timer) {
  Timer *t = static_cast<Timer *>(timer);
  RAI_REQUIRE(t, RAI_ERR_BAD_ARG, "timer is null");
  RAI_HIP_TRY(hipEventRecord(t->b, stream_of(t->dev)));
  return RAI_OK;
}
int rai_hip_timer_elapsed_ms(void *timer, float *ms) {
  Timer *t = static_cast<Timer *>(timer);
  RAI_REQUIRE(t && ms, RAI_ERR_BAD_ARG, "timer/ms is null");
  RAI_HIP_TRY(hipEventSynchronize(t->b));
  RAI_HIP_TRY(hipEventElapsedTime(ms, t->a, t->b));
  return RAI_OK;
}
int rai_hip_timer_destroy(void *timer) {
  Timer *t = static_cast<Timer *>(timer);
  if (!t) return RAI_OK;
  (void)hipEventDestroy(t->a);
  (void)hipEventDestroy(t->b);
  delete t;
  return RAI_OK;
}

int rai_hip_index_errors(int dev, uint64_t *count) {
  RAI_REQUIRE(count, RAI_ERR_BAD_ARG, "count is null");
  DeviceCtx *c = ctx(dev);
  if (!c) return RAI_ERR_HIP;
  unsigned long long v = 0;
  RAI_HIP_TRY(hipMemcpyAsync(&v, c->index_errors, sizeof(v), hipMemcpyDeviceToHost, c->stream));
  RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  *count = v;
  if (v) {
    unsigned long long zero = 0;
    RAI_HIP_TRY(hipMemcpyAsync(c->index_errors, &zero, sizeof(zero), hipMemcpyHostToDevice, c->stream));
    RAI_HIP_TRY(hipStreamSynchronize(c->stream));
  }
  return RAI_OK;
}

}  // extern "C"
