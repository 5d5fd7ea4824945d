// Context, buffer pool and the storage half of the C ABI (register / write / read /
// dispose / memory / time), i.e. the TensorStorage contract of the reference's
// KernelBackend (tfjs-core/src/backends/backend.ts:33-44, 92-126) on device memory.
#include "tfhip_internal.h"

using tfhip::Buf;

static thread_local std::string g_init_error;

int tfhip_ctx::fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  err = buf;
  return code;
}

Buf* tfhip_ctx::find(int64_t id) {
  auto it = bufs.find(id);
  if (it == bufs.end()) {
    fail(TFHIP_ENOENT, "unknown data id %lld", (long long)id);
    return nullptr;
  }
  return &it->second;
}

// Block sizes are rounded so that tensors of similar size share blocks: 512 B granules up
// to 1 MiB, then 1/8-octave steps (at most 12.5 % slack on large activations).
static size_t round_cap(size_t n) {
  if (n <= (1u << 20)) return (n + 511) & ~size_t(511);
  size_t step = size_t(1) << (63 - __builtin_clzll(n) - 3);
  return (n + step - 1) & ~(step - 1);
}

void* tfhip_ctx::alloc(size_t nbytes, size_t* cap) {
  const size_t want = round_cap(nbytes);
  auto it = pool.find(want);
  if (it != pool.end() && !it->second.empty()) {
    // most recently freed block first: it is the one most likely still in L2 / MALL
    void* p = it->second.back();
    it->second.pop_back();
    pooled -= want;
    in_use += want;
    *cap = want;
    if (capturing) capture_blocks.push_back(p);
    return p;
  }
  if (capturing) {
    // a capture must find every block in the pool (the same work has run once before it):
    // allocating here would put a device allocation into the middle of a stream capture
    fail(TFHIP_EDEVICE, "graph capture needs a block of %zu bytes that the pool does not hold; "
                        "run the captured work once before capturing it", want);
    return nullptr;
  }
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, want);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    trim();  // give parked blocks back to the driver and try once more
    e = hipMalloc(&p, want);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    fail(TFHIP_EDEVICE, "hipMalloc(%zu bytes): %s", want, hipGetErrorString(e));
    return nullptr;
  }
  in_use += want;
  *cap = want;
  return p;
}

void tfhip_ctx::release(void* p, size_t cap) {
  if (!p) return;
  in_use -= cap;
  auto own = owner.find(p);
  if (own != owner.end()) {  // a block that a captured graph writes on every replay
    graphs[own->second].parked.emplace_back(p, cap);
    return;
  }
  pooled += cap;
  pool[cap].push_back(p);
}

void tfhip_ctx::trim() {
  // (not while a graph exists: a replay may still read blocks that went back to the pool)
  if (pool.empty() || capturing || !graphs.empty()) return;
  (void)hipStreamSynchronize(stream);
  for (auto& kv : pool)
    for (void* p : kv.second) (void)hipFree(p);
  pool.clear();
  pooled = 0;
}

extern "C" {

int tfhip_init(int device, tfhip_ctx** out) {
  if (!out) return TFHIP_EINVAL;
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) {
    g_init_error = std::string("no HIP device available: ") +
                   (e != hipSuccess ? hipGetErrorString(e) : "device count is 0");
    (void)hipGetLastError();
    return TFHIP_EDEVICE;
  }
  if (device < 0 || device >= count) {
    g_init_error = "device index out of range";
    return TFHIP_EINVAL;
  }
  tfhip_ctx* ctx = new tfhip_ctx();
  ctx->device = device;
  hipDeviceProp_t prop;
  if ((e = hipSetDevice(device)) != hipSuccess ||
      (e = hipGetDeviceProperties(&prop, device)) != hipSuccess ||
      (e = hipStreamCreate(&ctx->stream)) != hipSuccess ||
      (e = hipEventCreate(&ctx->ev_begin)) != hipSuccess ||
      (e = hipEventCreate(&ctx->ev_end)) != hipSuccess) {
    g_init_error = std::string("device set-up failed: ") + hipGetErrorString(e);
    delete ctx;
    return TFHIP_EDEVICE;
  }
  if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0) {
    g_init_error = std::string("libtfjs_hip is built for gfx950 only, device is ") +
                   prop.gcnArchName;
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return TFHIP_ENOTSUP;
  }
  ctx->num_cus = prop.multiProcessorCount;
  *out = ctx;
  return TFHIP_OK;
}

void tfhip_destroy(tfhip_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& kv : ctx->bufs)
    if (kv.second.ptr) (void)hipFree(kv.second.ptr);
  for (auto& kv : ctx->pool)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : ctx->graphs) {
    (void)hipGraphExecDestroy(kv.second.exec);
    (void)hipGraphDestroy(kv.second.graph);
    for (auto& blk : kv.second.parked) (void)hipFree(blk.first);
  }
  (void)hipEventDestroy(ctx->ev_begin);
  (void)hipEventDestroy(ctx->ev_end);
  (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

const char* tfhip_last_error(tfhip_ctx* ctx) {
  return ctx ? ctx->err.c_str() : g_init_error.c_str();
}

int tfhip_register(tfhip_ctx* ctx, int64_t id, const int32_t* shape, int rank, int dtype) {
  if (!ctx) return TFHIP_EINVAL;
  if (rank < 0 || rank > 8 || (rank > 0 && !shape))
    return ctx->fail(TFHIP_EINVAL, "register: rank %d not in 0..8", rank);
  if (dtype < TFHIP_FLOAT32 || dtype > TFHIP_UINT8Q)
    return ctx->fail(TFHIP_EINVAL, "register: unknown dtype code %d", dtype);
  if (ctx->bufs.count(id))  // backend_cpu.ts:119-121
    return ctx->fail(TFHIP_EEXIST, "Data buffer is already registered");
  Buf b;
  b.dtype = dtype;
  b.rank = rank;
  b.numel = 1;
  for (int i = 0; i < rank; i++) {
    if (shape[i] < 0) return ctx->fail(TFHIP_EINVAL, "register: negative dimension");
    b.shape[i] = shape[i];
    b.numel *= shape[i];
  }
  b.nbytes = (size_t)b.numel * tfhip::dtype_size(dtype);
  if (b.nbytes) {
    b.ptr = ctx->alloc(b.nbytes, &b.cap);
    if (!b.ptr) return TFHIP_EDEVICE;
  }
  ctx->bufs.emplace(id, b);
  return TFHIP_OK;
}

int tfhip_write(tfhip_ctx* ctx, int64_t id, const void* host, size_t nbytes) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing)
    return ctx->fail(TFHIP_EINVAL, "write: host data cannot enter a graph capture (create the "
                                   "tensor before capturing)");
  TFHIP_GET(ctx, b, id);
  if (!host && nbytes)  // backend_cpu.ts:125-127
    return ctx->fail(TFHIP_EINVAL, "MathBackendHIP.write(): values can not be null");
  if (nbytes != b->nbytes)
    return ctx->fail(TFHIP_EINVAL, "write: got %zu bytes for a buffer of %zu", nbytes, b->nbytes);
  if (!nbytes) return TFHIP_OK;
  // The caller may reuse or free `host` as soon as this returns, so wait for the copy.
  TFHIP_HIP(ctx, hipMemcpyAsync(b->ptr, host, nbytes, hipMemcpyHostToDevice, ctx->stream));
  TFHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return TFHIP_OK;
}

int tfhip_read(tfhip_ctx* ctx, int64_t id, void* host, size_t nbytes) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "read: not during a graph capture");
  TFHIP_GET(ctx, b, id);
  if (nbytes != b->nbytes)
    return ctx->fail(TFHIP_EINVAL, "read: asked %zu bytes of a buffer of %zu", nbytes, b->nbytes);
  if (nbytes)
    TFHIP_HIP(ctx, hipMemcpyAsync(host, b->ptr, nbytes, hipMemcpyDeviceToHost, ctx->stream));
  TFHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return TFHIP_OK;
}

int tfhip_dispose(tfhip_ctx* ctx, int64_t id) {
  if (!ctx) return TFHIP_EINVAL;
  auto it = ctx->bufs.find(id);
  if (it == ctx->bufs.end()) return TFHIP_OK;  // backend_cpu.ts:228-237: unknown id is a no-op
  ctx->release(it->second.ptr, it->second.cap);
  ctx->bufs.erase(it);
  return TFHIP_OK;
}

int tfhip_mem_info(tfhip_ctx* ctx, size_t* in_use, size_t* pooled, size_t* num_ids) {
  if (!ctx) return TFHIP_EINVAL;
  if (in_use) *in_use = ctx->in_use;
  if (pooled) *pooled = ctx->pooled;
  if (num_ids) *num_ids = ctx->bufs.size();
  return TFHIP_OK;
}

int tfhip_sync(tfhip_ctx* ctx) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "sync: not during a graph capture");
  TFHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return TFHIP_OK;
}

int tfhip_time_begin(tfhip_ctx* ctx) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "time: not during a graph capture");
  TFHIP_HIP(ctx, hipEventRecord(ctx->ev_begin, ctx->stream));
  ctx->timing = true;
  return TFHIP_OK;
}

int tfhip_time_end(tfhip_ctx* ctx, float* ms) {
  if (!ctx || !ms) return TFHIP_EINVAL;
  if (!ctx->timing) return ctx->fail(TFHIP_EINVAL, "time_end without time_begin");
  ctx->timing = false;
  TFHIP_HIP(ctx, hipEventRecord(ctx->ev_end, ctx->stream));
  TFHIP_HIP(ctx, hipEventSynchronize(ctx->ev_end));
  TFHIP_HIP(ctx, hipEventElapsedTime(ms, ctx->ev_begin, ctx->ev_end));
  return TFHIP_OK;
}

// ---- captured graphs ---------------------------------------------------------------------
int tfhip_graph_begin(tfhip_ctx* ctx) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "graph_begin: a capture is already running");
  ctx->capture_blocks.clear();
  TFHIP_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
  ctx->capturing = true;
  return TFHIP_OK;
}

int tfhip_graph_end(tfhip_ctx* ctx, int64_t* graph_id) {
  if (!ctx || !graph_id) return TFHIP_EINVAL;
  if (!ctx->capturing) return ctx->fail(TFHIP_EINVAL, "graph_end without graph_begin");
  ctx->capturing = false;
  tfhip_ctx::Graph g;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g.graph);
  if (e == hipSuccess) e = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    if (g.graph) (void)hipGraphDestroy(g.graph);
    ctx->capture_blocks.clear();
    return ctx->fail(TFHIP_EDEVICE, "graph capture failed: %s", hipGetErrorString(e));
  }
  const int64_t id = ctx->next_graph++;
  // Every block the capture handed out now belongs to the graph: those lying free in the pool
  // are taken out of it, the others follow when their tensor lets go of them (release()).
  for (void* p : ctx->capture_blocks) {
    if (ctx->owner.count(p)) continue;
    ctx->owner[p] = id;
    for (auto& kv : ctx->pool) {
      auto& v = kv.second;
      for (size_t i = 0; i < v.size(); i++) {
        if (v[i] != p) continue;
        v.erase(v.begin() + i);
        ctx->pooled -= kv.first;
        g.parked.emplace_back(p, kv.first);
        break;
      }
    }
  }
  ctx->capture_blocks.clear();
  ctx->graphs.emplace(id, std::move(g));
  *graph_id = id;
  return TFHIP_OK;
}

int tfhip_graph_launch(tfhip_ctx* ctx, int64_t graph_id) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "graph_launch: not during a graph capture");
  auto it = ctx->graphs.find(graph_id);
  if (it == ctx->graphs.end()) return ctx->fail(TFHIP_ENOENT, "graph %lld does not exist", (long long)graph_id);
  TFHIP_HIP(ctx, hipGraphLaunch(it->second.exec, ctx->stream));
  return TFHIP_OK;
}

int tfhip_graph_destroy(tfhip_ctx* ctx, int64_t graph_id) {
  if (!ctx) return TFHIP_EINVAL;
  auto it = ctx->graphs.find(graph_id);
  if (it == ctx->graphs.end()) return TFHIP_OK;
  // queued replays may still run: wait before the blocks can be handed to anyone else
  (void)hipStreamSynchronize(ctx->stream);
  (void)hipGraphExecDestroy(it->second.exec);
  (void)hipGraphDestroy(it->second.graph);
  for (auto& blk : it->second.parked) {
    ctx->pooled += blk.second;
    ctx->pool[blk.second].push_back(blk.first);
  }
  for (auto o = ctx->owner.begin(); o != ctx->owner.end();)
    o = o->second == graph_id ? ctx->owner.erase(o) : std::next(o);
  ctx->graphs.erase(it);
  return TFHIP_OK;
}

const char* tfhip_last_kernel(tfhip_ctx* ctx) { return ctx ? ctx->last_kernel : ""; }

int tfhip_device_ptr(tfhip_ctx* ctx, int64_t id, void** ptr, size_t* nbytes) {
  if (!ctx || !ptr) return TFHIP_EINVAL;
  TFHIP_GET(ctx, b, id);
  *ptr = b->ptr;
  if (nbytes) *nbytes = b->nbytes;
  return TFHIP_OK;
}

}  // extern "C"

namespace tfhip {

int as_f32(tfhip_ctx* ctx, const Buf* b, Temp* tmp, const float** out) {
  if (b->dtype == TFHIP_FLOAT32 || b->numel == 0) {
    *out = static_cast<const float*>(b->ptr);
    return TFHIP_OK;
  }
  if (b->dtype == TFHIP_UINT8Q)
    return ctx->fail(TFHIP_EINVAL, "quantised buffer used where float data is expected");
  if (!tmp->get((size_t)b->numel * 4)) return TFHIP_EDEVICE;
  int rc = launch_convert(ctx, b->ptr, b->dtype, tmp->ptr, TFHIP_FLOAT32, b->numel);
  *out = static_cast<const float*>(tmp->ptr);
  return rc;
}

}  // namespace tfhip
