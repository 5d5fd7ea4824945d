// Context, buffer pool and the storage half of the C ABI (register / write / read /
// dispose / memory / time), i.e. the TensorStorage contract of the reference's
// KernelBackend (tfjs-core/src/backends/backend.ts:33-44, 92-126) on device memory.
#include "tfhip_internal.h"

using tfhip::Buf;

static thread_local std::string g_init_error;

// Pinned host memory is process-wide: buffers handed to callers (tfhip_host_alloc) outlive any
// one context, and finished reads leave their staging blocks here for the next read.
static std::mutex g_host_mu;
static std::map<uintptr_t, size_t> g_pinned;                  // start -> bytes
static std::map<size_t, std::vector<void*>> g_staging;        // capacity -> free blocks
static size_t g_staging_bytes = 0;                            // bytes parked in g_staging
// Page-locked memory is taken from what the whole machine can pin, so finished reads keep at most
// this much for the next read; a block that would go beyond it is given back to the driver.
static constexpr size_t kStagingKeepBytes = size_t(256) << 20;

namespace tfhip {
static bool host_is_pinned(const void* p, size_t nbytes) {
  std::lock_guard<std::mutex> lock(g_host_mu);
  auto it = g_pinned.upper_bound((uintptr_t)p);
  if (it == g_pinned.begin()) return false;
  --it;
  return (uintptr_t)p + nbytes <= it->first + it->second;
}
// Block sizes are rounded so that tensors of similar size share blocks: 512 B granules up
// to 1 MiB, then 1/8-octave steps (at most 12.5 % slack on large activations).
static size_t round_cap(size_t n) {
  if (n <= (1u << 20)) return (n + 511) & ~size_t(511);
  size_t step = size_t(1) << (63 - __builtin_clzll(n) - 3);
  return (n + step - 1) & ~(step - 1);
}

static void* staging_get(size_t nbytes, size_t* cap) {
  *cap = round_cap(nbytes);
  {
    std::lock_guard<std::mutex> lock(g_host_mu);
    auto it = g_staging.find(*cap);
    if (it != g_staging.end() && !it->second.empty()) {
      void* p = it->second.back();
      it->second.pop_back();
      g_staging_bytes -= *cap;
      return p;
    }
  }
  void* p = nullptr;
  if (hipHostMalloc(&p, *cap, hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}
static void staging_put(void* p, size_t cap) {
  if (!p) return;
  {
    std::lock_guard<std::mutex> lock(g_host_mu);
    if (g_staging_bytes + cap <= kStagingKeepBytes) {
      g_staging[cap].push_back(p);
      g_staging_bytes += cap;
      return;
    }
  }
  // (the copy that used the block is complete: tfhip_read_finish has waited for it)
  if (hipHostFree(p) != hipSuccess) (void)hipGetLastError();
}
}  // namespace tfhip

int tfhip_ctx::fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  err = buf;
  return code;
}

void tfhip_ctx::name_kernel(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_kernel, sizeof last_kernel, fmt, ap);
  va_end(ap);
  kernel_named = true;
}

// One more event on the stream, for the begin or the end of a region.
int tfhip_ctx::mark() {
  if (marks_used >= kMaxMarks) {
    fail(TFHIP_EINVAL, "time: more than %d regions inside one", kMaxMarks / 2);
    return -1;
  }
  if (marks_used == (int)mark_events.size()) {
    hipEvent_t ev;
    hipError_t e = hipEventCreate(&ev);
    if (e != hipSuccess) {
      fail(TFHIP_EDEVICE, "hipEventCreate: %s", hipGetErrorString(e));
      return -1;
    }
    mark_events.push_back(ev);
  }
  hipError_t e = hipEventRecord(mark_events[marks_used], stream);
  if (e != hipSuccess) {
    fail(TFHIP_EDEVICE, "hipEventRecord: %s", hipGetErrorString(e));
    return -1;
  }
  return marks_used++;
}

bool tfhip_ctx::next_rec(hipEvent_t* start, hipEvent_t* stop) {
  if (recs_used >= kMaxKernelRecs || (recs_used == (int)recs.size() && no_alloc)) {
    recs_dropped++;  // (a call that promises to create nothing creates no event either)
    return false;
  }
  if (recs_used == (int)recs.size()) {
    KernelRec r;
    if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) {
      (void)hipGetLastError();
      if (r.start) (void)hipEventDestroy(r.start);
      recs_dropped++;
      return false;
    }
    recs.push_back(r);
  }
  *start = recs[recs_used].start;
  *stop = recs[recs_used].stop;
  recs[recs_used].name.clear();
  pending_rec = recs_used++;
  return true;
}

Buf* tfhip_ctx::find(int64_t id, bool touch, bool on_last_stream) {
  auto it = bufs.find(id);
  if (it == bufs.end()) {
    fail(TFHIP_ENOENT, "unknown data id %lld", (long long)id);
    return nullptr;
  }
  Buf& b = it->second;
  if (touch) {
    if (b.uploaded) {  // the data is still on its way: the compute streams wait for the copy
      all_wait(b.uploaded);
      ev_put(b.uploaded);
      b.uploaded = nullptr;
      b.wsidx = -1;
      b.vis = kAllStreams;
    }
    if (!on_last_stream) {
      // Work under different stream indices is ordered through the buffers it shares.  The
      // first queued work on a buffer is what writes it (tensors are written once); a stream
      // that meets contents written under another index waits, once, for that stream's work
      // queued so far.
      const unsigned char bit = (unsigned char)(1u << cur);
      if (!b.vis) {
        b.wsidx = cur;
        b.vis = bit;
      } else if (!(b.vis & bit)) {
        if (b.wsidx >= 0) order(b.wsidx, cur);
        b.vis |= bit;
      }
      b.users |= bit;
      b.sidx = cur;
    }
    if (b.ready) {  // from here on the block is ordered by the compute stream alone
      ev_put(b.ready);
      b.ready = nullptr;
    }
    b.used = true;
  }
  return &b;
}

int tfhip_ctx::await_uploads() {
  for (auto& kv : bufs) {
    if (!kv.second.uploaded) continue;
    all_wait(kv.second.uploaded);
    ev_put(kv.second.uploaded);
    kv.second.uploaded = nullptr;
    kv.second.wsidx = -1;
    kv.second.vis = kAllStreams;
  }
  return TFHIP_OK;
}

void tfhip_ctx::all_wait(hipEvent_t uploaded) {
  for (hipStream_t st : streams)
    if (hipStreamWaitEvent(st, uploaded, 0) != hipSuccess) (void)hipGetLastError();
}

void tfhip_ctx::order(int earlier, int later) {
  if (earlier == later) return;
  hipEvent_t ev = capturing ? nullptr : ev_get();
  if (ev && hipEventRecord(ev, streams[earlier]) == hipSuccess &&
      hipStreamWaitEvent(streams[later], ev, 0) == hipSuccess) {
    ev_put(ev);  // the wait has been queued: the event may be recorded again
    return;
  }
  // (a stream under capture cannot wait for an event from outside the capture, and without an
  // event there is nothing to wait for: the host waits instead)
  (void)hipGetLastError();
  ev_put(ev);
  (void)hipStreamSynchronize(streams[earlier]);
}

hipEvent_t tfhip_ctx::ev_get() {
  if (!free_events.empty()) {
    hipEvent_t ev = free_events.back();
    free_events.pop_back();
    return ev;
  }
  hipEvent_t ev = nullptr;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return ev;
}

namespace tfhip {
static hipError_t create_streams(hipStream_t* out, int n) {
  for (int i = 0; i < n; i++) {
    hipError_t e = hipStreamCreate(&out[i]);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}
}  // namespace tfhip

void* tfhip_ctx::alloc(size_t nbytes, size_t* cap, hipEvent_t* ready, bool* recycled) {
  if (no_alloc) {  // a mistake in the library, not in the caller: fail instead of allocating
    fail(TFHIP_EDEVICE, "internal: a no-alloc entry point asked the pool for %zu bytes", nbytes);
    return nullptr;
  }
  const size_t want = tfhip::round_cap(nbytes);
  if (ready) *ready = nullptr;
  if (recycled) *recycled = false;
  auto& pool = pools[cur];
  auto it = pool.find(want);
  if (it != pool.end() && !it->second.empty()) {
    // most recently freed block first: it is the one most likely still in L2 / MALL
    auto& bucket = it->second;
    if (ready && !block_ready.empty() && !capturing) {
      // ... unless it left an event behind that has not fired yet (an upload target whose last
      // readers are still queued: the next upload into it would wait for them).  Then a block
      // whose event has fired, or a fresh one while the bucket is small, lets the copy start now.
      auto pending = [&](void* q) {
        auto ev = block_ready.find(q);
        return ev != block_ready.end() && hipEventQuery(ev->second) == hipErrorNotReady;
      };
      if (pending(bucket.back())) {
        size_t pick = bucket.size();
        for (size_t i = bucket.size() - 1; i-- > 0;)
          if (!pending(bucket[i])) {
            pick = i;
            break;
          }
        (void)hipGetLastError();  // (hipErrorNotReady is not an error here)
        if (pick < bucket.size()) {
          std::swap(bucket[pick], bucket.back());
        } else if (bucket.size() < 3) {
          void* fresh = nullptr;
          if (hipMalloc(&fresh, want) == hipSuccess) {
            in_use += want;
            *cap = want;
            return fresh;
          }
          (void)hipGetLastError();
        }
      }
    }
    void* p = bucket.back();
    bucket.pop_back();
    pooled -= want;
    in_use += want;
    *cap = want;
    if (capturing) capture_blocks.push_back(p);
    if (recycled) *recycled = true;
    if (!block_ready.empty()) {
      auto ev = block_ready.find(p);
      if (ev != block_ready.end()) {
        if (ready) *ready = ev->second;
        else ev_put(ev->second);  // the new owner is ordered by the compute stream
        block_ready.erase(ev);
      }
    }
    return p;
  }
  // (not while capturing: the wait below is for an event from outside the capture)
  for (size_t i = 0; i < held.size() && !capturing; i++) {
    if (held[i].cap != want) continue;
    // no free block of this size, but one whose read is still copying: take it and put the copy,
    // and whatever its last stream still has queued on it, in front of what the selected stream
    // does next
    const HeldBlock h = held[i];
    held[i] = held.back();
    held.pop_back();
    order(h.sidx, cur);
    (void)hipStreamWaitEvent(stream, h.done, 0);
    ev_put(h.left);
    pooled -= want;
    in_use += want;
    *cap = want;
    if (capturing) capture_blocks.push_back(h.p);
    if (recycled) *recycled = true;
    return h.p;
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

void tfhip_ctx::release(void* p, size_t cap, hipEvent_t ready, int sidx) {
  if (!p) {
    ev_put(ready);
    return;
  }
  in_use -= cap;
  pooled += cap;
  park(p, cap, ready, sidx < 0 ? cur : sidx);
}

void tfhip_ctx::park(void* p, size_t cap, hipEvent_t ready, int sidx) {
  if (ready) {
    auto old = block_ready.find(p);
    if (old != block_ready.end()) ev_put(old->second);
    block_ready[p] = ready;
  }
  auto own = owner.find(p);
  if (own != owner.end()) {  // a block that a captured graph writes on every replay
    pooled -= cap;
    graphs[own->second].parked.emplace_back(p, cap);
    return;
  }
  pools[sidx][cap].push_back(p);
}

void tfhip_ctx::unhold(hipEvent_t done) {
  for (size_t i = 0; i < held.size();) {
    if (held[i].done == done) {
      park(held[i].p, held[i].cap, held[i].left, held[i].sidx);
      held[i] = held.back();
      held.pop_back();
    } else {
      i++;
    }
  }
}

// A buffer lets go of its block.  Copies still in flight on the other streams are put in
// front of whatever the compute stream does with the block next; a block that was filled
// through the upload stream leaves an event behind, so that the next upload into it waits for
// the kernels that read it and for nothing queued later.
void tfhip_ctx::release_buf(Buf& b) {
  // (a stream under capture cannot be waited for from outside the capture: a block that it used
  // too goes back to its pool instead, behind the other streams' work)
  if (capturing && b.sidx != cur && (b.users >> cur & 1)) b.sidx = cur;
  hipStream_t last = streams[b.sidx];  // the stream whose pool the block goes back to
  // (work of the other streams on the block comes before whatever that stream does with it next)
  for (int s = 0; s < kStreams; s++)
    if (s != b.sidx && (b.users >> s & 1) && b.ptr) order(s, b.sidx);
  if (b.uploaded) {
    (void)hipStreamWaitEvent(last, b.uploaded, 0);
    ev_put(b.uploaded);
  }
  hipEvent_t left = nullptr;
  if (b.ready) {
    if (b.used) ev_put(b.ready);
    else left = b.ready;  // never touched: the block's history is still what the event says
  }
  if (!left && b.ptr && b.upload_target && !capturing && (left = ev_get())) {
    if (hipEventRecord(left, last) != hipSuccess) {
      (void)hipGetLastError();
      ev_put(left);
      left = nullptr;
    }
  }
  if (b.read_done && b.ptr) {
    // An asynchronous read is still copying out of the block: it goes back to the pool when the
    // read's ticket is finished.  (Waiting for the copy on the compute stream here would hold up
    // every kernel queued after this dispose for the length of a cross-stream round trip.)
    in_use -= b.cap;
    pooled += b.cap;
    held.push_back({b.ptr, b.cap, b.read_done, left, b.sidx});
  } else {
    release(b.ptr, b.cap, left, b.sidx);
  }
  b.ptr = nullptr;
  b.uploaded = b.read_done = b.ready = nullptr;
}

void tfhip_ctx::trim() {
  // (not while a graph exists: a replay may still read blocks that went back to the pool)
  bool any = false;
  for (auto& pool : pools) any = any || !pool.empty();
  if (!any || capturing || !graphs.empty()) return;
  for (hipStream_t st : streams) (void)hipStreamSynchronize(st);
  for (auto& pool : pools) {
    for (auto& kv : pool)
      for (void* p : kv.second) {
        auto ev = block_ready.find(p);
        if (ev != block_ready.end()) {
          ev_put(ev->second);
          block_ready.erase(ev);
        }
        (void)hipFree(p);
      }
    pool.clear();
  }
  pooled = 0;
  for (const HeldBlock& h : held) pooled += h.cap;  // (they wait for their reads, outside the pool)
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
      (e = tfhip::create_streams(ctx->streams, tfhip_ctx::kStreams)) != hipSuccess ||
      (e = hipStreamCreateWithFlags(&ctx->upload, hipStreamNonBlocking)) != hipSuccess ||
      (e = hipStreamCreateWithFlags(&ctx->download, hipStreamNonBlocking)) != hipSuccess) {
    g_init_error = std::string("device set-up failed: ") + hipGetErrorString(e);
    for (hipStream_t st : ctx->streams)
      if (st) (void)hipStreamDestroy(st);
    if (ctx->upload) (void)hipStreamDestroy(ctx->upload);
    if (ctx->download) (void)hipStreamDestroy(ctx->download);
    delete ctx;
    return TFHIP_EDEVICE;
  }
  ctx->stream = ctx->streams[0];
  if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0) {
    g_init_error = std::string("libtfjs_hip is built for gfx950 only, device is ") +
                   prop.gcnArchName;
    for (hipStream_t st : ctx->streams) (void)hipStreamDestroy(st);
    (void)hipStreamDestroy(ctx->upload);
    (void)hipStreamDestroy(ctx->download);
    delete ctx;
    return TFHIP_ENOTSUP;
  }
  ctx->num_cus = prop.multiProcessorCount;
  if (tfhip::scratch_init(ctx) != TFHIP_OK) {
    g_init_error = ctx->err;
    for (hipStream_t st : ctx->streams) (void)hipStreamDestroy(st);
    (void)hipStreamDestroy(ctx->upload);
    (void)hipStreamDestroy(ctx->download);
    delete ctx;
    return TFHIP_EDEVICE;
  }
  *out = ctx;
  return TFHIP_OK;
}

void tfhip_destroy(tfhip_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->upload);
  (void)hipStreamSynchronize(ctx->download);
  for (hipStream_t st : ctx->streams) (void)hipStreamSynchronize(st);
  // reads that were begun and not finished keep their ticket (tfhip_read_finish with a NULL
  // context frees it); their events are theirs
  for (auto& kv : ctx->bufs) {
    if (kv.second.ptr) (void)hipFree(kv.second.ptr);
    if (kv.second.ready) (void)hipEventDestroy(kv.second.ready);
    if (kv.second.uploaded) (void)hipEventDestroy(kv.second.uploaded);
  }
  for (auto& kv : ctx->block_ready) (void)hipEventDestroy(kv.second);
  for (hipEvent_t ev : ctx->free_events) (void)hipEventDestroy(ev);
  for (hipEvent_t ev : ctx->ring_done)
    if (ev) (void)hipEventDestroy(ev);
  if (ctx->ring) (void)hipHostFree(ctx->ring);
  for (auto& pool : ctx->pools)
    for (auto& kv : pool)
      for (void* p : kv.second) (void)hipFree(p);
  for (auto& h : ctx->held) {
    (void)hipFree(h.p);
    if (h.left) (void)hipEventDestroy(h.left);
  }
  for (auto& kv : ctx->graphs) {
    (void)hipGraphExecDestroy(kv.second.exec);
    (void)hipGraphDestroy(kv.second.graph);
    for (auto& blk : kv.second.parked) (void)hipFree(blk.first);
  }
  for (hipEvent_t ev : ctx->mark_events) (void)hipEventDestroy(ev);
  for (auto& r : ctx->recs) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  (void)hipStreamDestroy(ctx->upload);
  (void)hipStreamDestroy(ctx->download);
  for (hipStream_t st : ctx->streams) (void)hipStreamDestroy(st);
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
    b.ptr = ctx->alloc(b.nbytes, &b.cap, &b.ready, &b.recycled);
    if (!b.ptr) return TFHIP_EDEVICE;
  }
  b.sidx = ctx->cur;  // (the block came out of this stream's pool)
  ctx->bufs.emplace(id, b);
  return TFHIP_OK;
}

// Host-to-device copies take one of three roads:
//  * up to one ring slot (64 KiB): the bytes are copied into a pinned slot and from there by
//    the compute stream itself, in order with the kernels, without any wait on the host;
//  * larger, from memory of tfhip_host_alloc: a DMA on the upload stream straight from the
//    caller's buffer, which returns at once and overlaps with the kernels already queued;
//  * larger, from ordinary (pageable) memory: the same on the upload stream, and the host waits
//    for that stream only, so kernels queued earlier keep running during the copy.
// The upload stream may overwrite a block only after the compute-stream work that used it:
// it waits for the event the block's last owner left (release_buf), or, when the history is
// not known (a live buffer overwritten, a recycled block without an event), for everything
// queued on the compute stream so far.  A buffer fresh from the driver needs no wait.
int tfhip_write(tfhip_ctx* ctx, int64_t id, const void* host, size_t nbytes) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing)
    return ctx->fail(TFHIP_EINVAL, "write: host data cannot enter a graph capture (create the "
                                   "tensor before capturing)");
  Buf* b = ctx->find(id, /*touch=*/false);
  if (!b) return TFHIP_ENOENT;
  if (!host && nbytes)  // backend_cpu.ts:125-127
    return ctx->fail(TFHIP_EINVAL, "MathBackendHIP.write(): values can not be null");
  if (nbytes != b->nbytes)
    return ctx->fail(TFHIP_EINVAL, "write: got %zu bytes for a buffer of %zu", nbytes, b->nbytes);
  if (!nbytes) return TFHIP_OK;

  if (nbytes <= tfhip_ctx::kSlotBytes) {
    if (!ctx->ring)
      TFHIP_HIP(ctx, hipHostMalloc((void**)&ctx->ring, tfhip_ctx::kSlotBytes * tfhip_ctx::kSlots,
                                   hipHostMallocDefault));
    const int slot = ctx->ring_next;
    ctx->ring_next = (slot + 1) % tfhip_ctx::kSlots;
    if (ctx->ring_done[slot]) TFHIP_HIP(ctx, hipEventSynchronize(ctx->ring_done[slot]));
    else if (!(ctx->ring_done[slot] = ctx->ev_get()))
      return ctx->fail(TFHIP_EDEVICE, "write: could not create an event");
    char* staged = ctx->ring + (size_t)slot * tfhip_ctx::kSlotBytes;
    memcpy(staged, host, nbytes);
    b = ctx->find(id, /*touch=*/true);  // a copy on the compute stream is a use like any kernel
    // (and a write: behind the other streams' work on the old contents, and theirs to wait for)
    for (int s = 0; s < tfhip_ctx::kStreams; s++)
      if (s != ctx->cur && (b->users >> s & 1)) ctx->order(s, ctx->cur);
    b->wsidx = ctx->cur;
    b->vis = b->users = (unsigned char)(1u << ctx->cur);
    if (b->read_done) TFHIP_HIP(ctx, hipStreamWaitEvent(ctx->stream, b->read_done, 0));
    TFHIP_HIP(ctx, hipMemcpyAsync(b->ptr, staged, nbytes, hipMemcpyHostToDevice, ctx->stream));
    TFHIP_HIP(ctx, hipEventRecord(ctx->ring_done[slot], ctx->stream));
    return TFHIP_OK;
  }

  if (b->used || (b->recycled && !b->ready)) {
    hipEvent_t fence = ctx->ev_get();
    if (!fence) return ctx->fail(TFHIP_EDEVICE, "write: could not create an event");
    // behind every stream with work on the block (the one that got it, when none is known)
    const unsigned char users = b->users ? b->users : (unsigned char)(1u << b->sidx);
    hipError_t e = hipSuccess;
    for (int s = 0; s < tfhip_ctx::kStreams && e == hipSuccess; s++) {
      if (!(users >> s & 1)) continue;
      e = hipEventRecord(fence, ctx->streams[s]);
      if (e == hipSuccess) e = hipStreamWaitEvent(ctx->upload, fence, 0);
    }
    ctx->ev_put(fence);  // the waits have been queued: the event may be recorded again
    if (e != hipSuccess) return ctx->fail(TFHIP_EDEVICE, "write: %s", hipGetErrorString(e));
  } else if (b->ready) {
    TFHIP_HIP(ctx, hipStreamWaitEvent(ctx->upload, b->ready, 0));
  }
  ctx->ev_put(b->ready);
  b->ready = nullptr;
  if (b->read_done) TFHIP_HIP(ctx, hipStreamWaitEvent(ctx->upload, b->read_done, 0));
  b->used = false;
  b->recycled = false;
  b->upload_target = true;
  b->users = 0;
  b->wsidx = -1;
  b->vis = tfhip_ctx::kAllStreams;  // (with an upload on its way, find() makes every stream wait for it)
  TFHIP_HIP(ctx, hipMemcpyAsync(b->ptr, host, nbytes, hipMemcpyHostToDevice, ctx->upload));
  if (!tfhip::host_is_pinned(host, nbytes)) {
    // the copy reads the caller's pages until it is done, and the caller may change or free
    // them as soon as this returns
    TFHIP_HIP(ctx, hipStreamSynchronize(ctx->upload));
    ctx->ev_put(b->uploaded);
    b->uploaded = nullptr;
    return TFHIP_OK;
  }
  if (!b->uploaded && !(b->uploaded = ctx->ev_get()))
    return ctx->fail(TFHIP_EDEVICE, "write: could not create an event");
  TFHIP_HIP(ctx, hipEventRecord(b->uploaded, ctx->upload));
  return TFHIP_OK;
}

int tfhip_read(tfhip_ctx* ctx, int64_t id, void* host, size_t nbytes) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "read: not during a graph capture");
  Buf* b = ctx->find(id, /*touch=*/true, /*on_last_stream=*/true);
  if (!b) return TFHIP_ENOENT;
  if (nbytes != b->nbytes)
    return ctx->fail(TFHIP_EINVAL, "read: asked %zu bytes of a buffer of %zu", nbytes, b->nbytes);
  hipStream_t last = ctx->streams[b->sidx];  // the stream that produced (or last used) the buffer
  if (nbytes) TFHIP_HIP(ctx, hipMemcpyAsync(host, b->ptr, nbytes, hipMemcpyDeviceToHost, last));
  TFHIP_HIP(ctx, hipStreamSynchronize(last));
  return TFHIP_OK;
}

// ---- asynchronous read ----------------------------------------------------------------------
int tfhip_read_begin(tfhip_ctx* ctx, int64_t id, tfhip_pending_read** out) {
  if (!ctx || !out) return TFHIP_EINVAL;
  *out = nullptr;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "read: not during a graph capture");
  Buf* b = ctx->find(id, /*touch=*/true, /*on_last_stream=*/true);
  if (!b) return TFHIP_ENOENT;
  tfhip_pending_read* r = new tfhip_pending_read();
  r->device = ctx->device;
  r->nbytes = b->nbytes;
  if (b->nbytes) {
    r->staging = tfhip::staging_get(b->nbytes, &r->staging_cap);
    hipEvent_t produced = ctx->ev_get();
    r->done = ctx->ev_get();
    hipError_t e = (r->staging && produced && r->done) ? hipSuccess : hipErrorOutOfMemory;
    // the copy runs on the download stream, behind the kernels queued so far and no others
    if (e == hipSuccess) e = hipEventRecord(produced, ctx->streams[b->sidx]);
    if (e == hipSuccess) e = hipStreamWaitEvent(ctx->download, produced, 0);
    if (e == hipSuccess)
      e = hipMemcpyAsync(r->staging, b->ptr, b->nbytes, hipMemcpyDeviceToHost, ctx->download);
    if (e == hipSuccess) e = hipEventRecord(r->done, ctx->download);
    ctx->ev_put(produced);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      tfhip::staging_put(r->staging, r->staging_cap);
      ctx->ev_put(r->done);
      delete r;
      return ctx->fail(TFHIP_EDEVICE, "read: %s", hipGetErrorString(e));
    }
    b->read_done = r->done;
  }
  ctx->reads.emplace(r, id);
  *out = r;
  return TFHIP_OK;
}

int tfhip_read_wait(tfhip_pending_read* r) {
  if (!r) return TFHIP_EINVAL;
  if (!r->done) return TFHIP_OK;
  // may run on a thread that has never used the device
  if (hipSetDevice(r->device) != hipSuccess || hipEventSynchronize(r->done) != hipSuccess) {
    (void)hipGetLastError();
    r->failed = true;
    return TFHIP_EDEVICE;
  }
  return TFHIP_OK;
}

int tfhip_read_finish(tfhip_ctx* ctx, tfhip_pending_read* r, void* host, size_t nbytes) {
  if (!r) return TFHIP_EINVAL;
  int rc = TFHIP_OK;
  if (host && nbytes != r->nbytes) {
    rc = ctx ? ctx->fail(TFHIP_EINVAL, "read: asked %zu bytes of a buffer of %zu", nbytes, r->nbytes)
             : TFHIP_EINVAL;
  } else if (r->done && (r->failed || hipEventSynchronize(r->done) != hipSuccess)) {
    (void)hipGetLastError();
    rc = ctx ? ctx->fail(TFHIP_EDEVICE, "read: the copy from the device failed") : TFHIP_EDEVICE;
  } else if (host && nbytes) {
    memcpy(host, r->staging, nbytes);
  }
  if (ctx) {
    auto it = ctx->reads.find(r);
    if (it != ctx->reads.end()) {
      auto buf = ctx->bufs.find(it->second);
      if (buf != ctx->bufs.end() && buf->second.read_done == r->done) buf->second.read_done = nullptr;
      ctx->reads.erase(it);
    }
    if (r->done) ctx->unhold(r->done);  // the copy is complete (or failed for good)
    ctx->ev_put(r->done);
  } else if (r->done) {
    (void)hipEventDestroy(r->done);
  }
  tfhip::staging_put(r->staging, r->staging_cap);
  delete r;
  return rc;
}

int tfhip_host_alloc(size_t nbytes, void** ptr) {
  if (!ptr || !nbytes) return TFHIP_EINVAL;
  *ptr = nullptr;
  void* p = nullptr;
  if (hipHostMalloc(&p, nbytes, hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return TFHIP_EDEVICE;
  }
  std::lock_guard<std::mutex> lock(g_host_mu);
  g_pinned[(uintptr_t)p] = nbytes;
  *ptr = p;
  return TFHIP_OK;
}

int tfhip_host_free(void* ptr) {
  if (!ptr) return TFHIP_OK;
  {
    std::lock_guard<std::mutex> lock(g_host_mu);
    if (!g_pinned.erase((uintptr_t)ptr)) return TFHIP_EINVAL;
  }
  // waits for copies that still read the memory
  if (hipHostFree(ptr) != hipSuccess) {
    (void)hipGetLastError();
    return TFHIP_EDEVICE;
  }
  return TFHIP_OK;
}

int tfhip_dispose(tfhip_ctx* ctx, int64_t id) {
  if (!ctx) return TFHIP_EINVAL;
  auto it = ctx->bufs.find(id);
  if (it == ctx->bufs.end()) return TFHIP_OK;  // backend_cpu.ts:228-237: unknown id is a no-op
  ctx->release_buf(it->second);
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
  TFHIP_HIP(ctx, hipStreamSynchronize(ctx->upload));  // pinned sources are free again after this
  for (hipStream_t st : ctx->streams) TFHIP_HIP(ctx, hipStreamSynchronize(st));
  return TFHIP_OK;
}

int tfhip_select_stream(tfhip_ctx* ctx, int index) {
  if (!ctx) return TFHIP_EINVAL;
  if (index < 0 || index >= tfhip_ctx::kStreams)
    return ctx->fail(TFHIP_EINVAL, "select_stream: index %d, there are %d compute streams", index,
                     tfhip_ctx::kStreams);
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "select_stream: not during a graph capture");
  if (ctx->time_depth) return ctx->fail(TFHIP_EINVAL, "select_stream: not inside a timed region");
  ctx->cur = index;
  ctx->stream = ctx->streams[index];
  ctx->dirty |= (unsigned char)(1u << index);
  return TFHIP_OK;
}

int tfhip_time_begin(tfhip_ctx* ctx) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "time: not during a graph capture");
  if (ctx->time_depth == tfhip_ctx::kMaxTimeDepth)
    return ctx->fail(TFHIP_EINVAL, "time: more than %d nested regions", tfhip_ctx::kMaxTimeDepth);
  if (ctx->time_depth == 0) ctx->marks_used = ctx->recs_used = ctx->recs_dropped = 0;
  const int at = ctx->mark();
  if (at < 0) return TFHIP_EDEVICE;
  ctx->time_stack[ctx->time_depth++] = {at, ctx->recs_used};
  return TFHIP_OK;
}

int tfhip_time_end(tfhip_ctx* ctx, float* ms) {
  if (!ctx || !ms) return TFHIP_EINVAL;
  if (!ctx->time_depth) return ctx->fail(TFHIP_EINVAL, "time_end without time_begin");
  const tfhip_ctx::Region first = ctx->time_stack[--ctx->time_depth];
  const int last = ctx->mark();
  if (last < 0) return TFHIP_EDEVICE;
  TFHIP_HIP(ctx, hipEventSynchronize(ctx->mark_events[last]));
  TFHIP_HIP(ctx, hipEventElapsedTime(ms, ctx->mark_events[first.mark], ctx->mark_events[last]));
  ctx->kernel_times.clear();
  for (int i = first.rec; i < ctx->recs_used; i++) {
    float d = 0;
    TFHIP_HIP(ctx, hipEventElapsedTime(&d, ctx->recs[i].start, ctx->recs[i].stop));
    ctx->kernel_times.push_back({ctx->recs[i].name, d});
  }
  if (ctx->recs_dropped) {
    char note[64];
    snprintf(note, sizeof note, "(%d launches not recorded)", ctx->recs_dropped);
    ctx->kernel_times.push_back({note, 0.f});
  }
  return TFHIP_OK;
}

int tfhip_time_per_kernel(tfhip_ctx* ctx, int enable) {
  if (!ctx) return TFHIP_EINVAL;
  ctx->per_kernel = enable != 0;
  return TFHIP_OK;
}

int tfhip_time_kernel_count(tfhip_ctx* ctx, int* count) {
  if (!ctx || !count) return TFHIP_EINVAL;
  *count = (int)ctx->kernel_times.size();
  return TFHIP_OK;
}

int tfhip_time_kernel(tfhip_ctx* ctx, int index, const char** name, float* ms) {
  if (!ctx) return TFHIP_EINVAL;
  if (index < 0 || index >= (int)ctx->kernel_times.size())
    return ctx->fail(TFHIP_EINVAL, "time_kernel: index %d not in 0..%zu", index,
                     ctx->kernel_times.size());
  if (name) *name = ctx->kernel_times[index].name.c_str();
  if (ms) *ms = ctx->kernel_times[index].ms;
  return TFHIP_OK;
}

// ---- captured graphs ---------------------------------------------------------------------
int tfhip_graph_begin(tfhip_ctx* ctx) {
  if (!ctx) return TFHIP_EINVAL;
  if (ctx->capturing) return ctx->fail(TFHIP_EINVAL, "graph_begin: a capture is already running");
  ctx->capture_blocks.clear();
  ctx->capture_used_scratch = false;
  // uploads still on their way are waited for before the recording starts: a wait for an
  // event of another stream must not become part of the graph
  int rc = ctx->await_uploads();
  if (rc) return rc;
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
  g.sidx = ctx->cur;
  g.uses_scratch = ctx->capture_used_scratch;
  // Every block the capture handed out now belongs to the graph: those lying free in the pool
  // are taken out of it, the others follow when their tensor lets go of them (release()).
  for (void* p : ctx->capture_blocks) {
    if (ctx->owner.count(p)) continue;
    ctx->owner[p] = id;
    for (auto& pool : ctx->pools)
      for (auto& kv : pool) {
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
  // the recorded kernels read their inputs by address: new data written into those tensors
  // through the upload stream has to arrive first
  int rc = ctx->await_uploads();
  if (rc) return rc;
  tfhip_ctx::Graph& g = it->second;
  // A replay reads its inputs at their addresses and writes its blocks again, every time.  So it
  // runs behind everything the other compute streams have queued so far (a small write into an
  // input copied by the other stream, kernels there that still read the previous replay's
  // results), and behind asynchronous reads still copying out of its blocks ...
  for (int s = 0; s < tfhip_ctx::kStreams; s++) {
    if (s == g.sidx || !(ctx->dirty >> s & 1)) continue;
    ctx->order(s, g.sidx);
    if (s != ctx->cur) ctx->dirty &= (unsigned char)~(1u << s);
  }
  const unsigned char gbit = (unsigned char)(1u << g.sidx);
  for (auto& kv : ctx->bufs) {
    Buf& b = kv.second;
    if (!b.ptr) continue;
    auto own = ctx->owner.find(b.ptr);
    if (own == ctx->owner.end() || own->second != graph_id) continue;
    if (b.read_done) TFHIP_HIP(ctx, hipStreamWaitEvent(ctx->streams[g.sidx], b.read_done, 0));
    // ... and the tensors on its blocks are booked as written anew on the capture's stream: the
    // next consumer on another stream waits again, a host read follows this stream.
    b.wsidx = g.sidx;
    b.vis = gbit;
    b.users |= gbit;
    b.sidx = g.sidx;
    b.used = true;
  }
  if (g.uses_scratch) ctx->scratch_sidx = g.sidx;
  // (on the stream of the capture, whichever is selected)
  TFHIP_HIP(ctx, hipGraphLaunch(g.exec, ctx->streams[g.sidx]));
  return TFHIP_OK;
}

int tfhip_graph_destroy(tfhip_ctx* ctx, int64_t graph_id) {
  if (!ctx) return TFHIP_EINVAL;
  auto it = ctx->graphs.find(graph_id);
  if (it == ctx->graphs.end()) return TFHIP_OK;
  // queued replays may still run: wait before the blocks can be handed to anyone else
  for (hipStream_t st : ctx->streams) (void)hipStreamSynchronize(st);
  (void)hipGraphExecDestroy(it->second.exec);
  (void)hipGraphDestroy(it->second.graph);
  for (auto& blk : it->second.parked) {
    ctx->pooled += blk.second;
    ctx->pools[ctx->cur][blk.second].push_back(blk.first);  // (every stream is idle now)
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
