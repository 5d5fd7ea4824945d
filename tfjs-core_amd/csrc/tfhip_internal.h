// Internal declarations shared by the translation units of libtfjs_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>
#include <utility>
#include <vector>

#include "tfjs_hip.h"

namespace tfhip {

// Cache policy of a buffer store on gfx950 (last argument of __builtin_amdgcn_raw_buffer_store_*):
// sc1, device scope.  The store writes through the XCD's L2 to memory as it happens instead of
// leaving a dirty line behind.  A kernel is over only when the L2s have written back what is
// dirty, so a kernel that ends with its last megabytes dirty pays for them with an idle machine;
// written through, they leave while the kernel still computes.  The data still enters the
// memory-side cache, where the kernel that reads it next finds it (a non-temporal store goes
// past that cache too and made those readers slower than it made the writer faster).  Measured
// inside a batch-64 MobileNet step, the readers' times unchanged: 64 x 64 GEMM tiles
// [50176,128]x[128,256] 34.1 -> 32.5 us, [12544,512]x[512,512] 52.6 -> 51.6; the 3x3x3 stem
// 33.9 -> 32.5; the fused 128 -> 128 depthwise + pointwise block 76.9 -> 74.9; the step with
// the input resident 0.870 -> 0.854 ms.  The depthwise kernels do not use it: their own times
// fell (14x14x512: 9.8 -> 9.3 us) but the step that uploads its input while the previous batch
// computes got 8 us longer.
constexpr int STORE_WRITE_THROUGH = 16;

// Wave priority (s_setprio) that the kernels bound by memory give their wavefronts: the stem, the
// fused depthwise + pointwise blocks and the 3 x 3 depthwise kernels.  With two batches in flight
// on the two compute streams their wavefronts share SIMDs with those of a matrix-bound product of
// the other batch; a wavefront that has a load or a store to issue then goes first, and memory
// stays busy while the product, which has work for every slot it gets, fills the rest.  Alone in
// the machine a kernel's wavefronts all have the same priority and nothing changes.  Measured on
// a batch-64 MobileNet (400 steps, libraries alternating on one box): two batches in flight end
// to end 0.783 -> 0.775 ms per step, one batch resident 0.840 either way; the product's
// wavefronts raised instead: 0.798.
constexpr int WAVE_PRIORITY_MEMORY_BOUND = 3;

struct Buf {
  void* ptr = nullptr;
  size_t nbytes = 0;  // logical bytes (numel * element size)
  size_t cap = 0;     // bytes of the pool block behind ptr
  int dtype = TFHIP_FLOAT32;
  int64_t numel = 0;
  int rank = 0;
  int32_t shape[8] = {0};
  // Ordering between the compute stream and the copy streams (see tfhip_ctx::upload):
  hipEvent_t ready = nullptr;      // compute work that last read the block, recorded when it went
                                   // back to the pool: a copy stream waits for it before overwriting
  hipEvent_t uploaded = nullptr;   // a copy on the upload stream that the first consumer waits for
  hipEvent_t read_done = nullptr;  // the last asynchronous read of this buffer (owned by its ticket)
  bool recycled = false;           // the block came out of the pool (its history is unknown)
  bool used = false;               // queued work may have touched the buffer since it was written
  bool upload_target = false;      // written through the upload stream: worth an event on release
  int sidx = 0;                    // compute stream (tfhip_select_stream) of the last queued use
  // Ordering between the compute streams, one bit per stream:
  int wsidx = -1;                  // the stream whose queued work wrote the contents (-1: a copy did)
  unsigned char vis = 0;           // streams that are ordered behind that write (0: nothing written yet)
  unsigned char users = 0;         // streams with queued work on the block since the buffer got it
};

inline size_t dtype_size(int dtype) {
  return (dtype == TFHIP_BOOL || dtype == TFHIP_UINT8Q) ? 1 : 4;
}

}  // namespace tfhip

// An asynchronous read between tfhip_read_begin and tfhip_read_finish.  Self-contained, so that
// a thread which only waits (tfhip_read_wait) never looks into the context.
struct tfhip_pending_read {
  int device = 0;
  size_t nbytes = 0;
  void* staging = nullptr;  // pinned; the device copies into it on the download stream
  size_t staging_cap = 0;
  hipEvent_t done = nullptr;  // recorded behind that copy
  bool failed = false;
};

// One device, one in-order stream, one size-bucketed pool of device blocks.  Freed blocks
// go back to the pool at once: every consumer is queued on the same stream, so a block
// handed out again can only be touched after the work that last used it.
struct tfhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;  // every kernel runs here, in order
  // Copies that overlap with kernels: host-to-device on `upload`, asynchronous reads on
  // `download` (both at the default priority).  Events carry the order between the three.
  hipStream_t upload = nullptr, download = nullptr;
  std::vector<hipEvent_t> free_events;  // untimed events, reused
  hipEvent_t ev_get();
  void ev_put(hipEvent_t ev) {
    if (ev) free_events.push_back(ev);
  }
  std::unordered_map<void*, hipEvent_t> block_ready;  // pool block -> Buf::ready of its last owner
  // Blocks whose buffer was disposed while an asynchronous read of it was still copying: they
  // stay out of the pool until the read's ticket is finished (the copy is complete then), so the
  // compute stream never waits for the download stream at dispose time.  `done` belongs to the
  // ticket; `left` is the compute-stream event an upload target leaves behind.
  struct HeldBlock {
    void* p;
    size_t cap;
    hipEvent_t done, left;
    int sidx;  // the compute stream whose pool the block returns to
  };
  std::vector<HeldBlock> held;
  // Small writes travel through a ring of pinned slots on the compute stream itself.
  static constexpr size_t kSlotBytes = 64 << 10;
  static constexpr int kSlots = 32;
  char* ring = nullptr;
  hipEvent_t ring_done[kSlots] = {nullptr};
  int ring_next = 0;
  std::unordered_map<tfhip_pending_read*, int64_t> reads;  // asynchronous reads not yet finished
  std::unordered_map<int64_t, tfhip::Buf> bufs;
  // Two compute streams (tfhip_select_stream): work queued under one index runs in order, work
  // under different indices is ordered only through the buffers it shares (find()), so that two
  // independent passes (two batches of a serving loop) share the machine.  `stream` is the selected one.  Every
  // stream has a pool of its own: a block goes back to the pool of the stream that used it last,
  // where the next owner is ordered behind that use by the stream itself.
  static constexpr int kStreams = 2;  // (at most 8: Buf keeps a bit per stream)
  static constexpr unsigned char kAllStreams = (unsigned char)((1u << kStreams) - 1);
  hipStream_t streams[kStreams] = {};
  int cur = 0;  // index of `stream`
  // Streams that may hold queued work which a graph replay has not been ordered behind yet (a bit
  // per stream, set when the stream is selected): a replay waits for these, see tfhip_graph_launch.
  unsigned char dirty = 1;
  std::map<size_t, std::vector<void*>> pools[kStreams];  // capacity -> free blocks, reused LIFO
  size_t in_use = 0, pooled = 0;
  std::string err;
  char last_kernel[96] = "";  // variant chosen by the last dense / image launch
  bool kernel_named = false;  // last_kernel was written for the launch that is being queued
  void name_kernel(const char* fmt, ...);

  // KernelBackend.time with per-kernel figures (backends/backend.ts:27-31).  A region is
  // bracketed by two events on the stream ("marks"); regions nest, each remembers the mark it
  // started at.  While a region is open every kernel is launched with a start and a stop event
  // attached to its own dispatch (hipExtLaunchKernel), so its time is the execution of that
  // kernel on the device, as a profiler's kernel trace reports it, and no extra packet sits
  // between two kernels.
  static constexpr int kMaxMarks = 64;
  static constexpr int kMaxKernelRecs = 1 << 16;
  static constexpr int kMaxTimeDepth = 8;
  struct KernelTime {
    std::string name;
    float ms;
  };
  struct KernelRec {
    hipEvent_t start = nullptr, stop = nullptr;
    std::string name;
  };
  std::vector<hipEvent_t> mark_events;  // created on demand, reused by later regions
  int marks_used = 0;
  std::vector<KernelRec> recs;  // events created on demand, reused by later regions
  int recs_used = 0, recs_dropped = 0;
  struct Region {
    int mark, rec;
  };
  Region time_stack[kMaxTimeDepth];
  int time_depth = 0;
  bool per_kernel = true;
  std::vector<KernelTime> kernel_times;  // of the region that ended last
  int mark();  // index of the new mark, -1 when none could be recorded
  bool timing_kernels() const { return time_depth && per_kernel && !capturing; }
  // The event pair for the next launch (false: launch without).
  bool next_rec(hipEvent_t* start, hipEvent_t* stop);
  int pending_rec = -1;  // record of the launch that is being queued, waiting for its name
  void after_launch(const char* func) {
    if (pending_rec >= 0) {
      recs[pending_rec].name = kernel_named ? last_kernel : func;
      pending_rec = -1;
    }
    kernel_named = false;
  }

  int num_cus = 256;
  // Direction in which the next row-sweeping kernel should walk its rows: 1 = from the end.
  // A kernel leaves the rows it wrote last in the L2 of the XCD that wrote them (32 MB over the
  // chip); its consumer, which cuts the rows into the same per-XCD runs, finds them there if it
  // starts with those rows, so consecutive sweeps alternate.  Measured on MI355X in a batch-64
  // MobileNet: the stride-2 depthwise layers after the two largest activations run 49 us
  // instead of 58 us and 27 us instead of 31 us.
  // (One state for both compute streams: a direction per stream, so that each pass alternates by
  // itself, was measured 2.5 % slower with two batches in flight: 0.828 against 0.806 ms.)
  int sweep = 0;
  int take_sweep() {
    const int s = sweep;
    sweep ^= 1;
    return s;
  }

  // Captured graphs (tfhip_graph_*): while `capturing`, every block handed out is noted; when
  // the capture ends those blocks belong to the graph (`owner`), which keeps them out of the
  // pool for as long as it lives, because a replay writes them again.
  struct Graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<void*, size_t>> parked;  // owned blocks that no tensor holds
    int sidx = 0;  // the compute stream it was recorded on, and replays on
    bool uses_scratch = false;  // a recorded kernel keeps partial tiles in the static scratch array
  };
  bool capturing = false;
  bool capture_used_scratch = false;
  std::vector<void*> capture_blocks;
  std::unordered_map<void*, int64_t> owner;  // block -> graph that owns it
  std::unordered_map<int64_t, Graph> graphs;
  int64_t next_graph = 1;

  // tfhip_matmul_noalloc: this device's copy of the library's static scratch array (asked from
  // the driver once, at init), and the flag that routes scratch needs there while it runs.
  void* scratch = nullptr;
  bool no_alloc = false;
  int scratch_sidx = -1;  // the compute stream whose queued work used the scratch array last
  bool separable_off = false;  // tfhip_separable_conv2d always runs its two-kernel form

  int fail(int code, const char* fmt, ...);
  // Looks an id up (sets err when missing).  `touch` = the caller queues work on the compute
  // stream that reads or writes the buffer: a pending upload is waited for first.
  // touch: the caller queues work that uses the buffer, on the selected compute stream, or (for
  // host reads of a buffer, which follow its producer) on the stream that used it last.
  tfhip::Buf* find(int64_t id, bool touch = true, bool on_last_stream = false);
  // nullptr + err on failure (nbytes > 0).  *ready receives the event that the block's last
  // owner left with it, or nullptr; *recycled whether the block was used before.
  void* alloc(size_t nbytes, size_t* cap, hipEvent_t* ready = nullptr, bool* recycled = nullptr);
  // (sidx: the compute stream that used the block last; -1 = the selected one)
  void release(void* p, size_t cap, hipEvent_t ready = nullptr, int sidx = -1);
  void park(void* p, size_t cap, hipEvent_t ready, int sidx);  // release() after the accounting
  void unhold(hipEvent_t done);                       // held blocks of a finished read -> pool
  void release_buf(tfhip::Buf& b);
  int await_uploads();  // the compute streams wait for every upload still on its way
  // Puts compute stream `later` behind everything queued on compute stream `earlier` so far.
  void order(int earlier, int later);
  // Every compute stream waits for the copy that `uploaded` stands for.
  void all_wait(hipEvent_t uploaded);
  void trim();
};

#define TFHIP_HIP(ctx, expr)                                                          \
  do {                                                                                \
    hipError_t e_ = (expr);                                                           \
    if (e_ != hipSuccess)                                                             \
      return (ctx)->fail(TFHIP_EDEVICE, "%s: %s", #expr, hipGetErrorString(e_));      \
  } while (0)

#define TFHIP_GET(ctx, var, id)           \
  tfhip::Buf* var = (ctx)->find(id);      \
  if (!var) return TFHIP_ENOENT

// After every kernel launch: report a launch error, and note the launch for an open time() region.
#define TFHIP_LAUNCH_CHECK(ctx)            \
  do {                                     \
    TFHIP_HIP(ctx, hipGetLastError());     \
    (ctx)->after_launch(__func__);         \
  } while (0)
// The same for a launch that has a name of its own (a second kernel of one call).
#define TFHIP_LAUNCH_CHECK_NAMED(ctx, name) \
  do {                                      \
    TFHIP_HIP(ctx, hipGetLastError());      \
    (ctx)->kernel_named = false;            \
    (ctx)->after_launch(name);              \
  } while (0)

namespace tfhip {

// Scoped device scratch taken from the pool (returned when the object dies; safe because
// later users are ordered behind the kernels already queued on the stream).
struct Temp {
  tfhip_ctx* ctx;
  void* ptr = nullptr;
  size_t cap = 0;
  explicit Temp(tfhip_ctx* c) : ctx(c) {}
  bool get(size_t nbytes) {
    ptr = ctx->alloc(nbytes, &cap);
    return ptr != nullptr;
  }
  ~Temp() {
    if (ptr) ctx->release(ptr, cap);
  }
};

// Returns a float32 view of `b`: the buffer itself when it is stored as float32, else a
// converted copy in `tmp` (int32 / bool storage under a float32 tensor: widening casts
// alias the same data id, backends/backend_util.ts:49-55).
int as_f32(tfhip_ctx* ctx, const Buf* b, Temp* tmp, const float** out);

// gemm.hip: looks up this device's address of the static scratch array (tfhip_init calls it)
int scratch_init(tfhip_ctx* ctx);

// elementwise.hip
int launch_convert(tfhip_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype,
                   int64_t n);

// image.hip
int depthwise_forward_f32(tfhip_ctx* ctx, const float* x, const float* w, float* y,
                          const tfhip_conv2d_info* ci);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Every kernel of the library is launched through here, on the context's stream.  The
// arguments are converted to the kernel's parameter types as a <<<>>> launch would.  Inside a
// time() region the launch carries its own start / stop events.
template <typename... Params, typename... Args>
inline void launch(tfhip_ctx* ctx, void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds,
                   Args&&... args) {
  static_assert(sizeof...(Params) == sizeof...(Args), "wrong number of kernel arguments");
  std::tuple<Params...> values{static_cast<Params>(std::forward<Args>(args))...};
  void* ptrs[sizeof...(Params) ? sizeof...(Params) : 1];
  {
    int i = 0;
    std::apply([&](auto&... v) { ((ptrs[i++] = (void*)&v), ...); }, values);
  }
  hipEvent_t start = nullptr, stop = nullptr;
  if (ctx->timing_kernels() && ctx->next_rec(&start, &stop))
    (void)hipExtLaunchKernel((const void*)kernel, grid, block, ptrs, lds, ctx->stream, start, stop, 0);
  else
    (void)hipLaunchKernel((const void*)kernel, grid, block, ptrs, lds, ctx->stream);
}

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has its own
// L2.  Remap the id so that every XCD receives one contiguous run of the work: neighbours
// that share data (A rows / B columns of a GEMM, halo rows of a convolution) then meet in
// the same L2 instead of each fetching its own copy over the fabric.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  constexpr int XCDS = 8;
  const int per = total / XCDS, rem = total % XCDS;
  const int x = bid % XCDS, i = bid / XCDS;
  // XCD x owns `per` items (+1 for the first `rem` XCDs)
  const int start = x * per + (x < rem ? x : rem);
  return start + i;
}
// The same runs, each walked from its end when `reverse` is set.
__device__ __forceinline__ int xcd_remap_dir(int bid, int total, int reverse) {
  constexpr int XCDS = 8;
  const int per = total / XCDS, rem = total % XCDS;
  const int x = bid % XCDS, i = bid / XCDS;
  const int start = x * per + (x < rem ? x : rem);
  const int len = per + (x < rem ? 1 : 0);
  return start + (reverse ? len - 1 - i : i);
}

}  // namespace tfhip
