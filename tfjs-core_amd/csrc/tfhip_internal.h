// Internal declarations shared by the translation units of libtfjs_hip.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "tfjs_hip.h"

namespace tfhip {

struct Buf {
  void* ptr = nullptr;
  size_t nbytes = 0;  // logical bytes (numel * element size)
  size_t cap = 0;     // bytes of the pool block behind ptr
  int dtype = TFHIP_FLOAT32;
  int64_t numel = 0;
  int rank = 0;
  int32_t shape[8] = {0};
};

inline size_t dtype_size(int dtype) {
  return (dtype == TFHIP_BOOL || dtype == TFHIP_UINT8Q) ? 1 : 4;
}

}  // namespace tfhip

// One device, one in-order stream, one size-bucketed pool of device blocks.  Freed blocks
// go back to the pool at once: every consumer is queued on the same stream, so a block
// handed out again can only be touched after the work that last used it.
struct tfhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev_begin = nullptr, ev_end = nullptr;
  bool timing = false;
  std::unordered_map<int64_t, tfhip::Buf> bufs;
  std::map<size_t, std::vector<void*>> pool;  // capacity -> free blocks, reused LIFO
  size_t in_use = 0, pooled = 0;
  std::string err;
  char last_kernel[96] = "";  // variant chosen by the last dense / image launch
  int num_cus = 256;
  // Direction in which the next row-sweeping kernel should walk its rows: 1 = from the end.
  // A kernel leaves the rows it wrote last in the L2 of the XCD that wrote them (32 MB over the
  // chip); its consumer, which cuts the rows into the same per-XCD runs, finds them there if it
  // starts with those rows, so consecutive sweeps alternate.  Measured on MI355X in a batch-64
  // MobileNet: the stride-2 depthwise layers after the two largest activations run 49 us
  // instead of 58 us and 27 us instead of 31 us.
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
  };
  bool capturing = false;
  std::vector<void*> capture_blocks;
  std::unordered_map<void*, int64_t> owner;  // block -> graph that owns it
  std::unordered_map<int64_t, Graph> graphs;
  int64_t next_graph = 1;

  int fail(int code, const char* fmt, ...);
  tfhip::Buf* find(int64_t id);          // sets err when missing
  void* alloc(size_t nbytes, size_t* cap);  // nullptr + err on failure (nbytes > 0)
  void release(void* p, size_t cap);
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

#define TFHIP_LAUNCH_CHECK(ctx) TFHIP_HIP(ctx, hipGetLastError())

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

// elementwise.hip
int launch_convert(tfhip_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype,
                   int64_t n);

// image.hip
int depthwise_forward_f32(tfhip_ctx* ctx, const float* x, const float* w, float* y,
                          const tfhip_conv2d_info* ci);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

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
