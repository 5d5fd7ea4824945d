// Device-side helpers shared by the product kernels (gemm.hip, separable.hip).
#pragma once
#include "tfhip_internal.h"

namespace tfhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));


// Buffer descriptor over [base, base + bytes): loads through it return 0 for any offset at or
// beyond `bytes`, which is how out-of-range items of a tile are zero-filled without a branch
// or a select on the loaded value.  OOB_OFFSET is such an offset for every extent below 2 GiB.
constexpr unsigned OOB_OFFSET = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  // the base is the same for the whole workgroup: say so, or the descriptor lands in VGPRs
  const unsigned long long b = reinterpret_cast<unsigned long long>(base);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  void* ub = reinterpret_cast<void*>(((unsigned long long)hi << 32) | lo);
  return __builtin_amdgcn_make_buffer_rsrc(ub, (short)0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ f32x4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
}

// w = q*scale + min evaluated in double, rounded once (io/io_utils.ts:133-136).
__device__ __forceinline__ float dequant(unsigned q, double scale, double mn) {
#pragma clang fp contract(off)
  double v = (double)q * scale;
  v = v + mn;
  return (float)v;
}

// Activation of the reference (backend_cpu.ts:50-62) with JavaScript's NaN behaviour:
// Math.max(0, NaN) is NaN (:1191-1201), clip keeps NaN (:1265-1275).  Branch-free: the kind
// is unpacked once into flags that are the same for every lane.
struct ActCfg {
  bool linear, use_alpha;
  float hi;
};
__device__ __forceinline__ ActCfg act_cfg(int act) {
  ActCfg c;
  c.linear = act == TFHIP_ACT_LINEAR;
  c.use_alpha = act == TFHIP_ACT_PRELU;
  c.hi = act == TFHIP_ACT_RELU6 ? 6.f : __builtin_inff();
  return c;
}
__device__ __forceinline__ float activate(float v, const ActCfg& c, float alpha) {
  const float neg = c.linear ? v : (c.use_alpha ? alpha * v : 0.f);
  const float r = v < 0.f ? neg : v;  // NaN is not < 0: it passes through
  return r > c.hi ? c.hi : r;
}

// relu / relu6 / linear as a clamp to [lo, hi] that lets NaN through (no comparison with NaN
// holds), which is what the reference's Math.max(0, x) and clip do (backend_cpu.ts:1191-1201,
// :1265-1275): two vector instructions per value, against nine of the general form above.  The matrix instructions share their pipe with the vector ALU, so the
// stores of the dense kernels use this form and leave prelu to their general path.
struct Clamp {
  float lo, hi;
};
__device__ __forceinline__ Clamp clamp_of(int act) {
  Clamp c;
  c.lo = act == TFHIP_ACT_LINEAR ? -__builtin_inff() : 0.f;
  c.hi = act == TFHIP_ACT_RELU6 ? 6.f : __builtin_inff();
  return c;
}
__device__ __forceinline__ float clamp(float v, const Clamp& c) {
  // IEEE 754-2019 maximum / minimum return NaN when an operand is NaN, so NaN passes through;
  // gfx950 has them as v_maximum3_f32 / v_minimum3_f32: two vector instructions per value
  // (the median of three plus a NaN select took three, two compare-and-select pairs four).
  return __builtin_elementwise_minimum(__builtin_elementwise_maximum(v, c.lo), c.hi);
}

}  // namespace tfhip
