// Device-side integer requantisation shared by every quantized kernel.
// Semantics follow Glow's CPU backend bit for bit (reference
// lib/LLVMIRCodeGen/libjit/libjit_defs.h:147-233): 32-bit wrap-around
// arithmetic, arithmetic right shifts, round-to-nearest on the post-shift,
// activation applied after the requantisation and before the int8 clip.
#ifndef GLOW_MI355X_REQUANT_H
#define GLOW_MI355X_REQUANT_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355x {

// libjit_scale<int32_t>: ((((in >> pre) * scale) + rtn) >> post) + offset.
__device__ __forceinline__ int32_t scale_i32(int32_t in, int32_t pre,
                                             int32_t post, int32_t scale,
                                             int32_t offset) {
  uint32_t rtn = (post > 0) ? (1u << (post - 1)) : 0u;
  uint32_t m = (uint32_t)(in >> pre) * (uint32_t)scale + rtn;
  return (int32_t)((uint32_t)((int32_t)m >> post) + (uint32_t)offset);
}

// The same for |in >> pre| and |scale| below 2^23: the 24-bit multiplier gives
// the identical low 32 bits of the product at four times the rate of the
// 32-bit one. Callers check the bound on the host.
__device__ __forceinline__ int32_t scale_i32_small(int32_t in, int32_t pre,
                                                   int32_t post, int32_t scale,
                                                   int32_t offset) {
  uint32_t rtn = (post > 0) ? (1u << (post - 1)) : 0u;
  uint32_t m = (uint32_t)__mul24(in >> pre, scale) + rtn;
  return (int32_t)((uint32_t)((int32_t)m >> post) + (uint32_t)offset);
}

template <bool SMALL>
__device__ __forceinline__ int32_t scale_i32_sel(int32_t in, int32_t pre, int32_t post,
                                                 int32_t scale, int32_t offset) {
  if constexpr (SMALL) return scale_i32_small(in, pre, post, scale, offset);
  else return scale_i32(in, pre, post, scale, offset);
}

__device__ __forceinline__ int32_t clip_i8(int32_t v) {
  return min(max(v, -128), 127);
}

// min(max(v, lo), hi) for lo <= hi as one instruction (the compiler cannot
// merge the pair itself without knowing lo <= hi).
__device__ __forceinline__ int32_t med3_i32(int32_t v, int32_t lo, int32_t hi) {
  int32_t r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
  return r;
}

// libjit_activation_i32; act follows glow::FusedActivation.
__device__ __forceinline__ int32_t activation_i32(int32_t v, int32_t offset,
                                                  int32_t act, int32_t a0,
                                                  int32_t a1, int32_t a2) {
  switch (act) {
  case 1: // RELU
    return max(v, offset);
  case 2: // CLIP
    return min(max(v, a0), a1);
  case 5: // LEAKY_RELU
    return v >= offset
               ? v
               : scale_i32((int32_t)((uint32_t)v - (uint32_t)offset), a0, a1,
                           a2, offset);
  default: // NONE (fused tanh / sigmoid are rejected on the host)
    return v;
  }
}

} // namespace mi355x
#endif
