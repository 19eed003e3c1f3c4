// Shared by the sources of libvla_seq_gfx950.so: dtype dispatch, block reductions, error slot.
#pragma once

#include "../../include/vla_sequence_ops.h"
#include "vla_common.h"

namespace vla {
namespace seq {

void set_hip_error(int e);

#define VLA_SEQ_HIP_CHECK(expr)          \
  do {                                   \
    hipError_t e_ = (expr);              \
    if (e_ != hipSuccess) {              \
      vla::seq::set_hip_error((int)e_);  \
      return VLA_ERR_HIP;                \
    }                                    \
  } while (0)

// calls f(S{}) with the scalar traits of a dtype code; VLA_ERR_DTYPE for an unknown code
template <class F>
inline int with_dtype(int dtype, F&& f) {
  switch (dtype) {
    case VLA_F16: return f(F16{});
    case VLA_BF16: return f(BF16{});
    case VLA_F32: return f(F32{});
    default: return VLA_ERR_DTYPE;
  }
}

// Orders one wave's LDS traffic: what its lanes wrote before is visible to what they read after.
// (The hardware keeps a wave's LDS instructions in order; the fences keep the compiler from
// moving accesses of different types across the point.)
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// the two 16-bit values of a packed word, and back
template <class S>
__device__ __forceinline__ float lo16(uint32_t w) {
  return S::to_f32(__builtin_bit_cast(typename S::T, (uint16_t)(w & 0xffffu)));
}
template <class S>
__device__ __forceinline__ float hi16(uint32_t w) {
  return S::to_f32(__builtin_bit_cast(typename S::T, (uint16_t)(w >> 16)));
}
template <class S>
__device__ __forceinline__ uint32_t pack16(float lo, float hi) {
  return (uint32_t)__builtin_bit_cast(uint16_t, S::from_f32(lo)) |
         ((uint32_t)__builtin_bit_cast(uint16_t, S::from_f32(hi)) << 16);
}

// sum over a workgroup of up to 1024 threads; red holds 16 floats; every thread gets the sum
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  if (lane == 0) red[w] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  __syncthreads();
  return r;
}

}  // namespace seq
}  // namespace vla
