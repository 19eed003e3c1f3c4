// Row-wise steps of a decoder stack whose residual stream stays in fp32: embedding lookup with
// sinusoidal positions, RMS norm with a single gain (and the additions that precede it at the
// start of a pass over looped layers), residual accumulation, the PolyNorm activation and the
// gated per-head RMS norm that closes a linear-recurrence mixer.  One workgroup per row (or per
// row and head), fp32 arithmetic throughout, activations read / written in the model dtype.
// All of them move bytes: a row is read once (kept in registers between the reduction and the
// scaling pass when it fits) and written once.
#include "seq_common.h"

namespace vla {
namespace seq {

static thread_local int g_last_hip_error = 0;
void set_hip_error(int e) { g_last_hip_error = e; }

namespace {

constexpr int kThreads = 256;
constexpr int kKeep = 8;  // row elements a thread keeps in registers: rows up to 2048 are read once

template <class S>
__global__ __launch_bounds__(kThreads) void embed_positions_kernel(
    float* __restrict__ out, const typename S::T* __restrict__ table,
    const int64_t* __restrict__ ids, const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, int width, int vocab) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const float p = (float)positions[t];
  const typename S::T* row = table + id * (int64_t)width;
  for (int c = threadIdx.x; c < width; c += kThreads) {
    float v = S::to_f32(row[c]);
    if (inv_freq != nullptr) {
      const float a = p * inv_freq[c >> 1];
      v += (c & 1) ? cosf(a) : sinf(a);
    }
    out[(int64_t)t * width + c] = v;
  }
}

template <class S>
__global__ __launch_bounds__(kThreads) void scalar_rms_norm_kernel(
    typename S::T* __restrict__ out, float* __restrict__ x, const float* __restrict__ add_rows,
    const float* __restrict__ add_row, const float* __restrict__ gain, float eps, int width) {
  __shared__ float red[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  const bool adds = add_rows != nullptr || add_row != nullptr;
  float keep[kKeep];
  float ss = 0.f;
  auto take = [&](int c) {
    float v = x[base + c];
    if (add_rows != nullptr) v += add_rows[base + c];
    if (add_row != nullptr) v += add_row[c];
    if (adds) x[base + c] = v;
    ss += v * v;
    return v;
  };
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < width) keep[i] = take(c);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads) take(c);
  ss = block_sum(ss, red);
  const float inv = gain[0] / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < width) out[base + c] = S::from_f32(keep[i] * inv);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < width; c += kThreads)
    out[base + c] = S::from_f32(x[base + c] * inv);
}

template <class S>
__global__ __launch_bounds__(kThreads) void residual_add_kernel(float* __restrict__ x,
                                                               const typename S::T* __restrict__ y,
                                                               int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) x[i] += S::to_f32(y[i]);
}

template <class S>
__global__ __launch_bounds__(kThreads) void poly_norm_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ z,
    int64_t z_stride, const float* __restrict__ coef, float eps, int features) {
  __shared__ float red[16];
  const typename S::T* zr = z + (int64_t)blockIdx.x * z_stride;
  typename S::T* orow = out + (int64_t)blockIdx.x * out_stride;
  float keep[kKeep];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  auto take = [&](int c) {
    const float v = S::to_f32(zr[c]);
    const float v2 = v * v, v3 = v2 * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v3 * v3;
    return v;
  };
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < features) keep[i] = take(c);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < features; c += kThreads) take(c);
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  s3 = block_sum(s3, red);
  const float n = (float)features;
  const float k1 = coef[0] / sqrtf(s1 / n + eps), k2 = coef[1] / sqrtf(s2 / n + eps),
              k3 = coef[2] / sqrtf(s3 / n + eps), k0 = coef[3];
  auto put = [&](int c, float v) {
    const float v2 = v * v;
    orow[c] = S::from_f32(k1 * v + k2 * v2 + k3 * (v2 * v) + k0);
  };
#pragma unroll
  for (int i = 0; i < kKeep; ++i) {
    const int c = threadIdx.x + i * kThreads;
    if (c < features) put(c, keep[i]);
  }
  for (int c = threadIdx.x + kKeep * kThreads; c < features; c += kThreads)
    put(c, S::to_f32(zr[c]));
}

// 16-bit rows whose length is a multiple of four and whose ends are 8-byte aligned: four values
// per access, the row (up to 4096 values) kept in registers between the two passes.
template <class S>
__global__ __launch_bounds__(kThreads) void poly_norm_vec_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ z,
    int64_t z_stride, const float* __restrict__ coef, float eps, int features) {
  __shared__ float red[16];
  constexpr int STEPS = 4;
  const typename S::T* zr = z + (int64_t)blockIdx.x * z_stride;
  typename S::T* orow = out + (int64_t)blockIdx.x * out_stride;
  float keep[STEPS][4];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  auto take = [&](int c, float (&v)[4]) {
    const u32x2 w = *reinterpret_cast<const u32x2*>(zr + c);
    v[0] = lo16<S>(w.x);
    v[1] = hi16<S>(w.x);
    v[2] = lo16<S>(w.y);
    v[3] = hi16<S>(w.y);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v2 = v[e] * v[e], v3 = v2 * v[e];
      s1 += v2;
      s2 += v2 * v2;
      s3 += v3 * v3;
    }
  };
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    const int c = (threadIdx.x + i * kThreads) * 4;
    if (c < features) take(c, keep[i]);
  }
  for (int c = (threadIdx.x + STEPS * kThreads) * 4; c < features; c += kThreads * 4) {
    float v[4];
    take(c, v);
  }
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  s3 = block_sum(s3, red);
  const float n = (float)features;
  const float k1 = coef[0] / sqrtf(s1 / n + eps), k2 = coef[1] / sqrtf(s2 / n + eps),
              k3 = coef[2] / sqrtf(s3 / n + eps), k0 = coef[3];
  auto put = [&](int c, const float (&v)[4]) {
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v2 = v[e] * v[e];
      r[e] = k1 * v[e] + k2 * v2 + k3 * (v2 * v[e]) + k0;
    }
    *reinterpret_cast<u32x2*>(orow + c) = u32x2{pack16<S>(r[0], r[1]), pack16<S>(r[2], r[3])};
  };
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    const int c = (threadIdx.x + i * kThreads) * 4;
    if (c < features) put(c, keep[i]);
  }
  for (int c = (threadIdx.x + STEPS * kThreads) * 4; c < features; c += kThreads * 4) {
    const u32x2 w = *reinterpret_cast<const u32x2*>(zr + c);
    const float v[4] = {lo16<S>(w.x), hi16<S>(w.x), lo16<S>(w.y), hi16<S>(w.y)};
    put(c, v);
  }
}

// one wave per (token, head)
template <class S>
__global__ __launch_bounds__(kWave) void gated_head_rms_norm_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
    const float* __restrict__ weight, const typename S::T* __restrict__ gate, int64_t gate_stride,
    float eps, float scale, int heads, int vdim) {
  const int h = blockIdx.x, t = blockIdx.y;
  const float* orow = o + ((int64_t)t * heads + h) * vdim;
  float ss = 0.f;
  for (int c = threadIdx.x; c < vdim; c += kWave) ss += orow[c] * orow[c];
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss / (float)vdim + eps);
  for (int c = threadIdx.x; c < vdim; c += kWave) {
    const float g = S::to_f32(gate[(int64_t)t * gate_stride + (int64_t)h * vdim + c]);
    const float silu = g / (1.f + expf(-g));
    out[(int64_t)t * out_stride + (int64_t)h * vdim + c] =
        S::from_f32(orow[c] * inv * weight[c] * silu);
  }
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_last_hip_error(void) { return g_last_hip_error; }

extern "C" int vla_seq_embed_positions(float* out, const void* table, const int64_t* ids,
                                       const int64_t* positions, const float* inv_freq,
                                       int num_tokens, int width, int vocab, int dtype,
                                       void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !table || !ids || !positions || num_tokens < 0 || width <= 0 || vocab <= 0)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    embed_positions_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        out, (const typename S::T*)table, ids, positions, inv_freq, width, vocab);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_scalar_rms_norm(void* out, float* x, const float* add_rows,
                                       const float* add_row, const float* gain, float eps,
                                       int num_tokens, int width, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !x || !gain || num_tokens < 0 || width <= 0) return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    scalar_rms_norm_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        (typename S::T*)out, x, add_rows, add_row, gain, eps, width);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_residual_add(float* x, const void* y, int64_t n, int dtype, void* stream) {
  if (n == 0) return VLA_OK;
  if (!x || !y || n < 0) return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    residual_add_kernel<S><<<(unsigned)((n + kThreads - 1) / kThreads), kThreads, 0,
                             (hipStream_t)stream>>>(x, (const typename S::T*)y, n);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_poly_norm(void* out, int64_t out_stride, const void* z, int64_t z_stride,
                                 const float* coef, float eps, int num_tokens, int features,
                                 int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !z || !coef || num_tokens < 0 || features <= 0 || out_stride < features ||
      z_stride < features)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    if constexpr (sizeof(typename S::T) == 2) {
      if (features % 4 == 0 && ((uintptr_t)z % 8) == 0 && ((uintptr_t)out % 8) == 0 && (z_stride % 4) == 0 &&
          (out_stride % 4) == 0) {
        poly_norm_vec_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
            (typename S::T*)out, out_stride, (const typename S::T*)z, z_stride, coef, eps, features);
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      }
    }
    poly_norm_kernel<S><<<num_tokens, kThreads, 0, (hipStream_t)stream>>>(
        (typename S::T*)out, out_stride, (const typename S::T*)z, z_stride, coef, eps, features);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_gated_head_rms_norm(void* out, int64_t out_stride, const float* o,
                                           const float* weight, const void* gate,
                                           int64_t gate_stride, float eps, float scale,
                                           int num_tokens, int heads, int vdim, int dtype,
                                           void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !o || !weight || !gate || num_tokens < 0 || heads <= 0 || vdim <= 0 ||
      out_stride < (int64_t)heads * vdim || gate_stride < (int64_t)heads * vdim)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    gated_head_rms_norm_kernel<S><<<dim3(heads, num_tokens), kWave, 0, (hipStream_t)stream>>>(
        (typename S::T*)out, out_stride, o, weight, (const typename S::T*)gate, gate_stride, eps,
        scale, heads, vdim);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
