// Gated linear attention with a decay per key channel: the recurrence
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t       (S: [dim, vdim] per head)
// with its state kept in fp32 slots between steps.
//
// gla_log_decay_kernel: ln a_t = ln(sigmoid(z_t)) / tau = -softplus(-z_t) / tau from the low-rank
// projection z_t = W2 y_t + b, in fp32, one thread per (token, channel).
//
// gla_scan_kernel<ROWS>: one workgroup per (sequence, head) walks the sequence's rows of the step
// in order -- a decode step is a walk of one row, a prompt portion a walk of many, so both leave
// the same state.  Thread (r, v) owns rows r*ROWS .. r*ROWS+ROWS-1 of column v of S in registers;
// q, k, a and v of a token are staged in LDS (the next token's loads are issued before the current
// token's arithmetic), partial dot products over the row groups are combined through LDS.  Buffers
// alternate between even and odd tokens, so one workgroup barrier per token orders everything.
// The state is read from its slot unless the sequence starts here (context length 0), and
// written back at the end: a slot needs no clearing before it is used again.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

template <class S>
__global__ __launch_bounds__(256) void gla_log_decay_kernel(
    float* __restrict__ out, const typename S::T* __restrict__ y, int64_t y_stride,
    const typename S::T* __restrict__ w2, const float* __restrict__ bias, float inv_tau,
    int channels, int rank) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= channels) return;
  float z = bias != nullptr ? bias[c] : 0.f;
  const typename S::T* yr = y + (int64_t)t * y_stride;
  const typename S::T* wr = w2 + (int64_t)c * rank;
  for (int r = 0; r < rank; ++r) z += S::to_f32(wr[r]) * S::to_f32(yr[r]);
  // softplus(-z) = max(-z, 0) + log1p(exp(-|z|))
  const float sp = fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)));
  out[(int64_t)t * channels + c] = -sp * inv_tau;
}

template <class S, int ROWS>
__global__ __launch_bounds__(1024) void gla_scan_kernel(
    float* __restrict__ o, const typename S::T* __restrict__ q, int64_t q_stride,
    const typename S::T* __restrict__ k, int64_t k_stride, const typename S::T* __restrict__ v,
    int64_t v_stride, const float* __restrict__ log_decay, float* __restrict__ state,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, float q_scale, int heads, int dim, int vdim, int groups) {
  extern __shared__ float lds[];
  // per parity: q[dim] k[dim] a[dim] v[vdim] partial[groups][vdim]
  const int per = 3 * dim + vdim + groups * vdim;
  const int h = blockIdx.x, b = blockIdx.y;
  const int t0 = query_start_loc[b], t1 = query_start_loc[b + 1];
  if (t1 <= t0) return;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int col = tid % vdim, grp = tid / vdim;
  const bool owner = grp < groups;  // threads beyond groups * vdim only help with staging
  const int row0 = grp * ROWS;
  float* sp = state + (((int64_t)state_slots[b] * heads + h) * dim) * vdim;

  float s[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int d = row0 + i;
    s[i] = (owner && d < dim && context_lens[b] > 0) ? sp[(int64_t)d * vdim + col] : 0.f;
  }

  auto stage = [&](int t, float* buf) {
    for (int i = tid; i < 3 * dim + vdim; i += nthreads) {
      float x;
      if (i < dim) {
        x = S::to_f32(q[(int64_t)t * q_stride + (int64_t)h * dim + i]) * q_scale;
      } else if (i < 2 * dim) {
        x = S::to_f32(k[(int64_t)t * k_stride + (int64_t)h * dim + (i - dim)]);
      } else if (i < 3 * dim) {
        x = expf(log_decay[((int64_t)t * heads + h) * dim + (i - 2 * dim)]);
      } else {
        x = S::to_f32(v[(int64_t)t * v_stride + (int64_t)h * vdim + (i - 3 * dim)]);
      }
      buf[i] = x;
    }
  };

  stage(t0, lds);
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    float* cur = lds + ((t - t0) & 1) * per;
    if (t + 1 < t1) stage(t + 1, lds + ((t + 1 - t0) & 1) * per);
    if (owner) {
      const float vv = cur[3 * dim + col];
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        const int d = row0 + i;
        if (d < dim) {
          s[i] = cur[2 * dim + d] * s[i] + cur[dim + d] * vv;
          part += s[i] * cur[d];
        }
      }
      cur[3 * dim + vdim + grp * vdim + col] = part;
    }
    __syncthreads();
    if (tid < vdim) {
      float sum = 0.f;
      for (int g = 0; g < groups; ++g) sum += cur[3 * dim + vdim + g * vdim + tid];
      o[((int64_t)t * heads + h) * vdim + tid] = sum;
    }
  }
  if (owner) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = row0 + i;
      if (d < dim) sp[(int64_t)d * vdim + col] = s[i];
    }
  }
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_gla_log_decay(float* out, const void* y, int64_t y_stride, const void* w2,
                                     const float* bias, float inv_tau, int num_tokens,
                                     int channels, int rank, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !y || !w2 || num_tokens < 0 || channels <= 0 || rank <= 0 || y_stride < rank)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    gla_log_decay_kernel<S><<<dim3((channels + 255) / 256, num_tokens), 256, 0,
                              (hipStream_t)stream>>>(out, (const typename S::T*)y, y_stride,
                                                     (const typename S::T*)w2, bias, inv_tau,
                                                     channels, rank);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_gla_scan(float* o, const void* q, int64_t q_stride, const void* k,
                                int64_t k_stride, const void* v, int64_t v_stride,
                                const float* log_decay, float* state, const int* query_start_loc,
                                const int* context_lens, const int* state_slots, float q_scale,
                                int num_seqs, int num_slots, int heads, int dim, int vdim,
                                int dtype, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!o || !q || !k || !v || !log_decay || !state || !query_start_loc || !context_lens ||
      !state_slots || num_seqs < 0 || num_slots <= 0 || heads <= 0 || dim <= 0 || vdim <= 0 ||
      q_stride < (int64_t)heads * dim || k_stride < (int64_t)heads * dim ||
      v_stride < (int64_t)heads * vdim)
    return VLA_ERR_ARG;
  if (vdim > 1024) return VLA_ERR_HEAD_SIZE;
  // row groups: as many as fit 256 threads (at least one), each holding `rows` rows of S
  int groups = 256 / vdim;
  if (groups < 1) groups = 1;
  if (groups > dim) groups = dim;
  int rows = (dim + groups - 1) / groups;
  int rows_pow2 = 1;
  while (rows_pow2 < rows) rows_pow2 <<= 1;
  if (rows_pow2 > 128) return VLA_ERR_HEAD_SIZE;
  groups = (dim + rows_pow2 - 1) / rows_pow2;
  int threads = groups * vdim;
  threads = (threads + 63) / 64 * 64;
  const size_t lds_bytes = 2 * (size_t)(3 * dim + vdim + groups * vdim) * sizeof(float);
  if (lds_bytes > 64 * 1024) return VLA_ERR_HEAD_SIZE;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const dim3 grid(heads, num_seqs);
    auto launch = [&](auto kernel) {
      kernel<<<grid, threads, lds_bytes, (hipStream_t)stream>>>(
          o, (const T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, log_decay, state,
          query_start_loc, context_lens, state_slots, q_scale, heads, dim, vdim, groups);
    };
    switch (rows_pow2) {
      case 1: launch(gla_scan_kernel<S, 1>); break;
      case 2: launch(gla_scan_kernel<S, 2>); break;
      case 4: launch(gla_scan_kernel<S, 4>); break;
      case 8: launch(gla_scan_kernel<S, 8>); break;
      case 16: launch(gla_scan_kernel<S, 16>); break;
      case 32: launch(gla_scan_kernel<S, 32>); break;
      case 64: launch(gla_scan_kernel<S, 64>); break;
      default: launch(gla_scan_kernel<S, 128>); break;
    }
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
