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
#include <atomic>
#include <cstdlib>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

std::atomic<int> g_scan_kernel{0};
std::atomic<int> g_scan_cols{[] {
  const char* e = getenv("VLA_SCAN_COLS");
  const int v = e ? atoi(e) : 16;
  return v >= 1 && v <= 256 ? v : 16;
}()};

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


// gla_scan_block_kernel<S, ROWS>: the same walk, several tokens per workgroup barrier.  One
// workgroup per (sequence, head, slice of `vb` value columns).  The walk of a sequence cannot be
// parallel over tokens (S_t needs S_(t-1)), but a thread's part of it needs nobody else: thread
// (r, v) updates its ROWS rows of column v from the token's k, a and v and adds its part of
// q . S[:, v].  So a block of up to kBlockTokens tokens is staged in LDS at once (the next block's
// global loads are in flight meanwhile and land in the other buffer), every thread walks the
// block alone, and the partial dot products of the row groups are summed after one barrier.
constexpr int kBlockTokens = 16;
constexpr int kStageLoads = 16;   // values a thread fetches per block at most

template <class S, int ROWS>
__global__ __launch_bounds__(256) void gla_scan_block_kernel(
    float* __restrict__ o, const typename S::T* __restrict__ q, int64_t q_stride,
    const typename S::T* __restrict__ k, int64_t k_stride, const typename S::T* __restrict__ v,
    int64_t v_stride, const float* __restrict__ log_decay, float* __restrict__ state,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const int* __restrict__ state_slots, float q_scale, int heads, int dim, int vdim, int vb,
    int groups, int tb, int dim_pad, int tok, int per) {
  extern __shared__ __align__(16) float lds[];
  // per parity (`per` floats): stage [tb][tok], tok = 3 * dim_pad + vb rounded up to a multiple
  // of four floats | partial [tb][groups][vb]
  const int h = blockIdx.x, b = blockIdx.y, v0 = blockIdx.z * vb;
  const int t0 = query_start_loc[b], t1 = query_start_loc[b + 1];
  if (t1 <= t0) return;
  using T = typename S::T;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int nv = min(vb, vdim - v0);                 // columns of this slice
  const int col = tid % vb, grp = tid / vb;
  const bool owner = grp < groups && col < nv;
  const int row0 = grp * ROWS;
  float* sp = state + (((int64_t)state_slots[b] * heads + h) * dim) * vdim + v0;
  float s[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int d = row0 + i;
    s[i] = (owner && d < dim && context_lens[b] > 0) ? sp[(int64_t)d * vdim + col] : 0.f;
  }
  float regs[kStageLoads];
  const int tt_step = nthreads / tok, e_step = nthreads - tt_step * tok;
  // global -> registers.  Every thread issues all its loads before it needs any of them: the
  // addresses of entries that do not exist (padding, tokens past the block) are bent to a row that
  // does, and the value is dropped afterwards, so no load sits behind a branch.
  auto fetch = [&](int tstart, int n) {
    int tt = tid / tok, e = tid - tt * tok;      // element tid + u * nthreads = (token tt, entry e)
    const T* safe_t = q + (int64_t)tstart * q_stride + (int64_t)h * dim;
    const float* safe_f = log_decay + ((int64_t)tstart * heads + h) * dim;
    float xt[kStageLoads], xf[kStageLoads];
    int kind[kStageLoads];                       // 0 q, 1 k, 2 decay, 3 v, -1 nothing
#pragma unroll
    for (int u = 0; u < kStageLoads; ++u) {
      const int64_t t = tstart + tt;
      const int sec = e < dim_pad ? 0 : (e < 2 * dim_pad ? 1 : (e < 3 * dim_pad ? 2 : 3));
      const int off = e - sec * dim_pad;
      const bool valid = tt < n && (sec < 3 ? off < dim : off < nv);
      const T* pt = sec == 0 ? q + t * q_stride + (int64_t)h * dim + off
                             : (sec == 1 ? k + t * k_stride + (int64_t)h * dim + off
                                         : v + t * v_stride + (int64_t)h * vdim + v0 + off);
      const float* pf = log_decay + (t * heads + h) * dim + off;
      pt = (valid && sec != 2) ? pt : safe_t;
      pf = (valid && sec == 2) ? pf : safe_f;
      xt[u] = S::to_f32(*pt);
      xf[u] = *pf;
      kind[u] = valid ? sec : -1;
      tt += tt_step;
      e += e_step;
      if (e >= tok) {
        e -= tok;
        ++tt;
      }
    }
#pragma unroll
    for (int u = 0; u < kStageLoads; ++u) {
      float x = kind[u] == 2 ? expf(xf[u]) : (kind[u] == 0 ? xt[u] * q_scale : xt[u]);
      regs[u] = kind[u] < 0 ? 0.f : x;
    }
  };
  auto put = [&](float* buf, int n) {            // registers -> LDS
#pragma unroll
    for (int u = 0; u < kStageLoads; ++u) {
      const int i = tid + u * nthreads;
      if (i < n * tok) buf[i] = regs[u];
    }
  };
  fetch(t0, min(tb, t1 - t0));
  put(lds, min(tb, t1 - t0));
  __syncthreads();
  int parity = 0;
  for (int ts = t0; ts < t1; ts += tb, parity ^= 1) {
    const int n = min(tb, t1 - ts);
    const int nn = min(tb, t1 - (ts + tb));          // next block's tokens (<= 0: none)
    float* cur = lds + parity * per;
    float* part = cur + tb * tok;
    if (nn > 0) fetch(ts + tb, nn);
    if (owner) {
      for (int tt = 0; tt < n; ++tt) {
        const float* in = cur + tt * tok;
        const float vv = in[3 * dim_pad + col];
        float acc = 0.f;
        if constexpr (ROWS % 4 == 0) {
#pragma unroll
          for (int i = 0; i < ROWS; i += 4) {
            const f32x4 q4 = *reinterpret_cast<const f32x4*>(in + row0 + i);
            const f32x4 k4 = *reinterpret_cast<const f32x4*>(in + dim_pad + row0 + i);
            const f32x4 a4 = *reinterpret_cast<const f32x4*>(in + 2 * dim_pad + row0 + i);
            s[i] = a4.x * s[i] + k4.x * vv;
            s[i + 1] = a4.y * s[i + 1] + k4.y * vv;
            s[i + 2] = a4.z * s[i + 2] + k4.z * vv;
            s[i + 3] = a4.w * s[i + 3] + k4.w * vv;
            acc += s[i] * q4.x + s[i + 1] * q4.y + s[i + 2] * q4.z + s[i + 3] * q4.w;
          }
        } else {
#pragma unroll
          for (int i = 0; i < ROWS; ++i) {
            const int d = row0 + i;
            s[i] = in[2 * dim_pad + d] * s[i] + in[dim_pad + d] * vv;
            acc += s[i] * in[d];
          }
        }
        part[(tt * groups + grp) * vb + col] = acc;
      }
    }
    if (nn > 0) put(lds + (parity ^ 1) * per, nn);
    __syncthreads();
    for (int i = tid; i < n * vb; i += nthreads) {
      const int tt = i / vb, c = i - tt * vb;
      if (c < nv) {
        float sum = 0.f;
        for (int g = 0; g < groups; ++g) sum += part[(tt * groups + g) * vb + c];
        o[((int64_t)(ts + tt) * heads + h) * vdim + v0 + c] = sum;
      }
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
                                int num_seqs, int num_slots, int max_query_len, int heads, int dim,
                                int vdim, int dtype, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!o || !q || !k || !v || !log_decay || !state || !query_start_loc || !context_lens ||
      !state_slots || num_seqs < 0 || num_slots <= 0 || heads <= 0 || dim <= 0 || vdim <= 0 ||
      q_stride < (int64_t)heads * dim || k_stride < (int64_t)heads * dim ||
      v_stride < (int64_t)heads * vdim)
    return VLA_ERR_ARG;
  // ---- the blocked walk: slices of at most kSliceCols value columns, up to 256 threads
  {
    const int cols = g_scan_cols.load(std::memory_order_relaxed);
    const int vb = vdim < cols ? vdim : cols;
    const int slices = (vdim + vb - 1) / vb;
    int groups = 256 / vb;
    if (groups > dim) groups = dim;
    int rows = (dim + groups - 1) / groups, rows_pow2 = 1;
    while (rows_pow2 < rows) rows_pow2 <<= 1;
    groups = (dim + rows_pow2 - 1) / rows_pow2;
    const int dim_pad = groups * rows_pow2;          // rows past dim stay zero: a = k = q = 0
    const int threads = (groups * vb + 63) / 64 * 64;
    const int tok = (3 * dim_pad + vb + 3) & ~3;     // 16-byte rows for the four-wide LDS reads
    int tb = kStageLoads * threads / tok;
    if (tb > kBlockTokens) tb = kBlockTokens;
    if (max_query_len > 0 && tb > max_query_len) tb = max_query_len;   // decode: small LDS, many workgroups
    const int per = tb * tok + ((tb * groups * vb + 3) & ~3);
    const size_t lds_bytes = 2 * (size_t)per * sizeof(float);
    if (g_scan_kernel.load(std::memory_order_relaxed) != 1 && rows_pow2 <= 64 && tb >= 1 &&
        lds_bytes <= 64 * 1024) {
      return with_dtype(dtype, [&](auto s) {
        using S = decltype(s);
        using T = typename S::T;
        const dim3 grid(heads, num_seqs, slices);
        auto launch = [&](auto kernel) {
          kernel<<<grid, threads, lds_bytes, (hipStream_t)stream>>>(
              o, (const T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, log_decay, state,
              query_start_loc, context_lens, state_slots, q_scale, heads, dim, vdim, vb, groups, tb,
              dim_pad, tok, per);
        };
        switch (rows_pow2) {
          case 1: launch(gla_scan_block_kernel<S, 1>); break;
          case 2: launch(gla_scan_block_kernel<S, 2>); break;
          case 4: launch(gla_scan_block_kernel<S, 4>); break;
          case 8: launch(gla_scan_block_kernel<S, 8>); break;
          case 16: launch(gla_scan_block_kernel<S, 16>); break;
          case 32: launch(gla_scan_block_kernel<S, 32>); break;
          default: launch(gla_scan_block_kernel<S, 64>); break;
        }
        VLA_SEQ_HIP_CHECK(hipGetLastError());
        return VLA_OK;
      });
    }
  }
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

// 0: pick per shape; 1: always the token-by-token kernel (tests run both)
extern "C" int vla_seq_set_scan_kernel(int mode) {
  if (mode < 0 || mode > 1) return VLA_ERR_ARG;
  g_scan_kernel.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}
