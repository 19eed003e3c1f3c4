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
//
// gla_scan_block_kernel (further down) is the same walk with 16 tokens per barrier, for runs of
// rows; gla_piece_prefix_kernel / gla_combine_states_kernel join the pieces of a long run that
// the layer walks at once (attention/recurrent.py).
#include <atomic>
#include <cstdlib>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

std::atomic<int> g_scan_kernel{0};
std::atomic<int> g_scan_cols{[] {
  const char* e = getenv("VLA_SCAN_COLS");
  const int v = e ? atoi(e) : 0;     // 0: by the step's longest run of rows
  return v >= 0 && v <= 256 ? v : 0;
}()};

constexpr int kDecayTokens = 16;   // tokens a thread of the row-held form walks
constexpr int kDecayRank = 32;     // widest projection whose row a thread holds in registers

__device__ __forceinline__ float log_sigmoid_over_tau(float z, float inv_tau) {
  // ln sigmoid(z) = -softplus(-z) = -(max(-z, 0) + log1p(exp(-|z|)))
  return -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)))) * inv_tau;
}

// one thread per (token, channel): any rank
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
  out[(int64_t)t * channels + c] = log_sigmoid_over_tau(z, inv_tau);
}

// rank <= kDecayRank: a thread keeps its channel's row of W2 in registers and walks
// kDecayTokens tokens, whose y rows it reads through wave-uniform addresses
template <class S>
__global__ __launch_bounds__(256) void gla_log_decay_rows_kernel(
    float* __restrict__ out, const typename S::T* __restrict__ y, int64_t y_stride,
    const typename S::T* __restrict__ w2, const float* __restrict__ bias, float inv_tau,
    int num_tokens, int channels, int rank) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= channels) return;
  float w[kDecayRank];
#pragma unroll
  for (int r = 0; r < kDecayRank; ++r) w[r] = r < rank ? S::to_f32(w2[(int64_t)c * rank + r]) : 0.f;
  const float b = bias != nullptr ? bias[c] : 0.f;
  const int t0 = blockIdx.y * kDecayTokens, t1 = min(num_tokens, t0 + kDecayTokens);
  for (int t = t0; t < t1; ++t) {
    const typename S::T* yr = y + (int64_t)t * y_stride;
    float z = b;
#pragma unroll
    for (int r = 0; r < kDecayRank; ++r)
      if (r < rank) z += w[r] * S::to_f32(yr[r]);
    out[(int64_t)t * channels + c] = log_sigmoid_over_tau(z, inv_tau);
  }
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
  float regs_a[kStageLoads], regs_b[kStageLoads];   // blocks in flight: odd ones in a, even in b
  const int tt_step = nthreads / tok, e_step = nthreads - tt_step * tok;
  // global -> registers.  Every thread issues all its loads before it needs any of them: the
  // addresses of entries that do not exist (padding, tokens past the block) are bent to a row that
  // does, and the value is dropped afterwards, so no load sits behind a branch.
  auto fetch = [&](int tstart, int n, float (&regs)[kStageLoads]) {
    int tt = tid / tok, e = tid - tt * tok;      // element tid + u * nthreads = (token tt, entry e)
    // row bases of the block's first token are wave-uniform (scalar arithmetic); what a lane adds
    // is a 32-bit offset from a 24-bit multiply (strides below 2^24 are a launch condition):
    // 64-bit per-lane multiplies here cost more than the walk itself
    const T* qb = q + (int64_t)tstart * q_stride + (int64_t)h * dim;
    const T* kb = k + (int64_t)tstart * k_stride + (int64_t)h * dim;
    const T* vbase = v + (int64_t)tstart * v_stride + (int64_t)h * vdim + v0;
    const float* db = log_decay + ((int64_t)tstart * heads + h) * dim;
    const T* safe_t = qb;
    const float* safe_f = db;
    const unsigned qs32 = (unsigned)q_stride, ks32 = (unsigned)k_stride, vs32 = (unsigned)v_stride,
                   ds32 = (unsigned)(heads * dim);
    float xt[kStageLoads], xf[kStageLoads];
    int kind[kStageLoads];                       // 0 q, 1 k, 2 decay, 3 v, -1 nothing
#pragma unroll
    for (int u = 0; u < kStageLoads; ++u) {
      const int sec = e < dim_pad ? 0 : (e < 2 * dim_pad ? 1 : (e < 3 * dim_pad ? 2 : 3));
      const int off = e - sec * dim_pad;
      const bool valid = tt < n && (sec < 3 ? off < dim : off < nv);
      const unsigned ut = (unsigned)tt;
      const T* pt = sec == 0 ? qb + (__umul24(ut, qs32) + off)
                             : (sec == 1 ? kb + (__umul24(ut, ks32) + off) : vbase + (__umul24(ut, vs32) + off));
      const float* pf = db + (__umul24(ut, ds32) + off);
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
  auto put = [&](float* buf, int n, const float (&regs)[kStageLoads]) {   // registers -> LDS
#pragma unroll
    for (int u = 0; u < kStageLoads; ++u) {
      const int i = tid + u * nthreads;
      if (i < n * tok) buf[i] = regs[u];
    }
  };
  // Block i is staged in LDS buffer i & 1 while block i + 1 is on its way in one register set and
  // the loads of block i + 2 are issued into the other: a block's loads have a whole iteration
  // before anyone waits for them.
  fetch(t0, min(tb, t1 - t0), regs_b);
  put(lds, min(tb, t1 - t0), regs_b);
  if (t0 + tb < t1) fetch(t0 + tb, min(tb, t1 - (t0 + tb)), regs_a);
  __syncthreads();
  auto iteration = [&](int ts, int parity, float (&arriving)[kStageLoads], float (&issue)[kStageLoads]) {
    const int n = min(tb, t1 - ts);
    const int nn = min(tb, t1 - (ts + tb));          // next block's tokens (<= 0: none)
    const int n2 = min(tb, t1 - (ts + 2 * tb));      // the one after
    float* cur = lds + parity * per;
    float* part = cur + tb * tok;
    if (owner) {
      if constexpr (ROWS % 4 == 0) {
        // TU tokens at a time: all their LDS reads first, then the walk, then the partial sums --
        // a read of the next token cannot wait behind the write of the previous one's sum.  Rows
        // of the stage past the block's tokens hold old values: they are read and not used.
        constexpr int TU = ROWS <= 4 ? 4 : (ROWS <= 8 ? 2 : 1);
        for (int tt = 0; tt < n; tt += TU) {
          f32x4 q4[TU][ROWS / 4], k4[TU][ROWS / 4], a4[TU][ROWS / 4];
          float vv[TU], acc[TU];
#pragma unroll
          for (int u = 0; u < TU; ++u) {
            const float* in = cur + min(tt + u, tb - 1) * tok;
            vv[u] = in[3 * dim_pad + col];
#pragma unroll
            for (int i = 0; i < ROWS / 4; ++i) {
              q4[u][i] = *reinterpret_cast<const f32x4*>(in + row0 + 4 * i);
              k4[u][i] = *reinterpret_cast<const f32x4*>(in + dim_pad + row0 + 4 * i);
              a4[u][i] = *reinterpret_cast<const f32x4*>(in + 2 * dim_pad + row0 + 4 * i);
            }
          }
#pragma unroll
          for (int u = 0; u < TU; ++u) {
            acc[u] = 0.f;
            if (tt + u < n) {
#pragma unroll
              for (int i = 0; i < ROWS / 4; ++i) {
                s[4 * i] = a4[u][i].x * s[4 * i] + k4[u][i].x * vv[u];
                s[4 * i + 1] = a4[u][i].y * s[4 * i + 1] + k4[u][i].y * vv[u];
                s[4 * i + 2] = a4[u][i].z * s[4 * i + 2] + k4[u][i].z * vv[u];
                s[4 * i + 3] = a4[u][i].w * s[4 * i + 3] + k4[u][i].w * vv[u];
                acc[u] += s[4 * i] * q4[u][i].x + s[4 * i + 1] * q4[u][i].y + s[4 * i + 2] * q4[u][i].z +
                          s[4 * i + 3] * q4[u][i].w;
              }
            }
          }
#pragma unroll
          for (int u = 0; u < TU; ++u)
            if (tt + u < n) part[((tt + u) * groups + grp) * vb + col] = acc[u];
        }
      } else {
        for (int tt = 0; tt < n; ++tt) {
          const float* in = cur + tt * tok;
          const float vv = in[3 * dim_pad + col];
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < ROWS; ++i) {
            const int d = row0 + i;
            s[i] = in[2 * dim_pad + d] * s[i] + in[dim_pad + d] * vv;
            acc += s[i] * in[d];
          }
          part[(tt * groups + grp) * vb + col] = acc;
        }
      }
    }
    if (nn > 0) put(lds + (parity ^ 1) * per, nn, arriving);
    if (n2 > 0) fetch(ts + 2 * tb, n2, issue);       // `issue` held this block: free since its put
    __syncthreads();
    for (int i = tid; i < n * vb; i += nthreads) {
      const int tt = i / vb, c = i - tt * vb;
      if (c < nv) {
        float sum = 0.f;
        for (int g = 0; g < groups; ++g) sum += part[(tt * groups + g) * vb + c];
        o[((int64_t)(ts + tt) * heads + h) * vdim + v0 + c] = sum;
      }
    }
  };
  for (int ts = t0; ts < t1; ts += 2 * tb) {
    iteration(ts, 0, regs_a, regs_b);
    if (ts + tb < t1) iteration(ts + tb, 1, regs_b, regs_a);
  }
  if (owner) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = row0 + i;
      if (d < dim) sp[(int64_t)d * vdim + col] = s[i];
    }
  }
}


// ---- pieces of a long run of rows, walked in parallel ------------------------------------------
// A run of many rows of one sequence is cut into pieces.  Every piece is walked from a zero state
// (the first from the sequence's own), all at once; that leaves, per piece, outputs that lack the
// state the piece should have started from, and the state the piece adds.  With
// c_t = sum of the log decays from the piece's first row to row t,
//   o_t += (q_t * exp(c_t))^T S_start          (a matrix product per piece and head)
//   S_end = diag(exp(c_last)) S_start + S_piece (a cheap walk over the pieces)
// give exactly what the one long walk computes.  Every exponent is <= 0: nothing can overflow.
//
// gla_piece_prefix_kernel: c_t by a running sum over the piece's rows, one thread per (piece,
// channel); writes q_t * q_scale * exp(c_t) and, per piece, exp(c_last).
template <class S>
__global__ __launch_bounds__(256) void gla_piece_prefix_kernel(
    float* __restrict__ q_decayed, float* __restrict__ totals, const typename S::T* __restrict__ q,
    int64_t q_stride, const float* __restrict__ log_decay, const int* __restrict__ piece_start_loc,
    float q_scale, int channels) {
  const int piece = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= channels) return;
  const int t0 = piece_start_loc[piece], t1 = piece_start_loc[piece + 1];
  float sum = 0.f;
#pragma unroll 8
  for (int t = t0; t < t1; ++t) {
    sum += log_decay[(int64_t)t * channels + c];
    q_decayed[(int64_t)t * channels + c] = S::to_f32(q[(int64_t)t * q_stride + c]) * q_scale * expf(sum);
  }
  totals[(int64_t)piece * channels + c] = expf(sum);
}

// gla_combine_states_kernel: the pieces' states of one sequence in order; state[slots[i]] becomes
// the state at the end of piece i, and the last one is copied to the sequence's own slot.
__global__ __launch_bounds__(256) void gla_combine_states_kernel(
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ pieces,
    const float* __restrict__ totals, int count, int final_slot, int heads, int dim, int vdim) {
  const int64_t per = (int64_t)heads * dim * vdim;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= per) return;
  const int channel = (int)(e / vdim);            // h * dim + d
  float run = state[slots[0] * per + e];
  for (int i = 1; i < count; ++i) {
    run = totals[(int64_t)pieces[i] * heads * dim + channel] * run + state[slots[i] * per + e];
    state[slots[i] * per + e] = run;
  }
  state[final_slot * per + e] = run;
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
    // (worth it once there are enough 16-token groups to fill the chip)
    if (rank <= kDecayRank && num_tokens >= 32 * kDecayTokens)
      gla_log_decay_rows_kernel<S><<<dim3((channels + 255) / 256, (num_tokens + kDecayTokens - 1) / kDecayTokens),
                                     256, 0, (hipStream_t)stream>>>(
          out, (const typename S::T*)y, y_stride, (const typename S::T*)w2, bias, inv_tau, num_tokens, channels,
          rank);
    else
      gla_log_decay_kernel<S><<<dim3((channels + 255) / 256, num_tokens), 256, 0, (hipStream_t)stream>>>(
          out, (const typename S::T*)y, y_stride, (const typename S::T*)w2, bias, inv_tau, channels, rank);
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
    // Slice width: a walk of many tokens is bound by its serial chain, so narrow slices (more
    // workgroups, fewer rows per thread) win; a walk of a token or two is bound by reading and
    // writing the state, which wide slices do in fewer, fuller workgroups.  Measured on
    // 16 heads x 64 x 128: 4096 tokens 1.45 ms at 16 columns against 2.03 ms at 64; 64 sequences
    // of one token 40 us at 64 columns against 120 us at 16.
    // Every slice of a head fetches the head's q, k and decays again, so slices are only as narrow
    // as it takes to give every CU a workgroup.
    int cols = g_scan_cols.load(std::memory_order_relaxed);
    if (cols == 0) {
      cols = 16;
      if (max_query_len > 0 && max_query_len <= 4) cols = 64;
      else if ((int64_t)num_seqs * heads * ((vdim + 63) / 64) >= 256) cols = 64;
      else if ((int64_t)num_seqs * heads * ((vdim + 31) / 32) >= 256) cols = 32;
    }
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
    // a step of single rows has nothing to block: the token-by-token kernel below does it with
    // less set-up (64 sequences x 16 heads x 64 x 128: 15 us against 40 us)
    const int64_t lim24 = (int64_t)1 << 24;
    if (g_scan_kernel.load(std::memory_order_relaxed) != 1 && max_query_len != 1 && rows_pow2 <= 64 &&
        q_stride < lim24 && k_stride < lim24 && v_stride < lim24 && (int64_t)heads * dim < lim24 &&
        tb >= 1 && lds_bytes <= 150 * 1024) {
      return with_dtype(dtype, [&](auto s) {
        using S = decltype(s);
        using T = typename S::T;
        const dim3 grid(heads, num_seqs, slices);
        int status = VLA_OK;
        auto launch = [&](auto kernel) {
          static std::atomic<size_t> allowed{64 * 1024};   // raised once per kernel, not per launch
          if (lds_bytes > allowed.load(std::memory_order_relaxed)) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds_bytes) != hipSuccess) {
              status = VLA_ERR_HIP;
              return;
            }
            allowed.store(lds_bytes, std::memory_order_relaxed);
          }
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
        if (status != VLA_OK) return status;
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

extern "C" int vla_seq_gla_piece_prefix(float* q_decayed, float* totals, const void* q,
                                        int64_t q_stride, const float* log_decay,
                                        const int* piece_start_loc, float q_scale, int num_pieces,
                                        int channels, int dtype, void* stream) {
  if (num_pieces == 0) return VLA_OK;
  if (!q_decayed || !totals || !q || !log_decay || !piece_start_loc || num_pieces < 0 ||
      channels <= 0 || q_stride < channels)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    gla_piece_prefix_kernel<S><<<dim3((channels + 255) / 256, num_pieces), 256, 0, (hipStream_t)stream>>>(
        q_decayed, totals, (const typename S::T*)q, q_stride, log_decay, piece_start_loc, q_scale, channels);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_gla_combine_states(float* state, const int* slots, const int* pieces,
                                          const float* totals, int count, int final_slot,
                                          int num_slots, int heads, int dim, int vdim, void* stream) {
  if (count == 0) return VLA_OK;
  if (!state || !slots || !pieces || !totals || count < 0 || final_slot < 0 || final_slot >= num_slots ||
      heads <= 0 || dim <= 0 || vdim <= 0)
    return VLA_ERR_ARG;
  const int64_t per = (int64_t)heads * dim * vdim;
  gla_combine_states_kernel<<<(unsigned)((per + 255) / 256), 256, 0, (hipStream_t)stream>>>(
      state, slots, pieces, totals, count, final_slot, heads, dim, vdim);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}
