// Element-wise gated recurrence (minGRU): every channel carries one fp32 number per sequence,
//   S_t = (1 - z_t) S_(t-1) + z_t c_t,   z = sigmoid(zp),   c = up + 1/2 (up >= 0), sigmoid(up) (up < 0),
//   out_t = S_t * silu(gp),
// where zp, up and gp are projections of the current token alone.  The state lives in slots
// [num_slots, channels]; a sequence whose context length is 0 starts from zero whatever its slot
// held.  Gates, candidate and state are fp32; the projections come in the activation dtype.
//
// Short runs of rows (decode steps, small portions): one thread per (sequence, channel) walks the
// run.  Long runs are cut into pieces of kPiece rows that are walked at the same time: the
// recurrence is linear in S, so a piece is summed up by (A, B) with S_end = A S_start + B; a second
// launch chains the pieces' sums into the state each piece starts from (and leaves the run's last
// state in the slot), a third walks every piece again from its true start and writes the outputs.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kThreads = 256;
constexpr int kPiece = 128;

__device__ __forceinline__ float sigmoidf(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float candidate(float u) { return u >= 0.f ? u + 0.5f : sigmoidf(u); }

template <class S>
struct Rows {
  const typename S::T* zp;
  int64_t z_stride;
  const typename S::T* up;
  int64_t u_stride;
  const typename S::T* gp;
  int64_t g_stride;
  typename S::T* out;
  int64_t out_stride;
};

// walks rows [r0, r1) of channel c from state s; writes outputs when WRITE; returns the state
template <class S, bool WRITE>
__device__ __forceinline__ float walk(const Rows<S>& r, int r0, int r1, int c, float s, float* decay) {
  float a = 1.f;
  constexpr int U = 4;
  int t = r0;
  for (; t + U <= r1; t += U) {
    float z[U], u[U], g[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
      z[i] = S::to_f32(r.zp[(int64_t)(t + i) * r.z_stride + c]);
      u[i] = S::to_f32(r.up[(int64_t)(t + i) * r.u_stride + c]);
      if (WRITE) g[i] = S::to_f32(r.gp[(int64_t)(t + i) * r.g_stride + c]);
    }
#pragma unroll
    for (int i = 0; i < U; ++i) {
      const float zz = sigmoidf(z[i]);
      s = (1.f - zz) * s + zz * candidate(u[i]);
      if (WRITE)
        r.out[(int64_t)(t + i) * r.out_stride + c] = S::from_f32(s * (g[i] * sigmoidf(g[i])));
      else
        a *= 1.f - zz;
    }
  }
  for (; t < r1; ++t) {
    const float zz = sigmoidf(S::to_f32(r.zp[(int64_t)t * r.z_stride + c]));
    s = (1.f - zz) * s + zz * candidate(S::to_f32(r.up[(int64_t)t * r.u_stride + c]));
    if (WRITE) {
      const float g = S::to_f32(r.gp[(int64_t)t * r.g_stride + c]);
      r.out[(int64_t)t * r.out_stride + c] = S::from_f32(s * (g * sigmoidf(g)));
    } else {
      a *= 1.f - zz;
    }
  }
  if (decay != nullptr) *decay = a;
  return s;
}

template <class S>
__global__ __launch_bounds__(kThreads) void mingru_walk_kernel(
    Rows<S> r, float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots, int channels) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  float* st = state + (int64_t)state_slots[b] * channels + c;
  const float s0 = context_lens[b] > 0 ? *st : 0.f;
  *st = walk<S, true>(r, query_start_loc[b], query_start_loc[b + 1], c, s0, nullptr);
}

// sums[b][piece][0 / 1][c] = (A, B) of the piece walked from zero
template <class S>
__global__ __launch_bounds__(kThreads) void mingru_piece_sums_kernel(
    Rows<S> r, float* __restrict__ sums, const int* __restrict__ query_start_loc, int channels,
    int max_pieces) {
  const int b = blockIdx.z, piece = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  const int start = query_start_loc[b] + piece * kPiece, end = query_start_loc[b + 1];
  if (c >= channels || start >= end) return;
  float a;
  const float s = walk<S, false>(r, start, min(end, start + kPiece), c, 0.f, &a);
  float* dst = sums + (((int64_t)b * max_pieces + piece) * 2) * channels + c;
  dst[0] = a;
  dst[channels] = s;
}

// sums[b][piece][0][c] <- the state the piece starts from; the slot gets the run's last state
__global__ __launch_bounds__(kThreads) void mingru_chain_kernel(
    float* __restrict__ sums, float* __restrict__ state, const int* __restrict__ query_start_loc,
    const int* __restrict__ context_lens, const int* __restrict__ state_slots, int channels,
    int max_pieces) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  const int n = query_start_loc[b + 1] - query_start_loc[b];
  const int pieces = (n + kPiece - 1) / kPiece;
  float* st = state + (int64_t)state_slots[b] * channels + c;
  float s = context_lens[b] > 0 ? *st : 0.f;
  for (int i = 0; i < pieces; ++i) {
    float* e = sums + (((int64_t)b * max_pieces + i) * 2) * channels + c;
    const float a = e[0], add = e[channels];
    e[0] = s;
    s = a * s + add;
  }
  *st = s;
}

template <class S>
__global__ __launch_bounds__(kThreads) void mingru_piece_walk_kernel(
    Rows<S> r, const float* __restrict__ sums, const int* __restrict__ query_start_loc,
    int channels, int max_pieces) {
  const int b = blockIdx.z, piece = blockIdx.y;
  const int c = blockIdx.x * kThreads + threadIdx.x;
  const int start = query_start_loc[b] + piece * kPiece, end = query_start_loc[b + 1];
  if (c >= channels || start >= end) return;
  const float s0 = sums[(((int64_t)b * max_pieces + piece) * 2) * channels + c];
  walk<S, true>(r, start, min(end, start + kPiece), c, s0, nullptr);
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int64_t vla_seq_mingru_scratch_floats(int num_seqs, int max_query_len, int channels) {
  if (max_query_len < 2 * kPiece) return 0;
  return (int64_t)num_seqs * ((max_query_len + kPiece - 1) / kPiece) * 2 * channels;
}

extern "C" int vla_seq_mingru_scan(void* out, int64_t out_stride, const void* zp, int64_t z_stride,
                                   const void* up, int64_t u_stride, const void* gp,
                                   int64_t g_stride, float* state, const int* query_start_loc,
                                   const int* context_lens, const int* state_slots, int num_seqs,
                                   int num_slots, int max_query_len, int channels, float* scratch,
                                   int64_t scratch_floats, int dtype, void* stream) {
  if (num_seqs == 0) return VLA_OK;
  if (!out || !zp || !up || !gp || !state || !query_start_loc || !context_lens || !state_slots ||
      num_seqs < 0 || num_seqs > 65535 || num_slots <= 0 || channels <= 0 || max_query_len < 0 ||
      out_stride < channels || z_stride < channels || u_stride < channels || g_stride < channels)
    return VLA_ERR_ARG;
  const int64_t need = vla_seq_mingru_scratch_floats(num_seqs, max_query_len, channels);
  const bool pieces = need > 0 && scratch != nullptr && scratch_floats >= need;
  const int max_pieces = (max_query_len + kPiece - 1) / kPiece;
  if (pieces && max_pieces > 65535) return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const Rows<S> r{(const T*)zp, z_stride, (const T*)up, u_stride, (const T*)gp, g_stride, (T*)out,
                    out_stride};
    const int cb = (channels + kThreads - 1) / kThreads;
    hipStream_t st = (hipStream_t)stream;
    if (!pieces) {
      mingru_walk_kernel<S><<<dim3(cb, num_seqs), kThreads, 0, st>>>(
          r, state, query_start_loc, context_lens, state_slots, channels);
    } else {
      mingru_piece_sums_kernel<S><<<dim3(cb, max_pieces, num_seqs), kThreads, 0, st>>>(
          r, scratch, query_start_loc, channels, max_pieces);
      mingru_chain_kernel<<<dim3(cb, num_seqs), kThreads, 0, st>>>(
          scratch, state, query_start_loc, context_lens, state_slots, channels, max_pieces);
      mingru_piece_walk_kernel<S><<<dim3(cb, max_pieces, num_seqs), kThreads, 0, st>>>(
          r, scratch, query_start_loc, channels, max_pieces);
    }
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
