// Sliding-window attention over a paged key cache whose values are its keys, with a linear
// distance bias per head, a position-dependent query temperature and a sigmoid output gate.
//
// Cache: [num_blocks, block_size, kv_heads, dim] in the model dtype -- token-major rows, so one
// tensor serves both contractions (q . k_j reads rows, sum_j p_j k_j reads them again from L2 /
// L1).  There is no value cache: a layer of this kind keeps half the bytes of an ordinary one.
//
// One kernel serves prompts, portions of prompts and decode steps: every query row reads its
// window from the cache (the step's own keys are written first), so a position's result cannot
// depend on how its sequence was cut into steps.  Scores, softmax and the weighted sum are fp32.
//
// window_attention_kernel: one wave per (token, query head).  A tile is 64 keys: lane j computes
// the score of key j against the query held in LDS (row reads of 16 bytes), the wave reduces
// max / sum (online softmax across tiles), then lane d accumulates sum_j p_j k_j[d] with
// coalesced column reads.  The four waves of a workgroup take consecutive query heads of one
// token, which share KV heads under grouped queries.
#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kMaxDim = 256;
constexpr int kAccum = kMaxDim / kWave;
constexpr int kHeadsPerGroup = 4;

template <class S>
__global__ __launch_bounds__(256) void key_cache_write_kernel(
    typename S::T* __restrict__ cache, const typename S::T* __restrict__ k, int64_t k_stride,
    const int64_t* __restrict__ slot_mapping, int row, int64_t num_slots) {
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_slots) return;
  for (int c = threadIdx.x; c < row; c += blockDim.x)
    cache[slot * row + c] = k[(int64_t)t * k_stride + c];
}

template <class S>
__global__ __launch_bounds__(kWave* kHeadsPerGroup) void window_attention_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float* __restrict__ slopes, int heads, int kv_heads, int dim, int block_size,
    int num_blocks, int window, float scale, float temp_coef, float temp_every, float out_scale) {
  __shared__ float q_lds[kHeadsPerGroup][kMaxDim];
  __shared__ float p_lds[kHeadsPerGroup][kWave];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.y;
  const int h = blockIdx.x * kHeadsPerGroup + w;
  if (h >= heads) return;  // whole wave; no workgroup barrier below
  const int g = h / (heads / kv_heads);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  float qs = scale;
  if (temp_coef != 0.f) qs *= 1.f + temp_coef * logf(floorf((float)(p + 1) / temp_every) + 1.f);
  for (int d = lane; d < dim; d += kWave)
    q_lds[w][d] = S::to_f32(q[(int64_t)t * q_stride + (int64_t)h * dim + d]) * qs;
  __builtin_amdgcn_wave_barrier();
  const float slope = slopes != nullptr ? slopes[h] : 0.f;
  const int64_t tok_stride = (int64_t)kv_heads * dim;
  // a block id outside the pool (a table the host filled wrongly) reads block 0 instead of faulting
  auto key_row = [&](int j) {
    int b = table[j / block_size];
    b = (unsigned)b < (unsigned)num_blocks ? b : 0;
    return cache + ((int64_t)b * block_size + j % block_size) * tok_stride + (int64_t)g * dim;
  };

  float acc[kAccum];
#pragma unroll
  for (int c = 0; c < kAccum; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = lo; j0 <= p; j0 += kWave) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const typename S::T* kr = key_row(j);
      float dot = 0.f;
      for (int d = 0; d < dim; ++d) dot += q_lds[w][d] * S::to_f32(kr[d]);
      s = dot - slope * (float)(p - j);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = j <= p ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    l = l * corr + wave_sum(pj);
    m = m_new;
    __builtin_amdgcn_wave_barrier();
    p_lds[w][lane] = pj;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < kAccum; ++c) acc[c] *= corr;
    const int n = min(kWave, p - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const int jk = j0 + jj;
      const typename S::T* kr = key_row(jk);
      const float pv = p_lds[w][jj];
#pragma unroll
      for (int c = 0; c < kAccum; ++c) {
        const int d = lane + c * kWave;
        if (d < dim) acc[c] += pv * S::to_f32(kr[d]);
      }
    }
  }
  const float inv = out_scale / l;
#pragma unroll
  for (int c = 0; c < kAccum; ++c) {
    const int d = lane + c * kWave;
    if (d < dim) {
      float v = acc[c] * inv;
      if (gate != nullptr) {
        const float gv = S::to_f32(gate[(int64_t)t * gate_stride + (int64_t)h * dim + d]);
        v *= 1.f / (1.f + expf(-gv));
      }
      out[(int64_t)t * out_stride + (int64_t)h * dim + d] = S::from_f32(v);
    }
  }
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_key_cache_write(void* cache, const void* k, int64_t k_stride,
                                       const int64_t* slot_mapping, int num_tokens, int kv_heads,
                                       int dim, int block_size, int num_blocks, int dtype,
                                       void* stream) {
  if (num_tokens == 0) return VLA_OK;
  const int row = kv_heads * dim;
  if (!cache || !k || !slot_mapping || num_tokens < 0 || kv_heads <= 0 || dim <= 0 ||
      block_size <= 0 || num_blocks <= 0 || k_stride < row)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    key_cache_write_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        (typename S::T*)cache, (const typename S::T*)k, k_stride, slot_mapping, row,
        (int64_t)num_blocks * block_size);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_window_attention(void* out, int64_t out_stride, const void* q,
                                        int64_t q_stride, const void* gate, int64_t gate_stride,
                                        const void* cache, const int* block_tables, int max_blocks,
                                        const int* token_seq, const int64_t* positions,
                                        const float* slopes, int num_tokens, int heads,
                                        int kv_heads, int dim, int block_size, int num_blocks,
                                        int window, float scale, float temp_coef, float temp_every,
                                        float out_scale, int dtype, void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !q || !cache || !block_tables || !token_seq || !positions || num_tokens < 0 ||
      heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || block_size <= 0 || num_blocks <= 0 ||
      max_blocks <= 0 || out_stride < (int64_t)heads * dim || q_stride < (int64_t)heads * dim ||
      (gate && gate_stride < (int64_t)heads * dim) || (temp_coef != 0.f && !(temp_every > 0.f)))
    return VLA_ERR_ARG;
  if (dim <= 0 || dim > kMaxDim) return VLA_ERR_HEAD_SIZE;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    const dim3 grid((heads + kHeadsPerGroup - 1) / kHeadsPerGroup, num_tokens);
    window_attention_kernel<S><<<grid, kWave * kHeadsPerGroup, 0, (hipStream_t)stream>>>(
        (typename S::T*)out, out_stride, (const typename S::T*)q, q_stride,
        (const typename S::T*)gate, gate_stride, (const typename S::T*)cache, block_tables,
        max_blocks, token_seq, positions, slopes, heads, kv_heads, dim, block_size, num_blocks, window,
        scale, temp_coef, temp_every, out_scale);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
