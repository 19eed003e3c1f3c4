// Causal softmax attention over paged key and value caches with rotary positions on queries and
// keys, values that are rotated by their own position when they are cached (the head's output is
// turned back by the query's position), an optional sliding window and a sigmoid gate of one
// number per head.
//
// Caches: keys [num_blocks, block_size, kv_heads, dim] and values [num_blocks, block_size, kv_heads,
// vdim] in the model dtype, token-major rows.  rotary_kv_write rotates the step's queries in place
// and writes the rotated keys and values to their slots; the attention kernels then read every
// query row's keys from the caches, so prompts, portions of prompts and decode steps are one case
// and a position's result cannot depend on how its sequence was cut into steps.  Angles, scores,
// softmax and the weighted sum are fp32.
//
// kv_attention_kernel: one wave per (token, query head), any dtype and head size up to 256.  A
// tile is 64 keys: lane j scores key j against the query held in LDS, the wave reduces max / sum
// (online softmax across tiles), then lane d accumulates sum_j p_j v_j[d] with coalesced reads.
#include <atomic>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

constexpr int kMaxDim = 256;
constexpr int kAccum = kMaxDim / kWave;
constexpr int kHeadsPerGroup = 4;

// the pair (a, b) turned by angle: (a cos - b sin, b cos + a sin)
__device__ __forceinline__ void turn(float& a, float& b, float angle) {
  float s, c;
  sincosf(angle, &s, &c);
  const float a2 = a * c - b * s;
  b = b * c + a * s;
  a = a2;
}

// element indices of pair i among `span` rotated elements
__device__ __forceinline__ void pair_index(int i, int span, int interleaved, int& ia, int& ib) {
  if (interleaved) {
    ia = 2 * i;
    ib = 2 * i + 1;
  } else {
    ia = i;
    ib = i + span / 2;
  }
}

// One workgroup per token: every head's rotated pairs, then the elements that are not rotated.
template <class S>
__global__ __launch_bounds__(256) void rotary_kv_write_kernel(
    typename S::T* __restrict__ q, int64_t q_stride, const typename S::T* __restrict__ k,
    int64_t k_stride, const typename S::T* __restrict__ v, int64_t v_stride,
    typename S::T* __restrict__ key_cache, typename S::T* __restrict__ value_cache,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slot_mapping,
    const float* __restrict__ inv_freq, const float* __restrict__ value_inv_freq, int heads,
    int kv_heads, int dim, int vdim, int rot_dims, int interleaved, int64_t num_slots) {
  using T = typename S::T;
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  int64_t slot = slot_mapping[t];
  const bool cached = slot >= 0 && slot < num_slots;
  const int half = rot_dims / 2;
  T* qr = q + (int64_t)t * q_stride;
  for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    int ia, ib;
    pair_index(f, rot_dims, interleaved, ia, ib);
    float a = S::to_f32(qr[h * dim + ia]), b = S::to_f32(qr[h * dim + ib]);
    turn(a, b, p * inv_freq[f]);
    qr[h * dim + ia] = S::from_f32(a);
    qr[h * dim + ib] = S::from_f32(b);
  }
  if (!cached) return;
  const T* kr = k + (int64_t)t * k_stride;
  T* kc = key_cache + slot * (int64_t)kv_heads * dim;
  for (int i = threadIdx.x; i < kv_heads * half; i += blockDim.x) {
    const int h = i / half, f = i - h * half;
    int ia, ib;
    pair_index(f, rot_dims, interleaved, ia, ib);
    float a = S::to_f32(kr[h * dim + ia]), b = S::to_f32(kr[h * dim + ib]);
    turn(a, b, p * inv_freq[f]);
    kc[h * dim + ia] = S::from_f32(a);
    kc[h * dim + ib] = S::from_f32(b);
  }
  const int rest = dim - rot_dims;
  for (int i = threadIdx.x; i < kv_heads * rest; i += blockDim.x) {
    const int h = i / rest, d = rot_dims + (i - h * rest);
    kc[h * dim + d] = kr[h * dim + d];
  }
  const T* vr = v + (int64_t)t * v_stride;
  T* vc = value_cache + slot * (int64_t)kv_heads * vdim;
  if (value_inv_freq == nullptr) {
    for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x) vc[i] = vr[i];
    return;
  }
  const int vhalf = vdim / 2;
  for (int i = threadIdx.x; i < kv_heads * vhalf; i += blockDim.x) {
    const int h = i / vhalf, f = i - h * vhalf;
    int ia, ib;
    pair_index(f, vdim, interleaved, ia, ib);
    float a = S::to_f32(vr[h * vdim + ia]), b = S::to_f32(vr[h * vdim + ib]);
    turn(a, b, p * value_inv_freq[f]);
    vc[h * vdim + ia] = S::from_f32(a);
    vc[h * vdim + ib] = S::from_f32(b);
  }
  if (vdim & 1) {
    for (int h = threadIdx.x; h < kv_heads; h += blockDim.x)
      vc[h * vdim + vdim - 1] = vr[h * vdim + vdim - 1];
  }
}

// The epilogue every attention kernel of this file shares: o_lds holds one head's normalized
// output [vdim] in fp32; turn pair m back by the query's position, gate, write.
template <class S>
__device__ __forceinline__ void write_head_output(typename S::T* __restrict__ orow,
                                                  const float* __restrict__ o_lds, int vdim, float p,
                                                  const float* __restrict__ out_inv_freq,
                                                  int interleaved, float gate, int first, int step) {
  const int vhalf = vdim / 2;
  for (int d = first; d < vdim; d += step) {
    float val = o_lds[d];
    if (out_inv_freq != nullptr && d < 2 * vhalf) {
      int f, other;
      bool is_a;
      if (interleaved) {
        f = d >> 1;
        is_a = (d & 1) == 0;
        other = d ^ 1;
      } else {
        is_a = d < vhalf;
        f = is_a ? d : d - vhalf;
        other = is_a ? d + vhalf : d - vhalf;
      }
      float s, c;
      sincosf(p * out_inv_freq[f], &s, &c);
      // turned by the negative angle: (a cos + b sin, b cos - a sin)
      val = is_a ? val * c + o_lds[other] * s : val * c - o_lds[other] * s;
    }
    orow[d] = S::from_f32(val * gate);
  }
}

template <class S>
__global__ __launch_bounds__(kWave* kHeadsPerGroup) void kv_attention_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ key_cache, const typename S::T* __restrict__ value_cache,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ token_seq,
    const int64_t* __restrict__ positions, const float* __restrict__ out_inv_freq, int interleaved,
    int heads, int kv_heads, int dim, int vdim, int block_size, int num_blocks, int window,
    float scale) {
  __shared__ float q_lds[kHeadsPerGroup][kMaxDim];
  __shared__ float p_lds[kHeadsPerGroup][kWave];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.x;
  const int h = blockIdx.y * kHeadsPerGroup + w;
  if (h >= heads) return;  // whole wave; no workgroup barrier below
  const int g = h / (heads / kv_heads);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  for (int d = lane; d < dim; d += kWave)
    q_lds[w][d] = S::to_f32(q[(int64_t)t * q_stride + (int64_t)h * dim + d]) * scale;
  wave_sync();
  // a block id outside the pool (a table the host filled wrongly) reads block 0 instead of faulting
  auto token_row = [&](int j) {
    int b = table[j / block_size];
    b = (unsigned)b < (unsigned)num_blocks ? b : 0;
    return ((int64_t)b * block_size + j % block_size) * kv_heads + g;
  };

  float acc[kAccum];
#pragma unroll
  for (int c = 0; c < kAccum; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = lo; j0 <= p; j0 += kWave) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const typename S::T* kr = key_cache + token_row(j) * dim;
      float dot = 0.f;
      for (int d = 0; d < dim; ++d) dot += q_lds[w][d] * S::to_f32(kr[d]);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = j <= p ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    l = l * corr + wave_sum(pj);
    m = m_new;
    wave_sync();
    p_lds[w][lane] = pj;
    wave_sync();
#pragma unroll
    for (int c = 0; c < kAccum; ++c) acc[c] *= corr;
    const int n = min(kWave, p - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const typename S::T* vr = value_cache + token_row(j0 + jj) * vdim;
      const float pv = p_lds[w][jj];
#pragma unroll
      for (int c = 0; c < kAccum; ++c) {
        const int d = lane + c * kWave;
        if (d < vdim) acc[c] += pv * S::to_f32(vr[d]);
      }
    }
  }
  wave_sync();
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < kAccum; ++c) {
    const int d = lane + c * kWave;
    if (d < vdim) q_lds[w][d] = acc[c] * inv;   // the query is done with
  }
  wave_sync();
  float gv = 1.f;
  if (gate != nullptr) gv = 1.f / (1.f + expf(-S::to_f32(gate[(int64_t)t * gate_stride + h])));
  write_head_output<S>(out + (int64_t)t * out_stride + (int64_t)h * vdim, q_lds[w], vdim, (float)p,
                       out_inv_freq, interleaved, gv, lane, kWave);
}

}  // namespace
}  // namespace seq
}  // namespace vla

using namespace vla;
using namespace vla::seq;

extern "C" int vla_seq_rotary_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                       const void* v, int64_t v_stride, void* key_cache,
                                       void* value_cache, const int64_t* positions,
                                       const int64_t* slot_mapping, const float* inv_freq,
                                       const float* value_inv_freq, int num_tokens, int heads,
                                       int kv_heads, int dim, int vdim, int rot_dims,
                                       int interleaved, int block_size, int num_blocks, int dtype,
                                       void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!q || !k || !v || !key_cache || !value_cache || !positions || !slot_mapping || num_tokens < 0 ||
      heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || rot_dims < 0 || rot_dims > dim ||
      (rot_dims & 1) || (rot_dims > 0 && !inv_freq) || block_size <= 0 || num_blocks <= 0 ||
      q_stride < (int64_t)heads * dim || k_stride < (int64_t)kv_heads * dim ||
      v_stride < (int64_t)kv_heads * vdim)
    return VLA_ERR_ARG;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    rotary_kv_write_kernel<S><<<num_tokens, 256, 0, (hipStream_t)stream>>>(
        (T*)q, q_stride, (const T*)k, k_stride, (const T*)v, v_stride, (T*)key_cache,
        (T*)value_cache, positions, slot_mapping, inv_freq, value_inv_freq, heads, kv_heads, dim,
        vdim, rot_dims, interleaved, (int64_t)num_blocks * block_size);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

extern "C" int vla_seq_kv_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                    const void* gate, int64_t gate_stride, const void* key_cache,
                                    const void* value_cache, const int* block_tables,
                                    int max_blocks, const int* token_seq, const int64_t* positions,
                                    const float* out_inv_freq, int interleaved, int num_tokens,
                                    int heads, int kv_heads, int dim, int vdim, int block_size,
                                    int num_blocks, int window, float scale, int dtype,
                                    void* stream) {
  if (num_tokens == 0) return VLA_OK;
  if (!out || !q || !key_cache || !value_cache || !block_tables || !token_seq || !positions ||
      num_tokens < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || block_size <= 0 ||
      num_blocks <= 0 || max_blocks <= 0 || out_stride < (int64_t)heads * vdim ||
      q_stride < (int64_t)heads * dim || (gate && gate_stride < heads))
    return VLA_ERR_ARG;
  if (dim <= 0 || dim > kMaxDim || vdim <= 0 || vdim > kMaxDim) return VLA_ERR_HEAD_SIZE;
  return with_dtype(dtype, [&](auto s) {
    using S = decltype(s);
    using T = typename S::T;
    const dim3 grid(num_tokens, (heads + kHeadsPerGroup - 1) / kHeadsPerGroup);
    kv_attention_kernel<S><<<grid, kWave * kHeadsPerGroup, 0, (hipStream_t)stream>>>(
        (T*)out, out_stride, (const T*)q, q_stride, (const T*)gate, gate_stride,
        (const T*)key_cache, (const T*)value_cache, block_tables, max_blocks, token_seq, positions,
        out_inv_freq, interleaved, heads, kv_heads, dim, vdim, block_size, num_blocks, window, scale);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}
