// Sliding-window attention over a paged key cache whose values are its keys, with a linear
// distance bias per head, a position-dependent query temperature and a sigmoid output gate.
//
// Cache: [num_blocks, block_size, kv_heads, dim] in the model dtype -- token-major rows, so one
// tensor serves both contractions (q . k_j reads rows, sum_j p_j k_j reads them again from L2 /
// L1).  There is no value cache: a layer of this kind keeps half the bytes of an ordinary one.
//
// Prompts, portions of prompts and decode steps are the same case: every query row reads its
// window from the cache (the step's own keys are written first), so a position's result cannot
// depend on how its sequence was cut into steps.  Scores, softmax and the weighted sum are fp32.
// Four kernels, by dtype and by how the step's rows come: window_attention_kernel and
// window_attention_group_kernel (any dtype, row by row), window_attention_heads_kernel (16-bit,
// single rows on the matrix cores), window_attention_tile_kernel (16-bit, runs of rows on the
// matrix cores); they differ by fp32 rounding.
//
// window_attention_kernel: one wave per (token, query head).  A tile is 64 keys: lane j computes
// the score of key j against the query held in LDS (row reads of 16 bytes), the wave reduces
// max / sum (online softmax across tiles), then lane d accumulates sum_j p_j k_j[d] with
// coalesced column reads.  The four waves of a workgroup take consecutive query heads of one
// token, which share KV heads under grouped queries.
#include <atomic>

#include "seq_common.h"

namespace vla {
namespace seq {
namespace {

std::atomic<int> g_window_kernel{0};

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
  wave_sync();
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
    wave_sync();
    p_lds[w][lane] = pj;
    wave_sync();
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


// ---------------------------------------------------------------------------------------------
// window_attention_group_kernel: one workgroup per (query row, KV head, chunk of up to kHeadChunk
// query heads of that KV head).  For rows that come one per sequence (decode steps) the launch is
// bound by reading each window once: the four waves split the window's 64-key tiles, each wave
// copies its tile into LDS with coalesced 16-byte loads (once, for all heads of the chunk), lane j
// scores key j against every head's query, the probabilities go through LDS, every lane
// accumulates two neighbouring dims of sum_j p_j k_j from the same tile, and the waves' (max, sum,
// acc) are merged at the end.  The queries are read through wave-uniform addresses (cache hits,
// no LDS traffic): the score loop's only LDS traffic is the key row.
constexpr int kHeadChunk = 4;
constexpr int kPairs = kMaxDim / (2 * kWave);   // passes of 128 dims in the weighted sum


template <class S>
__global__ __launch_bounds__(256) void window_attention_group_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float* __restrict__ slopes, int heads, int kv_heads, int dim, int block_size,
    int num_blocks, int window, float scale, float temp_coef, float temp_every, float out_scale,
    int row_pad) {
  using T = typename S::T;
  constexpr int VEC = 16 / sizeof(T);
  extern __shared__ __align__(16) unsigned char smem[];
  const int row_len = dim + row_pad;                       // elements; rows stay 16-byte aligned
  T* tiles = reinterpret_cast<T*>(smem);                   // [4][64][row_len]
  float* p_lds = reinterpret_cast<float*>(smem + (size_t)4 * kWave * row_len * sizeof(T));  // [4][64][chunk]
  float* merge = p_lds + 4 * kWave * kHeadChunk;           // [4][chunk][2 + dim]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int t = blockIdx.x;
  const int group = heads / kv_heads;
  const int chunks = (group + kHeadChunk - 1) / kHeadChunk;
  const int g = blockIdx.y / chunks;
  const int h0 = g * group + (blockIdx.y % chunks) * kHeadChunk;
  const int nh = min(kHeadChunk, g * group + group - h0);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  float qs = scale;
  if (temp_coef != 0.f) qs *= 1.f + temp_coef * logf(floorf((float)(p + 1) / temp_every) + 1.f);
  // heads past the chunk's last read the last one's query again (their results are dropped)
  const T* qrow[kHeadChunk];
  float slope[kHeadChunk];
#pragma unroll
  for (int hh = 0; hh < kHeadChunk; ++hh) {
    const int h = h0 + min(hh, nh - 1);
    qrow[hh] = q + (int64_t)t * q_stride + (int64_t)h * dim;
    slope[hh] = slopes != nullptr ? slopes[h] : 0.f;
  }

  T* tile = tiles + (size_t)w * kWave * row_len;
  float* pw = p_lds + w * kWave * kHeadChunk;
  const int64_t tok_stride = (int64_t)kv_heads * dim;
  float m[kHeadChunk], l[kHeadChunk], acc[kHeadChunk][kPairs][2];
#pragma unroll
  for (int hh = 0; hh < kHeadChunk; ++hh) {
    m[hh] = -INFINITY;
    l[hh] = 0.f;
#pragma unroll
    for (int c = 0; c < kPairs; ++c) acc[hh][c][0] = acc[hh][c][1] = 0.f;
  }
  const int vec_per_row = dim / VEC;   // dim % VEC == 0 is a launch condition
  for (int j0 = lo + w * kWave; j0 <= p; j0 += 4 * kWave) {
    const int n = min(kWave, p - j0 + 1);
    // the tile: n rows of dim elements, 16 bytes per lane and load
    for (int i = lane; i < n * vec_per_row; i += kWave) {
      const int r = i / vec_per_row, v = i - r * vec_per_row;
      const int j = j0 + r;
      int b = table[j / block_size];
      b = (unsigned)b < (unsigned)num_blocks ? b : 0;
      const T* src = cache + ((int64_t)b * block_size + j % block_size) * tok_stride + (int64_t)g * dim + v * VEC;
      *reinterpret_cast<u32x4*>(tile + (size_t)r * row_len + v * VEC) = *reinterpret_cast<const u32x4*>(src);
    }
    wave_sync();
    // scores: lane = key; its row comes from LDS 16 bytes at a time, the queries from scalar loads
    float s[kHeadChunk];
#pragma unroll
    for (int hh = 0; hh < kHeadChunk; ++hh) s[hh] = 0.f;
    const T* kr = tile + (size_t)min(lane, n - 1) * row_len;
    // (rows are read 4 bytes at a time: wider reads of lane-strided rows came back wrong on the
    // part, so the row costs dim / 2 reads in 16-bit models; the arithmetic still dominates)
    for (int d = 0; d < dim; d += 2) {
      float k0, k1;
      if constexpr (sizeof(T) == 4) {
        k0 = kr[d];
        k1 = kr[d + 1];
      } else {
        const uint32_t kk = *reinterpret_cast<const uint32_t*>(kr + d);
        k0 = lo16<S>(kk);
        k1 = hi16<S>(kk);
      }
#pragma unroll
      for (int hh = 0; hh < kHeadChunk; ++hh)      // the same address in every lane: scalar loads
        s[hh] += S::to_f32(qrow[hh][d]) * k0 + S::to_f32(qrow[hh][d + 1]) * k1;
    }
    const float dist = (float)(p - (j0 + lane));
    float corr[kHeadChunk];
#pragma unroll
    for (int hh = 0; hh < kHeadChunk; ++hh) {
      const float sv = lane < n ? s[hh] * qs - slope[hh] * dist : -INFINITY;
      const float m_new = fmaxf(m[hh], wave_max(sv));
      const float pj = lane < n ? expf(sv - m_new) : 0.f;
      corr[hh] = expf(m[hh] - m_new);
      l[hh] = l[hh] * corr[hh] + wave_sum(pj);
      m[hh] = m_new;
      pw[lane * kHeadChunk + hh] = pj;
    }
    wave_sync();
#pragma unroll
    for (int hh = 0; hh < kHeadChunk; ++hh)
#pragma unroll
      for (int c = 0; c < kPairs; ++c) {
        acc[hh][c][0] *= corr[hh];
        acc[hh][c][1] *= corr[hh];
      }
    // weighted sum: lane = dims 2 lane, 2 lane + 1 (+ 128 per pass); dim is even (dim % VEC == 0)
    for (int jj = 0; jj < n; ++jj) {
      const f32x4 pv = *reinterpret_cast<const f32x4*>(pw + jj * kHeadChunk);
      const float ph[kHeadChunk] = {pv.x, pv.y, pv.z, pv.w};
#pragma unroll
      for (int c = 0; c < kPairs; ++c) {
        const int d = 2 * lane + c * 2 * kWave;
        if (d < dim) {
          float k0, k1;
          if constexpr (sizeof(T) == 4) {
            const f32x2 kk = *reinterpret_cast<const f32x2*>(tile + (size_t)jj * row_len + d);
            k0 = kk.x;
            k1 = kk.y;
          } else {
            const uint32_t kk = *reinterpret_cast<const uint32_t*>(tile + (size_t)jj * row_len + d);
            k0 = lo16<S>(kk);
            k1 = hi16<S>(kk);
          }
#pragma unroll
          for (int hh = 0; hh < kHeadChunk; ++hh) {
            acc[hh][c][0] += ph[hh] * k0;
            acc[hh][c][1] += ph[hh] * k1;
          }
        }
      }
    }
    wave_sync();
  }
  // merge the four waves
  float* mine = merge + (size_t)w * kHeadChunk * (2 + dim);
#pragma unroll
  for (int hh = 0; hh < kHeadChunk; ++hh) {
    if (lane == 0) {
      mine[hh * (2 + dim)] = m[hh];
      mine[hh * (2 + dim) + 1] = l[hh];
    }
#pragma unroll
    for (int c = 0; c < kPairs; ++c) {
      const int d = 2 * lane + c * 2 * kWave;
      if (d < dim) {
        mine[hh * (2 + dim) + 2 + d] = acc[hh][c][0];
        mine[hh * (2 + dim) + 2 + d + 1] = acc[hh][c][1];
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < nh * dim; i += 256) {
    const int hh = i / dim, d = i - hh * dim;
    float mm = -INFINITY;
    for (int ww = 0; ww < 4; ++ww) mm = fmaxf(mm, merge[((size_t)ww * kHeadChunk + hh) * (2 + dim)]);
    float ll = 0.f, o = 0.f;
    for (int ww = 0; ww < 4; ++ww) {
      const float* src = merge + ((size_t)ww * kHeadChunk + hh) * (2 + dim);
      const float f = src[0] == -INFINITY ? 0.f : expf(src[0] - mm);
      ll += src[1] * f;
      o += src[2 + d] * f;
    }
    float v = o * (out_scale / ll);
    if (gate != nullptr) {
      const float gv = S::to_f32(gate[(int64_t)t * gate_stride + (int64_t)(h0 + hh) * dim + d]);
      v *= 1.f / (1.f + expf(-gv));
    }
    out[(int64_t)t * out_stride + (int64_t)(h0 + hh) * dim + d] = S::from_f32(v);
  }
}

// ---------------------------------------------------------------------------------------------
// window_attention_tile_kernel<S, DB>: prompts and portions of prompts in 16-bit models, on the
// matrix cores.  One workgroup per (sequence, tile of 32 consecutive query rows, KV head, chunk of
// up to four of its query heads); wave w takes query head w of the chunk.  The keys from the
// first row's window start to the last row walk through LDS in tiles of 32, staged once for all
// waves, row-major for the first product and transposed for the second.  Both products run in
// transposed form on 32x32x8 MFMAs, lane = (hf, c) = (lane >> 5, lane & 31):
//   S^T = K q^T   A = K    lane: key c, dims 8 ks + 4 hf .. + 3
//                 B = q^T  lane: query c, the same dims (registers, loaded once)
//                 C        lane: query c, keys (i & 3) + 8 (i >> 2) + 4 hf, i = 0 .. 15
//   O^T = K^T P^T A = K^T  lane: dim 32 n + c, keys 8 s + 4 hf .. + 3
//                 B = P^T  lane: query c, the same keys = registers 4 s .. 4 s + 3 of C above
//                 C        lane: query c, dims 32 n + (i & 3) + 8 (i >> 2) + 4 hf
// so a lane owns one query's scores, running max / sum and output column; the softmax reduces
// over registers and one exchange with the partner lane.  Scores leave the first product in fp32
// and stay there; a weight enters the second product as the sum of two 16-bit numbers (its
// rounding and the rounding of what the rounding lost), which keeps 16 bits of it and lets the
// accumulation stay on the matrix cores.
// Operands travel as two packed 32-bit words (four 16-bit values) and are cast to the builtin's
// vector type at the call.
template <class S>
struct Mfma8;
template <>
struct Mfma8<BF16> {
  typedef short V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c,
                                                    0, 0, 0);
  }
};
template <>
struct Mfma8<F16> {
  typedef _Float16 V4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x16 run(u32x2 a, u32x2 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(V4, a), __builtin_bit_cast(V4, b), c, 0,
                                                0, 0);
  }
};
template <class S>
__device__ __forceinline__ uint32_t bits16(float v) {
  return (uint32_t)__builtin_bit_cast(uint16_t, S::from_f32(v));
}
template <class S>
__device__ __forceinline__ float from_bits16(uint32_t b) {
  return S::to_f32(__builtin_bit_cast(typename S::T, (uint16_t)b));
}

constexpr int kTile = 32;

template <class S, int DB>
__global__ __launch_bounds__(256) void window_attention_tile_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ query_start_loc, const int* __restrict__ context_lens,
    const float* __restrict__ slopes, int heads, int kv_heads, int block_size, int num_blocks,
    int window, float scale, float temp_coef, float temp_every, float out_scale) {
  using T = typename S::T;
  using M = Mfma8<S>;
  constexpr int D = 32 * DB;
  constexpr int KROW = D + 4, TROW = kTile + 4;      // elements; both keep 8-byte alignment
  __shared__ __align__(16) T k_lds[kTile * KROW];    // [key][dim]
  __shared__ __align__(16) T kt_lds[D * TROW];       // [dim][key]
  const int b = blockIdx.z;
  const int t0 = query_start_loc[b] + kTile * blockIdx.x;
  const int nq = min(kTile, query_start_loc[b + 1] - t0);
  if (nq <= 0) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int hf = lane >> 5, c = lane & 31;
  const int group = heads / kv_heads;
  const int chunks = (group + 3) / 4;
  const int g = blockIdx.y / chunks;
  const int h = g * group + (blockIdx.y % chunks) * 4 + w;
  const bool active = h < g * group + group;
  const int p0 = context_lens[b] + kTile * blockIdx.x, p_last = p0 + nq - 1;
  const int j_lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int* table = block_tables + (int64_t)b * max_blocks;
  const int64_t tok_stride = (int64_t)kv_heads * D;
  const int pq = p0 + c;
  float qs = scale;
  if (temp_coef != 0.f) qs *= 1.f + temp_coef * logf(floorf((float)(pq + 1) / temp_every) + 1.f);
  const float slope = (slopes != nullptr && active) ? slopes[h] : 0.f;

  u32x2 qf[D / 8];
#pragma unroll
  for (int ks = 0; ks < D / 8; ++ks) {
    u32x2 v = {0u, 0u};
    if (active && c < nq)
      v = *reinterpret_cast<const u32x2*>(q + (int64_t)(t0 + c) * q_stride + (int64_t)h * D + 8 * ks + 4 * hf);
    qf[ks] = v;
  }
  f32x16 o[DB];
#pragma unroll
  for (int n = 0; n < DB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // staging: DB pieces of 8 bytes per thread and tile, loaded one tile ahead (see the heads kernel)
  u32x2 x[DB];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int u = 0; u < DB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (D / 4), v = i % (D / 4);
      const int j = j0 + r;
      long long off = 0;
      if (j <= p_last) {
        int blk = table[j / block_size];
        blk = (unsigned)blk < (unsigned)num_blocks ? blk : 0;
        off = ((long long)blk * block_size + j % block_size) * tok_stride + (long long)g * D + 4 * v;
      }
      const u32x2 got = *reinterpret_cast<const u32x2*>(cache + off);
      x[u] = j <= p_last ? got : u32x2{0u, 0u};
    }
  };
  fetch(j_lo);
  for (int j0 = j_lo; j0 <= p_last; j0 += kTile) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < DB; ++u) {
      const int i = tid + 256 * u;
      const int r = i / (D / 4), v = i % (D / 4);
      *reinterpret_cast<u32x2*>(k_lds + r * KROW + 4 * v) = x[u];
      uint16_t* col = reinterpret_cast<uint16_t*>(kt_lds) + (4 * v) * TROW + r;
      col[0] = (uint16_t)(x[u][0] & 0xffffu);
      col[TROW] = (uint16_t)(x[u][0] >> 16);
      col[2 * TROW] = (uint16_t)(x[u][1] & 0xffffu);
      col[3 * TROW] = (uint16_t)(x[u][1] >> 16);
    }
    if (j0 + kTile <= p_last) fetch(j0 + kTile);
    __syncthreads();
    if (!active) continue;
    f32x16 st;
#pragma unroll
    for (int i = 0; i < 16; ++i) st[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < D / 8; ++ks) {
      const u32x2 a = *reinterpret_cast<const u32x2*>(k_lds + c * KROW + 8 * ks + 4 * hf);
      st = M::run(a, qf[ks], st);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = j0 + (i & 3) + 8 * (i >> 2) + 4 * hf;
      const int dist = pq - key;
      const bool ok = c < nq && dist >= 0 && (window <= 0 || dist < window);
      st[i] = ok ? st[i] * qs - slope * (float)dist : -INFINITY;
      mt = fmaxf(mt, st[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m, mt);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      st[i] = m_new == -INFINITY ? 0.f : expf(st[i] - m_new);
      psum += st[i];
    }
    l = l * corr + psum;          // this lane's keys; the partner's half is added at the end
    m = m_new;
#pragma unroll
    for (int n = 0; n < DB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[n][i] *= corr;
#pragma unroll
    for (int s8 = 0; s8 < 4; ++s8) {
      uint32_t hb[4], lb[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float pv = st[4 * s8 + e];
        hb[e] = bits16<S>(pv);
        lb[e] = bits16<S>(pv - from_bits16<S>(hb[e]));
      }
      const u32x2 hi = {hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16)};
      const u32x2 lo = {lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16)};
#pragma unroll
      for (int n = 0; n < DB; ++n) {
        const u32x2 a = *reinterpret_cast<const u32x2*>(kt_lds + (32 * n + c) * TROW + 8 * s8 + 4 * hf);
        o[n] = M::run(a, hi, o[n]);
        o[n] = M::run(a, lo, o[n]);
      }
    }
  }
  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  if (c >= nq) return;
  const float inv = out_scale / l;
#pragma unroll
  for (int n = 0; n < DB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * n + (i & 3) + 8 * (i >> 2) + 4 * hf;
      float v = o[n][i] * inv;
      if (gate != nullptr) {
        const float gv = S::to_f32(gate[(int64_t)(t0 + c) * gate_stride + (int64_t)h * D + d]);
        v *= 1.f / (1.f + expf(-gv));
      }
      out[(int64_t)(t0 + c) * out_stride + (int64_t)h * D + d] = S::from_f32(v);
    }
}

// ---------------------------------------------------------------------------------------------
// window_attention_heads_kernel<S, DB>: single rows (decode steps) of 16-bit models on the matrix
// cores.  One workgroup per (row, KV head, chunk of up to 32 of its query heads).  The products
// are those of the tile kernel with the 32 columns holding the chunk's query heads instead of 32
// rows of one head: S^T = K q^T scores one 32-key tile against every head at once, so each key
// byte is read once per KV head whatever the group size.  The four waves split the window's
// tiles (wave w of kRowWaves takes tiles w, w + kRowWaves, ...), each with its own tile in LDS and its own running
// max / sum / output, merged at the end.
constexpr int kRowWaves = 8;   // waves that split a row's window

template <class S, int DB>
__global__ __launch_bounds__(64 * kRowWaves) void window_attention_heads_kernel(
    typename S::T* __restrict__ out, int64_t out_stride, const typename S::T* __restrict__ q,
    int64_t q_stride, const typename S::T* __restrict__ gate, int64_t gate_stride,
    const typename S::T* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int64_t* __restrict__ positions,
    const float* __restrict__ slopes, int heads, int kv_heads, int block_size, int num_blocks,
    int window, float scale, float temp_coef, float temp_every, float out_scale, int merge_heads) {
  using T = typename S::T;
  using M = Mfma8<S>;
  constexpr int D = 32 * DB;
  constexpr int KROW = D + 4;
  constexpr int WAVE_ELEMS = kTile * KROW;                // one wave's tile, in elements
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int hf = lane >> 5, c = lane & 31;
  T* k_lds = reinterpret_cast<T*>(smem) + (size_t)w * WAVE_ELEMS;
  const int t = blockIdx.x;
  const int group = heads / kv_heads;
  const int chunks = (group + 31) / 32;
  const int g = blockIdx.y / chunks;
  const int h0 = g * group + (blockIdx.y % chunks) * 32;
  const int nh = min(32, g * group + group - h0);
  const int p = (int)positions[t];
  const int* table = block_tables + (int64_t)token_seq[t] * max_blocks;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int64_t tok_stride = (int64_t)kv_heads * D;
  float qs = scale;
  if (temp_coef != 0.f) qs *= 1.f + temp_coef * logf(floorf((float)(p + 1) / temp_every) + 1.f);
  const bool live = c < nh;
  const float slope = (slopes != nullptr && live) ? slopes[h0 + c] : 0.f;
  u32x2 qf[D / 8];
#pragma unroll
  for (int ks = 0; ks < D / 8; ++ks) {
    u32x2 v = {0u, 0u};
    if (live)
      v = *reinterpret_cast<const u32x2*>(q + (int64_t)t * q_stride + (int64_t)(h0 + c) * D + 8 * ks + 4 * hf);
    qf[ks] = v;
  }
  f32x16 o[DB];
#pragma unroll
  for (int n = 0; n < DB; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[n][i] = 0.f;
  float m = -INFINITY, l = 0.f;

  // A wave's share of a tile is D / 8 pieces of 8 bytes per lane.  Their loads are all issued
  // before any is used, and one tile ahead: while a tile is in the matrix cores the next one is
  // on its way from HBM.  (A piece's address needs the key's block from the table: lanes 0..31
  // look the 32 keys of the tile up once and hand the row offsets round with shuffles.)
  constexpr int PIECES = D / 8;
  u32x2 x[PIECES];
  auto fetch = [&](int j0) {
    const int jr = j0 + c;
    long long base = -1;
    if (jr <= p) {
      int blk = table[jr / block_size];
      blk = (unsigned)blk < (unsigned)num_blocks ? blk : 0;
      base = ((long long)blk * block_size + jr % block_size) * tok_stride + (long long)g * D;
    }
#pragma unroll
    for (int u = 0; u < PIECES; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (D / 4), v = i % (D / 4);
      const long long rb = __shfl(base, r, 64);
      const T* src = cache + (rb >= 0 ? rb + 4 * v : 0);     // a valid address either way
      const u32x2 got = *reinterpret_cast<const u32x2*>(src);
      x[u] = rb >= 0 ? got : u32x2{0u, 0u};
    }
  };
  fetch(lo + w * kTile);
  for (int j0 = lo + w * kTile; j0 <= p; j0 += kRowWaves * kTile) {
#pragma unroll
    for (int u = 0; u < PIECES; ++u) {
      const int i = lane + kWave * u;
      const int r = i / (D / 4), v = i % (D / 4);
      *reinterpret_cast<u32x2*>(k_lds + r * KROW + 4 * v) = x[u];
    }
    if (j0 + kRowWaves * kTile <= p) fetch(j0 + kRowWaves * kTile);
    wave_sync();
    f32x16 st;
#pragma unroll
    for (int i = 0; i < 16; ++i) st[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < D / 8; ++ks) {
      const u32x2 a = *reinterpret_cast<const u32x2*>(k_lds + c * KROW + 8 * ks + 4 * hf);
      st = M::run(a, qf[ks], st);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int dist = p - (j0 + (i & 3) + 8 * (i >> 2) + 4 * hf);
      st[i] = (live && dist >= 0) ? st[i] * qs - slope * (float)dist : -INFINITY;
      mt = fmaxf(mt, st[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m, mt);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      st[i] = m_new == -INFINITY ? 0.f : expf(st[i] - m_new);
      psum += st[i];
    }
    l = l * corr + psum;
    m = m_new;
#pragma unroll
    for (int n = 0; n < DB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[n][i] *= corr;
#pragma unroll
    for (int s8 = 0; s8 < 4; ++s8) {
      uint32_t hb[4], lb[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float pv = st[4 * s8 + e];
        hb[e] = bits16<S>(pv);
        lb[e] = bits16<S>(pv - from_bits16<S>(hb[e]));
      }
      const u32x2 hi = {hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16)};
      const u32x2 lo2 = {lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16)};
#pragma unroll
      for (int n = 0; n < DB; ++n) {
        // K^T operand from the row-major tile: dim 32 n + c of keys 8 s8 + 4 hf .. + 3 (a
        // transposed copy of the tile costs 16-bit scatter writes that collide in the LDS banks
        // and, with eight waves a CU, took most of the kernel's time)
        const uint16_t* col = reinterpret_cast<const uint16_t*>(k_lds) + (8 * s8 + 4 * hf) * KROW + 32 * n + c;
        const u32x2 a = {(uint32_t)col[0] | ((uint32_t)col[KROW] << 16),
                         (uint32_t)col[2 * KROW] | ((uint32_t)col[3 * KROW] << 16)};
        o[n] = M::run(a, hi, o[n]);
        o[n] = M::run(a, lo2, o[n]);
      }
    }
    wave_sync();
  }
  l += __shfl_xor(l, 32, 64);
  // merge the four waves through LDS (the tiles are done with): [wave][head][2 + D]
  __syncthreads();
  float* merge = reinterpret_cast<float*>(smem);
  if (live) {
    float* mine = merge + ((size_t)w * merge_heads + c) * (2 + D);
    if (hf == 0) {
      mine[0] = m;
      mine[1] = l;
    }
#pragma unroll
    for (int n = 0; n < DB; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) mine[2 + 32 * n + (i & 3) + 8 * (i >> 2) + 4 * hf] = o[n][i];
  }
  __syncthreads();
  for (int i = tid; i < nh * D; i += 64 * kRowWaves) {
    const int hh = i / D, d = i - hh * D;
    float mm = -INFINITY;
    for (int ww = 0; ww < kRowWaves; ++ww) mm = fmaxf(mm, merge[((size_t)ww * merge_heads + hh) * (2 + D)]);
    float ll = 0.f, ov = 0.f;
    for (int ww = 0; ww < kRowWaves; ++ww) {
      const float* src = merge + ((size_t)ww * merge_heads + hh) * (2 + D);
      const float f = src[0] == -INFINITY ? 0.f : expf(src[0] - mm);
      ll += src[1] * f;
      ov += src[2 + d] * f;
    }
    float v = ov * (out_scale / ll);
    if (gate != nullptr) {
      const float gv = S::to_f32(gate[(int64_t)t * gate_stride + (int64_t)(h0 + hh) * D + d]);
      v *= 1.f / (1.f + expf(-gv));
    }
    out[(int64_t)t * out_stride + (int64_t)(h0 + hh) * D + d] = S::from_f32(v);
  }
}

template <class S, int DB>
size_t heads_kernel_lds(int merge_heads) {
  constexpr int D = 32 * DB;
  const size_t tiles = (size_t)kRowWaves * kTile * (D + 4) * sizeof(typename S::T);
  const size_t merge = (size_t)kRowWaves * merge_heads * (2 + D) * sizeof(float);
  return tiles > merge ? tiles : merge;
}

template <class S, int DB>
int launch_heads_one(dim3 grid, hipStream_t stream, typename S::T* out, int64_t out_stride,
                     const typename S::T* q, int64_t q_stride, const typename S::T* gate,
                     int64_t gate_stride, const typename S::T* cache, const int* block_tables,
                     int max_blocks, const int* token_seq, const int64_t* positions,
                     const float* slopes, int heads, int kv_heads, int block_size, int num_blocks,
                     int window, float scale, float temp_coef, float temp_every, float out_scale) {
  const int group = heads / kv_heads;
  const int merge_heads = group < 32 ? group : 32;
  const size_t lds = heads_kernel_lds<S, DB>(merge_heads);
  static std::atomic<size_t> allowed{64 * 1024};   // raised once per kernel, not per launch
  if (lds > allowed.load(std::memory_order_relaxed)) {
    VLA_SEQ_HIP_CHECK(hipFuncSetAttribute(
        reinterpret_cast<const void*>(&window_attention_heads_kernel<S, DB>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed.store(lds, std::memory_order_relaxed);
  }
  window_attention_heads_kernel<S, DB><<<grid, 64 * kRowWaves, lds, stream>>>(
      out, out_stride, q, q_stride, gate, gate_stride, cache, block_tables, max_blocks, token_seq,
      positions, slopes, heads, kv_heads, block_size, num_blocks, window, scale, temp_coef,
      temp_every, out_scale, merge_heads);
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
}

template <class S, class... A>
int launch_heads(int db, A... a) {
  switch (db) {
    case 1: return launch_heads_one<S, 1>(a...);
    case 2: return launch_heads_one<S, 2>(a...);
    case 3: return launch_heads_one<S, 3>(a...);
    case 4: return launch_heads_one<S, 4>(a...);
    default: return VLA_ERR_HEAD_SIZE;
  }
}

template <class S>
int launch_tiles(int db, dim3 grid, hipStream_t stream, typename S::T* out, int64_t out_stride,
                 const typename S::T* q, int64_t q_stride, const typename S::T* gate,
                 int64_t gate_stride, const typename S::T* cache, const int* block_tables,
                 int max_blocks, const int* qsl, const int* ctx, const float* slopes, int heads,
                 int kv_heads, int block_size, int num_blocks, int window, float scale,
                 float temp_coef, float temp_every, float out_scale) {
#define VLA_TILE(DB)                                                                             \
  window_attention_tile_kernel<S, DB><<<grid, 256, 0, stream>>>(                                 \
      out, out_stride, q, q_stride, gate, gate_stride, cache, block_tables, max_blocks, qsl, ctx, \
      slopes, heads, kv_heads, block_size, num_blocks, window, scale, temp_coef, temp_every,     \
      out_scale)
  switch (db) {
    case 1: VLA_TILE(1); break;
    case 2: VLA_TILE(2); break;
    case 3: VLA_TILE(3); break;
    case 4: VLA_TILE(4); break;
    default: return VLA_ERR_HEAD_SIZE;
  }
#undef VLA_TILE
  VLA_SEQ_HIP_CHECK(hipGetLastError());
  return VLA_OK;
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
    using T = typename S::T;
    constexpr int VEC = 16 / sizeof(T);
    // the grouped kernel wants 16-byte rows everywhere it loads vectors and its tiles in LDS
    const int row_pad = VEC;
    const size_t lds = (size_t)4 * kWave * (dim + row_pad) * sizeof(T) +
                       sizeof(float) * ((size_t)4 * kWave * kHeadChunk + (size_t)4 * kHeadChunk * (2 + dim));
    const int mode = g_window_kernel.load(std::memory_order_relaxed);
    if constexpr (sizeof(T) == 2) {
      // 16-bit rows on the matrix cores when the head size and the alignment allow
      if (mode == 0 && dim % 32 == 0 && dim <= 128 && ((uintptr_t)q % 8) == 0 &&
          ((q_stride * 2) % 8) == 0 && ((uintptr_t)cache % 8) == 0) {
        const int group = heads / kv_heads;
        const dim3 grid(num_tokens, kv_heads * ((group + 31) / 32));
        return launch_heads<S>(dim / 32, grid, (hipStream_t)stream, (T*)out, out_stride, (const T*)q,
                               q_stride, (const T*)gate, gate_stride, (const T*)cache, block_tables,
                               max_blocks, token_seq, positions, slopes, heads, kv_heads, block_size,
                               num_blocks, window, scale, temp_coef, temp_every, out_scale);
      }
    }
    const bool grouped = mode != 1 && dim % VEC == 0 &&
                         ((uintptr_t)cache % 16) == 0 && lds <= 150 * 1024;
    if (grouped) {
      const int group = heads / kv_heads;
      const dim3 grid(num_tokens, kv_heads * ((group + kHeadChunk - 1) / kHeadChunk));
      static std::atomic<size_t> allowed{64 * 1024};   // raised once per kernel, not per launch
      if (lds > allowed.load(std::memory_order_relaxed)) {
        VLA_SEQ_HIP_CHECK(hipFuncSetAttribute(
            reinterpret_cast<const void*>(&window_attention_group_kernel<S>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        allowed.store(lds, std::memory_order_relaxed);
      }
      window_attention_group_kernel<S><<<grid, 256, lds, (hipStream_t)stream>>>(
          (T*)out, out_stride, (const T*)q, q_stride, (const T*)gate, gate_stride, (const T*)cache,
          block_tables, max_blocks, token_seq, positions, slopes, heads, kv_heads, dim, block_size,
          num_blocks, window, scale, temp_coef, temp_every, out_scale, row_pad);
      VLA_SEQ_HIP_CHECK(hipGetLastError());
      return VLA_OK;
    }
    const dim3 grid((heads + kHeadsPerGroup - 1) / kHeadsPerGroup, num_tokens);
    window_attention_kernel<S><<<grid, kWave * kHeadsPerGroup, 0, (hipStream_t)stream>>>(
        (T*)out, out_stride, (const T*)q, q_stride, (const T*)gate, gate_stride, (const T*)cache,
        block_tables, max_blocks, token_seq, positions, slopes, heads, kv_heads, dim, block_size,
        num_blocks, window, scale, temp_coef, temp_every, out_scale);
    VLA_SEQ_HIP_CHECK(hipGetLastError());
    return VLA_OK;
  });
}

// 0: pick per shape; 1: the one-wave-per-(row, head) kernel; 2: no matrix-core kernel for rows
// (tests run all)
extern "C" int vla_seq_set_window_kernel(int mode) {
  if (mode < 0 || mode > 2) return VLA_ERR_ARG;
  g_window_kernel.store(mode, std::memory_order_relaxed);
  return VLA_OK;
}

extern "C" int vla_seq_window_attention_tiles_supported(int dim, int dtype) {
  return (dtype == VLA_F16 || dtype == VLA_BF16) && dim % 32 == 0 && dim >= 32 && dim <= 128;
}

extern "C" int vla_seq_window_attention_tiles(
    void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
    int64_t gate_stride, const void* cache, const int* block_tables, int max_blocks,
    const int* query_start_loc, const int* context_lens, const float* slopes, int num_seqs,
    int max_query_len, int heads, int kv_heads, int dim, int block_size, int num_blocks, int window,
    float scale, float temp_coef, float temp_every, float out_scale, int dtype, void* stream) {
  if (num_seqs == 0 || max_query_len == 0) return VLA_OK;
  if (!out || !q || !cache || !block_tables || !query_start_loc || !context_lens || num_seqs < 0 ||
      max_query_len < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || block_size <= 0 ||
      num_blocks <= 0 || max_blocks <= 0 || out_stride < (int64_t)heads * dim ||
      q_stride < (int64_t)heads * dim || (gate && gate_stride < (int64_t)heads * dim) ||
      (temp_coef != 0.f && !(temp_every > 0.f)))
    return VLA_ERR_ARG;
  if (!vla_seq_window_attention_tiles_supported(dim, dtype)) return VLA_ERR_HEAD_SIZE;
  // 8-byte fragment loads: query rows and cache rows must allow them
  if (((uintptr_t)q % 8) || ((q_stride * 2) % 8) || ((uintptr_t)cache % 8)) return VLA_ERR_ARG;
  const int group = heads / kv_heads;
  const dim3 grid((max_query_len + kTile - 1) / kTile, kv_heads * ((group + 3) / 4), num_seqs);
  if (dtype == VLA_BF16)
    return launch_tiles<BF16>(dim / 32, grid, (hipStream_t)stream, (__bf16*)out, out_stride,
                              (const __bf16*)q, q_stride, (const __bf16*)gate, gate_stride,
                              (const __bf16*)cache, block_tables, max_blocks, query_start_loc,
                              context_lens, slopes, heads, kv_heads, block_size, num_blocks, window,
                              scale, temp_coef, temp_every, out_scale);
  return launch_tiles<F16>(dim / 32, grid, (hipStream_t)stream, (_Float16*)out, out_stride,
                           (const _Float16*)q, q_stride, (const _Float16*)gate, gate_stride,
                           (const _Float16*)cache, block_tables, max_blocks, query_start_loc,
                           context_lens, slopes, heads, kv_heads, block_size, num_blocks, window, scale,
                           temp_coef, temp_every, out_scale);
}
