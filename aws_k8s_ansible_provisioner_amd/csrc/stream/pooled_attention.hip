// Attention over a sliding window plus mean-pooled blocks before it, on a paged cache.
//
//   bias_rope_cache        q / k / v slices of a fused projection + biases, rotate-half rotary
//                          positions on q and k, q out, K / V cache write
//   pool_cache_blocks      mean key / value (fp32) of every block that a token of the step
//                          completed, stored with the page of the block's first token
//   pooled_window_attention  one online softmax over pooled entries and window tokens, optionally
//                          starting from a sink of score 0 (a 1 in the denominator)
//
// K [NB, G, BS, D] token-major and V [NB, G, BS / 8, Dv, 8] (groups of 8 tokens,
// dimension-major inside a group: the layout the matrix-core kernels read) in the activation
// type; pooled K / V [NB, G, PS, D / Dv] fp32.  Biases, angles, scores, softmax and the weighted sums are fp32.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::wave_max;
using akap::wave_sum;

namespace {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ int seq_of_row(const int32_t* q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// dot of a staged fp32 query with a cached row, 8 (bf16) or 4 (fp32) entries per load when the
// row allows it
__device__ __forceinline__ float dot_row(const float* q, const bf16* k, int D) {
  float acc = 0.f;
  if ((D & 7) == 0) {
    for (int i = 0; i < D; i += 8) {
      const akap::bf16x8 a = *(const akap::bf16x8*)(k + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += q[i + j] * (float)a[j];
    }
  } else {
    for (int i = 0; i < D; ++i) acc += q[i] * (float)k[i];
  }
  return acc;
}
__device__ __forceinline__ float dot_row(const float* q, const float* k, int D) {
  float acc = 0.f;
  if ((D & 3) == 0) {
    for (int i = 0; i < D; i += 4) {
      const float4 a = *(const float4*)(k + i);
      acc += q[i] * a.x + q[i + 1] * a.y + q[i + 2] * a.z + q[i + 3] * a.w;
    }
  } else {
    for (int i = 0; i < D; ++i) acc += q[i] * k[i];
  }
  return acc;
}

// ------------------------------------------------------------------ biases, rotation, cache
template <typename T>
__global__ __launch_bounds__(256) void bias_rope_cache_kernel(const RopeCacheParams p) {
  const int t = blockIdx.x;
  const T* row = (const T*)p.proj + (size_t)t * p.proj_stride;
  const int64_t pos = p.positions[t];
  const int64_t slot = p.slots[t];
  const int half = p.rot_dims / 2;
  const float* cs = p.cos_sin ? p.cos_sin + (size_t)(pos < p.max_pos ? pos : p.max_pos - 1) *
                                                p.rot_dims : nullptr;
  const int nq = p.H * p.D, nk = p.G * p.D, nv = p.G * p.Dv;
  for (int e = threadIdx.x; e < nq + nk + nv; e += 256) {
    int col, i, head;
    bool rot = false;
    if (e < nq) {
      col = p.q_off + e; head = e / p.D; i = e - head * p.D; rot = true;
    } else if (e < nq + nk) {
      const int f = e - nq;
      col = p.k_off + f; head = f / p.D; i = f - head * p.D; rot = true;
    } else {
      const int f = e - nq - nk;
      col = p.v_off + f; head = f / p.Dv; i = f - head * p.Dv;
    }
    float val = ldf(row + col) + (p.bias ? p.bias[col] : 0.f);
    if (rot && cs && i < p.rot_dims) {
      if (i < half) {
        const float v = ldf(row + col + half) + (p.bias ? p.bias[col + half] : 0.f);
        val = val * cs[i] - v * cs[half + i];
      } else {
        const int j = i - half;
        const float u = ldf(row + col - half) + (p.bias ? p.bias[col - half] : 0.f);
        val = val * cs[j] + u * cs[half + j];
      }
    }
    if (e < nq) {
      stf((T*)p.q_out + (size_t)t * nq + e, val);
    } else if (slot >= 0 && slot < p.num_slots) {
      const int64_t blk = slot / p.BS, off = slot - blk * p.BS;
      if (e < nq + nk)
        stf((T*)p.k_cache + ((blk * p.G + head) * p.BS + off) * p.D + i, val);
      else
        stf((T*)p.v_cache + (((blk * p.G + head) * (p.BS >> 3) + (off >> 3)) * p.Dv + i) * 8 +
                (off & 7), val);
    }
  }
}

// ------------------------------------------------------------------ pooled entries
// one workgroup per (RB rows, key/value head): 32 rows for large steps (few rows end a block,
// a workgroup per row would mostly launch and leave), one otherwise; rows that do not end a
// block are passed over
constexpr int kPoolRows = 32;

template <typename T>
__global__ __launch_bounds__(128) void pool_cache_blocks_kernel(const PoolParams p, const int RB) {
  const int g = blockIdx.y;
  for (int t = blockIdx.x * RB; t < min(p.T, (int)(blockIdx.x + 1) * RB); ++t) {
  const int pos = (int)p.positions[t];
  if (p.slots[t] < 0 || (pos + 1) % p.pool) continue;
  const int b = p.q_start ? seq_of_row(p.q_start, p.B, t) : t;
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const int first = pos + 1 - p.pool;
  const int page0 = bt[first / p.BS];
  const int idx = (first % p.BS) / p.pool;
  const float inv = 1.0f / (float)p.pool;
  const T* kc = (const T*)p.k_cache;
  const T* vc = (const T*)p.v_cache;
  for (int i = threadIdx.x; i < p.D + p.Dv; i += 128) {
    const bool isk = i < p.D;
    const int e = isk ? i : i - p.D;
    float acc = 0.f;
    int q = first;
    while (q <= pos) {                       // page by page
      const int page = bt[q / p.BS], off0 = q % p.BS;
      const int cnt = min(pos + 1 - q, p.BS - off0);
      const size_t row = (size_t)page * p.G + g;
      if (isk) {
        const T* src = kc + (row * p.BS + off0) * p.D + e;
        for (int j = 0; j < cnt; ++j) acc += ldf(src + (size_t)j * p.D);
      } else {
        for (int j = 0; j < cnt; ++j) {
          const int off = off0 + j;
          acc += ldf(vc + ((row * (p.BS >> 3) + (off >> 3)) * p.Dv + e) * 8 + (off & 7));
        }
      }
      q += cnt;
    }
    if (isk) p.k_pool[(((size_t)page0 * p.G + g) * p.PS + idx) * p.D + e] = acc * inv;
    else p.v_pool[(((size_t)page0 * p.G + g) * p.PS + idx) * p.Dv + e] = acc * inv;
  }
  }
}

// ------------------------------------------------------------------ attention
// One workgroup per (row, key/value head, up to 16 query heads of the group), one wave per query
// head.  The visible
// keys are an index range: first the pooled entries 0 .. nb-1, then the window tokens lo .. i.
// Per piece of 64 keys a lane scores one key (its row read in 16-byte pieces), the wave updates
// the running maximum and sum, then every lane accumulates its output dimensions over the
// piece's values.  All waves of a workgroup walk the same range, so barriers are uniform.
constexpr int kMaxDv = 512;
constexpr int kRowWaves = 16;

template <typename T>
__global__ void pooled_window_attention_kernel(const PoolAttnParams p, const int nw) {
  extern __shared__ float lds[];   // per wave: [D] query, [64] weights
  const int t = blockIdx.x, g = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rep = p.H / p.G, h = g * rep + blockIdx.z * nw + wave;
  if (p.slots[t] < 0) return;
  const int b = p.q_start ? seq_of_row(p.q_start, p.B, t) : t;
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const int i = (int)p.positions[t];
  const int lo = p.window > 0 ? (i - p.window + 1 > 0 ? i - p.window + 1 : 0) : 0;
  const int nb = (p.pool > 0 && p.window > 0 && i - p.window + 1 > 0)
                     ? (i - p.window + 1) / p.pool : 0;
  const int n = nb + (i - lo + 1);
  float* qs = lds + (size_t)wave * (p.D + 64);
  float* ps = qs + p.D;
  const T* q = (const T*)p.q + ((size_t)t * p.H + h) * p.D;
  for (int e = lane; e < p.D; e += 64) qs[e] = ldf(q + e) * p.scale;
  __syncthreads();
  float m = p.unit_sink ? 0.f : -INFINITY;
  float l = p.unit_sink ? 1.f : 0.f;
  float acc[kMaxDv / 64];
#pragma unroll
  for (int k = 0; k < kMaxDv / 64; ++k) acc[k] = 0.f;
  const T* kc = (const T*)p.k_cache;
  const T* vc = (const T*)p.v_cache;
  for (int base = 0; base < n; base += 64) {
    const int idx = base + lane;
    float s = -INFINITY;
    if (idx < n) {
      if (idx < nb) {
        const int first = idx * p.pool, page = bt[first / p.BS];
        const int e = (first % p.BS) / p.pool;
        s = dot_row(qs, p.k_pool + (((size_t)page * p.G + g) * p.PS + e) * p.D, p.D);
      } else {
        const int j = lo + (idx - nb), page = bt[j / p.BS], off = j % p.BS;
        s = dot_row(qs, kc + (((size_t)page * p.G + g) * p.BS + off) * p.D, p.D);
      }
    }
    const float mx = fmaxf(m, wave_max(s));
    const float w = idx < n ? __expf(s - mx) : 0.f;
    const float corr = (mx == -INFINITY) ? 1.f : __expf(m - mx);
    l = l * corr + wave_sum(w);
#pragma unroll
    for (int k = 0; k < kMaxDv / 64; ++k) acc[k] *= corr;
    m = mx;
    ps[lane] = w;
    __syncthreads();
    const int cnt = n - base < 64 ? n - base : 64;
    for (int kk = 0; kk < cnt; ++kk) {
      const int id2 = base + kk;
      const float w2 = ps[kk];
      if (id2 < nb) {
        const int first = id2 * p.pool, page = bt[first / p.BS];
        const int e = (first % p.BS) / p.pool;
        const float* vr = p.v_pool + (((size_t)page * p.G + g) * p.PS + e) * p.Dv;
#pragma unroll
        for (int k = 0; k < kMaxDv / 64; ++k)
          if (lane + 64 * k < p.Dv) acc[k] += w2 * vr[lane + 64 * k];
      } else {
        const int j = lo + (id2 - nb), page = bt[j / p.BS], off = j % p.BS;
        const T* vr = vc + (((size_t)page * p.G + g) * (p.BS >> 3) + (off >> 3)) * p.Dv * 8 +
                      (off & 7);
#pragma unroll
        for (int k = 0; k < kMaxDv / 64; ++k)
          if (lane + 64 * k < p.Dv) acc[k] += w2 * ldf(vr + (size_t)(lane + 64 * k) * 8);
      }
    }
    __syncthreads();
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  T* o = (T*)p.out + (size_t)t * p.out_stride + (size_t)h * p.Dv;
#pragma unroll
  for (int k = 0; k < kMaxDv / 64; ++k)
    if (lane + 64 * k < p.Dv) stf(o + lane + 64 * k, acc[k] * inv);
}

}  // namespace

void launch_bias_rope_cache(const RopeCacheParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  if (f32) bias_rope_cache_kernel<float><<<p.T, 256, 0, s>>>(p);
  else bias_rope_cache_kernel<bf16><<<p.T, 256, 0, s>>>(p);
}

void launch_pool_cache_blocks(const PoolParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  const int RB = p.T >= 1024 ? kPoolRows : 1;
  const dim3 grid((p.T + RB - 1) / RB, p.G);
  if (f32) pool_cache_blocks_kernel<float><<<grid, 128, 0, s>>>(p, RB);
  else pool_cache_blocks_kernel<bf16><<<grid, 128, 0, s>>>(p, RB);
}

void launch_pooled_window_attention(const PoolAttnParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  // rep = nz * nw: every workgroup has the same number of waves (heads)
  const int rep = p.H / p.G;
  int nw = rep < kRowWaves ? rep : kRowWaves;
  while (rep % nw) --nw;
  const dim3 grid(p.T, p.G, rep / nw);
  const size_t lds = (size_t)nw * (p.D + 64) * sizeof(float);
  if (f32) pooled_window_attention_kernel<float><<<grid, 64 * nw, lds, s>>>(p, nw);
  else pooled_window_attention_kernel<bf16><<<grid, 64 * nw, lds, s>>>(p, nw);
}

}  // namespace akap_stream
