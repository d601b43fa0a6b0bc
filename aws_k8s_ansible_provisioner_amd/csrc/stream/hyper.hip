// Kernels of layers over several residual streams (learned read / mix / write weights per
// sublayer), a tanh cap on logits, sigmoid group routing, and the selective state-space mixer:
// causal convolution + silu with carried inputs, the recurrence with the state in registers, the
// silu gate with a grouped RMS norm.
//
// Sums over streams, norms, router scores, step sizes, decays and the whole recurrence are fp32
// whatever the storage type; every size is a run-time argument.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::block_sum;
using akap::wave_sum;

namespace {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ float ldv(const void* p, bool f32, size_t i) {
  return f32 ? ((const float*)p)[i] : (float)((const bf16*)p)[i];
}
__device__ __forceinline__ void ld4v(const void* p, bool f32, size_t i, float (&v)[4]) {
  if (f32) {
    const float4 a = *(const float4*)((const float*)p + i);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  } else {
    const akap::bf16x4 a = *(const akap::bf16x4*)((const bf16*)p + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = (float)a[k];
  }
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(bf16* p, const float (&v)[4]) {
  akap::bf16x4 o;
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = (bf16)v[k];
  *(akap::bf16x4*)p = o;
}

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + __expf(-z)); }
__device__ __forceinline__ float siluf(float z) { return z * sigmoidf(z); }

// the sequence that owns row t: the last b with q_start[b] <= t (q_start ascending, B + 1 entries)
__device__ __forceinline__ int seq_of_row(const int32_t* q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

constexpr int kMaxStreams = 8;

// ------------------------------------------------------------------ stream write + read + norm
// one workgroup per token; W columns per thread and turn (W = 4: 16-byte accesses).  A thread
// keeps to its own columns in both phases, so the LDS row needs no barrier beyond the block sum.
struct HyperArgs {
  float* xs;            // [T, S, d]
  const float* fresh;   // [T, d] or null
  const void* ya;       // [T, d] rows of ya_stride, or null
  const void* yb;
  const float* bias;    // [d] or null
  const float* mix;     // [S, S] (from, to)
  const float* w_out;   // [S]
  const float* w_in;    // [S]
  const float* norm_w;  // [d]
  int ya_stride, yb_stride, ya_f32, yb_f32;
  int S, d;
  float eps;
};

template <typename TO, int W>
__global__ __launch_bounds__(256) void hyper_step_kernel(TO* __restrict__ out, int out_stride,
                                                         const HyperArgs a) {
  extern __shared__ float lds[];   // [d] u, then [S S + 2 S] coefficients, then 16 scratch
  float* us = lds;
  float* cf = lds + a.d;
  float* scratch = cf + a.S * a.S + 2 * a.S;
  const int t = blockIdx.x, S = a.S, d = a.d;
  for (int i = threadIdx.x; i < S * S + 2 * S; i += 256) {
    float v;
    if (i < S * S) v = a.mix ? a.mix[i] : 0.f;
    else if (i < S * S + S) v = a.w_out ? a.w_out[i - S * S] : 0.f;
    else v = a.w_in[i - S * S - S];
    cf[i] = v;
  }
  __syncthreads();
  const float* mixs = cf;
  const float* outs = cf + S * S;
  const float* ins = cf + S * S + S;
  float* xr = a.xs + (size_t)t * S * d;
  float ssq = 0.f;
  for (int c = threadIdx.x * W; c < d; c += 256 * W) {
    float nw[kMaxStreams][W];
    float u[W];
#pragma unroll
    for (int k = 0; k < W; ++k) u[k] = 0.f;
    if (a.fresh) {
      float e[W];
      if constexpr (W == 4) ld4v(a.fresh, true, (size_t)t * d + c, (float(&)[4])e);
      else e[0] = a.fresh[(size_t)t * d + c];
#pragma unroll
      for (int r = 0; r < kMaxStreams; ++r)
        if (r < S) {
#pragma unroll
          for (int k = 0; k < W; ++k) nw[r][k] = e[k];
        }
    } else {
      float y[W];
#pragma unroll
      for (int k = 0; k < W; ++k) y[k] = 0.f;
      if (a.ya) {
        float v[W];
        if constexpr (W == 4) ld4v(a.ya, a.ya_f32, (size_t)t * a.ya_stride + c, (float(&)[4])v);
        else v[0] = ldv(a.ya, a.ya_f32, (size_t)t * a.ya_stride + c);
#pragma unroll
        for (int k = 0; k < W; ++k) y[k] += v[k];
      }
      if (a.yb) {
        float v[W];
        if constexpr (W == 4) ld4v(a.yb, a.yb_f32, (size_t)t * a.yb_stride + c, (float(&)[4])v);
        else v[0] = ldv(a.yb, a.yb_f32, (size_t)t * a.yb_stride + c);
#pragma unroll
        for (int k = 0; k < W; ++k) y[k] += v[k];
      }
      if (a.bias) {
#pragma unroll
        for (int k = 0; k < W; ++k) y[k] += a.bias[c + k];
      }
      float old[kMaxStreams][W];
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < S) {
          if constexpr (W == 4) ld4v(xr, true, (size_t)s * d + c, (float(&)[4])old[s]);
          else old[s][0] = xr[(size_t)s * d + c];
        }
#pragma unroll
      for (int r = 0; r < kMaxStreams; ++r)
        if (r < S) {
          const float wo = outs[r];
#pragma unroll
          for (int k = 0; k < W; ++k) nw[r][k] = wo * y[k];
#pragma unroll
          for (int s = 0; s < kMaxStreams; ++s)
            if (s < S) {
              const float m = mixs[s * S + r];
#pragma unroll
              for (int k = 0; k < W; ++k) nw[r][k] += m * old[s][k];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kMaxStreams; ++r)
      if (r < S) {
        if constexpr (W == 4) st4(xr + (size_t)r * d + c, (const float(&)[4])nw[r]);
        else xr[(size_t)r * d + c] = nw[r][0];
        const float wi = ins[r];
#pragma unroll
        for (int k = 0; k < W; ++k) u[k] += wi * nw[r][k];
      }
#pragma unroll
    for (int k = 0; k < W; ++k) {
      us[c + k] = u[k];
      ssq += u[k] * u[k];
    }
  }
  ssq = block_sum(ssq, scratch);
  const float inv = rsqrtf(ssq / (float)d + a.eps);
  TO* o = out + (size_t)t * out_stride;
  for (int c = threadIdx.x * W; c < d; c += 256 * W) {
    if constexpr (W == 4) {
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = us[c + k] * inv * a.norm_w[c + k];
      st4(o + c, v);
    } else {
      stf(o + c, us[c] * inv * a.norm_w[c]);
    }
  }
}

// ------------------------------------------------------------------ tanh cap
template <typename T>
__global__ __launch_bounds__(256) void softcap_kernel(T* __restrict__ x, size_t n, float cap,
                                                      float inv_cap) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    stf(x + i, cap * tanhf(ldf(x + i) * inv_cap));
}

// ------------------------------------------------------------------ gate + grouped norm
// one workgroup per (row, part)
template <typename T>
__global__ __launch_bounds__(256) void gate_group_norm_kernel(T* __restrict__ out, int out_stride,
                                                              const float* __restrict__ y,
                                                              const T* __restrict__ gate,
                                                              int gate_stride,
                                                              const float* __restrict__ w, int n,
                                                              int groups, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, part = n / groups, c0 = blockIdx.y * part;
  const float* yr = y + (size_t)t * n + c0;
  const T* gr = gate + (size_t)t * gate_stride + c0;
  float ssq = 0.f;
  for (int c = threadIdx.x; c < part; c += 256) {
    const float v = yr[c] * siluf(ldf(gr + c));
    ssq += v * v;
  }
  ssq = block_sum(ssq, scratch);
  const float inv = rsqrtf(ssq / (float)part + eps);
  T* o = out + (size_t)t * out_stride + c0;
  for (int c = threadIdx.x; c < part; c += 256)
    stf(o + c, yr[c] * siluf(ldf(gr + c)) * inv * w[c0 + c]);
}

// ------------------------------------------------------------------ sigmoid group routing
// one workgroup of four waves per token: the row staged in LDS, a logit per wave and turn, then
// one thread picks groups and experts (ties: the lower index)
template <typename T>
__global__ __launch_bounds__(256) void route_sigmoid_kernel(int32_t* __restrict__ ids,
                                                            float* __restrict__ wts,
                                                            const T* __restrict__ h, int h_stride,
                                                            const float* __restrict__ router, int d,
                                                            int E, int top, int groups, int keep,
                                                            int group_top) {
  extern __shared__ __align__(16) float lds[];   // [d] row (padded to 4), [E] scores, [E] choice
  float* hs = lds;                               // values, [groups] group scores
  float* sc = lds + ((d + 3) & ~3);
  float* ch = sc + E;
  float* gs = ch + E;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + (size_t)t * h_stride;
  for (int c = threadIdx.x; c < d; c += 256) hs[c] = ldf(hr + c);
  __syncthreads();
  for (int e = wave; e < E; e += 4) {
    const float* r = router + (size_t)e * d;
    float acc = 0.f;
    if ((d & 3) == 0 && ((uintptr_t)router & 15) == 0) {
      float a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll 4
      for (int c = lane * 4; c < d; c += 256) {
        const float4 w4 = *(const float4*)(r + c), h4 = *(const float4*)(hs + c);
        acc += h4.x * w4.x; a1 += h4.y * w4.y; a2 += h4.z * w4.z; a3 += h4.w * w4.w;
      }
      acc = (acc + a1) + (a2 + a3);
    } else {
      for (int c = lane; c < d; c += 64) acc += hs[c] * r[c];
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      const float s = 1.0f / (1.0f + expf(-acc));
      sc[e] = s;
      ch[e] = s;
    }
  }
  __syncthreads();
  const int per = E / groups;
  if (groups > 1) {
    // group score: the sum of its group_top largest scores (ch is consumed and restored)
    for (int g = threadIdx.x; g < groups; g += 256) {
      float sum = 0.f;
      const int n = group_top < per ? group_top : per;
      for (int k = 0; k < n; ++k) {
        int best = -1;
        float bv = -1.f;
        for (int e = g * per; e < (g + 1) * per; ++e)
          if (ch[e] > bv) { bv = ch[e]; best = e; }
        sum += bv;
        ch[best] = -2.f;
      }
      for (int e = g * per; e < (g + 1) * per; ++e) ch[e] = sc[e];
      gs[g] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      // keep the best groups: mark kept groups by a negative score - 10
      for (int k = 0; k < keep; ++k) {
        int best = -1;
        float bv = -1.f;
        for (int g = 0; g < groups; ++g)
          if (gs[g] > bv) { bv = gs[g]; best = g; }
        gs[best] = -10.f;
      }
      for (int g = 0; g < groups; ++g)
        if (gs[g] != -10.f)
          for (int e = g * per; e < (g + 1) * per; ++e) ch[e] = -1.f;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    for (int k = 0; k < top; ++k) {
      int best = 0;
      float bv = -3.f;
      for (int e = 0; e < E; ++e)
        if (ch[e] > bv) { bv = ch[e]; best = e; }
      ids[(size_t)t * top + k] = best;
      wts[(size_t)t * top + k] = sc[best];
      ch[best] = -4.f;
    }
  }
}

// ------------------------------------------------------------------ causal convolution + silu
constexpr int kMaxTaps = 8;

struct ConvArgs {
  float* out;              // [T, C]
  const void* proj;        // rows of proj_stride; the convolution's columns start at off
  void* state;             // [slots, taps - 1, C] of proj's type, oldest first
  const float* w;          // [C, taps]
  const float* b;          // [C]
  const int32_t* seq_slot; // [T]
  const int64_t* positions;
  const int32_t* q_start;  // [B + 1] or null (a row is a sequence)
  int proj_stride, off, C, taps, T, B;
};

// a thread per (row, channel): inputs before the step's first row of the sequence come from the
// slot (zeros before position 0)
template <typename TY>
__global__ __launch_bounds__(256) void conv_silu_kernel(const ConvArgs a) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.C) return;
  const int r0 = a.q_start ? a.q_start[seq_of_row(a.q_start, a.B, t)] : t;
  const int slot = a.seq_slot[r0];
  if (slot < 0) return;
  const int64_t pos0 = a.positions[r0];
  const TY* proj = (const TY*)a.proj;
  const TY* st = (const TY*)a.state + (size_t)slot * (a.taps - 1) * a.C;
  float acc = a.b[c];
  for (int j = 0; j < a.taps; ++j) {
    const int src = t - (a.taps - 1 - j);
    float u = 0.f;
    if (src >= r0) {
      u = ldf(proj + (size_t)src * a.proj_stride + a.off + c);
    } else {
      const int k = src - r0;   // -1: the input just before the step
      if (pos0 + k >= 0) u = ldf(st + (size_t)(a.taps - 1 + k) * a.C + c);
    }
    acc += a.w[(size_t)c * a.taps + j] * u;
  }
  a.out[(size_t)t * a.C + c] = siluf(acc);
}

// four channels per thread over a tile of RB rows (kConvRows for prompt chunks, 1 for steps of
// single rows, where every row starts from its slot anyway; C % 4 == 0, rows and pointers aligned
// for 8- / 16-byte accesses): the weights are read once, the last taps - 1 inputs slide through
// registers, a row costs one load and one store; at a sequence's first row of the step the
// history comes from its slot
constexpr int kConvRows = 16;

template <typename TY>
__global__ __launch_bounds__(256) void conv_silu_vec_kernel(const ConvArgs a, const int RB) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= a.C) return;
  const int tb = blockIdx.x * RB, te = min(a.T, tb + RB);
  constexpr bool F32 = sizeof(TY) == 4;
  const TY* proj = (const TY*)a.proj;
  float bias[4], w[4][kMaxTaps], hist[kMaxTaps][4];   // hist[j]: the input taps - 1 - j rows back
  ld4v(a.b, true, c, bias);
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) w[k][j] = j < a.taps ? a.w[(size_t)(c + k) * a.taps + j] : 0.f;
  int b = a.q_start ? seq_of_row(a.q_start, a.B, tb) : tb;
  int r1 = tb;                                        // forces the first row to load its history
  int slot = -1;
  for (int t = tb; t < te; ++t) {
    if (t >= r1) {                                    // a new sequence (or the tile's first row)
      int r0;
      if (a.q_start) {
        if (t > tb) ++b;
        while (a.q_start[b + 1] <= t) ++b;            // empty sequences
        r0 = a.q_start[b];
        r1 = a.q_start[b + 1];
      } else {
        r0 = t;
        r1 = t + 1;
      }
      slot = a.seq_slot[r0];
      const int pos0 = (int)a.positions[r0];
      const TY* st = (const TY*)a.state + (size_t)(slot < 0 ? 0 : slot) * (a.taps - 1) * a.C;
#pragma unroll
      for (int j = 0; j < kMaxTaps - 1; ++j) {
        if (j < a.taps - 1) {
          const int src = t - (a.taps - 1 - j);
#pragma unroll
          for (int k = 0; k < 4; ++k) hist[j][k] = 0.f;
          if (slot >= 0) {
            if (src >= r0) {
              ld4v(proj, F32, (size_t)src * a.proj_stride + a.off + c, hist[j]);
            } else {
              const int kk = src - r0;                // -1: the input just before the step
              if (pos0 + kk >= 0) ld4v(st, F32, (size_t)(a.taps - 1 + kk) * a.C + c, hist[j]);
            }
          }
        }
      }
    }
    float cur[4];
    ld4v(proj, F32, (size_t)t * a.proj_stride + a.off + c, cur);
    float acc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = bias[k];
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j)
      if (j < a.taps - 1) {
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] += w[k][j] * hist[j][k];
      }
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float wl = 0.f;
#pragma unroll
      for (int j = 0; j < kMaxTaps; ++j)
        if (j == a.taps - 1) wl = w[k][j];
      o[k] = siluf(acc[k] + wl * cur[k]);
    }
    if (slot >= 0) st4(a.out + (size_t)t * a.C + c, o);
#pragma unroll
    for (int j = 0; j < kMaxTaps - 2; ++j)
      if (j < a.taps - 2) {
#pragma unroll
        for (int k = 0; k < 4; ++k) hist[j][k] = hist[j + 1][k];
      }
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j)
      if (j == a.taps - 2) {
#pragma unroll
        for (int k = 0; k < 4; ++k) hist[j][k] = cur[k];
      }
  }
}

// a thread per (sequence, channel): the last taps - 1 inputs of the sequence go to its slot
template <typename TY>
__global__ __launch_bounds__(256) void conv_state_kernel(const ConvArgs a) {
  const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.C) return;
  const int r0 = a.q_start ? a.q_start[b] : b;
  const int r1 = a.q_start ? a.q_start[b + 1] : b + 1;
  if (r1 <= r0) return;
  const int slot = a.seq_slot[r0];
  if (slot < 0) return;
  const int64_t pos0 = a.positions[r0];
  const int n = r1 - r0, keep = a.taps - 1;
  const TY* proj = (const TY*)a.proj;
  TY* st = (TY*)a.state + (size_t)slot * keep * a.C;
  TY nv[kMaxTaps];
#pragma unroll
  for (int m = 0; m < kMaxTaps; ++m) {
    if (m < keep) {
      const int e = n + m - keep;   // row offset from r0 of the entry's input
      TY v = (TY)0.f;
      if (e >= 0) v = proj[(size_t)(r0 + e) * a.proj_stride + a.off + c];
      else if (pos0 + e >= 0) v = st[(size_t)(keep + e) * a.C + c];
      nv[m] = v;
    }
  }
#pragma unroll
  for (int m = 0; m < kMaxTaps; ++m)
    if (m < keep) st[(size_t)m * a.C + c] = nv[m];
}

// ------------------------------------------------------------------ selective scan
struct ScanArgs {
  float* y;                // [T, H V]
  const float* xbc;        // [T, H V + 2 G N] = [x | B | C]
  const void* proj;        // dt at column dt_off + h of rows of proj_stride
  const float* dt_bias;    // [H]
  const float* a_log;      // [H]
  const float* d_skip;     // [H]
  float* state;            // [slots, H, N, V]
  const int32_t* seq_slot;
  const int64_t* positions;
  const int32_t* q_start;  // [B + 1] or null
  int proj_stride, dt_off, H, V, N, G, T, B;
  int VL;                  // state columns of a workgroup (V / VL workgroups per head)
};

constexpr int kScanTokens = 16;

__host__ __device__ __forceinline__ int up4(int n) { return (n + 3) & ~3; }

// One workgroup per (sequence, head, VL state columns) -- the columns of a state are independent;
// the launcher gives a workgroup the whole head.  Thread (v, part) owns column v of the R
// consecutive state rows part R .. part R + R - 1 (NP = 256 / VL parts), in registers over all
// rows of the step.  Tokens are staged TK at a time (x, B, C, step size and decay; TK = 16 for
// prompt chunks, fetched into registers one stage ahead; 1 for steps of single rows); per token
// a thread updates its rows and adds its share of S^T C, reading B and C from LDS four rows at a
// time (all lanes of a wave read the same addresses); the parts' shares meet in LDS after the
// staged tokens.
template <typename TY, int R>
__global__ __launch_bounds__(256) void selective_scan_kernel(const ScanArgs a, const int TK) {
  extern __shared__ __align__(16) float lds[];
  const int V = a.VL, N = a.N, NP = 256 / V;    // V: the columns of this workgroup
  float* xs = lds;                              // [TK][V]
  float* bs = xs + up4(TK * V);                 // [TK][N]
  float* cs = bs + up4(TK * N);                 // [TK][N]
  float* dts = cs + up4(TK * N);                // [TK] step, [TK] decay
  float* ys = dts + up4(2 * TK);                // [TK][NP][V]
  const int nsplit = a.V / V;
  const int b = blockIdx.x, h = blockIdx.y / nsplit, v0 = (blockIdx.y - h * nsplit) * V;
  const int r0 = a.q_start ? a.q_start[b] : b;
  const int r1 = a.q_start ? a.q_start[b + 1] : b + 1;
  if (r1 <= r0) return;
  const int slot = a.seq_slot[r0];
  if (slot < 0) return;
  const int g = h / (a.H / a.G);
  const int inner = a.H * a.V, C = inner + 2 * a.G * N;
  const int tid = threadIdx.x;
  const int v = tid % V, part = tid / V;
  const int n0 = part * R;
  const bool active = part < NP && n0 < N;
  const bool vec = (N & 3) == 0 && (R & 3) == 0;
  float* sp = a.state + ((size_t)slot * a.H + h) * N * a.V + v0;
  float S[R];
  const bool carry = a.positions[r0] > 0;
#pragma unroll
  for (int r = 0; r < R; ++r)
    S[r] = (carry && active && n0 + r < N) ? sp[(size_t)(n0 + r) * a.V + v] : 0.f;
  const float ea = expf(a.a_log[h]), dsk = a.d_skip[h], dtb = a.dt_bias[h];
  const TY* proj = (const TY*)a.proj;
  // prompt chunks with sizes in fours: the next 16 tokens are fetched into registers (16-byte
  // loads, all issued together) while the current 16 are computed
  const bool vstage = TK == kScanTokens && (V & 3) == 0 && (N & 3) == 0 && (a.V & 3) == 0 &&
                      V <= 256 && N <= 256;
  const int V4 = V >> 2, N4 = N >> 2;
  float4 px[4], pb[4], pc[4];
  float pdt = 0.f;
  auto prefetch = [&](int c0) {
    const int nt = min(TK, r1 - c0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = tid + 256 * u;
      if (i < nt * V4) {
        const int tk = i / V4, e = i - tk * V4;
        px[u] = *(const float4*)(a.xbc + (size_t)(c0 + tk) * C + h * a.V + v0 + 4 * e);
      }
      if (i < nt * N4) {
        const int tk = i / N4, e = i - tk * N4;
        const float* row = a.xbc + (size_t)(c0 + tk) * C + inner + g * N + 4 * e;
        pb[u] = *(const float4*)row;
        pc[u] = *(const float4*)(row + a.G * N);
      }
    }
    if (tid < nt) pdt = ldf(proj + (size_t)(c0 + tid) * a.proj_stride + a.dt_off + h);
  };
  if (vstage) prefetch(r0);
  for (int c0 = r0; c0 < r1; c0 += TK) {
    const int nt = min(TK, r1 - c0);
    __syncthreads();
    if (vstage) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = tid + 256 * u;
        if (i < nt * V4) *(float4*)(xs + 4 * i) = px[u];
        if (i < nt * N4) {
          *(float4*)(bs + 4 * i) = pb[u];
          *(float4*)(cs + 4 * i) = pc[u];
        }
      }
      if (tid < nt) {
        const float z = pdt + dtb;
        const float dt = z > 20.f ? z : log1pf(expf(z));
        dts[tid] = dt;
        dts[TK + tid] = expf(-ea * dt);
      }
      __syncthreads();
      if (c0 + TK < r1) prefetch(c0 + TK);
    } else {
    for (int i = tid; i < nt * V; i += 256) {
      const int tk = i / V, e = i - tk * V;
      xs[tk * V + e] = a.xbc[(size_t)(c0 + tk) * C + h * a.V + v0 + e];
    }
    for (int i = tid; i < nt * N; i += 256) {
      const int tk = i / N, e = i - tk * N;
      const float* row = a.xbc + (size_t)(c0 + tk) * C + inner + g * N + e;
      bs[tk * N + e] = row[0];
      cs[tk * N + e] = row[a.G * N];
    }
    if (tid < nt) {
      const float z = ldf(proj + (size_t)(c0 + tid) * a.proj_stride + a.dt_off + h) + dtb;
      const float dt = z > 20.f ? z : log1pf(expf(z));
      dts[tid] = dt;
      dts[TK + tid] = expf(-ea * dt);
    }
    __syncthreads();
    }
    if (active) {
      for (int tk = 0; tk < nt; ++tk) {
        const float dt = dts[tk], dec = dts[TK + tk];
        const float dx = dt * xs[tk * V + v];
        const float* bt = bs + tk * N + n0;
        const float* ct = cs + tk * N + n0;
        float acc = 0.f;
        if (vec) {
          float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;   // four chains instead of one
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            if (n0 + r < N) {
              const float4 b4 = *(const float4*)(bt + r), c4 = *(const float4*)(ct + r);
              S[r] = dec * S[r] + dx * b4.x;
              S[r + 1] = dec * S[r + 1] + dx * b4.y;
              S[r + 2] = dec * S[r + 2] + dx * b4.z;
              S[r + 3] = dec * S[r + 3] + dx * b4.w;
              a0 += S[r] * c4.x;
              a1 += S[r + 1] * c4.y;
              a2 += S[r + 2] * c4.z;
              a3 += S[r + 3] * c4.w;
            }
          }
          acc = (a0 + a1) + (a2 + a3);
        } else {
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (n0 + r < N) {
              S[r] = dec * S[r] + dx * bt[r];
              acc += S[r] * ct[r];
            }
          }
        }
        ys[(tk * NP + part) * V + v] = acc;
      }
    } else if (part < NP) {
      for (int tk = 0; tk < nt; ++tk) ys[(tk * NP + part) * V + v] = 0.f;
    }
    __syncthreads();
    for (int i = tid; i < nt * V; i += 256) {
      const int tk = i / V, e = i - tk * V;
      float acc = dsk * xs[tk * V + e];
      for (int p = 0; p < NP; ++p) acc += ys[(tk * NP + p) * V + e];
      a.y[(size_t)(c0 + tk) * inner + h * a.V + v0 + e] = acc;
    }
  }
  if (active) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (n0 + r < N) sp[(size_t)(n0 + r) * a.V + v] = S[r];
  }
}

// The same recurrence with FOUR neighbouring state columns per thread (V a multiple of 4 with
// V / 4 a power of two up to 64): thread (cg, part) owns columns 4 cg .. 4 cg + 3 of the R rows
// part R .. part R + R - 1 (NP = 1024 / V parts).  A staged B or C value now serves four
// columns, so a token costs a quarter of the LDS reads (the one-column form is bound by them),
// and the state moves in 16-byte pieces.  The parts of a wave add their shares of S^T C by lane
// exchange, the four waves' sums meet in LDS.  PRE: prompt chunks, the next 16 tokens are
// fetched into registers while the current 16 are computed.
template <typename TY, int R, bool PRE>
__global__ __launch_bounds__(256) void selective_scan4_kernel(const ScanArgs a, const int TK) {
  extern __shared__ __align__(16) float lds[];
  const int V = a.V, N = a.N, V4 = V >> 2, N4 = N >> 2, NP = 256 / V4;
  float* xs = lds;                              // [TK][V]
  float* bs = xs + up4(TK * V);                 // [TK][N]
  float* cs = bs + up4(TK * N);                 // [TK][N]
  float* dts = cs + up4(TK * N);                // [TK] step, [TK] decay
  float* ys = dts + up4(2 * TK);                // [TK][4][V]
  const int b = blockIdx.x, h = blockIdx.y;
  const int r0 = a.q_start ? a.q_start[b] : b;
  const int r1 = a.q_start ? a.q_start[b + 1] : b + 1;
  if (r1 <= r0) return;
  const int slot = a.seq_slot[r0];
  if (slot < 0) return;
  const int g = h / (a.H / a.G);
  const int inner = a.H * V, C = inner + 2 * a.G * N;
  const int tid = threadIdx.x, wave = tid >> 6;
  const int cg = tid % V4, part = tid / V4;
  const int n0 = part * R;
  const bool active = n0 < N;
  float* sp = a.state + ((size_t)slot * a.H + h) * N * V + 4 * cg;
  float4 S[R];
  const bool carry = a.positions[r0] > 0;
#pragma unroll
  for (int r = 0; r < R; ++r)
    S[r] = (carry && active && n0 + r < N) ? *(const float4*)(sp + (size_t)(n0 + r) * V)
                                           : make_float4(0.f, 0.f, 0.f, 0.f);
  const float ea = expf(a.a_log[h]), dsk = a.d_skip[h], dtb = a.dt_bias[h];
  const TY* proj = (const TY*)a.proj;
  float4 px[PRE ? 4 : 1], pb[PRE ? 4 : 1], pc[PRE ? 4 : 1];
  float pdt = 0.f;
  auto prefetch = [&](int c0) {
    const int nt = min(TK, r1 - c0);
#pragma unroll
    for (int u = 0; u < (PRE ? 4 : 1); ++u) {
      const int i = tid + 256 * u;
      if (i < nt * V4) {
        const int tk = i / V4, e = i - tk * V4;
        px[u] = *(const float4*)(a.xbc + (size_t)(c0 + tk) * C + h * V + 4 * e);
      }
      if (i < nt * N4) {
        const int tk = i / N4, e = i - tk * N4;
        const float* row = a.xbc + (size_t)(c0 + tk) * C + inner + g * N + 4 * e;
        pb[u] = *(const float4*)row;
        pc[u] = *(const float4*)(row + a.G * N);
      }
    }
    if (tid < nt) pdt = ldf(proj + (size_t)(c0 + tid) * a.proj_stride + a.dt_off + h);
  };
  prefetch(r0);
  for (int c0 = r0; c0 < r1; c0 += TK) {
    const int nt = min(TK, r1 - c0);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < (PRE ? 4 : 1); ++u) {
      const int i = tid + 256 * u;
      if (i < nt * V4) *(float4*)(xs + 4 * i) = px[u];
      if (i < nt * N4) {
        *(float4*)(bs + 4 * i) = pb[u];
        *(float4*)(cs + 4 * i) = pc[u];
      }
    }
    if (tid < nt) {
      const float z = pdt + dtb;
      const float dt = z > 20.f ? z : log1pf(expf(z));
      dts[tid] = dt;
      dts[TK + tid] = expf(-ea * dt);
    }
    __syncthreads();
    if (PRE && c0 + TK < r1) prefetch(c0 + TK);
    for (int tk = 0; tk < nt; ++tk) {
      const float dt = dts[tk], dec = dts[TK + tk];
      const float4 x4 = *(const float4*)(xs + tk * V + 4 * cg);
      const float4 dx = make_float4(dt * x4.x, dt * x4.y, dt * x4.z, dt * x4.w);
      const float* bt = bs + tk * N + n0;
      const float* ct = cs + tk * N + n0;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      if (active) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          if (n0 + r < N) {
            const float4 b4 = *(const float4*)(bt + r), c4 = *(const float4*)(ct + r);
            const float bb[4] = {b4.x, b4.y, b4.z, b4.w}, cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              S[r + q].x = dec * S[r + q].x + dx.x * bb[q];
              S[r + q].y = dec * S[r + q].y + dx.y * bb[q];
              S[r + q].z = dec * S[r + q].z + dx.z * bb[q];
              S[r + q].w = dec * S[r + q].w + dx.w * bb[q];
              acc.x += S[r + q].x * cc[q];
              acc.y += S[r + q].y * cc[q];
              acc.z += S[r + q].z * cc[q];
              acc.w += S[r + q].w * cc[q];
            }
          }
        }
      }
      // the parts of this wave (lanes V4 apart)
      for (int o = V4; o < 64; o <<= 1) {
        acc.x += __shfl_xor(acc.x, o, 64);
        acc.y += __shfl_xor(acc.y, o, 64);
        acc.z += __shfl_xor(acc.z, o, 64);
        acc.w += __shfl_xor(acc.w, o, 64);
      }
      if ((tid & 63) < V4 || V4 >= 64) *(float4*)(ys + (tk * 4 + wave) * V + 4 * cg) = acc;
    }
    __syncthreads();
    // V4 >= 64: a wave holds one part of 64 column groups, its sums cover columns of its own
    for (int i = tid; i < nt * V; i += 256) {
      const int tk = i / V, e = i - tk * V;
      float acc = dsk * xs[tk * V + e];
#pragma unroll
      for (int w = 0; w < 4; ++w) acc += ys[(tk * 4 + w) * V + e];
      a.y[(size_t)(c0 + tk) * inner + h * V + e] = acc;
    }
  }
  if (active) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (n0 + r < N) *(float4*)(sp + (size_t)(n0 + r) * V) = S[r];
  }
}

}  // namespace

// ================================================================== launchers
void launch_hyper_step(void* out, bool out_f32, int out_stride, float* xs, const float* fresh,
                       const void* ya, bool ya_f32, int ya_stride, const void* yb, bool yb_f32,
                       int yb_stride, const float* bias, const float* mix, const float* w_out,
                       const float* w_in, const float* norm_w, int rows, int S, int d, float eps,
                       hipStream_t s) {
  if (rows <= 0) return;
  HyperArgs a{xs, fresh, ya, yb, bias, mix, w_out, w_in, norm_w, ya_stride, yb_stride,
              ya_f32 ? 1 : 0, yb_f32 ? 1 : 0, S, d, eps};
  const size_t lds = (size_t)(d + S * S + 2 * S + 16) * sizeof(float);
  auto al = [](const void* p, int bytes) { return p == nullptr || ((uintptr_t)p % bytes) == 0; };
  const bool vec = d % 4 == 0 && out_stride % 4 == 0 && ya_stride % 4 == 0 && yb_stride % 4 == 0 &&
                   al(out, 16) && al(xs, 16) && al(fresh, 16) && al(ya, 16) && al(yb, 16);
  if (out_f32) {
    if (vec) hyper_step_kernel<float, 4><<<rows, 256, lds, s>>>((float*)out, out_stride, a);
    else hyper_step_kernel<float, 1><<<rows, 256, lds, s>>>((float*)out, out_stride, a);
  } else {
    if (vec) hyper_step_kernel<bf16, 4><<<rows, 256, lds, s>>>((bf16*)out, out_stride, a);
    else hyper_step_kernel<bf16, 1><<<rows, 256, lds, s>>>((bf16*)out, out_stride, a);
  }
}

void launch_softcap(void* x, bool f32, size_t n, float cap, hipStream_t s) {
  if (n == 0) return;
  const int grid = (int)min((size_t)4096, (n + 255) / 256);
  if (f32) softcap_kernel<float><<<grid, 256, 0, s>>>((float*)x, n, cap, 1.0f / cap);
  else softcap_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)x, n, cap, 1.0f / cap);
}

void launch_gate_group_norm(void* out, int out_stride, const float* y, const void* gate,
                            int gate_stride, const float* w, bool f32, int rows, int n,
                            int groups, float eps, hipStream_t s) {
  if (rows <= 0) return;
  const dim3 grid(rows, groups);
  if (f32)
    gate_group_norm_kernel<float><<<grid, 256, 0, s>>>((float*)out, out_stride, y,
                                                       (const float*)gate, gate_stride, w, n,
                                                       groups, eps);
  else
    gate_group_norm_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out, out_stride, y,
                                                      (const bf16*)gate, gate_stride, w, n, groups,
                                                      eps);
}

void launch_route_sigmoid(int32_t* ids, float* w, const void* h, int h_stride, bool f32,
                          const float* router, int rows, int d, int E, int top, int groups,
                          int keep, int group_top, hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)(((d + 3) & ~3) + 2 * E + groups) * sizeof(float);
  if (f32)
    route_sigmoid_kernel<float><<<rows, 256, lds, s>>>(ids, w, (const float*)h, h_stride, router,
                                                       d, E, top, groups, keep, group_top);
  else
    route_sigmoid_kernel<bf16><<<rows, 256, lds, s>>>(ids, w, (const bf16*)h, h_stride, router, d,
                                                      E, top, groups, keep, group_top);
}

void launch_conv_silu(float* out, const void* proj, int proj_stride, int off, bool f32,
                      void* state, const float* w, const float* b, const int32_t* seq_slot,
                      const int64_t* positions, const int32_t* q_start, int T, int B, int C,
                      int taps, hipStream_t s) {
  if (T <= 0) return;
  ConvArgs a{out, proj, state, w, b, seq_slot, positions, q_start, proj_stride, off, C, taps, T, B};
  const dim3 g1(T, (C + 255) / 256), g2(B, (C + 255) / 256), g4((T + (q_start ? kConvRows : 1) - 1) / (q_start ? kConvRows : 1), (C / 4 + 255) / 256);
  const int RB = q_start ? kConvRows : 1;
  const int es = f32 ? 4 : 2;
  const bool vec = C % 4 == 0 && off % 4 == 0 && proj_stride % 4 == 0 &&
                   (uintptr_t)proj % (4 * es) == 0 && (uintptr_t)state % (4 * es) == 0 &&
                   (uintptr_t)out % 16 == 0 && (uintptr_t)b % 16 == 0;
  if (vec) {
    if (f32) conv_silu_vec_kernel<float><<<g4, 256, 0, s>>>(a, RB);
    else conv_silu_vec_kernel<bf16><<<g4, 256, 0, s>>>(a, RB);
  } else if (f32) conv_silu_kernel<float><<<g1, 256, 0, s>>>(a);
  else conv_silu_kernel<bf16><<<g1, 256, 0, s>>>(a);
  if (taps > 1) {
    if (f32) conv_state_kernel<float><<<g2, 256, 0, s>>>(a);
    else conv_state_kernel<bf16><<<g2, 256, 0, s>>>(a);
  }
}

int selective_scan_rows(int V, int N) {
  const int NP = 256 / V;
  return (N + NP - 1) / NP;
}

// four columns per thread: V / 4 a power of two up to 32 (a wave holds whole parts), N in fours
// and at most 256, at most 32 rows per thread
static bool scan_four(int V, int N, int* rows) {
  const int V4 = V / 4;
  if (!(V % 4 == 0 && V4 >= 1 && V4 <= 32 && (V4 & (V4 - 1)) == 0 && N % 4 == 0 && N <= 256))
    return false;
  const int NP = 256 / V4;
  const int R = ((N + NP - 1) / NP + 3) & ~3;
  if (rows) *rows = R;
  return R <= 32;
}

bool selective_scan_supported(int V, int N) {
  return V >= 1 && V <= 256 && N >= 1 && (scan_four(V, N, nullptr) || selective_scan_rows(V, N) <= 64);
}

void launch_selective_scan(float* y, const float* xbc, const void* proj, int proj_stride,
                           int dt_off, bool f32, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, const int32_t* seq_slot,
                           const int64_t* positions, const int32_t* q_start, int T, int B, int H,
                           int V, int N, int G, hipStream_t s) {
  if (T <= 0) return;
  ScanArgs a{y, xbc, proj, dt_bias, a_log, d_skip, state, seq_slot, positions, q_start,
             proj_stride, dt_off, H, V, N, G, T, B, V};
  int TK = q_start ? kScanTokens : 1;      // halved below until the staging fits 64 KB of LDS
  const dim3 grid(B, H);
  int R4 = 0;
  if (scan_four(V, N, &R4)) {
    const int R = R4;
    auto need = [&](int tk) {
      return (size_t)(up4(tk * V) + 2 * up4(tk * N) + up4(2 * tk) + tk * 4 * V) * sizeof(float);
    };
    while (TK > 1 && need(TK) > 65536) TK >>= 1;
    const size_t lds = need(TK);
#define AKAP_SCAN4(TY, RR)                                                          \
  do {                                                                              \
    if (q_start) selective_scan4_kernel<TY, RR, true><<<grid, 256, lds, s>>>(a, TK); \
    else selective_scan4_kernel<TY, RR, false><<<grid, 256, lds, s>>>(a, TK);       \
  } while (0)
#define AKAP_SCAN4_R(TY)                \
  do {                                  \
    if (R <= 4) AKAP_SCAN4(TY, 4);        \
    else if (R <= 8) AKAP_SCAN4(TY, 8);   \
    else if (R <= 16) AKAP_SCAN4(TY, 16); \
    else AKAP_SCAN4(TY, 32);              \
  } while (0)
    if (f32) AKAP_SCAN4_R(float);
    else AKAP_SCAN4_R(bf16);
    return;
#undef AKAP_SCAN4_R
#undef AKAP_SCAN4
  }
  const int NP = 256 / V, R = selective_scan_rows(V, N);
  auto need = [&](int tk) {
    return (size_t)(up4(tk * V) + 2 * up4(tk * N) + up4(2 * tk) + tk * NP * V) * sizeof(float);
  };
  while (TK > 1 && need(TK) > 65536) TK >>= 1;
  const size_t lds = need(TK);
#define AKAP_SCAN(TY, RR) selective_scan_kernel<TY, RR><<<grid, 256, lds, s>>>(a, TK)
#define AKAP_SCAN_R(TY)                  \
  do {                                   \
    if (R <= 4) AKAP_SCAN(TY, 4);        \
    else if (R <= 8) AKAP_SCAN(TY, 8);   \
    else if (R <= 16) AKAP_SCAN(TY, 16); \
    else if (R <= 32) AKAP_SCAN(TY, 32); \
    else AKAP_SCAN(TY, 64);              \
  } while (0)
  if (f32) AKAP_SCAN_R(float);
  else AKAP_SCAN_R(bf16);
#undef AKAP_SCAN_R
#undef AKAP_SCAN
}

}  // namespace akap_stream
