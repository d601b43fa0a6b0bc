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
  extern __shared__ float lds[];   // [d] row, [E] scores, [E] choice values, [groups] group scores
  float* hs = lds;
  float* sc = lds + d;
  float* ch = sc + E;
  float* gs = ch + E;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + (size_t)t * h_stride;
  for (int c = threadIdx.x; c < d; c += 256) hs[c] = ldf(hr + c);
  __syncthreads();
  for (int e = wave; e < E; e += 4) {
    const float* r = router + (size_t)e * d;
    float acc = 0.f;
    for (int c = lane; c < d; c += 64) acc += hs[c] * r[c];
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
};

constexpr int kScanTokens = 16;

__host__ __device__ __forceinline__ int up4(int n) { return (n + 3) & ~3; }

// One workgroup per (sequence, head).  Thread (v, part) owns column v of the R consecutive
// state rows part R .. part R + R - 1 (NP = 256 / V parts), in registers over all rows of the
// step.  Tokens are staged TK at a time (x, B, C, step size and decay; TK = 16 for prompt
// chunks, 1 for steps of single rows); per token a thread updates its rows and adds its share
// of S^T C, reading B and C from LDS four rows at a time (all lanes of a wave read the same
// addresses); the parts' shares meet in LDS after the staged tokens.
template <typename TY, int R>
__global__ __launch_bounds__(256) void selective_scan_kernel(const ScanArgs a, const int TK) {
  extern __shared__ __align__(16) float lds[];
  const int V = a.V, N = a.N, NP = 256 / V;
  float* xs = lds;                              // [TK][V]
  float* bs = xs + up4(TK * V);                 // [TK][N]
  float* cs = bs + up4(TK * N);                 // [TK][N]
  float* dts = cs + up4(TK * N);                // [TK] step, [TK] decay
  float* ys = dts + up4(2 * TK);                // [TK][NP][V]
  const int b = blockIdx.x, h = blockIdx.y;
  const int r0 = a.q_start ? a.q_start[b] : b;
  const int r1 = a.q_start ? a.q_start[b + 1] : b + 1;
  if (r1 <= r0) return;
  const int slot = a.seq_slot[r0];
  if (slot < 0) return;
  const int g = h / (a.H / a.G);
  const int inner = a.H * V, C = inner + 2 * a.G * N;
  const int tid = threadIdx.x;
  const int v = tid % V, part = tid / V;
  const int n0 = part * R;
  const bool active = part < NP && n0 < N;
  const bool vec = (N & 3) == 0 && (R & 3) == 0;
  float* sp = a.state + ((size_t)slot * a.H + h) * N * V;
  float S[R];
  const bool carry = a.positions[r0] > 0;
#pragma unroll
  for (int r = 0; r < R; ++r)
    S[r] = (carry && active && n0 + r < N) ? sp[(size_t)(n0 + r) * V + v] : 0.f;
  const float ea = expf(a.a_log[h]), dsk = a.d_skip[h], dtb = a.dt_bias[h];
  const TY* proj = (const TY*)a.proj;
  for (int c0 = r0; c0 < r1; c0 += TK) {
    const int nt = min(TK, r1 - c0);
    __syncthreads();
    for (int i = tid; i < nt * V; i += 256) {
      const int tk = i / V, e = i - tk * V;
      xs[tk * V + e] = a.xbc[(size_t)(c0 + tk) * C + h * V + e];
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
    if (active) {
      for (int tk = 0; tk < nt; ++tk) {
        const float dt = dts[tk], dec = dts[TK + tk];
        const float dx = dt * xs[tk * V + v];
        const float* bt = bs + tk * N + n0;
        const float* ct = cs + tk * N + n0;
        float acc = 0.f;
        if (vec) {
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            if (n0 + r < N) {
              const float4 b4 = *(const float4*)(bt + r), c4 = *(const float4*)(ct + r);
              S[r] = dec * S[r] + dx * b4.x;
              S[r + 1] = dec * S[r + 1] + dx * b4.y;
              S[r + 2] = dec * S[r + 2] + dx * b4.z;
              S[r + 3] = dec * S[r + 3] + dx * b4.w;
              acc += S[r] * c4.x + S[r + 1] * c4.y + S[r + 2] * c4.z + S[r + 3] * c4.w;
            }
          }
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
      a.y[(size_t)(c0 + tk) * inner + h * V + e] = acc;
    }
  }
  if (active) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (n0 + r < N) sp[(size_t)(n0 + r) * V + v] = S[r];
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
  const size_t lds = (size_t)(d + 2 * E + groups) * sizeof(float);
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
  const dim3 g1(T, (C + 255) / 256), g2(B, (C + 255) / 256);
  if (f32) conv_silu_kernel<float><<<g1, 256, 0, s>>>(a);
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

void launch_selective_scan(float* y, const float* xbc, const void* proj, int proj_stride,
                           int dt_off, bool f32, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, const int32_t* seq_slot,
                           const int64_t* positions, const int32_t* q_start, int T, int B, int H,
                           int V, int N, int G, hipStream_t s) {
  if (T <= 0) return;
  ScanArgs a{y, xbc, proj, dt_bias, a_log, d_skip, state, seq_slot, positions, q_start,
             proj_stride, dt_off, H, V, N, G, T, B};
  const int NP = 256 / V, R = selective_scan_rows(V, N);
  const int TK = q_start ? kScanTokens : 1;
  const size_t lds = (size_t)(up4(TK * V) + 2 * up4(TK * N) + up4(2 * TK) + TK * NP * V) *
                     sizeof(float);
  const dim3 grid(B, H);
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
