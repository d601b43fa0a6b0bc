// Kernels of layers with a norm before and after each sublayer, decayed linear attention
// ("retention") with a recurrent state, softmax attention whose heads mix their weights, and
// logit-top-k routed gated experts.
//
// Sums of squares, norm scales, angles and rotations, decays, the recurrent state, attention
// scores / softmax / head mixing / gates, router logits and the residual sum are fp32 whatever
// the storage type; every size is a run-time argument.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::block_sum;
using akap::wave_max;
using akap::wave_sum;

namespace {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + __expf(-z)); }

// 4 consecutive elements (16- resp. 8-byte aligned) as floats
__device__ __forceinline__ void ld4(const float* p, float (&v)[4]) {
  const float4 a = *(const float4*)p;
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void ld4(const bf16* p, float (&v)[4]) {
  const akap::bf16x4 a = *(const akap::bf16x4*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = (float)a[i];
}

// 8 consecutive elements (32- resp. 16-byte aligned) as floats
__device__ __forceinline__ void ld8(const float* p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void ld8(const bf16* p, float (&v)[8]) {
  const akap::bf16x8 a = *(const akap::bf16x8*)p;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
}

// ------------------------------------------------------------------ post-norm + residual + norm
// one workgroup per row; a thread keeps to its own columns in every phase, so the two LDS rows
// need no barrier beyond those of the block sums
// 8 weights from column c: a vector of d entries (stride 1) or one number (stride 0)
__device__ __forceinline__ void ldw8(const float* w, int stride, int c, float (&v)[8]) {
  if (stride) {
    ld8(w + c, v);
  } else {
    const float f = w[0];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = f;
  }
}
__device__ __forceinline__ void st8(float* p, const float (&v)[8]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
  *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void st8(bf16* p, const float (&v)[8]) {
  akap::bf16x8 o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (bf16)v[i];
  *(akap::bf16x8*)p = o;
}

// VEC: 8 columns per thread and turn, 16-byte accesses (d, the row strides and the pointers are
// multiples of 8 elements resp. 16 bytes)
template <typename TY, typename TO, bool VEC>
__global__ __launch_bounds__(256) void post_norm_add_norm_kernel(
    TO* __restrict__ out, int out_stride, float* __restrict__ x, const TY* __restrict__ ya,
    int ya_stride, const TY* __restrict__ yb, int yb_stride, const float* __restrict__ wa, int was,
    const float* __restrict__ wb, int wbs, const float* __restrict__ post_w, int pws,
    const float* __restrict__ next_w, int nws, int d, float eps, int fresh) {
  extern __shared__ float lds[];
  __shared__ float scratch[16];
  float* ra = lds;
  float* rb = lds + d;
  const int row = blockIdx.x;
  const TY* a = ya + (size_t)row * ya_stride;
  const TY* b = yb ? yb + (size_t)row * yb_stride : nullptr;
  float* xr = x + (size_t)row * d;
  TO* o = out + (size_t)row * out_stride;
  const float inv_d = 1.0f / (float)d;
  constexpr int W = VEC ? 8 : 1;
  const int c0 = threadIdx.x * W, step = 256 * W;
  float ss = 0.f, sb = 0.f;
  for (int c = c0; c < d; c += step) {
    if (VEC) {
      float f[8];
      ld8(a + c, f);
      st8(ra + c, f);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += f[i] * f[i];
      if (b) {
        ld8(b + c, f);
        st8(rb + c, f);
#pragma unroll
        for (int i = 0; i < 8; ++i) sb += f[i] * f[i];
      }
    } else {
      const float f = ldf(a + c);
      ra[c] = f;
      ss += f * f;
      if (b) {
        const float g = ldf(b + c);
        rb[c] = g;
        sb += g * g;
      }
    }
  }
  ss = block_sum(ss, scratch);
  if (b) {
    sb = block_sum(sb, scratch);
    const float ia = 1.0f / sqrtf(ss * inv_d + eps), ib = 1.0f / sqrtf(sb * inv_d + eps);
    ss = 0.f;
    for (int c = c0; c < d; c += step) {
      if (VEC) {
        float fa[8], fb[8], ua[8], ub[8];
        ld8(ra + c, fa);
        ld8(rb + c, fb);
        ldw8(wa, was, c, ua);
        ldw8(wb, wbs, c, ub);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          fa[i] = 0.5f * (fa[i] * ia * ua[i] + fb[i] * ib * ub[i]);
          ss += fa[i] * fa[i];
        }
        st8(ra + c, fa);
      } else {
        const float m = 0.5f * (ra[c] * ia * wa[c * was] + rb[c] * ib * wb[c * wbs]);
        ra[c] = m;
        ss += m * m;
      }
    }
    ss = block_sum(ss, scratch);
  }
  const float im = 1.0f / sqrtf(ss * inv_d + eps);
  float sx = 0.f;
  for (int c = c0; c < d; c += step) {
    if (VEC) {
      float f[8], xv[8], pw[8];
      ld8(ra + c, f);
      ldw8(post_w, pws, c, pw);
      if (fresh) {
#pragma unroll
        for (int i = 0; i < 8; ++i) xv[i] = 0.f;
      } else {
        ld8(xr + c, xv);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        f[i] = xv[i] + f[i] * im * pw[i];
        sx += f[i] * f[i];
      }
      st8(xr + c, f);
      st8(ra + c, f);
    } else {
      const float f = (fresh ? 0.f : xr[c]) + ra[c] * im * post_w[c * pws];
      xr[c] = f;
      ra[c] = f;
      sx += f * f;
    }
  }
  sx = block_sum(sx, scratch);
  const float ix = 1.0f / sqrtf(sx * inv_d + eps);
  for (int c = c0; c < d; c += step) {
    if (VEC) {
      float f[8], nw[8];
      ld8(ra + c, f);
      ldw8(next_w, nws, c, nw);
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = f[i] * ix * nw[i];
      st8(o + c, f);
    } else {
      stf(o + c, ra[c] * ix * next_w[c * nws]);
    }
  }
}

// ------------------------------------------------------------------ per-head norms + cache write
// one workgroup per token; a wave per head (query heads, then key heads, then value heads)
template <typename T>
__global__ __launch_bounds__(256) void head_norm_cache_kernel(HeadNormParams p) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* row = (const T*)p.proj + (size_t)t * p.proj_stride;
  const int64_t slot = p.slots[t];
  const bool cached = slot >= 0 && slot < p.num_slots;
  const int64_t blk = cached ? slot / p.BS : 0;
  const int off = cached ? (int)(slot % p.BS) : 0;
  for (int u = wave; u < p.H + 2 * p.G; u += 4) {
    const T* src;
    T* dst;
    int n, vstep = 1;
    bool norm;
    if (u < p.H) {
      src = row + p.q_off + u * p.D;
      dst = (T*)p.q_out + ((size_t)t * p.H + u) * p.D;
      n = p.D;
      norm = p.norm_qk;
    } else if (u < p.H + p.G) {
      if (!cached) continue;
      const int g = u - p.H;
      src = row + p.k_off + g * p.D;
      dst = (T*)p.k_cache + ((size_t)(blk * p.G + g) * p.BS + off) * p.D;
      n = p.D;
      norm = p.norm_qk;
    } else {
      if (!cached) continue;
      const int g = u - p.H - p.G;
      src = row + p.v_off + g * p.Dv;
      // values go in groups of 8 tokens, dimension-major inside a group: entry c of token
      // `off` sits at [off / 8][c][off % 8]
      dst = (T*)p.v_cache + (((size_t)(blk * p.G + g) * (p.BS >> 3) + (off >> 3)) * p.Dv) * 8 +
            (off & 7);
      n = p.Dv;
      norm = p.norm_v;
      vstep = 8;
    }
    float inv = 1.0f;
    if (norm) {
      float ss = 0.f;
      for (int c = lane; c < n; c += 64) {
        const float f = ldf(src + c);
        ss += f * f;
      }
      ss = wave_sum(ss);
      inv = 1.0f / sqrtf(ss / (float)n + p.eps);
    }
    for (int c = lane; c < n; c += 64) stf(dst + c * vstep, ldf(src + c) * inv);
  }
}

// ------------------------------------------------------------------ retention
// One workgroup per (sequence, head).  The state S[d][v] stays in registers over the sequence's
// rows of this step: a thread owns RET_VR neighbouring state columns v and, of their rows d,
// DREG / 4 groups of four (group j of lane part `part` covers d = 4 (j DP + part) ..+4, so that
// the DP lanes of a column read and write consecutive 16-byte pieces of the stored state and
// of the staged q / k rows).  Rows are staged TC at a time: q and k rotated (fp32) into LDS,
// then the recurrence runs over the TC tokens without a barrier (every staged k / q value
// serves RET_VR columns; the DP lanes that share columns add their partial outputs by lane
// exchange), then the outputs of the TC tokens are normed and gated, a wave per token.
constexpr int RET_TC = 16;   // tokens staged at a time (8 when the rows of 16 exceed 64 KB)
constexpr int RET_VR = 4;    // state columns per thread

// Long prompt chunks run in three launches over segments of p.SEG rows, so that a sequence's
// segments proceed side by side: MODE 1 leaves each segment's own state (started from zeros, no
// outputs) in seg_buf, retention_scan_kernel turns these into the state BEFORE each segment (and
// the sequence's final state in its slot), MODE 3 produces the outputs of each segment from
// that.  MODE 0 is the direct form: a workgroup walks all rows of its sequence.
// Segment buffers are indexed compactly: sequence b owns entries from q_start[b] / SEG + b.
__device__ __forceinline__ int seg_base(const int32_t* q_start, int b, int SEG) {
  return q_start[b] / SEG + b;
}

template <typename T, int DREG, int MODE>
__global__ __launch_bounds__(DREG == 16 ? 256 : 512) void retention_kernel(RetentionParams p) {
  extern __shared__ float lds[];
  constexpr int NJ = DREG / 4;
  const int DP = p.DP;                    // lanes per column group (power of two, <= 64)
  const int DPD = DP * DREG;              // D rounded up: the staged rows end in zeros
  const int VP = (p.V + 3) & ~3;
  const int TC = p.TC;
  float* qs = lds;                        // [TC][DPD]
  float* ks = qs + TC * DPD;
  float* vs = ks + TC * DPD;              // [TC][VP]
  float* os = vs + TC * VP;               // [TC][VP]
  int b = blockIdx.x;
  const int h = blockIdx.y;
  int r0, r1;
  if (MODE == 0) {
    r0 = p.q_start ? p.q_start[b] : b;
    r1 = p.q_start ? p.q_start[b + 1] : b + 1;
  } else {
    // blockIdx.x is a segment entry: its sequence is the last one whose base is not above it
    int lo = 0, hi = p.num_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (seg_base(p.q_start, mid, p.SEG) <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
    }
    b = lo;
    const int sg = blockIdx.x - seg_base(p.q_start, b, p.SEG);
    r0 = p.q_start[b] + sg * p.SEG;
    r1 = min(r0 + p.SEG, p.q_start[b + 1]);
  }
  if (r1 <= r0) return;
  const int slot = p.seq_slot[r0];
  if (slot < 0 || slot >= p.num_slots) return;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int v0 = (tid / DP) * RET_VR, part = tid % DP;
  float* sbase = MODE == 0 ? p.state + ((size_t)slot * p.H + h) * p.V * p.D
                           : p.seg_buf + ((size_t)blockIdx.x * p.H + h) * p.V * p.D;
  const bool vec = (p.D & 3) == 0;        // 16-byte pieces of the stored state
  float S[RET_VR][DREG];
  const bool fresh = MODE == 1 || (MODE == 0 && p.positions[r0] == 0);
#pragma unroll
  for (int r = 0; r < RET_VR; ++r) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int d = 4 * (j * DP + part);
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      if (!fresh && v0 + r < p.V) {
        const float* sp = sbase + (size_t)(v0 + r) * p.D + d;
        if (vec) {
          if (d < p.D) t = *(const float4*)sp;
        } else {
          if (d < p.D) t.x = sp[0];
          if (d + 1 < p.D) t.y = sp[1];
          if (d + 2 < p.D) t.z = sp[2];
          if (d + 3 < p.D) t.w = sp[3];
        }
      }
      S[r][4 * j] = t.x; S[r][4 * j + 1] = t.y; S[r][4 * j + 2] = t.z; S[r][4 * j + 3] = t.w;
    }
  }
  const float decay = exp2f(p.log2_decay[h]);
  const float kscale = 1.0f / sqrtf((float)p.D);
  const int half = p.rot_dims / 2;
  // vector staging: every slice starts and every row strides at a multiple of 4 elements
  const bool vstage = ((p.D | p.V | half | p.proj_stride | p.q_off | p.k_off | p.v_off) & 3) == 0 &&
                      ((uintptr_t)p.proj & 15) == 0;
  // lanes per token of the output phase: all TC tokens of a round at once
  int LPT = 64;
  while (LPT * TC > nt && LPT > 1) LPT >>= 1;
  for (int c0 = r0; c0 < r1; c0 += TC) {
    const int n = min(TC, r1 - c0);
    // stage: q, k (rotated, k scaled) and v of this head
    if (vstage) {
      // four dimensions per item: few rounds of independent vector loads
      const int Q4 = DPD >> 2;
      for (int e = tid; e < n * Q4; e += nt) {
        const int tk = e / Q4, d = (e - tk * Q4) << 2;
        const T* row = (const T*)p.proj + (size_t)(c0 + tk) * p.proj_stride;
        const T* q = row + p.q_off + h * p.D;
        const T* k = row + p.k_off + h * p.D;
        float q4[4] = {0.f, 0.f, 0.f, 0.f}, k4[4] = {0.f, 0.f, 0.f, 0.f};
        if (d < p.D) {
          ld4(q + d, q4);
          ld4(k + d, k4);
          if (d < p.rot_dims) {
            const int64_t pos = p.positions[c0 + tk];
            const float* cs = p.cos_sin + (size_t)pos * p.rot_dims;
            const bool low = d < half;
            const int i = low ? d : d - half, d2 = low ? d + half : d - half;
            float c4[4], s4[4], q2[4], k2[4];
            ld4(cs + i, c4);
            ld4(cs + half + i, s4);
            ld4(q + d2, q2);
            ld4(k + d2, k2);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const float sn = low ? -s4[u] : s4[u];
              q4[u] = q4[u] * c4[u] + q2[u] * sn;
              k4[u] = k4[u] * c4[u] + k2[u] * sn;
            }
          }
        }
        *(float4*)(qs + tk * DPD + d) = make_float4(q4[0], q4[1], q4[2], q4[3]);
        *(float4*)(ks + tk * DPD + d) =
            make_float4(k4[0] * kscale, k4[1] * kscale, k4[2] * kscale, k4[3] * kscale);
      }
      const int V4 = VP >> 2;
      for (int e = tid; e < n * V4; e += nt) {
        const int tk = e / V4, c = (e - tk * V4) << 2;
        float v4[4];
        ld4((const T*)p.proj + (size_t)(c0 + tk) * p.proj_stride + p.v_off + h * p.V + c, v4);
        *(float4*)(vs + tk * VP + c) = make_float4(v4[0], v4[1], v4[2], v4[3]);
      }
    } else {
    for (int e = tid; e < n * DPD; e += nt) {
      const int tk = e / DPD, d = e % DPD;
      const T* row = (const T*)p.proj + (size_t)(c0 + tk) * p.proj_stride;
      const T* q = row + p.q_off + h * p.D;
      const T* k = row + p.k_off + h * p.D;
      float qv = 0.f, kv = 0.f;
      if (d < p.D) {
        qv = ldf(q + d);
        kv = ldf(k + d);
      }
      if (d < p.rot_dims) {
        const int64_t pos = p.positions[c0 + tk];
        const float* cs = p.cos_sin + (size_t)pos * p.rot_dims;
        const int i = d < half ? d : d - half;
        const float c = cs[i], sn = cs[half + i];
        if (d < half) {
          const float q2 = ldf(q + d + half), k2 = ldf(k + d + half);
          qv = qv * c - q2 * sn;
          kv = kv * c - k2 * sn;
        } else {
          const float q1 = ldf(q + d - half), k1 = ldf(k + d - half);
          qv = qv * c + q1 * sn;
          kv = kv * c + k1 * sn;
        }
      }
      qs[e] = qv;
      ks[e] = kv * kscale;
    }
    for (int e = tid; e < n * VP; e += nt) {
      const int tk = e / VP, c = e % VP;
      vs[e] = c < p.V ? ldf((const T*)p.proj + (size_t)(c0 + tk) * p.proj_stride + p.v_off +
                            h * p.V + c)
                      : 0.f;
    }
    }
    __syncthreads();
    // the recurrence
    for (int tk = 0; tk < n; ++tk) {
      float4 vv = make_float4(0.f, 0.f, 0.f, 0.f);
      if (v0 < p.V) vv = *(const float4*)(vs + tk * VP + v0);
      const float vr[RET_VR] = {vv.x, vv.y, vv.z, vv.w};
      const float* kq = ks + tk * DPD + 4 * part;
      const float* qq = qs + tk * DPD + 4 * part;
      float acc[RET_VR] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float4 k4 = *(const float4*)(kq + 4 * j * DP);
        const float4 q4 = *(const float4*)(qq + 4 * j * DP);
#pragma unroll
        for (int r = 0; r < RET_VR; ++r) {
          S[r][4 * j] = fmaf(decay, S[r][4 * j], k4.x * vr[r]);
          S[r][4 * j + 1] = fmaf(decay, S[r][4 * j + 1], k4.y * vr[r]);
          S[r][4 * j + 2] = fmaf(decay, S[r][4 * j + 2], k4.z * vr[r]);
          S[r][4 * j + 3] = fmaf(decay, S[r][4 * j + 3], k4.w * vr[r]);
          if (MODE != 1) {
            acc[r] = fmaf(S[r][4 * j], q4.x, acc[r]);
            acc[r] = fmaf(S[r][4 * j + 1], q4.y, acc[r]);
            acc[r] = fmaf(S[r][4 * j + 2], q4.z, acc[r]);
            acc[r] = fmaf(S[r][4 * j + 3], q4.w, acc[r]);
          }
        }
      }
      if (MODE != 1) {
        for (int o = DP >> 1; o > 0; o >>= 1) {
#pragma unroll
          for (int r = 0; r < RET_VR; ++r) acc[r] += __shfl_xor(acc[r], o, 64);
        }
        if (v0 < p.V && part == 0)
          *(float4*)(os + tk * VP + v0) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      }
    }
    __syncthreads();
    if (MODE == 1) continue;
    // output norm over the head's V entries and the silu gate: LPT lanes per token
    for (int tk = tid / LPT; tk < n; tk += nt / LPT) {
      const int ln = tid % LPT;
      float ss = 0.f;
      for (int c = ln; c < p.V; c += LPT) {
        const float f = os[tk * VP + c];
        ss += f * f;
      }
      for (int o = LPT >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      const float inv = 1.0f / sqrtf(ss / (float)p.V + p.eps);
      const T* g = (const T*)p.proj + (size_t)(c0 + tk) * p.proj_stride + p.g_off + h * p.V;
      T* o = (T*)p.out + (size_t)(c0 + tk) * p.out_stride + h * p.V;
      for (int c = ln; c < p.V; c += LPT) {
        const float z = ldf(g + c);
        stf(o + c, os[tk * VP + c] * inv * z * sigmoidf(z));
      }
    }
    __syncthreads();
  }
  if (MODE != 3) {
#pragma unroll
    for (int r = 0; r < RET_VR; ++r) {
      if (v0 + r >= p.V) continue;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = 4 * (j * DP + part);
        float* sp = sbase + (size_t)(v0 + r) * p.D + d;
        if (vec) {
          if (d < p.D)
            *(float4*)sp = make_float4(S[r][4 * j], S[r][4 * j + 1], S[r][4 * j + 2], S[r][4 * j + 3]);
        } else {
          if (d < p.D) sp[0] = S[r][4 * j];
          if (d + 1 < p.D) sp[1] = S[r][4 * j + 1];
          if (d + 2 < p.D) sp[2] = S[r][4 * j + 2];
          if (d + 3 < p.D) sp[3] = S[r][4 * j + 3];
        }
      }
    }
  }
}

// state before each segment from the segments' own states, per (sequence, head); the state
// after the last segment goes to the sequence's slot
__global__ __launch_bounds__(256) void retention_scan_kernel(RetentionParams p) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int r0 = p.q_start[b], r1 = p.q_start[b + 1];
  if (r1 <= r0) return;
  const int slot = p.seq_slot[r0];
  if (slot < 0 || slot >= p.num_slots) return;
  const int n = r1 - r0, nseg = (n + p.SEG - 1) / p.SEG;
  const bool fresh = p.positions[r0] == 0;
  const float l2 = p.log2_decay[h];
  const size_t hs = (size_t)p.V * p.D;
  float* st = p.state + ((size_t)slot * p.H + h) * hs;
  float* sb = p.seg_buf + ((size_t)seg_base(p.q_start, b, p.SEG) * p.H + h) * hs;
  for (int e = threadIdx.x; e < p.V * p.D; e += 256) {
    float prev = fresh ? 0.f : st[e];
    for (int sg = 0; sg < nseg; ++sg) {
      float* cell = sb + (size_t)sg * p.H * hs + e;
      const float own = *cell;
      *cell = prev;
      prev = fmaf(exp2f(l2 * (float)min(p.SEG, n - sg * p.SEG)), prev, own);
    }
    st[e] = prev;
  }
}

// ------------------------------------------------------------------ head-mixed attention
// One workgroup per (query row, key partition); thread (c, dv) owns entry dv of value head c and
// keeps, for EVERY query head g, the unnormalised sum over the keys of exp(s_g - m_g) v_c[dv].
// Keys go by pieces of 64: the waves score the piece (a lane per key, a wave per key head and
// its query heads), publish the weights through LDS, then all threads accumulate.
constexpr int TA_PIECE = 64;

__device__ __forceinline__ int find_seq(const int32_t* q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// the finish shared by the one-partition kernel and the merge: normalise, mix the heads, gate
template <typename T, int HMAX>
__device__ __forceinline__ void talk_finish(const TalkParams& p, int t, int c, int dv,
                                            float (&acc)[HMAX], const float* inv_l) {
  const int rep = p.H / p.G;
#pragma unroll
  for (int g = 0; g < HMAX; ++g)
    if (g < p.H) acc[g] *= inv_l[g];
  for (int i = 0; i < rep; ++i) {
    const int h = c * rep + i;
    float o;
    if (p.talk) {
      o = 0.f;
      const float* tr = p.talk + (size_t)h * p.H;
#pragma unroll
      for (int g = 0; g < HMAX; ++g)
        if (g < p.H) o = fmaf(tr[g], acc[g], o);
    } else {
      o = 0.f;
#pragma unroll
      for (int g = 0; g < HMAX; ++g)
        if (g == h) o = acc[g];
    }
    const int col = h * p.Dv + dv;
    if (p.gate) o *= sigmoidf(ldf((const T*)p.gate + (size_t)t * p.gate_stride + col));
    stf((T*)p.out + (size_t)t * p.out_stride + col, o);
  }
}

template <typename T, int HMAX>
__global__ __launch_bounds__(1024) void talking_attention_kernel(TalkParams p) {
  extern __shared__ float lds[];
  float* qs = lds;                                 // [H][D]
  float* ps = qs + p.H * p.D;                      // [H][PIECE] weights of the piece
  float* alpha = ps + p.H * TA_PIECE;              // [H] rescale of the running sums
  float* ms = alpha + p.H;                         // [H] running max
  float* lsum = ms + p.H;                          // [H] running sum
  int* rowbase = (int*)(lsum + p.H);               // [PIECE] cache row of key j for head 0
  const int t = blockIdx.x, part = blockIdx.y;
  const int b = p.q_start ? find_seq(p.q_start, p.B, t) : t;
  if (p.seq_lens[b] <= 0) return;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int wave = tid >> 6, lane = tid & 63, nw = nt >> 6;
  const int nkeys = (int)p.positions[t] + 1;
  const int pieces = (nkeys + TA_PIECE - 1) / TA_PIECE;
  const int per = (pieces + p.num_parts - 1) / p.num_parts;
  const int lo = part * per * TA_PIECE;
  const int hi = min(nkeys, lo + per * TA_PIECE);
  const int rep = p.H / p.G;
  const int GV = p.G * p.Dv;
  const bool owner = tid < GV;
  const int c = owner ? tid / p.Dv : 0, dv = owner ? tid % p.Dv : 0;
  float acc[HMAX];
#pragma unroll
  for (int g = 0; g < HMAX; ++g) acc[g] = 0.f;
  for (int e = tid; e < p.H * p.D; e += nt) qs[e] = ldf((const T*)p.q + (size_t)t * p.H * p.D + e);
  for (int g = tid; g < p.H; g += nt) { ms[g] = -INFINITY; lsum[g] = 0.f; }
  __syncthreads();
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  for (int j0 = lo; j0 < hi; j0 += TA_PIECE) {
    const int j = j0 + lane;
    const bool live = j < hi;
    int base = 0;
    if (live) base = (bt[j / p.BS] * p.G) * p.BS + (j % p.BS);
    if (wave == 0) rowbase[lane] = base;
    // scores: wave w takes key heads w, w + nw, ...; lane = key
    for (int kc = wave; kc < p.G; kc += nw) {
      const T* kr = (const T*)p.k_cache + (size_t)(base + kc * p.BS) * p.D;
      for (int i0 = 0; i0 < rep; i0 += 4) {
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        const float* q0 = qs + (kc * rep + i0) * p.D;
        const int n = min(4, rep - i0);
        if (live && (p.D & 7) == 0) {
          for (int d = 0; d < p.D; d += 8) {
            float k8[8];
            ld8(kr + d, k8);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              s0 = fmaf(q0[d + e], k8[e], s0);
              if (n > 1) s1 = fmaf(q0[p.D + d + e], k8[e], s1);
              if (n > 2) s2 = fmaf(q0[2 * p.D + d + e], k8[e], s2);
              if (n > 3) s3 = fmaf(q0[3 * p.D + d + e], k8[e], s3);
            }
          }
        } else if (live) {
          for (int d = 0; d < p.D; ++d) {
            const float kv = ldf(kr + d);
            s0 = fmaf(q0[d], kv, s0);
            if (n > 1) s1 = fmaf(q0[p.D + d], kv, s1);
            if (n > 2) s2 = fmaf(q0[2 * p.D + d], kv, s2);
            if (n > 3) s3 = fmaf(q0[3 * p.D + d], kv, s3);
          }
        }
        const float sc[4] = {s0, s1, s2, s3};
        for (int i = 0; i < n; ++i) {
          const int g = kc * rep + i0 + i;
          const float s = live ? sc[i] * p.scale : -INFINITY;
          const float m_old = ms[g];
          const float m_new = fmaxf(m_old, wave_max(s));
          const float pw = live ? __expf(s - m_new) : 0.f;
          const float sum = wave_sum(pw);
          ps[g * TA_PIECE + lane] = pw;
          if (lane == 0) {
            const float a = m_old == -INFINITY ? 0.f : __expf(m_old - m_new);
            alpha[g] = a;
            ms[g] = m_new;
            lsum[g] = lsum[g] * a + sum;
          }
        }
      }
    }
    __syncthreads();
    if (owner) {
#pragma unroll
      for (int g = 0; g < HMAX; ++g)
        if (g < p.H) acc[g] *= alpha[g];
      const int nk = min(TA_PIECE, hi - j0);
      // values of 8 consecutive keys are one vector (pieces start at multiples of 64 keys and
      // blocks hold a multiple of 8): [..][key / 8][dv][key % 8]
      for (int jj = 0; jj < nk; jj += 8) {
        const int rb = rowbase[jj];                   // (blk G) BS + key offset in the block
        const int blkG = rb / p.BS, off = rb - blkG * p.BS;
        const T* vp = (const T*)p.v_cache +
                      ((((size_t)(blkG + c) * (p.BS >> 3) + (off >> 3)) * p.Dv) + dv) * 8;
        float v8[8];
        ld8(vp, v8);
#pragma unroll
        for (int g = 0; g < HMAX; ++g) {
          if (g < p.H) {
            const float4 w0 = *(const float4*)(ps + g * TA_PIECE + jj);
            const float4 w1 = *(const float4*)(ps + g * TA_PIECE + jj + 4);
            float a = acc[g];
            a = fmaf(w0.x, v8[0], a);
            a = fmaf(w0.y, v8[1], a);
            a = fmaf(w0.z, v8[2], a);
            a = fmaf(w0.w, v8[3], a);
            a = fmaf(w1.x, v8[4], a);
            a = fmaf(w1.y, v8[5], a);
            a = fmaf(w1.z, v8[6], a);
            a = fmaf(w1.w, v8[7], a);
            acc[g] = a;
          }
        }
      }
    }
    __syncthreads();
  }
  if (p.num_parts == 1) {
    // 1 / l per head (lsum > 0: key 0 is always visible)
    for (int g = tid; g < p.H; g += nt) alpha[g] = 1.0f / lsum[g];
    __syncthreads();
    if (owner) talk_finish<T, HMAX>(p, t, c, dv, acc, alpha);
    return;
  }
  const size_t cell = (size_t)t * p.num_parts + part;
  for (int g = tid; g < p.H; g += nt) {
    p.ws_ml[(cell * p.H + g) * 2] = ms[g];
    p.ws_ml[(cell * p.H + g) * 2 + 1] = lsum[g];
  }
  if (owner) {
#pragma unroll
    for (int g = 0; g < HMAX; ++g)
      if (g < p.H) p.ws_o[(cell * p.H + g) * GV + tid] = acc[g];
  }
}

template <typename T, int HMAX>
__global__ __launch_bounds__(1024) void talking_merge_kernel(TalkParams p) {
  extern __shared__ float lds[];
  float* wgt = lds;                  // [parts][H] weight of a partition's sums
  float* inv_l = wgt + p.num_parts * p.H;
  const int t = blockIdx.x + p.row0;
  const int b = p.q_start ? find_seq(p.q_start, p.B, t) : t;
  if (p.seq_lens[b] <= 0) return;
  const int tid = threadIdx.x, nt = blockDim.x;
  const int GV = p.G * p.Dv;
  for (int g = tid; g < p.H; g += nt) {
    float mx = -INFINITY;
    for (int q = 0; q < p.num_parts; ++q)
      mx = fmaxf(mx, p.ws_ml[(((size_t)t * p.num_parts + q) * p.H + g) * 2]);
    float tot = 0.f;
    for (int q = 0; q < p.num_parts; ++q) {
      const float* ml = p.ws_ml + (((size_t)t * p.num_parts + q) * p.H + g) * 2;
      const float w = ml[0] == -INFINITY ? 0.f : __expf(ml[0] - mx);
      wgt[q * p.H + g] = w;
      tot += ml[1] * w;
    }
    inv_l[g] = 1.0f / tot;
  }
  __syncthreads();
  if (tid >= GV) return;
  float acc[HMAX];
#pragma unroll
  for (int g = 0; g < HMAX; ++g) acc[g] = 0.f;
  for (int q = 0; q < p.num_parts; ++q) {
    // every partition wrote its sums (zeros when it had no keys): the loads of a partition go
    // out together, unconditionally
    const float* o = p.ws_o + ((size_t)t * p.num_parts + q) * p.H * GV + tid;
    float part[HMAX];
#pragma unroll
    for (int g = 0; g < HMAX; ++g) part[g] = g < p.H ? o[(size_t)g * GV] : 0.f;
#pragma unroll
    for (int g = 0; g < HMAX; ++g)
      if (g < p.H) acc[g] = fmaf(wgt[q * p.H + g], part[g], acc[g]);
  }
  talk_finish<T, HMAX>(p, t, tid / p.Dv, tid % p.Dv, acc, inv_l);
}

// ------------------------------------------------------------------ routing by the largest logits
template <typename T>
__global__ __launch_bounds__(256) void route_topk_kernel(int32_t* __restrict__ ids,
                                                         float* __restrict__ wout,
                                                         const T* __restrict__ h, int h_stride,
                                                         const float* __restrict__ router,
                                                         const float* __restrict__ bias, int d,
                                                         int n, int top) {
  extern __shared__ float lds[];   // [n] logits, then the row as fp32 [d]
  float* hs = lds + ((n + 3) & ~3);
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* hr = h + (size_t)t * h_stride;
  for (int c = threadIdx.x; c < d; c += 256) hs[c] = ldf(hr + c);
  __syncthreads();
  // a logit per wave and turn; 16-byte pieces of the router row and of the staged input
  const bool vec = (d & 3) == 0;
  for (int e = wave; e < n; e += 4) {
    const float* wr = router + (size_t)e * d;
    float a0 = 0.f, a1 = 0.f;
    if (vec) {
      int c = lane * 4;
      for (; c + 256 < d; c += 512) {
        const float4 w0 = *(const float4*)(wr + c), w1 = *(const float4*)(wr + c + 256);
        const float4 x0 = *(const float4*)(hs + c), x1 = *(const float4*)(hs + c + 256);
        a0 = fmaf(x0.x, w0.x, fmaf(x0.y, w0.y, fmaf(x0.z, w0.z, fmaf(x0.w, w0.w, a0))));
        a1 = fmaf(x1.x, w1.x, fmaf(x1.y, w1.y, fmaf(x1.z, w1.z, fmaf(x1.w, w1.w, a1))));
      }
      if (c < d) {
        const float4 w0 = *(const float4*)(wr + c);
        const float4 x0 = *(const float4*)(hs + c);
        a0 = fmaf(x0.x, w0.x, fmaf(x0.y, w0.y, fmaf(x0.z, w0.z, fmaf(x0.w, w0.w, a0))));
      }
    } else {
      for (int c = lane; c < d; c += 64) a0 = fmaf(hs[c], wr[c], a0);
    }
    const float a = wave_sum(a0 + a1);
    if (lane == 0) lds[e] = a + (bias ? bias[e] : 0.f);
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  float first = 0.f, total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = 0.f;
    for (int e = 0; e < n; ++e) {
      const float v = lds[e];
      if (v != v || v == -INFINITY) continue;     // taken (marked below) or unusable
      if (best < 0 || v > bv) { best = e; bv = v; }
    }
    if (best < 0) best = 0;
    lds[best] = -INFINITY;
    if (k == 0) first = bv;
    const float ev = __expf(bv - first);
    ids[(size_t)t * top + k] = best;
    wout[(size_t)t * top + k] = ev;
    total += ev;
  }
  const float inv = 1.0f / total;
  for (int k = 0; k < top; ++k) wout[(size_t)t * top + k] *= inv;
}

// out[t, e F + f] = w_e(t) act(gu[t, e 2F + f]) gu[t, e 2F + F + f]; ids null: weight 1;
// ACT 0: silu, 1: gelu in its tanh form
__device__ __forceinline__ float gelu_tanhf(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
template <typename T, int ACT>
__global__ __launch_bounds__(256) void swiglu_routed_kernel(T* __restrict__ out, int out_stride,
                                                            const T* __restrict__ gu, int gu_stride,
                                                            const int32_t* __restrict__ ids,
                                                            const float* __restrict__ w, int top,
                                                            int E, int F) {
  extern __shared__ float lds[];   // [E] routing weight of every expert
  const int t = blockIdx.x;
  for (int e = threadIdx.x; e < E; e += 256) lds[e] = ids ? 0.f : 1.f;
  __syncthreads();
  if (ids && threadIdx.x < top) {
    const int e = ids[(size_t)t * top + threadIdx.x];
    if (e >= 0 && e < E) lds[e] = w[(size_t)t * top + threadIdx.x];
  }
  __syncthreads();
  const T* g = gu + (size_t)t * gu_stride;
  T* o = out + (size_t)t * out_stride;
  for (int c = threadIdx.x; c < E * F; c += 256) {
    const int e = c / F, f = c - e * F;
    const float we = lds[e];
    float r = 0.f;
    if (we != 0.f) {
      const float z = ldf(g + e * 2 * F + f);
      r = we * (ACT == 1 ? gelu_tanhf(z) : z * sigmoidf(z)) * ldf(g + e * 2 * F + F + f);
    }
    stf(o + c, r);
  }
}

}  // namespace

// ================================================================== launchers
void launch_post_norm_add_norm(void* out, bool out_f32, int out_stride, float* x, const void* ya,
                               int ya_stride, const void* yb, int yb_stride, bool y_f32,
                               const float* wa, int was, const float* wb, int wbs,
                               const float* post_w, int pws, const float* next_w, int nws,
                               int rows, int d, float eps, bool fresh, hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)2 * d * sizeof(float);
  // 16-byte accesses when every row starts at a multiple of 16 bytes
  auto al = [](const void* p, int bytes) { return p == nullptr || ((uintptr_t)p % bytes) == 0; };
  const int ye = y_f32 ? 4 : 2, oe = out_f32 ? 4 : 2;
  const bool vec = d % 8 == 0 && out_stride % 8 == 0 && ya_stride % 8 == 0 && yb_stride % 8 == 0 &&
                   al(out, 16) && al(x, 16) && al(ya, 16) && al(yb, 16) && al(wa, 16) &&
                   al(wb, 16) && al(post_w, 16) && al(next_w, 16) && ye > 0 && oe > 0;
#define AKAP_PN1(TY, TO, V)                                                                      \
  post_norm_add_norm_kernel<TY, TO, V><<<rows, 256, lds, s>>>(                                   \
      (TO*)out, out_stride, x, (const TY*)ya, ya_stride, (const TY*)yb, yb_stride, wa, was, wb, \
      wbs, post_w, pws, next_w, nws, d, eps, fresh ? 1 : 0)
#define AKAP_PN(TY, TO)            \
  do {                             \
    if (vec) AKAP_PN1(TY, TO, true); \
    else AKAP_PN1(TY, TO, false);  \
  } while (0)
  if (y_f32 && out_f32) AKAP_PN(float, float);
  else if (y_f32) AKAP_PN(float, bf16);
  else if (out_f32) AKAP_PN(bf16, float);
  else AKAP_PN(bf16, bf16);
#undef AKAP_PN1
#undef AKAP_PN
}

void launch_head_norm_cache(const HeadNormParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  if (f32) head_norm_cache_kernel<float><<<p.T, 256, 0, s>>>(p);
  else head_norm_cache_kernel<bf16><<<p.T, 256, 0, s>>>(p);
}

int retention_dreg(int D, int V) {
  // state rows per thread: 16 (64 state registers, workgroups of at most 256 threads), else 32
  // (128 registers, at most 512 threads); the workgroup has ceil(V / 4) column groups x
  // D / DREG lanes each, the lanes of a group a power of two
  for (int dreg : {16, 32}) {
    int dp = 1;
    while (dp * dreg < D) dp <<= 1;
    if (dp <= 64 && (int64_t)((V + RET_VR - 1) / RET_VR) * dp <= (dreg == 16 ? 256 : 512))
      return dreg;
  }
  return 0;
}

void launch_retention(RetentionParams p, bool f32, hipStream_t s) {
  if (p.num_seqs <= 0) return;
  const int dreg = retention_dreg(p.D, p.V);
  int dp = 1;
  while (dp * dreg < p.D) dp <<= 1;
  p.DP = dp;
  const int nt = ((((p.V + RET_VR - 1) / RET_VR) * dp + 63) / 64) * 64;
  const int vp = (p.V + 3) & ~3;
  p.TC = RET_TC;
  size_t lds = (size_t)p.TC * (2 * dp * dreg + 2 * vp) * sizeof(float);
  if (lds > 65536) {
    p.TC = RET_TC / 2;
    lds /= 2;
  }
#define AKAP_RET1(TY, R, M) retention_kernel<TY, R, M><<<grid, nt, lds, s>>>(p)
#define AKAP_RET(M)                                                                   \
  do {                                                                                \
    if (f32) {                                                                        \
      if (dreg == 16) AKAP_RET1(float, 16, M); else AKAP_RET1(float, 32, M);          \
    } else {                                                                          \
      if (dreg == 16) AKAP_RET1(bf16, 16, M); else AKAP_RET1(bf16, 32, M);            \
    }                                                                                 \
  } while (0)
  if (p.seg_buf == nullptr) {
    const dim3 grid(p.num_seqs, p.H);
    AKAP_RET(0);
    return;
  }
  {
    const dim3 grid(p.num_segs, p.H);
    AKAP_RET(1);
  }
  retention_scan_kernel<<<dim3(p.num_seqs, p.H), 256, 0, s>>>(p);
  {
    const dim3 grid(p.num_segs, p.H);
    AKAP_RET(3);
  }
#undef AKAP_RET
#undef AKAP_RET1
}

size_t talking_attention_lds(int H, int D) {
  return (size_t)(H * D + H * TA_PIECE + 3 * H + TA_PIECE) * sizeof(float);
}

void launch_talking_attention(const TalkParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  const int nt = ((p.G * p.Dv + 63) / 64) * 64;
  const size_t lds = talking_attention_lds(p.H, p.D);
  const int rows = p.T;
  const dim3 grid(rows, p.num_parts);
  const size_t mlds = (size_t)(p.num_parts + 1) * p.H * sizeof(float);
#define AKAP_TA(TY, HM)                                                          \
  do {                                                                           \
    talking_attention_kernel<TY, HM><<<grid, nt, lds, s>>>(p);                   \
    if (p.num_parts > 1) talking_merge_kernel<TY, HM><<<rows, nt, mlds, s>>>(p); \
  } while (0)
  if (f32) {
    if (p.H <= 8) AKAP_TA(float, 8); else if (p.H <= 16) AKAP_TA(float, 16); else AKAP_TA(float, 32);
  } else {
    if (p.H <= 8) AKAP_TA(bf16, 8); else if (p.H <= 16) AKAP_TA(bf16, 16); else AKAP_TA(bf16, 32);
  }
#undef AKAP_TA
}

// the second launch alone, over rows [row0, T): normalise, mix the heads and gate what the
// matrix-core kernel (or the split row kernel) left in the workspace
void launch_talking_merge(const TalkParams& p, bool f32, hipStream_t s) {
  const int rows = p.T - p.row0;
  if (rows <= 0) return;
  const int nt = ((p.G * p.Dv + 63) / 64) * 64;
  const size_t mlds = (size_t)(p.num_parts + 1) * p.H * sizeof(float);
#define AKAP_TM(TY, HM) talking_merge_kernel<TY, HM><<<rows, nt, mlds, s>>>(p)
  if (f32) {
    if (p.H <= 8) AKAP_TM(float, 8); else if (p.H <= 16) AKAP_TM(float, 16); else AKAP_TM(float, 32);
  } else {
    if (p.H <= 8) AKAP_TM(bf16, 8); else if (p.H <= 16) AKAP_TM(bf16, 16); else AKAP_TM(bf16, 32);
  }
#undef AKAP_TM
}

void launch_route_topk(int32_t* ids, float* w, const void* h, int h_stride, const float* router,
                       const float* bias, int rows, int d, int n, int top, bool f32,
                       hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)(((n + 3) & ~3) + d) * sizeof(float);
  if (f32)
    route_topk_kernel<float><<<rows, 256, lds, s>>>(ids, w, (const float*)h, h_stride, router, bias,
                                                    d, n, top);
  else
    route_topk_kernel<bf16><<<rows, 256, lds, s>>>(ids, w, (const bf16*)h, h_stride, router, bias,
                                                   d, n, top);
}

void launch_swiglu_routed(void* out, int out_stride, const void* gu, int gu_stride,
                          const int32_t* ids, const float* w, int rows, int top, int E, int F,
                          bool f32, int act, hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)E * sizeof(float);
#define AKAP_GA(TY, A)                                                                          \
  swiglu_routed_kernel<TY, A><<<rows, 256, lds, s>>>((TY*)out, out_stride, (const TY*)gu,      \
                                                     gu_stride, ids, w, top, E, F)
  if (f32) {
    if (act == 1) AKAP_GA(float, 1); else AKAP_GA(float, 0);
  } else {
    if (act == 1) AKAP_GA(bf16, 1); else AKAP_GA(bf16, 0);
  }
#undef AKAP_GA
}

}  // namespace akap_stream
