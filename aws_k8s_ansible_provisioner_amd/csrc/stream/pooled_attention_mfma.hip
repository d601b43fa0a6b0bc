// Window + pooled-block attention of prompt chunks on the matrix cores (bf16 cache).
//
// v_mfma_f32_32x32x16_bf16 with the keys as the rows of the score tile (S^T = K Q^T), so a query
// is a lane column: its running maximum and sum live in the two lanes col and col + 32.  The K
// rows of a 32-key step are loaded in the order that swaps bits 2 and 3 of the row, which makes a
// lane's 16 accumulator registers exactly the keys 16 c + 8 hf + e (c = 0, 1; e = 0..7): the
// softmax weights become the B operand of O^T = V^T P^T without lane traffic, and the A operand
// is one 16-byte load from the value cache [NB, G, BS / 8, Dv, 8].  A wave owns 32 queries of one
// head; the four waves of a workgroup take the four quarters of a 128-token tile of the
// scheduler's map and share the tile's keys through the caches.  The visible range of a tile is
// walked as pooled entries first (fp32 in memory, rounded to bf16 operands, gathered), then
// window tokens in steps aligned to 32 positions; the sink of score 0 is the starting state of
// the online softmax.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::bf16x4;
using akap::bf16x8;
using akap::f32x16;

namespace {

__device__ __forceinline__ int swap23(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 v;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (bf16)0.f;
  return v;
}

// DVT: 32-wide tiles of the value size.  DEC: one query per sequence (a decode step, or the
// single rows of a mixed step): the columns of the tile are the query heads of one key/value
// head, the eight waves of the workgroup split the steps of the key range among themselves and
// add their shares in LDS.
constexpr int kDecWaves = 8;

template <int DVT, bool DEC>
__global__ __launch_bounds__(DEC ? 64 * kDecWaves : 256) void pooled_window_mfma_kernel(
    const PoolAttnParams p, const int32_t* __restrict__ tile_seq,
    const int32_t* __restrict__ tile_row) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int KS = p.D >> 4;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int rep = p.H / p.G;
  // Q operands [KS][64]: one set per wave (prompt tiles), one for the workgroup (DEC)
  bf16x8* qs = (bf16x8*)smem + (DEC ? 0 : (size_t)wave * KS * 64);
  int b, t0, nrows, g, h = 0;
  bool active = true;
  if (DEC) {
    t0 = blockIdx.x;
    g = blockIdx.y;
    b = t0;
    nrows = rep;                                   // columns in use: the heads of the group
    if (p.slots[t0] < 0) return;                   // a padding row (the whole workgroup)
    for (int e = tid; e < KS * 64; e += 64 * kDecWaves) {
      const int c = e >> 6, ln = e & 63;
      bf16x8 v = zero8();
      if ((ln & 31) < rep)
        v = *(const bf16x8*)((const bf16*)p.q + ((size_t)t0 * p.H + g * rep + (ln & 31)) * p.D +
                             16 * c + 8 * (ln >> 5));
      qs[e] = v;
    }
  } else {
    // the map is sorted by rising work: the grid walks it from its end, longest tiles first
    const int tile = (int)gridDim.x - 1 - (int)blockIdx.x;
    h = blockIdx.y;
    g = h / rep;
    b = tile_seq[tile];
    const int r_first = tile_row[tile] + 32 * wave;
    const int chunk = p.q_start[b + 1] - p.q_start[b];
    active = r_first < chunk;
    t0 = p.q_start[b] + (active ? r_first : 0);
    nrows = active ? min(32, chunk - r_first) : 0;
    if (active) {
      for (int c = 0; c < KS; ++c) {
        bf16x8 v = zero8();
        if (col < nrows)
          v = *(const bf16x8*)((const bf16*)p.q + ((size_t)(t0 + col) * p.H + h) * p.D + 16 * c +
                               8 * hf);
        qs[c * 64 + lane] = v;
      }
    }
  }
  __syncthreads();
  if (!active) return;

  const int pos0 = (int)p.positions[t0];
  const int plast = DEC ? pos0 : pos0 + nrows - 1;
  const int qpos = col < nrows ? (DEC ? pos0 : pos0 + col) : -1;      // -1: an unused column
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const float sc2 = p.scale * 1.44269504088896f;       // scores -> log2 units
  const int W = p.window, P = p.pool, BS = p.BS, G = p.G, D = p.D, Dv = p.Dv;
  const bf16* kc = (const bf16*)p.k_cache;
  const bf16* vc = (const bf16*)p.v_cache;

  f32x16 acc[DVT];
#pragma unroll
  for (int k = 0; k < DVT; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  float m_run = p.unit_sink ? 0.f : -INFINITY;
  // the two lanes of a column (and, DEC, the waves) are added at the end: the sink counts once
  float l_run = (p.unit_sink && hf == 0 && (!DEC || wave == 0)) ? 1.f : 0.f;

  // one step: scores s (raw dot products, masked with `seen`) -> weights -> acc
  auto softmax_step = [&](f32x16& s, const bool (&seen)[16], bf16x8 (&pb)[2]) -> bool {
    float cmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = seen[i] ? s[i] * sc2 : -INFINITY;
      cmax = fmaxf(cmax, s[i]);
    }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m_run, cmax);
    const bool any = m_new != -INFINITY;
    const float alpha = any ? exp2f(m_run - m_new) : 1.f;
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float w = any ? exp2f(s[8 * c + e] - m_new) : 0.f;
        sum += w;
        pb[c][e] = (bf16)w;
      }
    l_run = l_run * alpha + sum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int k = 0; k < DVT; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[k][i] *= alpha;
    }
    return __any(sum > 0.f);
  };

  // ---- pooled entries 0 .. nbt-1 (what the tile's last query sees)
  const int nbt = (P > 0 && W > 0 && plast - W + 1 > 0) ? (plast - W + 1) / P : 0;
  const int pool_steps = (nbt + 31) >> 5;
  for (int cb = 0; cb < nbt; cb += 32) {
    if (DEC && ((cb >> 5) % kDecWaves != wave)) continue;
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    {
      const int c = min(cb + swap23(col), nbt - 1);
      const int first = c * P, page = bt[first / BS], idx = (first % BS) / P;
      const float* kp = p.k_pool + ((size_t)(page * G + g) * p.PS + idx) * D + 8 * hf;
      for (int ks = 0; ks < KS; ++ks) {
        const float4 a = *(const float4*)(kp + 16 * ks), c4 = *(const float4*)(kp + 16 * ks + 4);
        bf16x8 kf;
        kf[0] = (bf16)a.x; kf[1] = (bf16)a.y; kf[2] = (bf16)a.z; kf[3] = (bf16)a.w;
        kf[4] = (bf16)c4.x; kf[5] = (bf16)c4.y; kf[6] = (bf16)c4.z; kf[7] = (bf16)c4.w;
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qs[ks * 64 + lane], s, 0, 0, 0);
      }
    }
    bool seen[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int c = cb + 16 * (i >> 3) + 8 * hf + (i & 7);
      seen[i] = c < nbt && qpos >= 0 && c * P + P - 1 <= qpos - W;
    }
    bf16x8 pb[2];
    if (!softmax_step(s, seen, pb)) continue;
    // values: entry rows gathered one by one (few steps: a tile sees n / pool entries)
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      const float* vrow[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int c = min(cb + 16 * c2 + 8 * hf + e, nbt - 1);
        const int first = c * P, page = bt[first / BS], idx = (first % BS) / P;
        vrow[e] = p.v_pool + ((size_t)(page * G + g) * p.PS + idx) * Dv + col;
      }
#pragma unroll
      for (int k = 0; k < DVT; ++k) {
        bf16x8 vf;
#pragma unroll
        for (int e = 0; e < 8; ++e) vf[e] = (bf16)vrow[e][32 * k];
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[c2], acc[k], 0, 0, 0);
      }
    }
  }

  // ---- window tokens, in steps aligned to 32 positions
  const int lo = W > 0 ? max(0, pos0 - W + 1) : 0;
  for (int kb = lo & ~31; kb <= plast; kb += 32) {
    if (DEC && ((pool_steps + ((kb - (lo & ~31)) >> 5)) % kDecWaves != wave)) continue;
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    {
      const int key = min(kb + swap23(col), plast);   // rows past the range are masked below
      const int bi = key / BS;
      const bf16* kp = kc + ((size_t)(bt[bi] * G + g) * BS + (key - bi * BS)) * D + 8 * hf;
      // fragment loads go out in batches ahead of their products
      for (int c0 = 0; c0 < KS; c0 += 4) {
        bf16x8 kf[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c0 + u < KS) kf[u] = *(const bf16x8*)(kp + 16 * (c0 + u));
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c0 + u < KS)
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[u], qs[(c0 + u) * 64 + lane], s, 0, 0, 0);
      }
    }
    // value operands of the step: groups of 8 keys, rows of the grouped cache
    const bf16* vp[2];
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      const int kk = min(kb + 16 * c2 + 8 * hf, plast);
      const int bi = kk / BS;
      vp[c2] = vc + ((size_t)(bt[bi] * G + g) * (BS >> 3) + ((kk - bi * BS) >> 3)) * Dv * 8 +
               (size_t)col * 8;
    }
    bf16x8 vf[2][DVT];
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
      for (int k = 0; k < DVT; ++k) vf[c2][k] = *(const bf16x8*)(vp[c2] + (size_t)32 * 8 * k);
    bool seen[16];
    const bool whole = kb + 31 <= pos0 && (W <= 0 || kb > plast - W);   // no query masks a key
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb + 16 * (i >> 3) + 8 * hf + (i & 7);
      seen[i] = qpos >= 0 && (whole || (key <= qpos && (W <= 0 || key > qpos - W)));
    }
    bf16x8 pb[2];
    if (!softmax_step(s, seen, pb)) continue;
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
      for (int k = 0; k < DVT; ++k)
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[c2][k], pb[c2], acc[k], 0, 0, 0);
  }

  // ---- out: register j of tile k is value entry 32 k + 8 (j / 4) + 4 hf + j % 4 of query col
  const float l = l_run + __shfl_xor(l_run, 32, 64);
  if (DEC) {
    // the waves' shares: maxima and sums through LDS, outputs added with LDS atomics
    __syncthreads();                               // every wave is done with the Q operands
    constexpr int NW = kDecWaves, NTH = 64 * kDecWaves;
    float* m_s = (float*)smem;                     // [NW][32]
    float* l_s = m_s + NW * 32;                    // [NW][32]
    float* ob = l_s + NW * 32;                     // [Dv][32]
    for (int e = tid; e < Dv * 32; e += NTH) ob[e] = 0.f;
    if (hf == 0) {
      m_s[wave * 32 + col] = m_run;
      l_s[wave * 32 + col] = l;
    }
    __syncthreads();
    float mg = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) mg = fmaxf(mg, m_s[w * 32 + col]);
    const float f = (m_run == -INFINITY || mg == -INFINITY) ? 0.f : exp2f(m_run - mg);
    if (col < nrows && f > 0.f) {
#pragma unroll
      for (int k = 0; k < DVT; ++k)
#pragma unroll
        for (int j = 0; j < 16; ++j)
          atomicAdd(&ob[(32 * k + 8 * (j >> 2) + 4 * hf + (j & 3)) * 32 + col], acc[k][j] * f);
    }
    __syncthreads();
    bf16* o = (bf16*)p.out + (size_t)t0 * p.out_stride + (size_t)g * rep * Dv;
    for (int e = tid; e < rep * Dv; e += NTH) {
      const int c = e / Dv, dv = e - c * Dv;
      float mg2 = -INFINITY, lg = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) mg2 = fmaxf(mg2, m_s[w * 32 + c]);
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float mw = m_s[w * 32 + c];
        if (mw != -INFINITY) lg += l_s[w * 32 + c] * exp2f(mw - mg2);
      }
      o[e] = (bf16)(lg > 0.f ? ob[dv * 32 + c] / lg : 0.f);
    }
    return;
  }
  if (col < nrows) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16* o = (bf16*)p.out + (size_t)(t0 + col) * p.out_stride + (size_t)h * Dv;
#pragma unroll
    for (int k = 0; k < DVT; ++k)
#pragma unroll
      for (int j4 = 0; j4 < 4; ++j4) {
        bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16)(acc[k][4 * j4 + i] * inv);
        *(bf16x4*)(o + 32 * k + 8 * j4 + 4 * hf) = v;
      }
  }
}

}  // namespace

bool pooled_mfma_supported(int H, int G, int D, int Dv, int BS) {
  return D % 16 == 0 && D <= 256 && (Dv == 32 || Dv == 64 || Dv == 128 || Dv == 256) &&
         BS % 8 == 0 && H % G == 0;
}

void launch_pooled_window_prefill_mfma(const PoolAttnParams& p, const int32_t* tile_seq,
                                       const int32_t* tile_row, int num_tiles, hipStream_t s) {
  if (num_tiles <= 0) return;
  const dim3 grid(num_tiles, p.H);
  const size_t lds = (size_t)4 * (p.D >> 4) * 64 * sizeof(bf16x8);
#define AKAP_PWM(N) \
  pooled_window_mfma_kernel<N, false><<<grid, 256, lds, s>>>(p, tile_seq, tile_row)
  switch (p.Dv >> 5) {
    case 1: AKAP_PWM(1); break;
    case 2: AKAP_PWM(2); break;
    case 4: AKAP_PWM(4); break;
    default: AKAP_PWM(8); break;
  }
#undef AKAP_PWM
}

// one query per sequence: rows [0, rows) of p, row t = sequence t (at most 32 query heads per
// key/value head)
void launch_pooled_window_decode_mfma(const PoolAttnParams& p, int rows, hipStream_t s) {
  if (rows <= 0) return;
  const dim3 grid(rows, p.G);
  const size_t q_bytes = (size_t)(p.D >> 4) * 64 * sizeof(bf16x8);
  const size_t m_bytes = (size_t)(2 * kDecWaves * 32 + p.Dv * 32) * sizeof(float);
  const size_t lds = q_bytes > m_bytes ? q_bytes : m_bytes;
#define AKAP_PWD(N) \
  pooled_window_mfma_kernel<N, true><<<grid, 64 * kDecWaves, lds, s>>>(p, nullptr, nullptr)
  switch (p.Dv >> 5) {
    case 1: AKAP_PWD(1); break;
    case 2: AKAP_PWD(2); break;
    case 4: AKAP_PWD(4); break;
    default: AKAP_PWD(8); break;
  }
#undef AKAP_PWD
}

}  // namespace akap_stream
