// Head-mixed attention of prompt chunks on the matrix cores (bf16 cache).
//
// One workgroup of four waves per (tile of 32 queries of one sequence, query head g).  Keys go
// by steps of 128: wave w scores keys [32 w, 32 w + 32) of the step (S^T = K Q^T on
// v_mfma_f32_32x32x16_bf16: a query is a lane column, so its running max and sum are per-lane
// values plus one exchange between the lane halves; the K rows are taken in an order -- bits 2
// and 3 of the row swapped -- that makes a lane's accumulator registers 8 consecutive keys,
// i.e. an operand of the next product without lane traffic).  The waves agree on the step's
// maximum through LDS and publish their bf16 weights there; then every wave accumulates, for
// ITS share of the (value head, 32 value entries) column tiles, O = P V over all 128 keys of
// the step (values come from the cache in groups of 8 keys, one 16-byte load per lane and
// operand).  A workgroup thus forms, for its query head, the unnormalised sums of ALL value
// heads; they go to a workspace (fp32) with the head's (max, sum), and the merge launch of the
// split row kernel normalises, mixes the heads and gates.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::bf16x8;
using akap::f32x16;

namespace {

__device__ __forceinline__ int swap23(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

template <int TPW, int NQ>
__global__ __launch_bounds__(256) void talk_prefill_mfma_kernel(TalkParams p, const int32_t* tile_seq,
                                                               const int32_t* tile_row,
                                                               int tile_rows) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int KS = p.D >> 4;                         // 16-wide steps of the head size
  bf16x8* qs = (bf16x8*)smem;                      // [NQ][KS][64] Q operands
  bf16x8* ps = qs + NQ * KS * 64;                  // [2][NQ][8][64] weights of a step
  float* m_loc = (float*)(ps + 2 * NQ * 8 * 64);   // [2][4][NQ][32] each wave's maxima
  float* alpha_s = m_loc + 2 * 4 * NQ * 32;        // [2][NQ][32] rescale of the step
  float* l_s = alpha_s + 2 * NQ * 32;              // [4][NQ][32] the waves' sums at the end

  constexpr int QT = 32 * NQ;                      // queries of a workgroup
  const int sub_per = tile_rows / QT;
  // the map is sorted by rising work: the grid walks it from its end, longest tiles first
  const int tslot = blockIdx.x / sub_per, sub = blockIdx.x - tslot * sub_per;
  const int tile = (int)(gridDim.x / sub_per) - 1 - tslot;
  const int g = blockIdx.y;
  const int b = tile_seq[tile];
  const int r_first = tile_row[tile] + QT * sub;
  const int chunk = p.q_start[b + 1] - p.q_start[b];
  if (r_first >= chunk) return;
  const int t0 = p.q_start[b] + r_first;
  const int nrows = min(QT, chunk - r_first);
  const int pos0 = (int)p.positions[t0];
  const int kmax = pos0 + nrows - 1;               // last key any query of the tile sees
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int rep = p.H / p.G, kvh = g / rep;
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const float sc2 = p.scale * 1.44269504088896f;   // scores -> log2 units
  const int DVT = p.Dv >> 5, NT = p.G * DVT;       // column tiles of 32 value entries

  // Q operands: lane (col = query, hf) of step c holds Q[t0 + 32 q + col][16 c + 8 hf ..+8]
  for (int e = tid; e < NQ * KS * 64; e += 256) {
    const int q = e / (KS * 64), c = (e >> 6) % KS, ln = e & 63;
    const int qc = 32 * q + (ln & 31), qh = ln >> 5;
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (bf16)0.f;
    if (qc < nrows)
      v = *(const bf16x8*)((const bf16*)p.q + ((size_t)(t0 + qc) * p.H + g) * p.D + 16 * c + 8 * qh);
    qs[e] = v;
  }
  f32x16 acc[TPW][NQ];
#pragma unroll
  for (int k = 0; k < TPW; ++k)
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[k][q][i] = 0.f;
  float m_run[NQ], l_run[NQ];
  int qpos[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    m_run[q] = -INFINITY;
    l_run[q] = 0.f;
    qpos[q] = 32 * q + col < nrows ? pos0 + 32 * q + col : -1;   // -1: an unused column
  }
  __syncthreads();

  int buf = 0;
  for (int key0 = 0; key0 <= kmax; key0 += 128, buf ^= 1) {
    // ---- scores of my 32 keys against the NQ query tiles: every K fragment is loaded once
    const int kb = key0 + 32 * wave;
    f32x16 s[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[q][i] = 0.f;
    if (kb <= kmax) {
      const int key = min(kb + swap23(col), kmax);  // rows past the range are masked below
      const int bi = key / p.BS;
      const bf16* kp = (const bf16*)p.k_cache +
                       ((size_t)(bt[bi] * p.G + kvh) * p.BS + (key - bi * p.BS)) * p.D + 8 * hf;
      // fragment loads go out in batches ahead of their products (a load per product would
      // make the step a chain of load latencies)
      for (int c0 = 0; c0 < KS; c0 += 4) {
        bf16x8 kf[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c0 + u < KS) kf[u] = *(const bf16x8*)(kp + 16 * (c0 + u));
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c0 + u < KS) {
#pragma unroll
            for (int q = 0; q < NQ; ++q)
              s[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  kf[u], qs[(q * KS + c0 + u) * 64 + lane], s[q], 0, 0, 0);
          }
      }
    }
    // cache rows of the step's eight 16-key operands of the values
    int vrow[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kk = min(key0 + 16 * j + 8 * hf, kmax);
      const int bi = kk / p.BS;
      vrow[j] = bt[bi] * p.G * (p.BS >> 3) + ((kk - bi * p.BS) >> 3);
    }
    // register i of this lane: key kb + 16 (i >> 3) + 8 hf + (i & 7), query column col
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      float bmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = kb + 16 * (i >> 3) + 8 * hf + (i & 7);
        s[q][i] = key <= qpos[q] ? s[q][i] * sc2 : -INFINITY;
        bmax = fmaxf(bmax, s[q][i]);
      }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
      if (hf == 0) m_loc[((buf * 4 + wave) * NQ + q) * 32 + col] = bmax;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const float* ml = m_loc + (buf * 4 * NQ + q) * 32 + col;
      const float mn = fmaxf(fmaxf(m_run[q], fmaxf(ml[0], ml[NQ * 32])),
                             fmaxf(ml[2 * NQ * 32], ml[3 * NQ * 32]));
      const float ms = mn == -INFINITY ? 0.f : mn;  // nothing visible yet: every exp below is 0
      const float alpha = __builtin_amdgcn_exp2f(m_run[q] - ms);
      m_run[q] = mn;
      float psum = 0.f;
      bf16x8 pb[2];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = __builtin_amdgcn_exp2f(s[q][i] - ms);
        psum += e;
        pb[i >> 3][i & 7] = (bf16)e;
      }
      l_run[q] = l_run[q] * alpha + psum;
      ps[((buf * NQ + q) * 8 + 2 * wave) * 64 + lane] = pb[0];
      ps[((buf * NQ + q) * 8 + 2 * wave + 1) * 64 + lane] = pb[1];
      if (wave == 0 && hf == 0) alpha_s[(buf * NQ + q) * 32 + col] = alpha;
    }
    __syncthreads();
    // ---- O += P V for my column tiles; accumulator register i: query row
    //      (i & 3) + 4 hf + 8 ((i >> 2) & 1) + 16 (i >> 3), value entry col of the tile
    float ar[NQ][16];
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const float4 a4 = *(const float4*)(alpha_s + (buf * NQ + q) * 32 + 4 * hf + 8 * (i4 & 1) +
                                           16 * (i4 >> 1));
        ar[q][4 * i4] = a4.x; ar[q][4 * i4 + 1] = a4.y; ar[q][4 * i4 + 2] = a4.z;
        ar[q][4 * i4 + 3] = a4.w;
      }
#pragma unroll
    for (int k = 0; k < TPW; ++k) {
      const int ti = wave + 4 * k;
      if (ti < NT) {
        const int cv = ti / DVT, dv0 = (ti - cv * DVT) << 5;
        // operand j: keys key0 + 16 j ..+16 (a group wholly past the range has weights 0);
        // every value fragment is loaded once for the NQ query tiles
        bf16x8 vf[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (key0 + 16 * j <= kmax)
            vf[j] = *(const bf16x8*)((const bf16*)p.v_cache +
                                     (((size_t)vrow[j] + (size_t)cv * (p.BS >> 3)) * p.Dv + dv0 + col) * 8);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[k][q][i] *= ar[q][i];
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (key0 + 16 * j <= kmax)
              acc[k][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  ps[((buf * NQ + q) * 8 + j) * 64 + lane], vf[j], acc[k][q], 0, 0, 0);
        }
      }
    }
  }
  // ---- the head's (max, sum) and its unnormalised sums
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    l_run[q] += __shfl_xor(l_run[q], 32, 64);
    if (hf == 0) l_s[(wave * NQ + q) * 32 + col] = l_run[q];
  }
  __syncthreads();
  const int GV = p.G * p.Dv;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    if (wave == 0 && hf == 0 && 32 * q + col < nrows) {
      const size_t cell = ((size_t)(t0 + 32 * q + col) * p.H + g) * 2;
      const float* lq = l_s + q * 32 + col;
      p.ws_ml[cell] = m_run[q] * 0.6931471805599453f;
      p.ws_ml[cell + 1] = lq[0] + lq[NQ * 32] + lq[2 * NQ * 32] + lq[3 * NQ * 32];
    }
#pragma unroll
    for (int k = 0; k < TPW; ++k) {
      const int ti = wave + 4 * k;
      if (ti < NT) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int row = 32 * q + (i & 3) + 4 * hf + 8 * ((i >> 2) & 1) + 16 * (i >> 3);
          if (row < nrows)
            p.ws_o[((size_t)(t0 + row) * p.H + g) * GV + (ti << 5) + col] = acc[k][q][i];
        }
      }
    }
  }
}

// Decode rows (one query per sequence): one workgroup per (row, key partition).  The 32 columns
// of a tile are the query HEADS of the token; wave w scores all 128 keys of a step for the
// key heads w, w + 4, ... (only the columns of a key head's own query heads are kept, and since
// a column belongs to one wave, its running max and sum stay in that wave), the weights of all
// heads meet in LDS, and every wave accumulates its share of the (value head, 32 entries)
// column tiles with the heads as rows: each cached key and value is read once per row for all
// heads.  The partition's unnormalised sums and (max, sum) go to the workspace of the split
// form; the merge launch combines the partitions, mixes the heads and gates.
template <int TPW>
__global__ __launch_bounds__(256) void talk_decode_mfma_kernel(TalkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int KS = p.D >> 4;
  bf16x8* qs = (bf16x8*)smem;                      // [KS][64] Q operands (column = head)
  bf16x8* ps = qs + KS * 64;                       // [2][4 blocks][2][64] weights of a step
  float* alpha_s = (float*)(ps + 2 * 4 * 2 * 64);  // [2][32]

  const int t = blockIdx.x, part = blockIdx.y;
  if (p.seq_lens[t] <= 0) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int rep = p.H / p.G;
  const int last = (int)p.positions[t];            // the row sees keys 0 .. last
  const int steps = (last + 128) >> 7;
  const int per = (steps + p.num_parts - 1) / p.num_parts;
  const int lo = part * per * 128;
  const int hi = min(last + 1, lo + per * 128);    // keys [lo, hi)
  const int32_t* bt = p.block_tables + (size_t)t * p.max_blocks;
  const float sc2 = p.scale * 1.44269504088896f;
  const int DVT = p.Dv >> 5, NT = p.G * DVT;
  const int my_c = col < p.H ? col / rep : -1;     // key head of this column's query head
  const bool mine = my_c >= 0 && (my_c & 3) == wave;

  for (int e = tid; e < KS * 64; e += 256) {
    const int c = e >> 6, ln = e & 63;
    const int qc = ln & 31, qh = ln >> 5;
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (bf16)0.f;
    if (qc < p.H)
      v = *(const bf16x8*)((const bf16*)p.q + ((size_t)t * p.H + qc) * p.D + 16 * c + 8 * qh);
    qs[e] = v;
  }
  {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
    for (int e = tid; e < 2 * 4 * 2 * 64; e += 256) ps[e] = z;   // columns past H stay zero
    if (tid < 64) alpha_s[tid] = 1.f;                            // rows past H: never rescaled
  }
  f32x16 acc[TPW];
#pragma unroll
  for (int k = 0; k < TPW; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  __syncthreads();

  int buf = 0;
  for (int key0 = lo; key0 < hi; key0 += 128, buf ^= 1) {
    for (int cc = wave; cc < p.G; cc += 4) {
      f32x16 s[4];
      const bf16* kp[4];
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[blk][i] = 0.f;
        const int key = min(key0 + 32 * blk + swap23(col), hi - 1);
        const int bi = key / p.BS;
        kp[blk] = (const bf16*)p.k_cache +
                  ((size_t)(bt[bi] * p.G + cc) * p.BS + (key - bi * p.BS)) * p.D + 8 * hf;
      }
      // one key block at a time, all of its fragments in flight together: the 32 rows of a
      // block are consumed whole while their cache lines are still in L1 (fragments of several
      // blocks side by side touch 4 x 32 rows per wave and evict each other)
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        if (key0 + 32 * blk < hi) {
          for (int c0 = 0; c0 < KS; c0 += 8) {
            bf16x8 kf[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (c0 + u < KS) kf[u] = *(const bf16x8*)(kp[blk] + 16 * (c0 + u));
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (c0 + u < KS)
                s[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[u], qs[(c0 + u) * 64 + lane],
                                                                 s[blk], 0, 0, 0);
          }
        }
      }
      // the columns of key head cc's query heads: softmax over the step's 128 keys
      const bool act = my_c == cc;
      float bmax = -INFINITY;
      if (key0 + 128 <= hi) {
        // a whole step: nothing to mask (lanes of other heads' columns compute along; what
        // they get is never stored)
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            s[blk][i] *= sc2;
            bmax = fmaxf(bmax, s[blk][i]);
          }
      } else {
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = key0 + 32 * blk + 16 * (i >> 3) + 8 * hf + (i & 7);
            s[blk][i] = key < hi ? s[blk][i] * sc2 : -INFINITY;
            bmax = fmaxf(bmax, s[blk][i]);
          }
      }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
      const float mn = fmaxf(m_run, bmax);
      const float ms = mn == -INFINITY ? 0.f : mn;
      const float alpha = __builtin_amdgcn_exp2f(m_run - ms);
      float psum = 0.f;
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        bf16x8 pb[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(s[blk][i] - ms);
          psum += e;
          pb[i >> 3][i & 7] = (bf16)e;
        }
        if (act) {
          ps[((buf * 4 + blk) * 2 + 0) * 64 + lane] = pb[0];
          ps[((buf * 4 + blk) * 2 + 1) * 64 + lane] = pb[1];
        }
      }
      if (act) {
        m_run = mn;
        l_run = l_run * alpha + psum;
        if (hf == 0) alpha_s[buf * 32 + col] = alpha;
      }
    }
    int vrow[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kk = min(key0 + 16 * j + 8 * hf, hi - 1);
      const int bi = kk / p.BS;
      vrow[j] = bt[bi] * p.G * (p.BS >> 3) + ((kk - bi * p.BS) >> 3);
    }
    __syncthreads();
    float ar[16];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const float4 a4 = *(const float4*)(alpha_s + buf * 32 + 4 * hf + 8 * (i4 & 1) + 16 * (i4 >> 1));
      ar[4 * i4] = a4.x; ar[4 * i4 + 1] = a4.y; ar[4 * i4 + 2] = a4.z; ar[4 * i4 + 3] = a4.w;
    }
    // the accumulators are rescaled only when some head's maximum moved (wave-uniform)
    bool moved = false;
#pragma unroll
    for (int i = 0; i < 16; ++i) moved |= ar[i] != 1.0f;
    const bool rescale = __any(moved);
    // the value operands of two column tiles go out together
#pragma unroll
    for (int k0 = 0; k0 < TPW; k0 += 2) {
      bf16x8 vf[2][8];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ti = wave + 4 * (k0 + u);
        if (ti < NT) {
          const int cv = ti / DVT, dv0 = (ti - cv * DVT) << 5;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (key0 + 16 * j < hi)
              vf[u][j] = *(const bf16x8*)((const bf16*)p.v_cache +
                                          (((size_t)vrow[j] + (size_t)cv * (p.BS >> 3)) * p.Dv + dv0 + col) * 8);
        }
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ti = wave + 4 * (k0 + u);
        if (ti < NT) {
          if (rescale) {
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[k0 + u][i] *= ar[i];
          }
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (key0 + 16 * j < hi)
              acc[k0 + u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  ps[(buf * 8 + j) * 64 + lane], vf[u][j], acc[k0 + u], 0, 0, 0);
        }
      }
    }
  }
  // (max, sum) of the columns this wave owns, and the sums of its column tiles
  const size_t cell = (size_t)t * p.num_parts + part;
  l_run += __shfl_xor(l_run, 32, 64);
  if (mine && hf == 0) {
    p.ws_ml[(cell * p.H + col) * 2] = m_run * 0.6931471805599453f;
    p.ws_ml[(cell * p.H + col) * 2 + 1] = l_run;
  }
  const int GV = p.G * p.Dv;
#pragma unroll
  for (int k = 0; k < TPW; ++k) {
    const int ti = wave + 4 * k;
    if (ti < NT) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = (i & 3) + 4 * hf + 8 * ((i >> 2) & 1) + 16 * (i >> 3);
        if (row < p.H) p.ws_o[(cell * p.H + row) * GV + (ti << 5) + col] = acc[k][i];
      }
    }
  }
}

}  // namespace

void launch_talking_decode_mfma(const TalkParams& p, hipStream_t s) {
  if (p.T <= 0) return;
  const int NT = p.G * (p.Dv / 32);
  const dim3 grid(p.T, p.num_parts);
  const size_t lds = (size_t)(p.D / 16) * 64 * 16 + 2 * 4 * 2 * 64 * 16 + 2 * 32 * sizeof(float);
  if (NT <= 8) talk_decode_mfma_kernel<2><<<grid, 256, lds, s>>>(p);
  else if (NT <= 16) talk_decode_mfma_kernel<4><<<grid, 256, lds, s>>>(p);
  else talk_decode_mfma_kernel<8><<<grid, 256, lds, s>>>(p);
}

bool talk_mfma_supported(int H, int G, int D, int Dv, int BS) {
  return H <= 32 && D % 16 == 0 && D <= 256 && Dv % 32 == 0 && G * (Dv / 32) <= 32 && BS % 16 == 0;
}

void launch_talking_prefill_mfma(const TalkParams& p, const int32_t* tile_seq,
                                 const int32_t* tile_row, int num_tiles, int tile_rows,
                                 hipStream_t s) {
  if (num_tiles <= 0) return;
  const int NT = p.G * (p.Dv / 32);
  // two query tiles per workgroup (every key and value fragment serves 64 queries) when the
  // accumulators of the wave's column tiles leave room for it
  const int nq = (tile_rows % 64 == 0 && NT <= 16) ? 2 : 1;
  const dim3 grid(num_tiles * (tile_rows / (32 * nq)), p.H);
  const size_t lds = (size_t)nq * (p.D / 16) * 64 * 16 + (size_t)2 * nq * 8 * 64 * 16 +
                     (size_t)nq * (2 * 4 * 32 + 2 * 32 + 4 * 32) * sizeof(float);
#define AKAP_TP(TP, NQ) \
  talk_prefill_mfma_kernel<TP, NQ><<<grid, 256, lds, s>>>(p, tile_seq, tile_row, tile_rows)
  if (nq == 2) {
    if (NT <= 8) AKAP_TP(2, 2); else AKAP_TP(4, 2);
  } else {
    if (NT <= 8) AKAP_TP(2, 1); else if (NT <= 16) AKAP_TP(4, 1); else AKAP_TP(8, 1);
  }
#undef AKAP_TP
}

}  // namespace akap_stream
