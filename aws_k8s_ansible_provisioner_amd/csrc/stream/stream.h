// Launchers of the fp32-residual-stream kernels (library _C_stream.so, torch.ops.akap_stream).
//
// Activations, weights and the KV cache are bf16 or fp32 (`f32` flags below); norms, rotary
// angles, attention scores / softmax / gates and the residual sum are fp32 in both.  Every size
// (width, heads, GQA ratio, head size, block size) is a run-time argument.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace akap_stream {

void launch_embed_scaled(float* out, const int64_t* ids, const void* table, bool f32, int rows,
                         int d, int vocab, float scale, hipStream_t s);
// x (fp32, contiguous rows of d) += mult * y (y may be null); out = rmsnorm(x) * w
// (bias: d values of y's type added to every row of y, or null)
void launch_add_norm(void* out, bool out_f32, float* x, const void* y, bool y_f32, int y_stride,
                     const void* bias, float mult, const float* w, int rows, int d,
                     int out_stride, float eps, hipStream_t s);
void launch_relu2(void* out, const void* x, bool f32, int rows, int F, int x_stride,
                  int out_stride, hipStream_t s);

struct ProjParams {
  const void* proj;   // [T, N] fused projection rows
  int proj_stride;
  void* q_out;        // [T, H, D]
  void* k_cache;      // [NB, G, BS, D]
  void* v_cache;
  const int64_t* positions;
  const int64_t* slots;
  const float* cos_sin;  // [max_pos, rot_dims] = [cos | sin], or null
  int max_pos, rot_dims;
  const float* q_w;      // [H D]
  const float* k_w;      // [G D]
  const void* q_b;       // [H D] / [G D] of the projection's type, added to the q / k slices
  const void* k_b;       //   before anything else (the projection's biases), or null
  int T, H, G, D, BS, q_off, k_off;
  int64_t num_slots;     // NB * BS
  float eps;
};
void launch_proj_norm_rope_cache(const ProjParams& p, bool f32, hipStream_t s);

struct AttnParams {
  void* out;            // rows of out_stride elements; head h at columns [h D, (h+1) D)
  int out_stride;
  const void* q;        // [T, H, D]
  const void* k_cache;  // [NB, G, BS, D]
  const void* v_cache;
  const int32_t* block_tables;  // [B, max_blocks]
  int max_blocks;
  const int32_t* seq_lens;      // [B]
  const int32_t* q_start;       // [B + 1] (prefill)
  const int32_t* tile_seq;      // prefill tile map
  const int32_t* tile_row;
  int num_tiles, tile_rows;
  const void* gate;     // [T, H] logits with row stride gate_stride, or null
  int gate_stride;
  const float* sink;    // [H] or null
  float scale;
  int chunk, window;    // 0 = off
  int B, H, G, D, BS, NB;
  // decode split: partial (max, sum) [B, H, parts, 2] and outputs [B, H, parts, D]
  float* ws_ml;
  float* ws_o;
  int num_parts;
};
void launch_sink_attention_prefill(const AttnParams& p, bool f32, hipStream_t s);
void launch_sink_attention_decode(const AttnParams& p, bool f32, hipStream_t s);

// ---- grouped norms, token shift, latent attention, routed experts (latent.hip) ----------------
// x (fp32 rows of d) += y + bias + y2 (each may be null; y / bias of the activation type, y2
// fp32), then out1 = gnorm(x) * w1 and out2 = gnorm(x) * w2 (out2 / w2 may be null), the norm
// taken over `groups` equal consecutive parts of the row
// optional token shift of out1 inside the norm kernel, for batches whose every row is a sequence
// of its own with a distinct slot (decode steps): out1 = h + (state[slot] - h) * mu with h the
// normed row as stored (zeros for position 0), and state[slot] = h.  mu null: no shift.
struct ShiftArgs {
  const float* mu;       // [d]
  void* state;           // [slots, d] of out1's type
  const int32_t* slot;   // [rows]
  const int64_t* pos;    // [rows]
};
void launch_add_group_norm(void* out1, void* out2, bool out_f32, int out1_stride, int out2_stride,
                           float* x, const void* y, bool y_f32, int y_stride, const float* y2,
                           const void* bias, const float* w1, const float* w2, int rows, int d,
                           int groups, float eps, const ShiftArgs& sh, hipStream_t s);
// out[t] = h[t] + (prev - h[t]) * mu; then the last row of each sequence goes to state[slot].
// single: every row is a sequence of its own with a distinct slot (one launch instead of two)
void launch_token_shift(void* out, const void* h, const float* mu, void* state,
                        const int32_t* slot, const int64_t* pos, bool f32, int rows, int d,
                        bool single, hipStream_t s);

struct LatentPrepParams {
  const void* proj;   // [T, N] fused down-projection rows
  int proj_stride;
  void* cq_out;       // [T, q_rank]
  void* cache;        // [NB * BS, kv_rank + rot_dim] or null
  void* vgroups;      // [NB * BS / 8, kv_rank, 8]: the latent again, in 8-token groups, or null
  const int64_t* positions;
  const int64_t* slots;
  const float* cos_sin;  // [max_pos, rot_dim] = [cos | sin]
  int max_pos;
  const float* q_w;      // [q_rank]
  const float* kv_w;     // [kv_rank]
  int T, q_rank, kv_rank, rot_dim, q_off, kv_off;
  int64_t num_slots;
  float eps;
};
void launch_latent_prep(const LatentPrepParams& p, bool f32, hipStream_t s);
// in place: `dims` entries from `offset` of each of the H heads (n entries per head) of a row
void launch_rotate_heads(void* q, int q_stride, int T, int H, int n, int offset, int dims,
                         const int64_t* positions, const float* cos_sin, int max_pos, bool f32,
                         hipStream_t s);

struct LatentAttnParams {
  void* out;            // [H, T, R]
  const void* q_lat;    // [H, T, R]
  const void* q;        // [T, H, q_head]; the rotated part at rot_off of every head
  int q_stride, q_head, rot_off;
  const void* cache;    // [NB * BS, R + r]
  const int32_t* block_tables;  // [B, max_blocks]
  int max_blocks;
  const int32_t* seq_lens;      // [B]
  const int32_t* q_start;       // [B + 1], or null: row t is sequence t
  const int64_t* positions;     // [T]
  float scale;
  int T, B, H, R, r, BS;
  int vec;              // rows of the cache can be read in 16-byte pieces
  // matrix-core kernels only
  const void* vgroups;          // [NB * BS / 8, R, 8]
  int NB;
  const int32_t* tile_seq;      // prefill tile map: sequence and first chunk row of a tile
  const int32_t* tile_row;
  int num_tiles, tile_rows;
  float* ws_ml;                 // decode split: (max, sum) [B, H, parts, 2]
  float* ws_o;                  //               outputs    [B, H, parts, R]
  int num_parts;
};
void launch_latent_attention(const LatentAttnParams& p, bool f32, hipStream_t s);
// bf16, R / r among the built sizes (latent_mfma_sizes), BS % 32 == 0, 16-byte aligned rows
bool latent_mfma_sizes(int R, int r);
void launch_latent_prefill_mfma(const LatentAttnParams& p, hipStream_t s);
void launch_latent_decode_mfma(const LatentAttnParams& p, hipStream_t s);

// out [H, T, N] = a [H, T, K] (strides a_hs / a_ts, unit in k) x w [H, N, K]^T, bf16, K % 16 == 0,
// N % 32 == 0, 16-byte aligned rows; meant for a few rows (one wave per 32 x 32 tile)
void launch_head_matmul(void* out, const void* a, int64_t a_hs, int64_t a_ts, const void* w, int H,
                        int T, int N, int K, hipStream_t s);
void launch_head_gate(void* out, int out_stride, const void* o, const void* gate, int gate_stride,
                      bool per_head, int rows, int H, int V, bool f32, hipStream_t s);
void launch_xielu(void* out, int out_stride, const void* x, int x_stride, const void* bias,
                  const float* act, int rows, int F, bool f32, hipStream_t s);
void launch_moe_route(int32_t* ids, float* w, const void* h, int h_stride, const float* router,
                      const float* corr, int rows, int d, int n, int top, int groups, int keep,
                      bool f32, hipStream_t s);
void launch_relu2_routed(void* out, int out_stride, const void* up, int up_stride,
                         const int32_t* ids, const float* w, int rows, int top, int E, int F,
                         bool f32, hipStream_t s);
void launch_moe_combine(float* out, const void* y, const int32_t* inv, const int32_t* ids,
                        const float* w, const void* h, int h_stride, int rows, int d, int top,
                        int E, int y_rows, bool f32, hipStream_t s);

// ---- sandwich norms, retention, head-mixed attention, logit-top-k routing (retention.hip) -------
// m = ya, or (rms(ya) wa + rms(yb) wb) / 2 when yb is given; x (fp32 rows of d) <- x + rms(m)
// post_w (fresh: x is not read); out = rms(x) next_w.  Every weight has a stride of 1 (d
// entries) or 0 (one number).  ya / yb are both fp32 or both of the activation type.
void launch_post_norm_add_norm(void* out, bool out_f32, int out_stride, float* x, const void* ya,
                               int ya_stride, const void* yb, int yb_stride, bool y_f32,
                               const float* wa, int was, const float* wb, int wbs,
                               const float* post_w, int pws, const float* next_w, int nws,
                               int rows, int d, float eps, bool fresh, hipStream_t s);

struct HeadNormParams {
  const void* proj;   // [T, N] fused projection rows
  int proj_stride;
  void* q_out;        // [T, H, D]
  void* k_cache;      // [NB, G, BS, D]
  void* v_cache;      // [NB, G, BS / 8, Dv, 8]
  const int64_t* slots;
  int T, H, G, D, Dv, BS, q_off, k_off, v_off;
  int64_t num_slots;  // NB * BS
  float eps;
  bool norm_qk, norm_v;
};
void launch_head_norm_cache(const HeadNormParams& p, bool f32, hipStream_t s);

struct RetentionParams {
  void* out;            // rows of out_stride elements; head h at columns [h V, (h + 1) V)
  int out_stride;
  const void* proj;     // [T, N] fused projection rows
  int proj_stride;
  int q_off, k_off, v_off, g_off;
  float* state;         // [slots, H, V, D]: the transposed state of every slot and head
  int num_slots;
  const int32_t* seq_slot;   // [T]
  const int64_t* positions;  // [T]
  const int32_t* q_start;    // [num_seqs + 1] or null (row t is sequence t)
  const float* cos_sin;      // [max_pos, rot_dims] = [cos | sin] or null
  int rot_dims;
  const float* log2_decay;   // [H]
  int num_seqs, H, D, V;
  float eps;
  // segmented form (long prompt chunks, q_start given): states of the segments of SEG rows,
  // [num_segs, H, V, D] with num_segs = T / SEG + num_seqs; null: the direct form
  float* seg_buf;
  int SEG, num_segs;
  int DP, TC;           // set by the launcher
};
// 0 when the sizes do not fit a workgroup (ceil(V / 4) column groups x D / 32 lanes > 512)
int retention_dreg(int D, int V);
void launch_retention(RetentionParams p, bool f32, hipStream_t s);

struct TalkParams {
  void* out;            // rows of out_stride elements; head h at columns [h Dv, (h + 1) Dv)
  int out_stride;
  const void* q;        // [T, H, D]
  const void* k_cache;  // [NB, G, BS, D]
  const void* v_cache;  // [NB, G, BS / 8, Dv, 8]
  const int32_t* block_tables;  // [B, max_blocks]
  int max_blocks;
  const int32_t* seq_lens;      // [B]
  const int32_t* q_start;       // [B + 1] or null (row t is sequence t)
  const int64_t* positions;     // [T]
  const float* talk;    // [H, H] or null
  const void* gate;     // [T, H Dv] logits with row stride gate_stride, or null
  int gate_stride;
  float scale;
  int T, B, H, G, D, Dv, BS;
  // split form: (max, sum) [T, parts, H, 2] and unnormalised sums [T, parts, H, G Dv]
  float* ws_ml;
  float* ws_o;
  int num_parts;
  int row0;             // first row of a merge-only launch
};
size_t talking_attention_lds(int H, int D);
void launch_talking_attention(const TalkParams& p, bool f32, hipStream_t s);
void launch_talking_merge(const TalkParams& p, bool f32, hipStream_t s);
// matrix-core form for prompt chunks (bf16): fills the workspace of a one-partition split for
// the rows of the tile map (tile_seq / tile_row: sequence and first chunk row of a tile of
// tile_rows tokens, a multiple of 32); launch_talking_merge finishes
bool talk_mfma_supported(int H, int G, int D, int Dv, int BS);
// matrix-core form for one query per sequence (q_start null): fills the workspace of the
// num_parts-way split; launch_talking_merge finishes
void launch_talking_decode_mfma(const TalkParams& p, hipStream_t s);
void launch_talking_prefill_mfma(const TalkParams& p, const int32_t* tile_seq,
                                 const int32_t* tile_row, int num_tiles, int tile_rows,
                                 hipStream_t s);

void launch_route_topk(int32_t* ids, float* w, const void* h, int h_stride, const float* router,
                       const float* bias, int rows, int d, int n, int top, bool f32,
                       hipStream_t s);
// ids null: every weight is 1 (E = 1: a plain gated activation of [gate | up] rows)
// act 0: silu on the gate, 1: the tanh form of gelu
void launch_swiglu_routed(void* out, int out_stride, const void* gu, int gu_stride,
                          const int32_t* ids, const float* w, int rows, int top, int E, int F,
                          bool f32, int act, hipStream_t s);

// ---- several residual streams, state-space mixer, sigmoid group routing (hyper.hip) -----------
// xs [rows, S, d] fp32 in place: every stream from the old ones, xs_r <- sum_s mix[s, r] xs_s +
// w_out[r] (ya + yb + bias) (fresh: every stream <- fresh row); then u = sum_s w_in[s] xs_s and
// out = rmsnorm(u) * norm_w.  ya / yb rows of bf16 or fp32, each may be null.  S <= 8.
void launch_hyper_step(void* out, bool out_f32, int out_stride, float* xs, const float* fresh,
                       const void* ya, bool ya_f32, int ya_stride, const void* yb, bool yb_f32,
                       int yb_stride, const float* bias, const float* mix, const float* w_out,
                       const float* w_in, const float* norm_w, int rows, int S, int d, float eps,
                       hipStream_t s);
void launch_softcap(void* x, bool f32, size_t n, float cap, hipStream_t s);
// out = gnorm(y * silu(gate)) * w over `groups` equal parts of the n columns
void launch_gate_group_norm(void* out, int out_stride, const float* y, const void* gate,
                            int gate_stride, const float* w, bool f32, int rows, int n,
                            int groups, float eps, hipStream_t s);
void launch_route_sigmoid(int32_t* ids, float* w, const void* h, int h_stride, bool f32,
                          const float* router, int rows, int d, int E, int top, int groups,
                          int keep, int group_top, hipStream_t s);
// causal per-channel convolution + silu of columns [off, off + C) of proj, then the sequences'
// last taps - 1 inputs to their slots; B sequences (q_start null: B = T, one row each)
void launch_conv_silu(float* out, const void* proj, int proj_stride, int off, bool f32,
                      void* state, const float* w, const float* b, const int32_t* seq_slot,
                      const int64_t* positions, const int32_t* q_start, int T, int B, int C,
                      int taps, hipStream_t s);
// state rows a thread of the one-column scan keeps in registers (at most 64); can a head of V
// channels with N-entry states run (either form)?
int selective_scan_rows(int V, int N);
bool selective_scan_supported(int V, int N);
void launch_selective_scan(float* y, const float* xbc, const void* proj, int proj_stride,
                           int dt_off, bool f32, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, const int32_t* seq_slot,
                           const int64_t* positions, const int32_t* q_start, int T, int B, int H,
                           int V, int N, int G, hipStream_t s);

// ---- window + pooled blocks attention (pooled_attention.hip) -----------------------------------
struct RopeCacheParams {
  const void* proj;      // [T, N] fused projection rows
  int proj_stride;
  void* q_out;           // [T, H, D]
  void* k_cache;         // [NB, G, BS, D]
  void* v_cache;         // [NB, G, BS / 8, Dv, 8]
  const int64_t* positions;
  const int64_t* slots;
  const float* cos_sin;  // [max_pos, rot_dims] = [cos | sin], or null
  const float* bias;     // [N] laid out like proj's columns, or null
  int max_pos, rot_dims;
  int T, H, G, D, Dv, BS, q_off, k_off, v_off;
  int64_t num_slots;
};
void launch_bias_rope_cache(const RopeCacheParams& p, bool f32, hipStream_t s);

struct PoolParams {
  const void* k_cache;
  const void* v_cache;
  float* k_pool;         // [NB, G, PS, D]
  float* v_pool;
  const int64_t* positions;
  const int64_t* slots;
  const int32_t* block_tables;
  const int32_t* q_start;   // [B + 1] or null
  int max_blocks, T, B, G, D, Dv, BS, PS, pool;
};
void launch_pool_cache_blocks(const PoolParams& p, bool f32, hipStream_t s);

struct PoolAttnParams {
  void* out;             // rows of out_stride; head h at columns [h Dv, (h + 1) Dv)
  int out_stride;
  const void* q;         // [T, H, D]
  const void* k_cache;
  const void* v_cache;
  const float* k_pool;   // or null (pool 0)
  const float* v_pool;
  const int32_t* block_tables;
  const int32_t* q_start;
  const int64_t* positions;
  const int64_t* slots;
  float scale;
  int max_blocks, T, B, H, G, D, Dv, BS, PS, window, pool, unit_sink;
};
void launch_pooled_window_attention(const PoolAttnParams& p, bool f32, hipStream_t s);
// matrix-core form for prompt chunks (bf16): the rows of the tile map (tile_seq / tile_row:
// sequence and first chunk row of a tile of 128 tokens)
bool pooled_mfma_supported(int H, int G, int D, int Dv, int BS);
void launch_pooled_window_prefill_mfma(const PoolAttnParams& p, const int32_t* tile_seq,
                                       const int32_t* tile_row, int num_tiles, hipStream_t s);
// matrix-core form for one query per sequence (row t = sequence t, the first `rows` rows): the
// query heads of a key/value head are the columns of a tile, the key range is split over the
// workgroup's waves
void launch_pooled_window_decode_mfma(const PoolAttnParams& p, int rows, hipStream_t s);

}  // namespace akap_stream
