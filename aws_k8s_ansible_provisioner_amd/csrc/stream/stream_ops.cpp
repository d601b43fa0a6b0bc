// torch custom-op registrations (namespace `akap_stream`) of the fp32-residual-stream kernels.
//
// Like the core ops: every op launches on the caller's current HIP stream, allocates nothing
// and never synchronises (hipGraph-capturable).  Operand shapes are checked here, on the host,
// against what the kernels index.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include "stream.h"

namespace {

using at::Tensor;

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define CHECK_GPU(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_LAST_CONTIG(x) TORCH_CHECK((x).stride(-1) == 1, #x " must have unit last stride")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_F32(x) TORCH_CHECK((x).scalar_type() == at::kFloat, #x " must be fp32")

// the activation type of an op: bf16 (false) or fp32 (true)
bool is_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name,
              " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

void embed_scaled(Tensor out, Tensor ids, Tensor table, double scale) {
  CHECK_GPU(out); CHECK_GPU(ids); CHECK_GPU(table);
  CHECK_F32(out); CHECK_CONTIG(out); CHECK_CONTIG(table); CHECK_CONTIG(ids);
  TORCH_CHECK(ids.scalar_type() == at::kLong, "ids must be int64");
  TORCH_CHECK(table.dim() == 2 && out.dim() == 2 && out.size(1) == table.size(1) &&
                  out.size(0) == ids.numel(), "embed_scaled: shapes");
  const c10::DeviceGuard g(out.device());
  akap_stream::launch_embed_scaled(out.data_ptr<float>(), ids.data_ptr<int64_t>(), table.data_ptr(),
                                   is_f32(table, "table"), (int)ids.numel(), (int)table.size(1),
                                   (int)table.size(0), (float)scale, cur_stream());
}

void add_norm(Tensor out, Tensor x, std::optional<Tensor> y, double mult, Tensor w, double eps,
              std::optional<Tensor> bias) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_GPU(w);
  CHECK_F32(x); CHECK_CONTIG(x); CHECK_F32(w); CHECK_CONTIG(w); CHECK_LAST_CONTIG(out);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes(), "add_norm: shapes");
  const int rows = x.size(0), d = x.size(1);
  TORCH_CHECK(w.numel() == d, "add_norm: weight size");
  const void* yp = nullptr;
  bool yf = false;
  int ys = 0;
  if (y.has_value()) {
    CHECK_GPU(*y); CHECK_LAST_CONTIG(*y);
    TORCH_CHECK(y->dim() == 2 && y->sizes() == x.sizes(), "add_norm: y shape");
    yp = y->data_ptr();
    yf = is_f32(*y, "y");
    ys = y->stride(0);
  }
  const void* bp = nullptr;
  if (bias.has_value()) {
    TORCH_CHECK(y.has_value(), "add_norm: a bias needs y");
    CHECK_GPU(*bias); CHECK_CONTIG(*bias);
    TORCH_CHECK(bias->numel() == d && bias->scalar_type() == y->scalar_type(),
                "add_norm: bias must be [d] of y's dtype");
    bp = bias->data_ptr();
  }
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_add_norm(out.data_ptr(), is_f32(out, "out"), x.data_ptr<float>(), yp, yf, ys,
                               bp, (float)mult, w.data_ptr<float>(), rows, d, (int)out.stride(0),
                               (float)eps, cur_stream());
}

void relu2(Tensor out, Tensor x) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(x);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes(), "relu2: shapes");
  TORCH_CHECK(out.scalar_type() == x.scalar_type(), "relu2: dtypes differ");
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_relu2(out.data_ptr(), x.data_ptr(), is_f32(x, "x"), (int)x.size(0),
                            (int)x.size(1), (int)x.stride(0), (int)out.stride(0), cur_stream());
}

void check_cache(const Tensor& k_cache, const Tensor& v_cache, int64_t G, int64_t D) {
  CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 5 &&
                  k_cache.scalar_type() == v_cache.scalar_type(),
              "caches must be K [NB, G, BS, D] and V [NB, G, BS/8, D, 8]");
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D, "cache does not match G / D");
  TORCH_CHECK(k_cache.size(2) % 8 == 0 && v_cache.size(0) == k_cache.size(0) &&
                  v_cache.size(1) == G && v_cache.size(2) * 8 == k_cache.size(2) &&
                  v_cache.size(3) == D && v_cache.size(4) == 8, "V cache does not match K cache");
  TORCH_CHECK(k_cache.size(0) * G * k_cache.size(2) < (1LL << 31), "cache has too many rows");
}

void proj_norm_rope_cache(Tensor proj, Tensor q_out, Tensor k_cache, Tensor v_cache,
                          Tensor positions, Tensor slots, std::optional<Tensor> cos_sin,
                          Tensor q_w, Tensor k_w, int64_t H, int64_t G, int64_t D, int64_t q_off,
                          int64_t k_off, double eps, std::optional<Tensor> q_b,
                          std::optional<Tensor> k_b) {
  CHECK_GPU(proj); CHECK_LAST_CONTIG(proj); CHECK_GPU(q_out); CHECK_CONTIG(q_out);
  CHECK_GPU(positions); CHECK_GPU(slots); CHECK_GPU(q_w); CHECK_GPU(k_w);
  CHECK_F32(q_w); CHECK_F32(k_w); CHECK_CONTIG(q_w); CHECK_CONTIG(k_w);
  TORCH_CHECK(positions.scalar_type() == at::kLong && slots.scalar_type() == at::kLong,
              "positions/slots must be int64");
  CHECK_CONTIG(positions); CHECK_CONTIG(slots);
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
                  k_cache.scalar_type() == proj.scalar_type(), "q_out / cache dtype != proj dtype");
  check_cache(k_cache, v_cache, G, D);
  TORCH_CHECK(proj.dim() == 2 && H > 0 && G > 0 && D > 0 && D % 2 == 0, "bad H / G / D");
  const int64_t T = proj.size(0);
  TORCH_CHECK(q_off >= 0 && k_off >= 0 && q_off + H * D <= proj.size(1) &&
                  k_off + G * D <= proj.size(1), "q / k slices outside the projection");
  TORCH_CHECK(q_out.numel() == T * H * D, "q_out size");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "positions/slots too short");
  TORCH_CHECK(q_w.numel() == H * D && k_w.numel() == G * D, "norm weight sizes");
  akap_stream::ProjParams p{};
  if (cos_sin.has_value()) {
    CHECK_GPU(*cos_sin); CHECK_F32(*cos_sin); CHECK_CONTIG(*cos_sin);
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) % 2 == 0 && cos_sin->size(1) <= D,
                "cos_sin must be [max_pos, rot_dims <= D]");
    p.cos_sin = cos_sin->data_ptr<float>();
    p.max_pos = cos_sin->size(0);
    p.rot_dims = cos_sin->size(1);
  }
  if (q_b.has_value()) {
    CHECK_GPU(*q_b); CHECK_CONTIG(*q_b);
    TORCH_CHECK(q_b->numel() == H * D && q_b->scalar_type() == proj.scalar_type(), "q_b: [H D]");
    p.q_b = q_b->data_ptr();
  }
  if (k_b.has_value()) {
    CHECK_GPU(*k_b); CHECK_CONTIG(*k_b);
    TORCH_CHECK(k_b->numel() == G * D && k_b->scalar_type() == proj.scalar_type(), "k_b: [G D]");
    p.k_b = k_b->data_ptr();
  }
  p.proj = proj.data_ptr();
  p.proj_stride = proj.stride(0);
  p.q_out = q_out.data_ptr();
  p.k_cache = k_cache.data_ptr();
  p.v_cache = v_cache.data_ptr();
  p.positions = positions.data_ptr<int64_t>();
  p.slots = slots.data_ptr<int64_t>();
  p.q_w = q_w.data_ptr<float>();
  p.k_w = k_w.data_ptr<float>();
  p.T = T; p.H = H; p.G = G; p.D = D; p.BS = k_cache.size(2);
  p.q_off = q_off; p.k_off = k_off;
  p.num_slots = k_cache.size(0) * k_cache.size(2);
  p.eps = (float)eps;
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_proj_norm_rope_cache(p, f32, cur_stream());
}

// fields shared by the prefill and decode attention ops
akap_stream::AttnParams attn_params(const Tensor& out, const Tensor& q, const Tensor& k_cache,
                                    const Tensor& v_cache, const Tensor& block_tables,
                                    const Tensor& seq_lens, const std::optional<Tensor>& gate,
                                    const std::optional<Tensor>& sink, double scale, int64_t chunk,
                                    int64_t window) {
  CHECK_GPU(out); CHECK_GPU(q); CHECK_GPU(block_tables); CHECK_GPU(seq_lens);
  CHECK_LAST_CONTIG(out); CHECK_CONTIG(q); CHECK_CONTIG(block_tables); CHECK_CONTIG(seq_lens);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 2, "q must be [T, H, D], out [T, >= H D]");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  const int64_t G = k_cache.size(1);
  check_cache(k_cache, v_cache, G, D);
  TORCH_CHECK(H % G == 0, "H must be a multiple of G");
  TORCH_CHECK(D <= 256, "head size above 256 is not supported");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && k_cache.scalar_type() == q.scalar_type(),
              "out / cache dtype != q dtype");
  TORCH_CHECK(out.size(0) == T && out.size(1) >= H * D, "out too small");
  TORCH_CHECK(block_tables.scalar_type() == at::kInt && seq_lens.scalar_type() == at::kInt &&
                  block_tables.dim() == 2 && block_tables.size(0) >= seq_lens.numel(),
              "block_tables [B, max_blocks] / seq_lens [B] must be int32");
  TORCH_CHECK(chunk >= 0 && window >= 0, "chunk / window must be >= 0");
  akap_stream::AttnParams p{};
  p.out = out.data_ptr();
  p.out_stride = out.stride(0);
  p.q = q.data_ptr();
  p.k_cache = k_cache.data_ptr();
  p.v_cache = v_cache.data_ptr();
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.max_blocks = block_tables.size(1);
  p.seq_lens = seq_lens.data_ptr<int32_t>();
  p.B = seq_lens.numel();
  if (gate.has_value()) {
    CHECK_GPU(*gate); CHECK_LAST_CONTIG(*gate);
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H &&
                    gate->scalar_type() == q.scalar_type(), "gate must be [T, H] of q's dtype");
    p.gate = gate->data_ptr();
    p.gate_stride = gate->stride(0);
  }
  if (sink.has_value()) {
    CHECK_GPU(*sink); CHECK_F32(*sink); CHECK_CONTIG(*sink);
    TORCH_CHECK(sink->numel() == H, "sink must be [H]");
    p.sink = sink->data_ptr<float>();
  }
  p.scale = (float)scale;
  p.chunk = chunk; p.window = window;
  p.H = H; p.G = G; p.D = D; p.BS = k_cache.size(2); p.NB = k_cache.size(0);
  p.num_parts = 1;
  return p;
}

void sink_attention_prefill(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                            Tensor block_tables, Tensor seq_lens, Tensor q_start, Tensor tile_seq,
                            Tensor tile_row, int64_t tile_rows, std::optional<Tensor> gate,
                            std::optional<Tensor> sink, double scale, int64_t chunk,
                            int64_t window) {
  auto p = attn_params(out, q, k_cache, v_cache, block_tables, seq_lens, gate, sink, scale, chunk,
                       window);
  CHECK_GPU(q_start); CHECK_GPU(tile_seq); CHECK_GPU(tile_row);
  CHECK_CONTIG(q_start); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_row);
  TORCH_CHECK(q_start.scalar_type() == at::kInt && tile_seq.scalar_type() == at::kInt &&
                  tile_row.scalar_type() == at::kInt, "q_start / tile map must be int32");
  TORCH_CHECK(q_start.numel() >= p.B + 1 && tile_seq.numel() == tile_row.numel(),
              "q_start / tile map sizes");
  TORCH_CHECK(tile_rows > 0, "tile_rows must be positive");
  p.q_start = q_start.data_ptr<int32_t>();
  p.tile_seq = tile_seq.data_ptr<int32_t>();
  p.tile_row = tile_row.data_ptr<int32_t>();
  p.num_tiles = tile_seq.numel();
  p.tile_rows = tile_rows;
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_sink_attention_prefill(p, is_f32(q, "q"), cur_stream());
}

void sink_attention_decode(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                           Tensor block_tables, Tensor seq_lens, std::optional<Tensor> gate,
                           std::optional<Tensor> sink, double scale, int64_t chunk, int64_t window,
                           std::optional<Tensor> ws_ml, std::optional<Tensor> ws_o,
                           int64_t num_parts) {
  auto p = attn_params(out, q, k_cache, v_cache, block_tables, seq_lens, gate, sink, scale, chunk,
                       window);
  TORCH_CHECK(q.size(0) == p.B, "decode: one query row per sequence");
  TORCH_CHECK(num_parts >= 1 && num_parts <= 65535, "num_parts out of range");
  TORCH_CHECK(p.H <= 65535, "too many heads");
  p.num_parts = num_parts;
  if (num_parts > 1) {
    TORCH_CHECK(ws_ml.has_value() && ws_o.has_value(), "split decode needs a workspace");
    CHECK_GPU(*ws_ml); CHECK_GPU(*ws_o); CHECK_F32(*ws_ml); CHECK_F32(*ws_o);
    CHECK_CONTIG(*ws_ml); CHECK_CONTIG(*ws_o);
    const int64_t n = (int64_t)p.B * p.H * num_parts;
    TORCH_CHECK(ws_ml->numel() >= 2 * n && ws_o->numel() >= n * p.D, "decode workspace too small");
    p.ws_ml = ws_ml->data_ptr<float>();
    p.ws_o = ws_o->data_ptr<float>();
  }
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_sink_attention_decode(p, is_f32(q, "q"), cur_stream());
}


// ---- grouped norms, token shift, latent attention, routed experts ----------------------------
void add_group_norm(Tensor out1, std::optional<Tensor> out2, Tensor x, std::optional<Tensor> y,
                    std::optional<Tensor> y2, std::optional<Tensor> bias, Tensor w1,
                    std::optional<Tensor> w2, int64_t groups, double eps,
                    std::optional<Tensor> shift_mu, std::optional<Tensor> shift_state,
                    std::optional<Tensor> seq_slot, std::optional<Tensor> positions) {
  CHECK_GPU(out1); CHECK_GPU(x); CHECK_GPU(w1);
  CHECK_F32(x); CHECK_CONTIG(x); CHECK_F32(w1); CHECK_CONTIG(w1); CHECK_LAST_CONTIG(out1);
  TORCH_CHECK(x.dim() == 2 && out1.dim() == 2 && out1.sizes() == x.sizes(),
              "add_group_norm: shapes");
  const int rows = x.size(0), d = x.size(1);
  TORCH_CHECK(groups >= 1 && d % groups == 0, "add_group_norm: d must split into the groups");
  TORCH_CHECK(w1.numel() == d, "add_group_norm: weight size");
  TORCH_CHECK(out1.data_ptr() != x.data_ptr(), "add_group_norm: out1 must not alias x");
  const bool of = is_f32(out1, "out1");
  void* o2 = nullptr;
  const float* w2p = nullptr;
  int o2s = 0;
  if (out2.has_value()) {
    TORCH_CHECK(w2.has_value(), "add_group_norm: out2 needs w2");
    CHECK_GPU(*out2); CHECK_LAST_CONTIG(*out2); CHECK_GPU(*w2); CHECK_F32(*w2); CHECK_CONTIG(*w2);
    TORCH_CHECK(out2->sizes() == x.sizes() && out2->scalar_type() == out1.scalar_type() &&
                    w2->numel() == d, "add_group_norm: out2 / w2");
    o2 = out2->data_ptr();
    o2s = out2->stride(0);
    w2p = w2->data_ptr<float>();
  }
  const void* yp = nullptr;
  bool yf = of;
  int ys = 0;
  if (y.has_value()) {
    CHECK_GPU(*y); CHECK_LAST_CONTIG(*y);
    TORCH_CHECK(y->dim() == 2 && y->sizes() == x.sizes(), "add_group_norm: y shape");
    yp = y->data_ptr();
    yf = is_f32(*y, "y");
    ys = y->stride(0);
  }
  const void* bp = nullptr;
  if (bias.has_value()) {
    CHECK_GPU(*bias); CHECK_CONTIG(*bias);
    TORCH_CHECK(bias->numel() == d, "add_group_norm: bias must be [d]");
    if (y.has_value()) {
      TORCH_CHECK(bias->scalar_type() == y->scalar_type(), "bias dtype != y dtype");
    } else {
      yf = is_f32(*bias, "bias");
    }
    bp = bias->data_ptr();
  }
  const float* y2p = nullptr;
  if (y2.has_value()) {
    CHECK_GPU(*y2); CHECK_F32(*y2); CHECK_CONTIG(*y2);
    TORCH_CHECK(y2->sizes() == x.sizes(), "add_group_norm: y2 shape");
    y2p = y2->data_ptr<float>();
  }
  akap_stream::ShiftArgs sh{};
  if (shift_mu.has_value()) {
    TORCH_CHECK(shift_state.has_value() && seq_slot.has_value() && positions.has_value(),
                "add_group_norm: the shift needs state, slots and positions");
    CHECK_GPU(*shift_mu); CHECK_F32(*shift_mu); CHECK_CONTIG(*shift_mu);
    CHECK_GPU(*shift_state); CHECK_CONTIG(*shift_state); CHECK_GPU(*seq_slot); CHECK_CONTIG(*seq_slot);
    CHECK_GPU(*positions); CHECK_CONTIG(*positions);
    TORCH_CHECK(shift_mu->numel() == d && shift_state->dim() == 2 && shift_state->size(1) == d &&
                    shift_state->scalar_type() == out1.scalar_type(), "add_group_norm: shift shapes");
    TORCH_CHECK(seq_slot->scalar_type() == at::kInt && positions->scalar_type() == at::kLong &&
                    seq_slot->numel() >= rows && positions->numel() >= rows,
                "add_group_norm: seq_slot int32 / positions int64 per row");
    sh.mu = shift_mu->data_ptr<float>();
    sh.state = shift_state->data_ptr();
    sh.slot = seq_slot->data_ptr<int32_t>();
    sh.pos = positions->data_ptr<int64_t>();
  }
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_add_group_norm(out1.data_ptr(), o2, of, (int)out1.stride(0), o2s,
                                     x.data_ptr<float>(), yp, yf, ys, y2p, bp,
                                     w1.data_ptr<float>(), w2p, rows, d, (int)groups, (float)eps,
                                     sh, cur_stream());
}

void token_shift(Tensor out, Tensor h, Tensor mu, Tensor state, Tensor seq_slot, Tensor positions,
                 bool single) {
  CHECK_GPU(out); CHECK_GPU(h); CHECK_GPU(mu); CHECK_GPU(state); CHECK_GPU(seq_slot);
  CHECK_GPU(positions);
  CHECK_CONTIG(out); CHECK_CONTIG(h); CHECK_CONTIG(mu); CHECK_CONTIG(state); CHECK_CONTIG(seq_slot);
  CHECK_CONTIG(positions); CHECK_F32(mu);
  TORCH_CHECK(h.dim() == 2 && out.sizes() == h.sizes() && state.dim() == 2, "token_shift: shapes");
  const int64_t T = h.size(0), d = h.size(1);
  TORCH_CHECK(out.scalar_type() == h.scalar_type() && state.scalar_type() == h.scalar_type(),
              "token_shift: dtypes differ");
  TORCH_CHECK(out.data_ptr() != h.data_ptr(), "token_shift: out must not alias h");
  TORCH_CHECK(mu.numel() == d && state.size(1) == d, "token_shift: width");
  TORCH_CHECK(seq_slot.scalar_type() == at::kInt && positions.scalar_type() == at::kLong,
              "token_shift: seq_slot int32, positions int64");
  TORCH_CHECK(seq_slot.numel() >= T && positions.numel() >= T, "token_shift: per-row inputs");
  // slots index state rows: checked on the host side of the scheduler (slots < pool size)
  const c10::DeviceGuard g(h.device());
  akap_stream::launch_token_shift(out.data_ptr(), h.data_ptr(), mu.data_ptr<float>(),
                                  state.data_ptr(), seq_slot.data_ptr<int32_t>(),
                                  positions.data_ptr<int64_t>(), is_f32(h, "h"), (int)T, (int)d,
                                  single, cur_stream());
}

void latent_prep(Tensor proj, Tensor cq_out, std::optional<Tensor> cache, Tensor positions,
                 Tensor slots, Tensor cos_sin, Tensor q_w, std::optional<Tensor> kv_w,
                 int64_t q_rank, int64_t kv_rank, int64_t rot_dim, int64_t q_off, int64_t kv_off,
                 double eps, std::optional<Tensor> vgroups) {
  CHECK_GPU(proj); CHECK_LAST_CONTIG(proj); CHECK_GPU(cq_out); CHECK_CONTIG(cq_out);
  CHECK_GPU(positions); CHECK_GPU(slots); CHECK_CONTIG(positions); CHECK_CONTIG(slots);
  CHECK_GPU(cos_sin); CHECK_F32(cos_sin); CHECK_CONTIG(cos_sin);
  CHECK_GPU(q_w); CHECK_F32(q_w); CHECK_CONTIG(q_w);
  TORCH_CHECK(positions.scalar_type() == at::kLong && slots.scalar_type() == at::kLong,
              "positions/slots must be int64");
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(proj.dim() == 2 && cq_out.scalar_type() == proj.scalar_type(), "latent_prep: proj");
  const int64_t T = proj.size(0);
  TORCH_CHECK(q_rank > 0 && q_off >= 0 && q_off + q_rank <= proj.size(1), "q slice");
  TORCH_CHECK(cq_out.numel() == T * q_rank && q_w.numel() == q_rank, "cq_out / q_w size");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "positions/slots too short");
  akap_stream::LatentPrepParams p{};
  p.proj = proj.data_ptr();
  p.proj_stride = proj.stride(0);
  p.cq_out = cq_out.data_ptr();
  p.positions = positions.data_ptr<int64_t>();
  p.slots = slots.data_ptr<int64_t>();
  p.cos_sin = cos_sin.data_ptr<float>();
  p.max_pos = cos_sin.size(0);
  p.q_w = q_w.data_ptr<float>();
  p.T = T; p.q_rank = q_rank; p.kv_rank = kv_rank; p.rot_dim = rot_dim; p.q_off = q_off;
  p.kv_off = kv_off;
  p.eps = (float)eps;
  if (cache.has_value()) {
    CHECK_GPU(*cache); CHECK_CONTIG(*cache);
    TORCH_CHECK(kv_w.has_value(), "latent_prep: a cache needs kv_w");
    CHECK_GPU(*kv_w); CHECK_F32(*kv_w); CHECK_CONTIG(*kv_w);
    TORCH_CHECK(cache->dim() == 3 && cache->size(2) == kv_rank + rot_dim &&
                    cache->scalar_type() == proj.scalar_type(), "latent cache [NB, BS, R + r]");
    TORCH_CHECK(kv_rank > 0 && rot_dim > 0 && rot_dim % 2 == 0 && kv_off >= 0 &&
                    kv_off + kv_rank + rot_dim <= proj.size(1), "kv slice");
    TORCH_CHECK(kv_w->numel() == kv_rank && cos_sin.dim() == 2 && cos_sin.size(1) == rot_dim,
                "kv_w / rotary table size");
    p.cache = cache->data_ptr();
    p.kv_w = kv_w->data_ptr<float>();
    p.num_slots = cache->size(0) * cache->size(1);
    if (vgroups.has_value()) {
      CHECK_GPU(*vgroups); CHECK_CONTIG(*vgroups);
      TORCH_CHECK(vgroups->scalar_type() == cache->scalar_type() && cache->size(1) % 8 == 0 &&
                      vgroups->numel() == cache->size(0) * cache->size(1) * kv_rank,
                  "latent groups must be [NB, BS / 8, R, 8]");
      p.vgroups = vgroups->data_ptr();
    }
  }
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_latent_prep(p, f32, cur_stream());
}

void rotate_heads(Tensor q, Tensor positions, Tensor cos_sin, int64_t offset) {
  CHECK_GPU(q); CHECK_GPU(positions); CHECK_GPU(cos_sin); CHECK_F32(cos_sin); CHECK_CONTIG(cos_sin);
  CHECK_CONTIG(positions);
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2), "q must be [T, H, n]");
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.numel() >= q.size(0), "positions");
  const int64_t dims = cos_sin.size(1);
  TORCH_CHECK(cos_sin.dim() == 2 && dims % 2 == 0 && offset >= 0 && offset + dims <= q.size(2),
              "rotated part outside the head");
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_rotate_heads(q.data_ptr(), (int)q.stride(0), (int)q.size(0), (int)q.size(1),
                                   (int)q.size(2), (int)offset, (int)dims,
                                   positions.data_ptr<int64_t>(), cos_sin.data_ptr<float>(),
                                   (int)cos_sin.size(0), is_f32(q, "q"), cur_stream());
}

void latent_attention(Tensor out, Tensor q_lat, Tensor q, int64_t rot_off, Tensor cache,
                      Tensor block_tables, Tensor seq_lens, std::optional<Tensor> q_start,
                      Tensor positions, double scale) {
  CHECK_GPU(out); CHECK_GPU(q_lat); CHECK_GPU(q); CHECK_GPU(cache); CHECK_GPU(block_tables);
  CHECK_GPU(seq_lens); CHECK_GPU(positions);
  CHECK_CONTIG(out); CHECK_CONTIG(q_lat); CHECK_CONTIG(cache); CHECK_CONTIG(seq_lens);
  CHECK_CONTIG(positions);
  const bool f32 = is_f32(q, "q");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && q_lat.scalar_type() == q.scalar_type() &&
                  cache.scalar_type() == q.scalar_type(), "latent_attention: dtypes differ");
  TORCH_CHECK(q_lat.dim() == 3 && out.sizes() == q_lat.sizes() && q.dim() == 3 &&
                  q.stride(2) == 1 && q.stride(1) == q.size(2), "latent_attention: q shapes");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), R = q_lat.size(2);
  TORCH_CHECK(q.size(0) == T && q.size(1) == H, "latent_attention: q is [T, H, n]");
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) > R, "latent cache [NB, BS, R + r]");
  const int64_t r = cache.size(2) - R;
  TORCH_CHECK(rot_off >= 0 && rot_off + r <= q.size(2), "rotated query part outside the head");
  TORCH_CHECK(R <= 1024, "latent size over 1024");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.scalar_type() == at::kInt &&
                  block_tables.stride(1) == 1, "block_tables");
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && positions.scalar_type() == at::kLong &&
                  positions.numel() >= T, "seq_lens int32, positions int64");
  const int64_t B = seq_lens.numel();
  TORCH_CHECK(block_tables.size(0) >= B, "block table rows");
  TORCH_CHECK(block_tables.size(1) * cache.size(1) < (1LL << 31), "sequence too long");
  akap_stream::LatentAttnParams p{};
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_CONTIG(*q_start);
    TORCH_CHECK(q_start->scalar_type() == at::kInt && q_start->numel() >= B + 1, "q_start");
    p.q_start = q_start->data_ptr<int32_t>();
  } else {
    TORCH_CHECK(B >= T, "one query per sequence needs a sequence per row");
  }
  p.out = out.data_ptr();
  p.q_lat = q_lat.data_ptr();
  p.q = q.data_ptr();
  p.q_stride = q.stride(0);
  p.q_head = q.size(2);
  p.rot_off = rot_off;
  p.cache = cache.data_ptr();
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.max_blocks = block_tables.stride(0);
  p.seq_lens = seq_lens.data_ptr<int32_t>();
  p.positions = positions.data_ptr<int64_t>();
  p.scale = (float)scale;
  p.T = T; p.B = B; p.H = H; p.R = R; p.r = r; p.BS = cache.size(1);
  const int64_t es = f32 ? 4 : 2;
  p.vec = ((R + r) * es) % 16 == 0 && ((uintptr_t)cache.data_ptr() % 16) == 0;
  TORCH_CHECK(4 * (R + r) * 4 <= 64 * 1024, "query rows do not fit the LDS");
  TORCH_CHECK((H + 3) / 4 <= 65535, "too many heads");
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_latent_attention(p, f32, cur_stream());
}

// operands common to the two matrix-core launches
akap_stream::LatentAttnParams latent_mfma_params(const Tensor& out, const Tensor& q_lat,
                                                 const Tensor& q, int64_t rot_off,
                                                 const Tensor& cache, const Tensor& vgroups,
                                                 const Tensor& block_tables,
                                                 const Tensor& seq_lens, double scale) {
  CHECK_GPU(out); CHECK_GPU(q_lat); CHECK_GPU(q); CHECK_GPU(cache); CHECK_GPU(vgroups);
  CHECK_GPU(block_tables); CHECK_GPU(seq_lens);
  CHECK_CONTIG(out); CHECK_CONTIG(q_lat); CHECK_CONTIG(cache); CHECK_CONTIG(vgroups);
  CHECK_CONTIG(seq_lens);
  for (const Tensor* t : {&out, &q_lat, &q, &cache, &vgroups})
    TORCH_CHECK(t->scalar_type() == at::kBFloat16, "matrix-core latent attention is bf16");
  TORCH_CHECK(q_lat.dim() == 3 && out.sizes() == q_lat.sizes() && q.dim() == 3 &&
                  q.stride(2) == 1 && q.stride(1) == q.size(2), "latent attention: q shapes");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), R = q_lat.size(2);
  TORCH_CHECK(q.size(0) == T && q.size(1) == H, "latent attention: q is [T, H, n]");
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) > R, "latent cache [NB, BS, R + r]");
  const int64_t r = cache.size(2) - R, BS = cache.size(1);
  TORCH_CHECK(akap_stream::latent_mfma_sizes((int)R, (int)r) && BS % 32 == 0,
              "latent sizes / block size not built for the matrix cores");
  TORCH_CHECK(vgroups.numel() == cache.size(0) * BS * R, "latent groups [NB, BS / 8, R, 8]");
  TORCH_CHECK(rot_off >= 0 && rot_off + r <= q.size(2) && rot_off % 8 == 0 && q.size(2) % 8 == 0 &&
                  q.stride(0) % 8 == 0 && scale > 0, "rotated query part: place / alignment");
  for (const Tensor* t : {&q_lat, &q, &cache, &vgroups})
    TORCH_CHECK((uintptr_t)t->data_ptr() % 16 == 0, "operands must be 16-byte aligned");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.scalar_type() == at::kInt &&
                  block_tables.stride(1) == 1 && seq_lens.scalar_type() == at::kInt &&
                  block_tables.size(0) >= seq_lens.numel(), "block_tables / seq_lens");
  TORCH_CHECK(cache.size(0) * BS < (1LL << 31), "cache has too many rows");
  // (wide latents keep one row index per 32-key block of a sequence in LDS)
  TORCH_CHECK(block_tables.size(1) * (BS / 32) <= 16384, "block table too long for the LDS");
  akap_stream::LatentAttnParams p{};
  p.out = out.data_ptr();
  p.q_lat = q_lat.data_ptr();
  p.q = q.data_ptr();
  p.q_stride = q.stride(0);
  p.q_head = q.size(2);
  p.rot_off = rot_off;
  p.cache = cache.data_ptr();
  p.vgroups = vgroups.data_ptr();
  p.NB = cache.size(0);
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.max_blocks = block_tables.stride(0);
  p.seq_lens = seq_lens.data_ptr<int32_t>();
  p.scale = (float)scale;
  p.T = T; p.B = seq_lens.numel(); p.H = H; p.R = R; p.r = r; p.BS = BS;
  p.num_parts = 1;
  return p;
}

void latent_attention_prefill_mfma(Tensor out, Tensor q_lat, Tensor q, int64_t rot_off,
                                   Tensor cache, Tensor vgroups, Tensor block_tables,
                                   Tensor seq_lens, Tensor q_start, Tensor tile_seq,
                                   Tensor tile_row, int64_t tile_rows, double scale) {
  auto p = latent_mfma_params(out, q_lat, q, rot_off, cache, vgroups, block_tables, seq_lens, scale);
  CHECK_GPU(q_start); CHECK_GPU(tile_seq); CHECK_GPU(tile_row);
  CHECK_CONTIG(q_start); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_row);
  TORCH_CHECK(q_start.scalar_type() == at::kInt && tile_seq.scalar_type() == at::kInt &&
                  tile_row.scalar_type() == at::kInt, "int32 tile map");
  TORCH_CHECK(q_start.numel() >= p.B + 1 && tile_row.numel() >= tile_seq.numel(), "tile map sizes");
  TORCH_CHECK(tile_rows >= 32 && tile_rows % 32 == 0, "tiles are whole 32-token pieces");
  p.q_start = q_start.data_ptr<int32_t>();
  p.tile_seq = tile_seq.data_ptr<int32_t>();
  p.tile_row = tile_row.data_ptr<int32_t>();
  p.num_tiles = tile_seq.numel();
  p.tile_rows = tile_rows;
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_latent_prefill_mfma(p, cur_stream());
}

void latent_attention_decode_mfma(Tensor out, Tensor q_lat, Tensor q, int64_t rot_off,
                                  Tensor cache, Tensor vgroups, Tensor block_tables,
                                  Tensor seq_lens, double scale, std::optional<Tensor> ws_ml,
                                  std::optional<Tensor> ws_o, int64_t num_parts) {
  auto p = latent_mfma_params(out, q_lat, q, rot_off, cache, vgroups, block_tables, seq_lens, scale);
  TORCH_CHECK(p.T == p.B, "decode: one query row per sequence");
  TORCH_CHECK(num_parts >= 1 && num_parts <= 65535 && p.H <= 65535 * 32, "grid limits");
  p.num_parts = num_parts;
  if (num_parts > 1) {
    TORCH_CHECK(ws_ml.has_value() && ws_o.has_value(), "split decode needs a workspace");
    CHECK_GPU(*ws_ml); CHECK_GPU(*ws_o); CHECK_F32(*ws_ml); CHECK_F32(*ws_o);
    CHECK_CONTIG(*ws_ml); CHECK_CONTIG(*ws_o);
    const int64_t n = (int64_t)p.B * p.H * num_parts;
    TORCH_CHECK(ws_ml->numel() >= 2 * n && ws_o->numel() >= n * p.R, "decode workspace too small");
    p.ws_ml = ws_ml->data_ptr<float>();
    p.ws_o = ws_o->data_ptr<float>();
  }
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_latent_decode_mfma(p, cur_stream());
}

bool latent_mfma_supported(int64_t R, int64_t r) {
  return akap_stream::latent_mfma_sizes((int)R, (int)r);
}

void head_matmul(Tensor out, Tensor a, Tensor w) {
  CHECK_GPU(out); CHECK_GPU(a); CHECK_GPU(w); CHECK_CONTIG(out); CHECK_CONTIG(w);
  TORCH_CHECK(a.dim() == 3 && w.dim() == 3 && out.dim() == 3 && a.stride(2) == 1, "head_matmul: ranks");
  const int64_t H = a.size(0), T = a.size(1), K = a.size(2), N = w.size(1);
  TORCH_CHECK(w.size(0) == H && w.size(2) == K && out.size(0) == H && out.size(1) == T &&
                  out.size(2) == N, "head_matmul: shapes");
  for (const Tensor* t : {&out, &a, &w})
    TORCH_CHECK(t->scalar_type() == at::kBFloat16, "head_matmul is bf16");
  TORCH_CHECK(K % 16 == 0 && N % 32 == 0 && a.stride(0) % 8 == 0 && a.stride(1) % 8 == 0 &&
                  (uintptr_t)a.data_ptr() % 16 == 0 && (uintptr_t)w.data_ptr() % 16 == 0,
              "head_matmul: sizes / alignment");
  TORCH_CHECK(H <= 65535 && (N / 32) * ((T + 31) / 32) < (1LL << 31), "head_matmul: grid");
  const c10::DeviceGuard g(a.device());
  akap_stream::launch_head_matmul(out.data_ptr(), a.data_ptr(), a.stride(0), a.stride(1),
                                  w.data_ptr(), (int)H, (int)T, (int)N, (int)K, cur_stream());
}

void head_gate(Tensor out, Tensor o, Tensor gate) {
  CHECK_GPU(out); CHECK_GPU(o); CHECK_GPU(gate); CHECK_CONTIG(o); CHECK_LAST_CONTIG(out);
  CHECK_LAST_CONTIG(gate);
  TORCH_CHECK(o.dim() == 3 && out.dim() == 2 && gate.dim() == 2, "head_gate: shapes");
  const int64_t H = o.size(0), T = o.size(1), V = o.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * V && gate.size(0) == T &&
                  (gate.size(1) == H || gate.size(1) == H * V), "head_gate: sizes");
  TORCH_CHECK(out.scalar_type() == o.scalar_type() && gate.scalar_type() == o.scalar_type(),
              "head_gate: dtypes differ");
  const c10::DeviceGuard g(o.device());
  // H == H V only when V == 1: per-head and per-entry gates coincide
  akap_stream::launch_head_gate(out.data_ptr(), (int)out.stride(0), o.data_ptr(), gate.data_ptr(),
                                (int)gate.stride(0), gate.size(1) == H, (int)T, (int)H, (int)V,
                                is_f32(o, "o"), cur_stream());
}

void xielu(Tensor out, Tensor x, std::optional<Tensor> bias, Tensor act) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_GPU(act); CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(x);
  CHECK_F32(act); CHECK_CONTIG(act);
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && out.scalar_type() == x.scalar_type() &&
                  act.numel() == 2, "xielu: shapes");
  const void* bp = nullptr;
  if (bias.has_value()) {
    CHECK_GPU(*bias); CHECK_CONTIG(*bias);
    TORCH_CHECK(bias->numel() == x.size(1) && bias->scalar_type() == x.scalar_type(), "xielu: bias");
    bp = bias->data_ptr();
  }
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_xielu(out.data_ptr(), (int)out.stride(0), x.data_ptr(), (int)x.stride(0), bp,
                            act.data_ptr<float>(), (int)x.size(0), (int)x.size(1), is_f32(x, "x"),
                            cur_stream());
}

void moe_route(Tensor ids, Tensor w, Tensor h, Tensor router, std::optional<Tensor> correction,
               int64_t groups, int64_t keep) {
  CHECK_GPU(ids); CHECK_GPU(w); CHECK_GPU(h); CHECK_GPU(router);
  CHECK_CONTIG(ids); CHECK_CONTIG(w); CHECK_LAST_CONTIG(h); CHECK_CONTIG(router);
  CHECK_F32(w); CHECK_F32(router);
  TORCH_CHECK(h.dim() == 2 && router.dim() == 2 && router.size(1) == h.size(1), "moe_route: width");
  const int64_t T = h.size(0), n = router.size(0);
  TORCH_CHECK(ids.scalar_type() == at::kInt && ids.dim() == 2 && ids.size(0) == T &&
                  w.sizes() == ids.sizes(), "moe_route: ids / w [T, top]");
  const int64_t top = ids.size(1);
  TORCH_CHECK(groups >= 1 && n % groups == 0 && keep >= 1 && keep <= groups &&
                  top >= 1 && top <= keep * (n / groups), "moe_route: groups / keep / top");
  TORCH_CHECK((2 * n + groups) * 4 <= 48 * 1024, "moe_route: too many router outputs");
  const float* cp = nullptr;
  if (correction.has_value()) {
    CHECK_GPU(*correction); CHECK_F32(*correction); CHECK_CONTIG(*correction);
    TORCH_CHECK(correction->numel() == n, "moe_route: correction size");
    cp = correction->data_ptr<float>();
  }
  const c10::DeviceGuard g(h.device());
  akap_stream::launch_moe_route(ids.data_ptr<int32_t>(), w.data_ptr<float>(), h.data_ptr(),
                                (int)h.stride(0), router.data_ptr<float>(), cp, (int)T,
                                (int)h.size(1), (int)n, (int)top, (int)groups, (int)keep,
                                is_f32(h, "h"), cur_stream());
}

void relu2_routed(Tensor out, Tensor up, Tensor ids, Tensor w, int64_t experts) {
  CHECK_GPU(out); CHECK_GPU(up); CHECK_GPU(ids); CHECK_GPU(w);
  CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(up); CHECK_CONTIG(ids); CHECK_CONTIG(w); CHECK_F32(w);
  TORCH_CHECK(up.dim() == 2 && out.sizes() == up.sizes() && out.scalar_type() == up.scalar_type(),
              "relu2_routed: shapes");
  TORCH_CHECK(experts >= 1 && up.size(1) % experts == 0 && experts * 4 <= 48 * 1024,
              "relu2_routed: experts");
  TORCH_CHECK(ids.scalar_type() == at::kInt && ids.dim() == 2 && ids.size(0) == up.size(0) &&
                  w.sizes() == ids.sizes() && ids.size(1) <= 256, "relu2_routed: ids / w");
  const c10::DeviceGuard g(up.device());
  akap_stream::launch_relu2_routed(out.data_ptr(), (int)out.stride(0), up.data_ptr(),
                                   (int)up.stride(0), ids.data_ptr<int32_t>(), w.data_ptr<float>(),
                                   (int)up.size(0), (int)ids.size(1), (int)experts,
                                   (int)(up.size(1) / experts), is_f32(up, "up"), cur_stream());
}

void moe_combine(Tensor out, Tensor y, std::optional<Tensor> inv, Tensor ids, Tensor w, Tensor h,
                 int64_t experts) {
  CHECK_GPU(out); CHECK_GPU(y); CHECK_GPU(ids); CHECK_GPU(w); CHECK_GPU(h);
  CHECK_F32(out); CHECK_CONTIG(out); CHECK_CONTIG(y); CHECK_CONTIG(ids); CHECK_CONTIG(w);
  CHECK_F32(w); CHECK_LAST_CONTIG(h);
  TORCH_CHECK(out.dim() == 2 && h.dim() == 2 && h.sizes() == out.sizes() && y.dim() == 2 &&
                  y.size(1) == out.size(1) && y.scalar_type() == h.scalar_type(),
              "moe_combine: shapes");
  const int64_t T = out.size(0);
  TORCH_CHECK(ids.scalar_type() == at::kInt && ids.dim() == 2 && ids.size(0) == T &&
                  w.sizes() == ids.sizes(), "moe_combine: ids / w");
  const int32_t* ip = nullptr;
  if (inv.has_value()) {
    CHECK_GPU(*inv); CHECK_CONTIG(*inv);
    TORCH_CHECK(inv->scalar_type() == at::kInt && inv->numel() == ids.numel(), "moe_combine: inv");
    ip = inv->data_ptr<int32_t>();
  } else {
    TORCH_CHECK(y.size(0) == T, "moe_combine: y rows");
  }
  const c10::DeviceGuard g(out.device());
  akap_stream::launch_moe_combine(out.data_ptr<float>(), y.data_ptr(), ip, ids.data_ptr<int32_t>(),
                                  w.data_ptr<float>(), h.data_ptr(), (int)h.stride(0), (int)T,
                                  (int)out.size(1), (int)ids.size(1), (int)experts, (int)y.size(0),
                                  is_f32(y, "y"), cur_stream());
}

// a norm weight: fp32 with d entries (stride 1) or one (stride 0)
int weight_stride(const Tensor& w, int64_t d, const char* name) {
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == at::kFloat && w.is_contiguous() &&
                  (w.numel() == d || w.numel() == 1), name, " must be fp32 with d entries or one");
  return w.numel() == 1 ? 0 : 1;
}

void post_norm_add_norm(Tensor out, Tensor x, Tensor ya, std::optional<Tensor> yb,
                        std::optional<Tensor> wa, std::optional<Tensor> wb, Tensor post_w,
                        Tensor next_w, double eps, bool fresh) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_GPU(ya);
  CHECK_F32(x); CHECK_CONTIG(x); CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(ya);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes() && ya.dim() == 2 &&
                  ya.sizes() == x.sizes(), "post_norm_add_norm: shapes");
  const int64_t rows = x.size(0), d = x.size(1);
  TORCH_CHECK(d * 8 <= 65536, "post_norm_add_norm: rows of at most 8192 entries");
  const bool yf = is_f32(ya, "ya");
  const void* ybp = nullptr;
  const float *wap = nullptr, *wbp = nullptr;
  int ybs = 0, was = 0, wbs = 0;
  if (yb.has_value()) {
    CHECK_GPU(*yb); CHECK_LAST_CONTIG(*yb);
    TORCH_CHECK(yb->sizes() == x.sizes() && yb->scalar_type() == ya.scalar_type() &&
                    wa.has_value() && wb.has_value(),
                "post_norm_add_norm: two branches need yb of ya's shape and type, wa and wb");
    ybp = yb->data_ptr();
    ybs = yb->stride(0);
    was = weight_stride(*wa, d, "wa");
    wbs = weight_stride(*wb, d, "wb");
    wap = wa->data_ptr<float>();
    wbp = wb->data_ptr<float>();
  }
  const int pws = weight_stride(post_w, d, "post_w"), nws = weight_stride(next_w, d, "next_w");
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_post_norm_add_norm(
      out.data_ptr(), is_f32(out, "out"), (int)out.stride(0), x.data_ptr<float>(), ya.data_ptr(),
      (int)ya.stride(0), ybp, ybs, yf, wap, was, wbp, wbs, post_w.data_ptr<float>(), pws,
      next_w.data_ptr<float>(), nws, (int)rows, (int)d, (float)eps, fresh, cur_stream());
}

void head_norm_cache(Tensor proj, Tensor q_out, Tensor k_cache, Tensor v_cache, Tensor slots,
                     int64_t H, int64_t G, int64_t D, int64_t Dv, int64_t q_off, int64_t k_off,
                     int64_t v_off, double eps, bool norm_qk, bool norm_v) {
  CHECK_GPU(proj); CHECK_GPU(q_out); CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_GPU(slots);
  CHECK_LAST_CONTIG(proj); CHECK_CONTIG(q_out); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_CONTIG(slots);
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
                  k_cache.scalar_type() == proj.scalar_type() &&
                  v_cache.scalar_type() == proj.scalar_type(), "head_norm_cache: dtypes differ");
  TORCH_CHECK(slots.scalar_type() == at::kLong, "slots must be int64");
  const int64_t T = proj.size(0), N = proj.size(1);
  TORCH_CHECK(proj.dim() == 2 && H > 0 && G > 0 && D > 0 && Dv > 0 && q_off >= 0 && k_off >= 0 &&
                  v_off >= 0 && q_off + H * D <= N && k_off + G * D <= N && v_off + G * Dv <= N,
              "head_norm_cache: slices outside the projection");
  TORCH_CHECK(q_out.numel() == T * H * D && slots.numel() == T, "head_norm_cache: q_out / slots");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 5 && k_cache.size(1) == G &&
                  k_cache.size(3) == D && v_cache.size(0) == k_cache.size(0) &&
                  v_cache.size(1) == G && v_cache.size(2) * 8 == k_cache.size(2) &&
                  v_cache.size(3) == Dv && v_cache.size(4) == 8,
              "head_norm_cache: K [NB, G, BS, D], V [NB, G, BS / 8, Dv, 8]");
  akap_stream::HeadNormParams p;
  p.proj = proj.data_ptr(); p.proj_stride = proj.stride(0);
  p.q_out = q_out.data_ptr(); p.k_cache = k_cache.data_ptr(); p.v_cache = v_cache.data_ptr();
  p.slots = slots.data_ptr<int64_t>();
  p.T = T; p.H = H; p.G = G; p.D = D; p.Dv = Dv; p.BS = k_cache.size(2);
  p.q_off = q_off; p.k_off = k_off; p.v_off = v_off;
  p.num_slots = k_cache.size(0) * k_cache.size(2);
  p.eps = (float)eps; p.norm_qk = norm_qk; p.norm_v = norm_v;
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_head_norm_cache(p, f32, cur_stream());
}

void retention(Tensor out, Tensor proj, int64_t q_off, int64_t k_off, int64_t v_off, int64_t g_off,
               Tensor state, Tensor seq_slot, Tensor positions, std::optional<Tensor> q_start,
               std::optional<Tensor> cos_sin, Tensor log2_decay, int64_t H, int64_t D, int64_t V,
               double eps, std::optional<Tensor> seg_buf, int64_t seg) {
  CHECK_GPU(out); CHECK_GPU(proj); CHECK_GPU(state); CHECK_GPU(seq_slot); CHECK_GPU(positions);
  CHECK_GPU(log2_decay);
  CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(proj); CHECK_CONTIG(state); CHECK_F32(state);
  CHECK_CONTIG(seq_slot); CHECK_CONTIG(positions); CHECK_CONTIG(log2_decay); CHECK_F32(log2_decay);
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type(), "retention: dtypes differ");
  TORCH_CHECK(seq_slot.scalar_type() == at::kInt && positions.scalar_type() == at::kLong,
              "retention: seq_slot int32, positions int64");
  const int64_t T = proj.size(0), N = proj.size(1);
  TORCH_CHECK(proj.dim() == 2 && out.dim() == 2 && out.size(0) == T && out.size(1) >= H * V &&
                  H > 0 && D > 0 && V > 0, "retention: shapes");
  TORCH_CHECK(q_off >= 0 && k_off >= 0 && v_off >= 0 && g_off >= 0 && q_off + H * D <= N &&
                  k_off + H * D <= N && v_off + H * V <= N && g_off + H * V <= N,
              "retention: slices outside the projection");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == V && state.size(3) == D,
              "retention: state must be [slots, H, V, D]");
  TORCH_CHECK(seq_slot.numel() >= T && positions.numel() >= T && log2_decay.numel() == H,
              "retention: seq_slot / positions / decay sizes");
  TORCH_CHECK(akap_stream::retention_dreg((int)D, (int)V) > 0,
              "retention: head sizes too large for one workgroup (V / 4 * D / 32 <= 512)");
  akap_stream::RetentionParams p;
  p.out = out.data_ptr(); p.out_stride = out.stride(0);
  p.proj = proj.data_ptr(); p.proj_stride = proj.stride(0);
  p.q_off = q_off; p.k_off = k_off; p.v_off = v_off; p.g_off = g_off;
  p.state = state.data_ptr<float>(); p.num_slots = state.size(0);
  p.seq_slot = seq_slot.data_ptr<int32_t>(); p.positions = positions.data_ptr<int64_t>();
  p.q_start = nullptr;
  p.num_seqs = T;
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_CONTIG(*q_start);
    TORCH_CHECK(q_start->scalar_type() == at::kInt && q_start->numel() >= 1, "retention: q_start");
    p.q_start = q_start->data_ptr<int32_t>();
    p.num_seqs = q_start->numel() - 1;
  }
  p.cos_sin = nullptr; p.rot_dims = 0;
  if (cos_sin.has_value()) {
    CHECK_GPU(*cos_sin); CHECK_CONTIG(*cos_sin); CHECK_F32(*cos_sin);
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) % 2 == 0 && cos_sin->size(1) <= D,
                "retention: cos_sin must be [max_pos, dims <= D]");
    p.cos_sin = cos_sin->data_ptr<float>();
    p.rot_dims = cos_sin->size(1);
  }
  p.log2_decay = log2_decay.data_ptr<float>();
  p.H = H; p.D = D; p.V = V; p.eps = (float)eps; p.DP = 1;
  p.seg_buf = nullptr; p.SEG = 0; p.num_segs = 0;
  if (seg_buf.has_value()) {
    CHECK_GPU(*seg_buf); CHECK_CONTIG(*seg_buf); CHECK_F32(*seg_buf);
    p.SEG = seg;
    TORCH_CHECK(q_start.has_value() && seg >= 16, "retention: segments need q_start and >= 16 rows");
    p.num_segs = T / seg + p.num_seqs;
    TORCH_CHECK(seg_buf->numel() >= (int64_t)p.num_segs * H * V * D, "retention: seg_buf size");
    p.seg_buf = seg_buf->data_ptr<float>();
  }
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_retention(p, f32, cur_stream());
}

// shared argument checks of the head-mixed attention ops; fills everything but the workspace
akap_stream::TalkParams talk_params(const Tensor& out, const Tensor& q, const Tensor& k_cache,
                                    const Tensor& v_cache, const Tensor& block_tables,
                                    const Tensor& seq_lens, const std::optional<Tensor>& q_start,
                                    const Tensor& positions, const std::optional<Tensor>& talk,
                                    const std::optional<Tensor>& gate, double scale) {
  CHECK_GPU(out); CHECK_GPU(q); CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_GPU(block_tables);
  CHECK_GPU(seq_lens); CHECK_GPU(positions);
  CHECK_LAST_CONTIG(out); CHECK_CONTIG(q); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_CONTIG(seq_lens); CHECK_CONTIG(positions);
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && k_cache.scalar_type() == q.scalar_type() &&
                  v_cache.scalar_type() == q.scalar_type(), "talking_attention: dtypes differ");
  TORCH_CHECK(q.dim() == 3 && k_cache.dim() == 4 && v_cache.dim() == 5, "talking_attention: ranks");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  const int64_t G = k_cache.size(1), BS = k_cache.size(2), Dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G &&
                  v_cache.size(2) * 8 == BS && v_cache.size(4) == 8 && G > 0 && H % G == 0,
              "talking_attention: K [NB, G, BS, D], V [NB, G, BS / 8, Dv, 8]");
  TORCH_CHECK(H <= 32 && G * Dv <= 1024,
              "talking_attention: at most 32 heads and 1024 value entries per token");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) >= H * Dv, "talking_attention: out");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.scalar_type() == at::kInt &&
                  block_tables.stride(1) == 1 && seq_lens.scalar_type() == at::kInt &&
                  positions.scalar_type() == at::kLong && positions.numel() >= T,
              "talking_attention: block_tables / seq_lens int32, positions int64");
  akap_stream::TalkParams p;
  p.out = out.data_ptr(); p.out_stride = out.stride(0);
  p.q = q.data_ptr(); p.k_cache = k_cache.data_ptr(); p.v_cache = v_cache.data_ptr();
  TORCH_CHECK(block_tables.stride(0) == block_tables.size(1) || block_tables.size(0) == 1,
              "talking_attention: block_tables rows must be dense");
  p.block_tables = block_tables.data_ptr<int32_t>(); p.max_blocks = block_tables.size(1);
  p.seq_lens = seq_lens.data_ptr<int32_t>();
  p.B = seq_lens.numel();
  TORCH_CHECK(block_tables.size(0) >= p.B, "talking_attention: a block-table row per sequence");
  p.q_start = nullptr;
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_CONTIG(*q_start);
    TORCH_CHECK(q_start->scalar_type() == at::kInt && q_start->numel() >= p.B + 1,
                "talking_attention: q_start");
    p.q_start = q_start->data_ptr<int32_t>();
  } else {
    TORCH_CHECK(p.B >= T, "talking_attention: a sequence per row when q_start is not given");
  }
  p.positions = positions.data_ptr<int64_t>();
  p.talk = nullptr;
  if (talk.has_value()) {
    CHECK_GPU(*talk); CHECK_CONTIG(*talk); CHECK_F32(*talk);
    TORCH_CHECK(talk->numel() == H * H, "talking_attention: talk must be [H, H]");
    p.talk = talk->data_ptr<float>();
  }
  p.gate = nullptr; p.gate_stride = 0;
  if (gate.has_value()) {
    CHECK_GPU(*gate); CHECK_LAST_CONTIG(*gate);
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H * Dv &&
                    gate->scalar_type() == q.scalar_type(), "talking_attention: gate [T, H Dv]");
    p.gate = gate->data_ptr(); p.gate_stride = gate->stride(0);
  }
  p.scale = (float)scale;
  p.T = T; p.H = H; p.G = G; p.D = D; p.Dv = Dv; p.BS = BS;
  p.ws_ml = nullptr; p.ws_o = nullptr; p.num_parts = 1; p.row0 = 0;
  TORCH_CHECK(akap_stream::talking_attention_lds(H, D) <= 65536,
              "talking_attention: heads x head size too large for the query row in LDS");
  return p;
}

void talk_workspace(akap_stream::TalkParams& p, const std::optional<Tensor>& ws_ml,
                    const std::optional<Tensor>& ws_o, int64_t num_parts) {
  TORCH_CHECK(ws_ml.has_value() && ws_o.has_value(), "talking_attention: a workspace is needed");
  CHECK_GPU(*ws_ml); CHECK_GPU(*ws_o); CHECK_F32(*ws_ml); CHECK_F32(*ws_o);
  TORCH_CHECK(ws_ml->numel() >= (int64_t)p.T * num_parts * p.H * 2 &&
                  ws_o->numel() >= (int64_t)p.T * num_parts * p.H * p.G * p.Dv,
              "talking_attention: workspace size");
  TORCH_CHECK((num_parts + 1) * p.H * 4 <= 65536, "talking_attention: too many partitions");
  p.ws_ml = ws_ml->data_ptr<float>(); p.ws_o = ws_o->data_ptr<float>();
  p.num_parts = num_parts;
}

void talking_attention(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_tables,
                       Tensor seq_lens, std::optional<Tensor> q_start, Tensor positions,
                       std::optional<Tensor> talk, std::optional<Tensor> gate, double scale,
                       std::optional<Tensor> ws_ml, std::optional<Tensor> ws_o, int64_t num_parts) {
  akap_stream::TalkParams p = talk_params(out, q, k_cache, v_cache, block_tables, seq_lens, q_start,
                                          positions, talk, gate, scale);
  if (num_parts > 1) talk_workspace(p, ws_ml, ws_o, num_parts);
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_talking_attention(p, is_f32(q, "q"), cur_stream());
}

void talking_attention_decode_mfma(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                                   Tensor block_tables, Tensor seq_lens, Tensor positions,
                                   std::optional<Tensor> talk, std::optional<Tensor> gate,
                                   double scale, Tensor ws_ml, Tensor ws_o, int64_t num_parts) {
  akap_stream::TalkParams p = talk_params(out, q, k_cache, v_cache, block_tables, seq_lens,
                                          std::nullopt, positions, talk, gate, scale);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16 &&
                  akap_stream::talk_mfma_supported(p.H, p.G, p.D, p.Dv, p.BS) && num_parts >= 1,
              "talking_attention_decode_mfma: bf16 and sizes the matrix-core kernel takes");
  talk_workspace(p, ws_ml, ws_o, num_parts);
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_talking_decode_mfma(p, cur_stream());
  akap_stream::launch_talking_merge(p, false, cur_stream());
}

bool talking_mfma_supported(int64_t H, int64_t G, int64_t D, int64_t Dv, int64_t BS) {
  return akap_stream::talk_mfma_supported((int)H, (int)G, (int)D, (int)Dv, (int)BS);
}

void talking_attention_prefill_mfma(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                                    Tensor block_tables, Tensor seq_lens, Tensor q_start,
                                    Tensor positions, Tensor tile_seq, Tensor tile_row,
                                    int64_t tile_rows, int64_t first_row,
                                    std::optional<Tensor> talk, std::optional<Tensor> gate,
                                    double scale, Tensor ws_ml, Tensor ws_o) {
  akap_stream::TalkParams p = talk_params(out, q, k_cache, v_cache, block_tables, seq_lens, q_start,
                                          positions, talk, gate, scale);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16 &&
                  akap_stream::talk_mfma_supported(p.H, p.G, p.D, p.Dv, p.BS),
              "talking_attention_prefill_mfma: bf16 and sizes the matrix-core kernel takes");
  talk_workspace(p, ws_ml, ws_o, 1);
  CHECK_GPU(tile_seq); CHECK_GPU(tile_row); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_row);
  TORCH_CHECK(tile_seq.scalar_type() == at::kInt && tile_row.scalar_type() == at::kInt &&
                  tile_row.numel() >= tile_seq.numel() && tile_rows >= 32 && tile_rows % 32 == 0,
              "talking_attention_prefill_mfma: tile map");
  TORCH_CHECK(first_row >= 0 && first_row <= p.T, "talking_attention_prefill_mfma: first_row");
  p.row0 = first_row;
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_talking_prefill_mfma(p, tile_seq.data_ptr<int32_t>(),
                                           tile_row.data_ptr<int32_t>(), (int)tile_seq.numel(),
                                           (int)tile_rows, cur_stream());
  akap_stream::launch_talking_merge(p, false, cur_stream());
}

void route_topk(Tensor ids, Tensor w, Tensor h, Tensor router, std::optional<Tensor> bias) {
  CHECK_GPU(ids); CHECK_GPU(w); CHECK_GPU(h); CHECK_GPU(router);
  CHECK_CONTIG(ids); CHECK_CONTIG(w); CHECK_F32(w); CHECK_LAST_CONTIG(h); CHECK_CONTIG(router);
  CHECK_F32(router);
  TORCH_CHECK(h.dim() == 2 && router.dim() == 2 && router.size(1) == h.size(1), "route_topk: shapes");
  const int64_t T = h.size(0), n = router.size(0);
  TORCH_CHECK(ids.scalar_type() == at::kInt && ids.dim() == 2 && ids.size(0) == T &&
                  w.sizes() == ids.sizes() && ids.size(1) >= 1 && ids.size(1) <= n &&
                  (n + h.size(1)) * 4 <= 60000,
              "route_topk: ids / w (and logits + one input row must fit LDS)");
  const float* bp = nullptr;
  if (bias.has_value()) {
    CHECK_GPU(*bias); CHECK_CONTIG(*bias); CHECK_F32(*bias);
    TORCH_CHECK(bias->numel() == n, "route_topk: bias");
    bp = bias->data_ptr<float>();
  }
  const c10::DeviceGuard g(h.device());
  akap_stream::launch_route_topk(ids.data_ptr<int32_t>(), w.data_ptr<float>(), h.data_ptr(),
                                 (int)h.stride(0), router.data_ptr<float>(), bp, (int)T,
                                 (int)h.size(1), (int)n, (int)ids.size(1), is_f32(h, "h"),
                                 cur_stream());
}

void swiglu_routed(Tensor out, Tensor gu, std::optional<Tensor> ids, std::optional<Tensor> w,
                   int64_t experts, int64_t act) {
  TORCH_CHECK(act == 0 || act == 1, "swiglu_routed: act is 0 (silu) or 1 (gelu, tanh form)");
  CHECK_GPU(out); CHECK_GPU(gu); CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(gu);
  TORCH_CHECK(out.scalar_type() == gu.scalar_type() && out.dim() == 2 && gu.dim() == 2 &&
                  out.size(0) == gu.size(0) && experts >= 1 && gu.size(1) == 2 * out.size(1) &&
                  out.size(1) % experts == 0 && experts <= 8192, "swiglu_routed: shapes");
  const int64_t T = gu.size(0);
  const int32_t* ip = nullptr;
  const float* wp = nullptr;
  int top = 0;
  if (ids.has_value()) {
    TORCH_CHECK(w.has_value(), "swiglu_routed: ids need weights");
    CHECK_GPU(*ids); CHECK_GPU(*w); CHECK_CONTIG(*ids); CHECK_CONTIG(*w); CHECK_F32(*w);
    TORCH_CHECK(ids->scalar_type() == at::kInt && ids->dim() == 2 && ids->size(0) == T &&
                    w->sizes() == ids->sizes() && ids->size(1) <= 256, "swiglu_routed: ids / w");
    ip = ids->data_ptr<int32_t>(); wp = w->data_ptr<float>(); top = ids->size(1);
  }
  const c10::DeviceGuard g(gu.device());
  akap_stream::launch_swiglu_routed(out.data_ptr(), (int)out.stride(0), gu.data_ptr(),
                                    (int)gu.stride(0), ip, wp, (int)T, top, (int)experts,
                                    (int)(out.size(1) / experts), is_f32(gu, "gu"), (int)act,
                                    cur_stream());
}

}  // namespace

TORCH_LIBRARY(akap_stream, m) {
  m.def("embed_scaled(Tensor(a!) out, Tensor ids, Tensor table, float scale) -> ()");
  m.def("add_norm(Tensor(a!) out, Tensor(b!) x, Tensor? y, float mult, Tensor w, float eps, "
        "Tensor? bias=None) -> ()");
  m.def("relu2(Tensor(a!) out, Tensor x) -> ()");
  m.def(
      "proj_norm_rope_cache(Tensor proj, Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache, "
      "Tensor positions, Tensor slots, Tensor? cos_sin, Tensor q_w, Tensor k_w, int H, int G, "
      "int D, int q_off, int k_off, float eps, Tensor? q_b=None, Tensor? k_b=None) -> ()");
  m.def(
      "sink_attention_prefill(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
      "Tensor block_tables, Tensor seq_lens, Tensor q_start, Tensor tile_seq, Tensor tile_row, "
      "int tile_rows, Tensor? gate, Tensor? sink, float scale, int chunk, int window) -> ()");
  m.def(
      "sink_attention_decode(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
      "Tensor block_tables, Tensor seq_lens, Tensor? gate, Tensor? sink, float scale, int chunk, "
      "int window, Tensor(b!)? ws_ml, Tensor(c!)? ws_o, int num_parts) -> ()");
  m.def("add_group_norm(Tensor(a!) out1, Tensor(b!)? out2, Tensor(c!) x, Tensor? y, Tensor? y2, "
        "Tensor? bias, Tensor w1, Tensor? w2, int groups, float eps, Tensor? shift_mu=None, "
        "Tensor(d!)? shift_state=None, Tensor? seq_slot=None, Tensor? positions=None) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor h, Tensor mu, Tensor(b!) state, Tensor seq_slot, "
        "Tensor positions, bool single=False) -> ()");
  m.def("latent_prep(Tensor proj, Tensor(a!) cq_out, Tensor(b!)? cache, Tensor positions, "
        "Tensor slots, Tensor cos_sin, Tensor q_w, Tensor? kv_w, int q_rank, int kv_rank, "
        "int rot_dim, int q_off, int kv_off, float eps, Tensor(c!)? vgroups=None) -> ()");
  m.def("latent_attention_prefill_mfma(Tensor(a!) out, Tensor q_lat, Tensor q, int rot_off, "
        "Tensor cache, Tensor vgroups, Tensor block_tables, Tensor seq_lens, Tensor q_start, "
        "Tensor tile_seq, Tensor tile_row, int tile_rows, float scale) -> ()");
  m.def("latent_attention_decode_mfma(Tensor(a!) out, Tensor q_lat, Tensor q, int rot_off, "
        "Tensor cache, Tensor vgroups, Tensor block_tables, Tensor seq_lens, float scale, "
        "Tensor(b!)? ws_ml, Tensor(c!)? ws_o, int num_parts) -> ()");
  m.def("latent_mfma_supported(int R, int r) -> bool", &latent_mfma_supported);
  m.def("rotate_heads(Tensor(a!) q, Tensor positions, Tensor cos_sin, int offset) -> ()");
  m.def("latent_attention(Tensor(a!) out, Tensor q_lat, Tensor q, int rot_off, Tensor cache, "
        "Tensor block_tables, Tensor seq_lens, Tensor? q_start, Tensor positions, float scale) "
        "-> ()");
  m.def("head_matmul(Tensor(a!) out, Tensor a, Tensor w) -> ()");
  m.def("head_gate(Tensor(a!) out, Tensor o, Tensor gate) -> ()");
  m.def("xielu(Tensor(a!) out, Tensor x, Tensor? bias, Tensor act) -> ()");
  m.def("moe_route(Tensor(a!) ids, Tensor(b!) w, Tensor h, Tensor router, Tensor? correction, "
        "int groups, int keep) -> ()");
  m.def("relu2_routed(Tensor(a!) out, Tensor up, Tensor ids, Tensor w, int experts) -> ()");
  m.def("moe_combine(Tensor(a!) out, Tensor y, Tensor? inv, Tensor ids, Tensor w, Tensor h, "
        "int experts) -> ()");
  m.def("post_norm_add_norm(Tensor(a!) out, Tensor(b!) x, Tensor ya, Tensor? yb, Tensor? wa, "
        "Tensor? wb, Tensor post_w, Tensor next_w, float eps, bool fresh) -> ()");
  m.def("head_norm_cache(Tensor proj, Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache, "
        "Tensor slots, int H, int G, int D, int Dv, int q_off, int k_off, int v_off, float eps, "
        "bool norm_qk, bool norm_v) -> ()");
  m.def("retention(Tensor(a!) out, Tensor proj, int q_off, int k_off, int v_off, int g_off, "
        "Tensor(b!) state, Tensor seq_slot, Tensor positions, Tensor? q_start, Tensor? cos_sin, "
        "Tensor log2_decay, int H, int D, int V, float eps, Tensor(c!)? seg_buf=None, "
        "int seg=0) -> ()");
  m.def("talking_attention(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
        "Tensor block_tables, Tensor seq_lens, Tensor? q_start, Tensor positions, Tensor? talk, "
        "Tensor? gate, float scale, Tensor(b!)? ws_ml, Tensor(c!)? ws_o, int num_parts) -> ()");
  m.def("talking_mfma_supported(int H, int G, int D, int Dv, int BS) -> bool",
        &talking_mfma_supported);
  m.def("talking_attention_prefill_mfma(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
        "Tensor block_tables, Tensor seq_lens, Tensor q_start, Tensor positions, Tensor tile_seq, "
        "Tensor tile_row, int tile_rows, int first_row, Tensor? talk, Tensor? gate, float scale, "
        "Tensor(b!) ws_ml, Tensor(c!) ws_o) -> ()");
  m.def("talking_attention_decode_mfma(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
        "Tensor block_tables, Tensor seq_lens, Tensor positions, Tensor? talk, Tensor? gate, "
        "float scale, Tensor(b!) ws_ml, Tensor(c!) ws_o, int num_parts) -> ()");
  m.def("route_topk(Tensor(a!) ids, Tensor(b!) w, Tensor h, Tensor router, Tensor? bias) -> ()");
  m.def("swiglu_routed(Tensor(a!) out, Tensor gu, Tensor? ids, Tensor? w, int experts, "
        "int act=0) -> ()");
}

TORCH_LIBRARY_IMPL(akap_stream, CUDA, m) {
  m.impl("add_group_norm", &add_group_norm);
  m.impl("token_shift", &token_shift);
  m.impl("latent_prep", &latent_prep);
  m.impl("rotate_heads", &rotate_heads);
  m.impl("latent_attention", &latent_attention);
  m.impl("latent_attention_prefill_mfma", &latent_attention_prefill_mfma);
  m.impl("latent_attention_decode_mfma", &latent_attention_decode_mfma);
  m.impl("head_matmul", &head_matmul);
  m.impl("head_gate", &head_gate);
  m.impl("xielu", &xielu);
  m.impl("moe_route", &moe_route);
  m.impl("relu2_routed", &relu2_routed);
  m.impl("moe_combine", &moe_combine);
  m.impl("post_norm_add_norm", &post_norm_add_norm);
  m.impl("head_norm_cache", &head_norm_cache);
  m.impl("retention", &retention);
  m.impl("talking_attention", &talking_attention);
  m.impl("talking_attention_prefill_mfma", &talking_attention_prefill_mfma);
  m.impl("talking_attention_decode_mfma", &talking_attention_decode_mfma);
  m.impl("route_topk", &route_topk);
  m.impl("swiglu_routed", &swiglu_routed);
  m.impl("embed_scaled", &embed_scaled);
  m.impl("add_norm", &add_norm);
  m.impl("relu2", &relu2);
  m.impl("proj_norm_rope_cache", &proj_norm_rope_cache);
  m.impl("sink_attention_prefill", &sink_attention_prefill);
  m.impl("sink_attention_decode", &sink_attention_decode);
}
