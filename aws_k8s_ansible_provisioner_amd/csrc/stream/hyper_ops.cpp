// torch custom-op registrations (namespace `akap_stream`, a fragment beside stream_ops.cpp) of
// the kernels in hyper.hip and pooled_attention.hip.
//
// Like the other ops: every op launches on the caller's current HIP stream, allocates nothing
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
#define CHECK_I32(x) TORCH_CHECK((x).scalar_type() == at::kInt, #x " must be int32")
#define CHECK_I64(x) TORCH_CHECK((x).scalar_type() == at::kLong, #x " must be int64")

bool is_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name,
              " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

const float* f32_vec(const std::optional<Tensor>& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() &&
                  t->numel() == n, name, " must be a contiguous fp32 GPU tensor of ", n, " entries");
  return t->data_ptr<float>();
}

void hyper_step(Tensor out, Tensor xs, std::optional<Tensor> ya, std::optional<Tensor> yb,
                std::optional<Tensor> bias, std::optional<Tensor> mix,
                std::optional<Tensor> w_out, Tensor w_in, Tensor norm_w, double eps,
                std::optional<Tensor> fresh) {
  CHECK_GPU(out); CHECK_GPU(xs); CHECK_F32(xs); CHECK_CONTIG(xs); CHECK_LAST_CONTIG(out);
  TORCH_CHECK(xs.dim() == 3 && out.dim() == 2 && out.size(0) == xs.size(0) &&
                  out.size(1) == xs.size(2), "hyper_step: shapes");
  const int64_t T = xs.size(0), S = xs.size(1), d = xs.size(2);
  TORCH_CHECK(S >= 1 && S <= 8, "hyper_step: 1 to 8 streams");
  TORCH_CHECK(d <= 12000, "hyper_step: rows of at most 12000 entries");
  const float* fp = nullptr;
  if (fresh.has_value()) {
    CHECK_GPU(*fresh); CHECK_F32(*fresh); CHECK_CONTIG(*fresh);
    TORCH_CHECK(fresh->dim() == 2 && fresh->size(0) == T && fresh->size(1) == d,
                "hyper_step: fresh shape");
    fp = fresh->data_ptr<float>();
  } else {
    TORCH_CHECK(mix.has_value() && w_out.has_value(), "hyper_step: an update needs mix and w_out");
  }
  const void* yp[2] = {nullptr, nullptr};
  bool yf[2] = {false, false};
  int ys[2] = {0, 0};
  const std::optional<Tensor>* yy[2] = {&ya, &yb};
  for (int i = 0; i < 2; ++i) {
    if (!yy[i]->has_value()) continue;
    const Tensor& y = **yy[i];
    CHECK_GPU(y); CHECK_LAST_CONTIG(y);
    TORCH_CHECK(y.dim() == 2 && y.size(0) == T && y.size(1) == d, "hyper_step: y shape");
    yp[i] = y.data_ptr(); yf[i] = is_f32(y, "y"); ys[i] = (int)y.stride(0);
  }
  const c10::DeviceGuard g(xs.device());
  akap_stream::launch_hyper_step(out.data_ptr(), is_f32(out, "out"), (int)out.stride(0),
                                 xs.data_ptr<float>(), fp, yp[0], yf[0], ys[0], yp[1], yf[1], ys[1],
                                 f32_vec(bias, d, "bias"), f32_vec(mix, S * S, "mix"),
                                 f32_vec(w_out, S, "w_out"), f32_vec(w_in, S, "w_in"),
                                 f32_vec(norm_w, d, "norm_w"), (int)T, (int)S, (int)d, (float)eps,
                                 cur_stream());
}

void softcap_(Tensor x, double cap) {
  CHECK_GPU(x); CHECK_CONTIG(x);
  TORCH_CHECK(cap > 0, "softcap_: cap must be positive");
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_softcap(x.data_ptr(), is_f32(x, "x"), (size_t)x.numel(), (float)cap,
                              cur_stream());
}

void gate_group_norm(Tensor out, Tensor y, Tensor gate, Tensor w, int64_t groups, double eps) {
  CHECK_GPU(out); CHECK_GPU(y); CHECK_GPU(gate); CHECK_F32(y); CHECK_CONTIG(y);
  CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(gate);
  TORCH_CHECK(y.dim() == 2 && out.dim() == 2 && gate.dim() == 2 && out.sizes() == y.sizes() &&
                  gate.sizes() == y.sizes() && out.scalar_type() == gate.scalar_type(),
              "gate_group_norm: shapes / dtypes");
  const int64_t n = y.size(1);
  TORCH_CHECK(groups >= 1 && groups <= 65535 && n % groups == 0, "gate_group_norm: groups");
  const c10::DeviceGuard g(y.device());
  akap_stream::launch_gate_group_norm(out.data_ptr(), (int)out.stride(0), y.data_ptr<float>(),
                                      gate.data_ptr(), (int)gate.stride(0),
                                      f32_vec(w, n, "w"), is_f32(out, "out"), (int)y.size(0),
                                      (int)n, (int)groups, (float)eps, cur_stream());
}

void route_sigmoid(Tensor ids, Tensor w, Tensor h, Tensor router, int64_t groups, int64_t keep,
                   int64_t group_top) {
  CHECK_GPU(ids); CHECK_GPU(w); CHECK_GPU(h); CHECK_GPU(router);
  CHECK_I32(ids); CHECK_F32(w); CHECK_CONTIG(ids); CHECK_CONTIG(w); CHECK_LAST_CONTIG(h);
  CHECK_F32(router); CHECK_CONTIG(router);
  TORCH_CHECK(h.dim() == 2 && router.dim() == 2 && router.size(1) == h.size(1) && ids.dim() == 2 &&
                  ids.size(0) == h.size(0) && w.sizes() == ids.sizes(), "route_sigmoid: shapes");
  const int64_t E = router.size(0), d = h.size(1), top = ids.size(1);
  TORCH_CHECK(E >= 1 && E <= 2048 && d <= 12000, "route_sigmoid: at most 2048 experts, rows of at "
              "most 12000 entries");
  TORCH_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && group_top >= 1 &&
                  top >= 1 && top <= keep * (E / groups), "route_sigmoid: groups / keep / top");
  const c10::DeviceGuard g(h.device());
  akap_stream::launch_route_sigmoid(ids.data_ptr<int32_t>(), w.data_ptr<float>(), h.data_ptr(),
                                    (int)h.stride(0), is_f32(h, "h"), router.data_ptr<float>(),
                                    (int)h.size(0), (int)d, (int)E, (int)top, (int)groups,
                                    (int)keep, (int)group_top, cur_stream());
}

// rows, sequences and the checks shared by the ops that walk sequences of a step
struct SeqArgs {
  const int32_t* slot;
  const int64_t* pos;
  const int32_t* q_start;
  int T, B;
};
SeqArgs seq_args(int64_t T, const Tensor& seq_slot, const Tensor& positions,
                 const std::optional<Tensor>& q_start) {
  CHECK_GPU(seq_slot); CHECK_GPU(positions); CHECK_I32(seq_slot); CHECK_I64(positions);
  CHECK_CONTIG(seq_slot); CHECK_CONTIG(positions);
  TORCH_CHECK(seq_slot.numel() >= T && positions.numel() >= T, "seq_slot / positions: one per row");
  SeqArgs a{seq_slot.data_ptr<int32_t>(), positions.data_ptr<int64_t>(), nullptr, (int)T, (int)T};
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_I32(*q_start); CHECK_CONTIG(*q_start);
    TORCH_CHECK(q_start->numel() >= 2, "q_start: B + 1 entries");
    a.q_start = q_start->data_ptr<int32_t>();
    a.B = (int)q_start->numel() - 1;
  }
  return a;
}

void conv_silu(Tensor out, Tensor proj, int64_t off, Tensor conv_w, Tensor conv_b, Tensor state,
               Tensor seq_slot, Tensor positions, std::optional<Tensor> q_start) {
  CHECK_GPU(out); CHECK_GPU(proj); CHECK_GPU(state); CHECK_F32(out); CHECK_CONTIG(out);
  CHECK_LAST_CONTIG(proj); CHECK_CONTIG(state);
  TORCH_CHECK(conv_w.dim() == 2 && out.dim() == 2 && proj.dim() == 2, "conv_silu: shapes");
  const int64_t T = proj.size(0), C = conv_w.size(0), taps = conv_w.size(1);
  TORCH_CHECK(out.size(0) == T && out.size(1) == C && off >= 0 && off + C <= proj.size(1),
              "conv_silu: columns");
  TORCH_CHECK(taps >= 1 && taps <= 8, "conv_silu: 1 to 8 taps");
  TORCH_CHECK(state.scalar_type() == proj.scalar_type() && state.dim() == 3 &&
                  state.size(2) == C && state.size(1) >= taps - 1 &&
                  (taps == 1 || state.size(1) == taps - 1), "conv_silu: state [slots, taps - 1, C]");
  const SeqArgs sa = seq_args(T, seq_slot, positions, q_start);
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_conv_silu(out.data_ptr<float>(), proj.data_ptr(), (int)proj.stride(0),
                                (int)off, is_f32(proj, "proj"), state.data_ptr(),
                                f32_vec(conv_w, C * taps, "conv_w"), f32_vec(conv_b, C, "conv_b"),
                                sa.slot, sa.pos, sa.q_start, sa.T, sa.B, (int)C, (int)taps,
                                cur_stream());
}

void selective_scan(Tensor y, Tensor xbc, Tensor proj, int64_t dt_off, Tensor dt_bias,
                    Tensor a_log, Tensor d_skip, Tensor state, Tensor seq_slot, Tensor positions,
                    std::optional<Tensor> q_start, int64_t H, int64_t V, int64_t N, int64_t G) {
  CHECK_GPU(y); CHECK_GPU(xbc); CHECK_GPU(proj); CHECK_GPU(state);
  CHECK_F32(y); CHECK_F32(xbc); CHECK_F32(state); CHECK_CONTIG(y); CHECK_CONTIG(xbc);
  CHECK_CONTIG(state); CHECK_LAST_CONTIG(proj);
  const int64_t T = xbc.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && V >= 1 && V <= 256 && N >= 1,
              "selective_scan: heads / groups / sizes (vdim at most 256)");
  TORCH_CHECK(akap_stream::selective_scan_supported((int)V, (int)N),
              "selective_scan: state x vdim too large for the register-resident state");
  TORCH_CHECK(xbc.dim() == 2 && xbc.size(1) == H * V + 2 * G * N && y.dim() == 2 &&
                  y.size(0) == T && y.size(1) == H * V && proj.dim() == 2 && proj.size(0) == T &&
                  dt_off >= 0 && dt_off + H <= proj.size(1), "selective_scan: shapes");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == N && state.size(3) == V,
              "selective_scan: state [slots, H, N, V]");
  const SeqArgs sa = seq_args(T, seq_slot, positions, q_start);
  const c10::DeviceGuard g(xbc.device());
  akap_stream::launch_selective_scan(y.data_ptr<float>(), xbc.data_ptr<float>(), proj.data_ptr(),
                                     (int)proj.stride(0), (int)dt_off, is_f32(proj, "proj"),
                                     f32_vec(dt_bias, H, "dt_bias"), f32_vec(a_log, H, "a_log"),
                                     f32_vec(d_skip, H, "d_skip"), state.data_ptr<float>(), sa.slot,
                                     sa.pos, sa.q_start, sa.T, sa.B, (int)H, (int)V, (int)N, (int)G,
                                     cur_stream());
}

void bias_rope_cache(Tensor proj, Tensor q_out, Tensor k_cache, Tensor v_cache, Tensor positions,
                     Tensor slots, std::optional<Tensor> cos_sin, std::optional<Tensor> bias,
                     int64_t H, int64_t G, int64_t D, int64_t Dv, int64_t q_off, int64_t k_off,
                     int64_t v_off) {
  CHECK_GPU(proj); CHECK_GPU(q_out); CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_GPU(positions);
  CHECK_GPU(slots); CHECK_LAST_CONTIG(proj); CHECK_CONTIG(q_out); CHECK_CONTIG(k_cache);
  CHECK_CONTIG(v_cache); CHECK_I64(positions); CHECK_I64(slots); CHECK_CONTIG(positions);
  CHECK_CONTIG(slots);
  const int64_t T = proj.size(0), N = proj.size(1);
  TORCH_CHECK(proj.dim() == 2 && q_out.numel() == T * H * D && positions.numel() >= T &&
                  slots.numel() >= T, "bias_rope_cache: shapes");
  TORCH_CHECK(q_off >= 0 && q_off + H * D <= N && k_off >= 0 && k_off + G * D <= N && v_off >= 0 &&
                  v_off + G * Dv <= N, "bias_rope_cache: column ranges");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 5 && k_cache.size(1) == G &&
                  k_cache.size(3) == D && v_cache.size(0) == k_cache.size(0) &&
                  v_cache.size(1) == G && v_cache.size(2) * 8 == k_cache.size(2) &&
                  v_cache.size(3) == Dv && v_cache.size(4) == 8, "bias_rope_cache: cache shapes");
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
                  k_cache.scalar_type() == proj.scalar_type() &&
                  v_cache.scalar_type() == proj.scalar_type(), "bias_rope_cache: dtypes differ");
  akap_stream::RopeCacheParams p{};
  p.proj = proj.data_ptr(); p.proj_stride = (int)proj.stride(0);
  p.q_out = q_out.data_ptr(); p.k_cache = k_cache.data_ptr(); p.v_cache = v_cache.data_ptr();
  p.positions = positions.data_ptr<int64_t>(); p.slots = slots.data_ptr<int64_t>();
  if (cos_sin.has_value()) {
    CHECK_GPU(*cos_sin); CHECK_F32(*cos_sin); CHECK_CONTIG(*cos_sin);
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) % 2 == 0 && cos_sin->size(1) <= D,
                "bias_rope_cache: cos_sin [max_pos, dims], dims even and at most D");
    p.cos_sin = cos_sin->data_ptr<float>();
    p.max_pos = (int)cos_sin->size(0); p.rot_dims = (int)cos_sin->size(1);
  }
  p.bias = f32_vec(bias, N, "bias");
  p.T = (int)T; p.H = (int)H; p.G = (int)G; p.D = (int)D; p.Dv = (int)Dv;
  p.BS = (int)k_cache.size(2); p.q_off = (int)q_off; p.k_off = (int)k_off; p.v_off = (int)v_off;
  p.num_slots = k_cache.size(0) * k_cache.size(2);
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_bias_rope_cache(p, f32, cur_stream());
}

void check_paged(const Tensor& k_cache, const Tensor& v_cache, const std::optional<Tensor>& k_pool,
                 const std::optional<Tensor>& v_pool, const Tensor& block_tables, int64_t pool,
                 int64_t* PS) {
  CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_GPU(block_tables); CHECK_I32(block_tables); CHECK_CONTIG(block_tables);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 5 && block_tables.dim() == 2 &&
                  v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == k_cache.size(1) &&
                  v_cache.size(2) * 8 == k_cache.size(2) && v_cache.size(4) == 8 &&
                  v_cache.scalar_type() == k_cache.scalar_type(), "paged cache shapes");
  *PS = 0;
  if (pool > 0) {
    TORCH_CHECK(k_pool.has_value() && v_pool.has_value(), "pooled blocks need k_pool / v_pool");
    CHECK_GPU(*k_pool); CHECK_GPU(*v_pool); CHECK_F32(*k_pool); CHECK_F32(*v_pool);
    CHECK_CONTIG(*k_pool); CHECK_CONTIG(*v_pool);
    const int64_t BS = k_cache.size(2), ps = (BS + pool - 1) / pool;
    TORCH_CHECK(k_pool->dim() == 4 && v_pool->dim() == 4 && k_pool->size(0) == k_cache.size(0) &&
                    k_pool->size(1) == k_cache.size(1) && k_pool->size(2) == ps &&
                    k_pool->size(3) == k_cache.size(3) && v_pool->size(0) == k_cache.size(0) &&
                    v_pool->size(1) == k_cache.size(1) && v_pool->size(2) == ps &&
                    v_pool->size(3) == v_cache.size(3),
                "pooled entries: [NB, G, ceil(BS / pool), D / Dv]");
    *PS = ps;
  }
}

void pool_cache_blocks(Tensor k_cache, Tensor v_cache, Tensor k_pool, Tensor v_pool,
                       Tensor positions, Tensor slots, Tensor block_tables,
                       std::optional<Tensor> q_start, int64_t pool) {
  TORCH_CHECK(pool > 0, "pool_cache_blocks: pool must be positive");
  int64_t PS;
  check_paged(k_cache, v_cache, k_pool, v_pool, block_tables, pool, &PS);
  CHECK_GPU(positions); CHECK_GPU(slots); CHECK_I64(positions); CHECK_I64(slots);
  CHECK_CONTIG(positions); CHECK_CONTIG(slots);
  const int64_t T = positions.numel();
  TORCH_CHECK(slots.numel() >= T, "pool_cache_blocks: one slot per row");
  akap_stream::PoolParams p{};
  p.k_cache = k_cache.data_ptr(); p.v_cache = v_cache.data_ptr();
  p.k_pool = k_pool.data_ptr<float>(); p.v_pool = v_pool.data_ptr<float>();
  p.positions = positions.data_ptr<int64_t>(); p.slots = slots.data_ptr<int64_t>();
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.max_blocks = (int)block_tables.size(1);
  p.T = (int)T; p.B = (int)T;
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_I32(*q_start); CHECK_CONTIG(*q_start);
    p.q_start = q_start->data_ptr<int32_t>();
    p.B = (int)q_start->numel() - 1;
  }
  TORCH_CHECK(p.B >= 1 && p.B <= block_tables.size(0), "pool_cache_blocks: a block-table row per "
              "sequence");
  p.G = (int)k_cache.size(1); p.D = (int)k_cache.size(3); p.Dv = (int)v_cache.size(3);
  p.BS = (int)k_cache.size(2); p.PS = (int)PS; p.pool = (int)pool;
  const c10::DeviceGuard g(k_cache.device());
  akap_stream::launch_pool_cache_blocks(p, is_f32(k_cache, "k_cache"), cur_stream());
}

akap_stream::PoolAttnParams attn_params(Tensor& out, Tensor& q, Tensor& k_cache, Tensor& v_cache,
                                        std::optional<Tensor>& k_pool,
                                        std::optional<Tensor>& v_pool, Tensor& block_tables,
                                        std::optional<Tensor>& q_start, Tensor& positions,
                                        Tensor& slots, double scale, int64_t window, int64_t pool,
                                        bool unit_sink) {
  int64_t PS;
  if (window <= 0) pool = 0;
  check_paged(k_cache, v_cache, k_pool, v_pool, block_tables, pool, &PS);
  CHECK_GPU(out); CHECK_GPU(q); CHECK_LAST_CONTIG(out); CHECK_CONTIG(q);
  CHECK_GPU(positions); CHECK_GPU(slots); CHECK_I64(positions); CHECK_I64(slots);
  CHECK_CONTIG(positions); CHECK_CONTIG(slots);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 2 && out.size(0) == q.size(0), "attention: shapes");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  const int64_t G = k_cache.size(1), Dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(2) % 8 == 0, "attention: the block size must be a multiple of 8");
  TORCH_CHECK(k_cache.size(3) == D && H % G == 0 && Dv <= 512 && D <= 512 &&
                  out.size(1) >= H * Dv, "attention: head sizes (heads a multiple of the "
              "key/value heads, keys and values of at most 512 entries)");
  TORCH_CHECK(q.scalar_type() == k_cache.scalar_type() && out.scalar_type() == q.scalar_type(),
              "attention: dtypes differ");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "attention: one position per row");
  akap_stream::PoolAttnParams p{};
  p.out = out.data_ptr(); p.out_stride = (int)out.stride(0); p.q = q.data_ptr();
  p.k_cache = k_cache.data_ptr(); p.v_cache = v_cache.data_ptr();
  if (pool > 0) { p.k_pool = k_pool->data_ptr<float>(); p.v_pool = v_pool->data_ptr<float>(); }
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.positions = positions.data_ptr<int64_t>(); p.slots = slots.data_ptr<int64_t>();
  p.scale = (float)scale;
  p.max_blocks = (int)block_tables.size(1);
  p.T = (int)T; p.B = (int)T;
  if (q_start.has_value()) {
    CHECK_GPU(*q_start); CHECK_I32(*q_start); CHECK_CONTIG(*q_start);
    p.q_start = q_start->data_ptr<int32_t>();
    p.B = (int)q_start->numel() - 1;
  }
  TORCH_CHECK(p.B >= 1 && p.B <= block_tables.size(0), "attention: a block-table row per sequence");
  p.H = (int)H; p.G = (int)G; p.D = (int)D; p.Dv = (int)Dv; p.BS = (int)k_cache.size(2);
  p.PS = (int)PS; p.window = (int)window; p.pool = (int)pool; p.unit_sink = unit_sink ? 1 : 0;
  return p;
}

void pooled_window_attention(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                             std::optional<Tensor> k_pool, std::optional<Tensor> v_pool,
                             Tensor block_tables, std::optional<Tensor> q_start, Tensor positions,
                             Tensor slots, double scale, int64_t window, int64_t pool,
                             bool unit_sink) {
  const akap_stream::PoolAttnParams p =
      attn_params(out, q, k_cache, v_cache, k_pool, v_pool, block_tables, q_start, positions,
                  slots, scale, window, pool, unit_sink);
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_pooled_window_attention(p, is_f32(q, "q"), cur_stream());
}

void pooled_window_attention_decode_mfma(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                                         std::optional<Tensor> k_pool,
                                         std::optional<Tensor> v_pool, Tensor block_tables,
                                         Tensor positions, Tensor slots, double scale,
                                         int64_t window, int64_t pool, bool unit_sink) {
  std::optional<Tensor> none;
  const akap_stream::PoolAttnParams p =
      attn_params(out, q, k_cache, v_cache, k_pool, v_pool, block_tables, none, positions, slots,
                  scale, window, pool, unit_sink);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16, "matrix-core attention: bf16 only");
  TORCH_CHECK(akap_stream::pooled_mfma_supported(p.H, p.G, p.D, p.Dv, p.BS) && p.H / p.G <= 32,
              "matrix-core attention: unsupported head sizes");
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_pooled_window_decode_mfma(p, p.T, cur_stream());
}

bool pooled_mfma_supported(int64_t H, int64_t G, int64_t D, int64_t Dv, int64_t BS) {
  return akap_stream::pooled_mfma_supported((int)H, (int)G, (int)D, (int)Dv, (int)BS);
}

void pooled_window_attention_prefill_mfma(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                                          std::optional<Tensor> k_pool,
                                          std::optional<Tensor> v_pool, Tensor block_tables,
                                          Tensor q_start, Tensor positions, Tensor slots,
                                          Tensor tile_seq, Tensor tile_row, int64_t tile_rows,
                                          double scale, int64_t window, int64_t pool,
                                          bool unit_sink) {
  std::optional<Tensor> qs(q_start);
  const akap_stream::PoolAttnParams p =
      attn_params(out, q, k_cache, v_cache, k_pool, v_pool, block_tables, qs, positions, slots,
                  scale, window, pool, unit_sink);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16, "matrix-core attention: bf16 only");
  TORCH_CHECK(akap_stream::pooled_mfma_supported(p.H, p.G, p.D, p.Dv, p.BS),
              "matrix-core attention: unsupported head sizes");
  TORCH_CHECK(tile_rows == 128, "matrix-core attention: tiles of 128 rows");
  TORCH_CHECK(out.stride(0) % 4 == 0 && (uintptr_t)out.data_ptr() % 8 == 0,
              "matrix-core attention: out rows must start at multiples of 8 bytes");
  CHECK_GPU(tile_seq); CHECK_GPU(tile_row); CHECK_I32(tile_seq); CHECK_I32(tile_row);
  CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_row);
  TORCH_CHECK(tile_seq.numel() == tile_row.numel(), "matrix-core attention: tile map");
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_pooled_window_prefill_mfma(p, tile_seq.data_ptr<int32_t>(),
                                                 tile_row.data_ptr<int32_t>(),
                                                 (int)tile_seq.numel(), cur_stream());
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(akap_stream, m) {
  m.def("hyper_step(Tensor(a!) out, Tensor(b!) xs, Tensor? ya, Tensor? yb, Tensor? bias, "
        "Tensor? mix, Tensor? w_out, Tensor w_in, Tensor norm_w, float eps, Tensor? fresh=None) "
        "-> ()");
  m.def("softcap_(Tensor(a!) x, float cap) -> ()");
  m.def("gate_group_norm(Tensor(a!) out, Tensor y, Tensor gate, Tensor w, int groups, float eps) "
        "-> ()");
  m.def("route_sigmoid(Tensor(a!) ids, Tensor(b!) w, Tensor h, Tensor router, int groups, "
        "int keep, int group_top) -> ()");
  m.def("conv_silu(Tensor(a!) out, Tensor proj, int off, Tensor conv_w, Tensor conv_b, "
        "Tensor(b!) state, Tensor seq_slot, Tensor positions, Tensor? q_start) -> ()");
  m.def("selective_scan(Tensor(a!) y, Tensor xbc, Tensor proj, int dt_off, Tensor dt_bias, "
        "Tensor a_log, Tensor d_skip, Tensor(b!) state, Tensor seq_slot, Tensor positions, "
        "Tensor? q_start, int H, int V, int N, int G) -> ()");
  m.def("bias_rope_cache(Tensor proj, Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache, "
        "Tensor positions, Tensor slots, Tensor? cos_sin, Tensor? bias, int H, int G, int D, "
        "int Dv, int q_off, int k_off, int v_off) -> ()");
  m.def("pool_cache_blocks(Tensor k_cache, Tensor v_cache, Tensor(a!) k_pool, Tensor(b!) v_pool, "
        "Tensor positions, Tensor slots, Tensor block_tables, Tensor? q_start, int pool) -> ()");
  m.def("pooled_window_attention(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
        "Tensor? k_pool, Tensor? v_pool, Tensor block_tables, Tensor? q_start, Tensor positions, "
        "Tensor slots, float scale, int window, int pool, bool unit_sink) -> ()");
  m.def("pooled_window_attention_decode_mfma(Tensor(a!) out, Tensor q, Tensor k_cache, "
        "Tensor v_cache, Tensor? k_pool, Tensor? v_pool, Tensor block_tables, Tensor positions, "
        "Tensor slots, float scale, int window, int pool, bool unit_sink) -> ()");
  m.def("pooled_mfma_supported(int H, int G, int D, int Dv, int BS) -> bool",
        &pooled_mfma_supported);
  m.def("pooled_window_attention_prefill_mfma(Tensor(a!) out, Tensor q, Tensor k_cache, "
        "Tensor v_cache, Tensor? k_pool, Tensor? v_pool, Tensor block_tables, Tensor q_start, "
        "Tensor positions, Tensor slots, Tensor tile_seq, Tensor tile_row, int tile_rows, "
        "float scale, int window, int pool, bool unit_sink) -> ()");
}

TORCH_LIBRARY_IMPL(akap_stream, CUDA, m) {
  m.impl("hyper_step", &hyper_step);
  m.impl("softcap_", &softcap_);
  m.impl("gate_group_norm", &gate_group_norm);
  m.impl("route_sigmoid", &route_sigmoid);
  m.impl("conv_silu", &conv_silu);
  m.impl("selective_scan", &selective_scan);
  m.impl("bias_rope_cache", &bias_rope_cache);
  m.impl("pool_cache_blocks", &pool_cache_blocks);
  m.impl("pooled_window_attention", &pooled_window_attention);
  m.impl("pooled_window_attention_prefill_mfma", &pooled_window_attention_prefill_mfma);
  m.impl("pooled_window_attention_decode_mfma", &pooled_window_attention_decode_mfma);
}
