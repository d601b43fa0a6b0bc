"""Sazepel: a layered decoder over an fp32 residual stream (LayeredConfig, arch "sazepel").

The embedding is normed once.  Layers are sequential with a norm before AND after each
sublayer:  x <- x + norm1b(mixer(norm1 x)),  x <- x + norm2b(ff(norm2 x)); every norm weight
is one number.  Mixers: "retention" -- linear attention with a fixed decay per head, rotary
positions (rotate-half pairs) on q and k, no softmax; its only memory is a state S [dim, vdim]
per head and live sequence (fp32), kept in the scheduler's sequence slots -- or "parallel": a
grouped-query softmax attention without positions (per-head RMS norm of q, k and the cached
values, a learned [H, H] matrix that mixes the heads' softmax weights before they meet the
values, a sigmoid gate per output entry) beside a retention, both reading the same input, each
output RMS-normed over the width with a weight vector of its own, then averaged.  The
feed-forward is routed: the `top` largest of (router h + bias) win, weights = softmax over the
winners, SwiGLU experts.  Logits are scaled by a constant.

MI355X mapping.  Everything that reads the normed stream of a mixer is ONE GEMM (retention:
[q | k | v | g]; parallel: the attention's [q | k | v | g] and the retention's side by side).
The retention kernel reads its slices straight from that projection, rotates in fp32, runs the
recurrence on the fp32 state, norms each head's output and applies the silu gate: one launch
from projection to the input of the output projection.  The attention is one kernel that
norms q / k / v per head and writes the paged cache, and one that keeps, per query head, the
unnormalised sums of all value heads under its weights (so the head mixing is a small matrix
product at the end and the keys are read once), split over key partitions for decode rows.
The post-norm of a sublayer, the residual sum and the pre-norm of the next sublayer are one
kernel.  Routed layers take the expert path by batch size like the framework's other routed
model: small batches (every decode step, hipGraph-captured) run ALL experts as one GEMM over
the stacked [gate | up] projections, scale the gated activations by the routing weights (0 for
experts not chosen) and sum the chosen experts inside one GEMM over the side-by-side
down-projections; prompt-sized batches sort the (token, choice) pairs by expert.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import stream as sops
from ..parallel.state import ParallelState, get_state
from .config import AttentionSpec, LayeredConfig, LayerSpec, ParallelMixerSpec, RetentionSpec
from .routed import MOE_DENSE_ROWS, routed_sorted
from .transformer import AttnBatch


@dataclasses.dataclass
class SandwichLayerWeights:
    spec: LayerSpec
    norm1: torch.Tensor                 # fp32 [1]
    norm1b: torch.Tensor
    w_in: torch.Tensor                  # [attention q | k | v | g | retention q | k | v | g, d]
    ret_off: int                        # first row of the retention's slices in w_in
    w_o: torch.Tensor                   # retention output projection [d, H V]
    log2_decay: torch.Tensor            # fp32 [H]
    cos_sin: Optional[torch.Tensor]
    w_ao: Optional[torch.Tensor] = None     # attention output projection [d, H Dv]
    talk: Optional[torch.Tensor] = None     # fp32 [H, H]
    out_a: Optional[torch.Tensor] = None    # fp32 [d]: branch norm weights
    out_r: Optional[torch.Tensor] = None
    norm2: Optional[torch.Tensor] = None
    norm2b: Optional[torch.Tensor] = None
    w_up: Optional[torch.Tensor] = None     # [E 2F, d]: per expert [gate | up]
    w_down: Optional[torch.Tensor] = None   # [d, E F]
    router: Optional[torch.Tensor] = None   # fp32 [E, d]
    router_b: Optional[torch.Tensor] = None
    w_down_e: Optional[torch.Tensor] = None  # [E, d, F]: w_down per expert, made on first use


class SazepelLM:
    """Weights + forward of one replica (same surface as DecoderLM for the model runner)."""

    supports_v_tail = False
    gemm_tunable = True
    # the stacked expert weights are GEMM weights of decode-sized batches too (all experts run
    # as one GEMM pair there)
    gemm_weight_names = ("w_in", "w_o", "w_ao", "w_up", "w_down")
    fused_gemm_chain = False
    dtypes = (torch.bfloat16, torch.float32)
    # the retention states of a live sequence sit in one of the scheduler's sequence slots: the
    # runner sizes the slot pool for it and turns prefix caching off
    state_slots = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cpu",
                 dtype: torch.dtype = torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, max_model_len: int = 4096,
                 full_then_shard: bool = False, init_std: float = 0.02):
        if dtype not in self.dtypes:
            raise ValueError(f"Sazepel runs in bfloat16 or float32, not {dtype}")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError("Sazepel: tensor parallelism is not implemented (tp must be 1)")
        if max_model_len > cfg.max_position:
            raise ValueError(f"max_model_len {max_model_len} exceeds max_position "
                             f"{cfg.max_position}")
        self.max_model_len = max_model_len
        self.init_std = init_std
        self.runs = cfg.layer_runs()
        self.hq, self.hkv, self.D = cfg.num_heads, max(1, cfg.num_kv_heads), cfg.head_dim
        self.ffn = cfg.intermediate_size
        self.vocab_start, self.vocab_end = 0, cfg.vocab_size
        self._tables: dict = {}
        self.state: Optional[list] = None
        self._ws: Optional[tuple] = None
        self._ws_kept: list = []
        self._seg_map: dict = {}
        self._init_weights(seed)

    # ------------------------------------------------------------------ weights
    @staticmethod
    def _parts(ls: LayerSpec):
        """(attention spec or None, retention spec) of a layer."""
        m = ls.mixer
        if isinstance(m, ParallelMixerSpec):
            return m.left, m.right
        return None, m

    def _table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        key = (rot.dims, rot.base)
        if key not in self._tables:
            self._tables[key] = sops.rotary_table(max(self.max_model_len, 16), rot.dims, rot.base,
                                                  None, device=self.device)
        return self._tables[key]

    @staticmethod
    def _att_rows(a: Optional[AttentionSpec]) -> int:
        if a is None:
            return 0
        return a.heads * a.dim + a.kv_heads * (a.dim + a.vdim) + a.heads * a.vdim

    def _init_weights(self, seed: int) -> None:
        cfg, d = self.cfg, self.cfg.hidden_size
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        std = self.init_std

        def rand(*shape, s=std, mean=0.0, dt=None):
            t = torch.empty(*shape, dtype=torch.float32).normal_(mean, s, generator=g)
            return t.to(torch.bfloat16).to(dt or self.dtype).to(self.device)

        f32 = torch.float32
        one = lambda: rand(1, s=0.1, mean=1.0, dt=f32)  # noqa: E731
        self.embed = rand(cfg.vocab_size, d, s=1.0)
        self.embed_norm = one()
        self.layers: list[SandwichLayerWeights] = []
        for ls in cfg.layer_specs:
            a, r = self._parts(ls)
            na = self._att_rows(a)
            n = na + r.heads * (2 * r.dim + 2 * r.vdim)
            npad = -(-n // 256) * 256
            if npad > 1.05 * n:
                npad = -(-n // 8) * 8
            w_in = torch.zeros(npad, d, dtype=self.dtype, device=self.device)
            w_in[:n] = rand(n, d)
            lw = SandwichLayerWeights(
                spec=ls, norm1=one(), norm1b=one(), w_in=w_in, ret_off=na,
                w_o=rand(d, r.heads * r.vdim),
                log2_decay=torch.tensor([math.log2(x) for x in r.decay], dtype=f32,
                                        device=self.device),
                cos_sin=self._table(r.rot))
            if a is not None:
                lw.w_ao = rand(d, a.heads * a.vdim)
                lw.talk = (torch.eye(a.heads) + 0.2 * torch.randn(a.heads, a.heads, generator=g)
                           ).to(torch.bfloat16).to(f32).to(self.device)
                lw.out_a = rand(d, s=0.1, mean=1.0, dt=f32)
                lw.out_r = rand(d, s=0.1, mean=1.0, dt=f32)
            ml = ls.mlp
            if ml is not None:
                E, F_ = ml.router.experts, ml.ff
                lw.norm2, lw.norm2b = one(), one()
                lw.w_up = rand(E * 2 * F_, d)
                lw.w_down = rand(d, E * F_)
                lw.router = rand(E, d, s=4 * std, dt=f32)
                lw.router_b = rand(E, s=0.1, dt=f32)
            self.layers.append(lw)
        self.final_norm = one()
        self.lm_head = rand(cfg.vocab_size, d)
        self._scale_final()

    def _scale_final(self) -> None:
        # the constant logit scale rides in the last norm's weight (fp32): the hidden rows are
        # rounded once, after the scale
        self._final_w = self.final_norm * float(self.cfg.logit_scale)

    def _names(self, i: int, lw: SandwichLayerWeights):
        """(checkpoint name, destination view) of layer i."""
        a, r = self._parts(lw.spec)
        p = f"l{i}."
        out = [(p + "norm1", lw.norm1), (p + "norm1b", lw.norm1b)]
        rp = p + ("mix.right." if a is not None else "mix.")
        o = lw.ret_off
        hd, hv = r.heads * r.dim, r.heads * r.vdim
        out += [(rp + "q", lw.w_in[o:o + hd]), (rp + "k", lw.w_in[o + hd:o + 2 * hd]),
                (rp + "v", lw.w_in[o + 2 * hd:o + 2 * hd + hv]),
                (rp + "g", lw.w_in[o + 2 * hd + hv:o + 2 * hd + 2 * hv]), (rp + "o", lw.w_o)]
        if a is not None:
            ap = p + "mix.left."
            q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
            out += [(ap + "q", lw.w_in[:q]), (ap + "k", lw.w_in[q:q + k]),
                    (ap + "v", lw.w_in[q + k:q + k + v]),
                    (ap + "g", lw.w_in[q + k + v:q + k + v + a.heads * a.vdim]),
                    (ap + "o", lw.w_ao), (ap + "talk", lw.talk),
                    (p + "mix.left.out", lw.out_a), (p + "mix.right.out", lw.out_r)]
        ml = lw.spec.mlp
        if ml is not None:
            F_ = ml.ff
            out += [(p + "norm2", lw.norm2), (p + "norm2b", lw.norm2b),
                    (p + "mlp.router", lw.router), (p + "mlp.router.b", lw.router_b)]
            for e in range(ml.router.experts):
                out += [(p + f"mlp.e{e}.gate", lw.w_up[e * 2 * F_:e * 2 * F_ + F_]),
                        (p + f"mlp.e{e}.up", lw.w_up[e * 2 * F_ + F_:(e + 1) * 2 * F_]),
                        (p + f"mlp.e{e}.down", lw.w_down[:, e * F_:(e + 1) * F_])]
        return out

    def _all_names(self):
        out = [("embed", self.embed), ("embed.norm", self.embed_norm),
               ("final.norm", self.final_norm), ("head", self.lm_head)]
        for i, lw in enumerate(self.layers):
            out += self._names(i, lw)
        return out

    def state_dict(self) -> dict:
        """The weights under the checkpoint's names (norm weights as single numbers)."""
        sd = {}
        for name, t in self._all_names():
            sd[name] = t.reshape(()).clone() if t.numel() == 1 and t.dtype == torch.float32 \
                and ("norm" in name.rsplit(".", 1)[-1]) else t.clone()
        return sd

    def load_state_dict(self, sd: dict) -> None:
        """Checkpoint tensors (bf16 safetensors) into the fused layout; shapes are checked
        against the config."""
        for name, dst in self._all_names():
            if name not in sd:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            src = sd[name]
            if src.numel() != dst.numel() or (src.dim() > 0 and dst.numel() > 1 and
                                              tuple(src.shape) != tuple(dst.shape)):
                raise ValueError(f"{name}: checkpoint shape {tuple(src.shape)} does not fit the "
                                 f"config (wanted {tuple(dst.shape)})")
            dst.copy_(src.reshape(dst.shape).to(dst.dtype))
        for lw in self.layers:
            lw.w_down_e = None
        self._scale_final()

    @property
    def graph_safe(self) -> bool:
        return True

    def weight_bytes(self) -> int:
        seen = [self.embed, self.embed_norm, self.final_norm, self.lm_head]
        for lw in self.layers:
            seen += [getattr(lw, f.name) for f in dataclasses.fields(lw)
                     if f.name not in ("cos_sin", "w_down_e")
                     and isinstance(getattr(lw, f.name), torch.Tensor)]
        return sum(t.numel() * t.element_size() for t in seen)

    # ------------------------------------------------------------------ cache and state
    def prefill_tile_plan(self) -> tuple:
        """(q rows per token, rows per tile, rows per tile of short steps) of the scheduler's
        prefill tile map; this model's kernels take their grids from the token rows and the
        sequence starts."""
        return 1, 128, 0

    def kv_block_bytes(self, block_size: int, kv_dtype: str = "auto") -> int:
        es = torch.empty(0, dtype=self.dtype).element_size()
        n = 0
        for i in self.runs:
            a, _ = self._parts(self.cfg.layer_specs[i])
            if a is not None:
                n += block_size * es * a.kv_heads * (a.dim + a.vdim)
        return max(n, es)

    def allocate_kv_segments(self, num_blocks: int, block_size: int, kv_dtype: str = "auto",
                             max_segment_bytes: Optional[int] = None) -> list:
        """Per layer run with an attention: K [NB, G, BS, D] (token-major rows) and V
        [NB, G, BS / 8, Dv, 8] (groups of 8 tokens, dimension-major inside a group: the 8 keys a
        matrix-core operand contracts over, or a decode lane accumulates, are one 16-byte
        load), zero-filled, in the model's dtype.  Retention layers cache nothing per token (a model
        of retention layers only gets one placeholder so the pool has a dtype)."""
        if kv_dtype not in ("auto", "bf16", "bfloat16"):
            raise ValueError("Sazepel: the KV cache is kept in the model's dtype (no fp8)")
        if block_size % 8:
            raise ValueError("Sazepel: the block size must be a multiple of 8")
        segs, self._seg_map = [], {}
        for r, i in enumerate(self.runs):
            a, _ = self._parts(self.cfg.layer_specs[i])
            if a is None:
                continue
            self._seg_map[r] = len(segs)
            segs.append(torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, dtype=self.dtype,
                                    device=self.device))
            segs.append(torch.zeros(num_blocks, a.kv_heads, block_size // 8, a.vdim, 8,
                                    dtype=self.dtype, device=self.device))
        if not segs:
            segs.append(torch.zeros(1, dtype=self.dtype, device=self.device))
        return segs

    def allocate_kv_cache(self, num_blocks: int, block_size: int, kv_dtype: str = "auto"):
        return self.allocate_kv_segments(num_blocks, block_size, kv_dtype)

    def cache_views(self, kv, block_size: int):
        segs = list(kv)
        ks, vs = [], []
        for r in range(len(self.runs)):
            j = self._seg_map.get(r)
            ks.append(segs[j] if j is not None else None)
            vs.append(segs[j + 1] if j is not None else None)
        return ks, vs

    def allocate_state(self, num_slots: int) -> None:
        """The retention state per layer run and sequence slot, transposed: [slots, H, V, D]
        fp32."""
        self.state = []
        for i in self.runs:
            _, r = self._parts(self.cfg.layer_specs[i])
            self.state.append(torch.zeros(max(1, num_slots), r.heads, r.vdim, r.dim,
                                          dtype=torch.float32, device=self.device))

    def state_bytes_per_slot(self) -> int:
        return sum(4 * self._parts(self.cfg.layer_specs[i])[1].state_floats for i in self.runs)

    # ------------------------------------------------------------------ forward
    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        if self.dtype == torch.bfloat16:
            return ops.linear(x, w)
        return F.linear(x, w)

    def _workspace(self, rows: int, a: AttentionSpec, parts: int):
        """Partial softmax state of the split attention; a buffer that has to grow (eager steps
        only: the runner warms a bucket before capturing it) is kept alive, since captured
        graphs may still point at it."""
        n_ml, n_o = 2 * rows * parts * a.heads, rows * parts * a.heads * a.kv_heads * a.vdim
        if self._ws is None or self._ws[0].numel() < n_ml or self._ws[1].numel() < n_o:
            if self._ws is not None:
                self._ws_kept.append(self._ws)
                n_ml, n_o = max(n_ml, self._ws[0].numel()), max(n_o, self._ws[1].numel())
            self._ws = (torch.empty(n_ml, dtype=torch.float32, device=self.device),
                        torch.empty(n_o, dtype=torch.float32, device=self.device))
        return self._ws

    def _attention(self, lw: SandwichLayerWeights, a: AttentionSpec, proj, batch: AttnBatch,
                   kc, vc, out) -> None:
        T = proj.shape[0]
        q = torch.empty(T, a.heads, a.dim, dtype=self.dtype, device=self.device)
        nq, nk, nv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        sops.head_norm_cache(proj, q, kc, vc, batch.slots, a.heads, a.kv_heads, a.dim, a.vdim,
                             0, nq, nq + nk, self.cfg.rms_eps, a.head_norm, a.v_norm)
        gate = proj[:, nq + nk + nv:nq + nk + nv + a.heads * a.vdim] if a.gate else None
        talk = lw.talk if a.talk else None
        if batch.is_prefill:
            sops.talking_attention_prefill(out, q, kc, vc, batch.block_tables, batch.seq_lens,
                                           batch.q_start, batch.positions, batch.tile_seq,
                                           batch.tile_row, batch.tile_rows, talk, gate, a.scale,
                                           first_seq=batch.num_decode)
            return
        parts, ws = 1, None
        if q.is_cuda:
            parts = sops.talking_attention_parts(T, a.kv_heads, self.max_model_len)
            ws = self._workspace(T, a, parts)
        sops.talking_attention_decode(out, q, kc, vc, batch.block_tables, batch.seq_lens,
                                      batch.positions, talk, gate, a.scale, ws, parts)

    def _grouped_ok(self, h2: torch.Tensor, ff: int) -> bool:
        """Can the core library's grouped expert GEMMs run this layer (bf16 on the GPU, the
        library loaded -- a replay engine that returns logits alone runs without it --, both
        reduction depths multiples of 64)?"""
        return (h2.is_cuda and self.dtype == torch.bfloat16 and ops.native_loaded()
                and h2.shape[1] % 64 == 0 and ff % 64 == 0)

    def _routed(self, lw: SandwichLayerWeights, h2: torch.Tensor, small: bool) -> torch.Tensor:
        """The routed feed-forward of h2 [T, d] (fp32, or the activation type from the grouped
        GEMMs)."""
        ml = lw.spec.mlp
        rt, F_ = ml.router, ml.ff
        T, d = h2.shape
        E = rt.experts
        ids, w = sops.route_topk(h2, lw.router, lw.router_b, rt.top)
        if small:
            out = torch.empty(T, d, dtype=torch.float32, device=h2.device)
            gu = self._linear(h2, lw.w_up)                       # every expert: [T, E 2F]
            act = torch.empty(T, E * F_, dtype=gu.dtype, device=gu.device)
            sops.swiglu_routed(gu, ids, w, E, act)
            sops.moe_combine(out, self._linear(act, lw.w_down), None, ids, w, h2, E)
            return out

        if self._grouped_ok(h2, F_):
            # prompt-sized batches on an engine that has the core library: the framework's
            # grouped expert GEMMs (device-side sort and tile map, SwiGLU in the epilogue, no
            # host round trip); they take the down-projections per expert, [E, d, F]
            if lw.w_down_e is None:
                lw.w_down_e = lw.w_down.view(d, E, F_).permute(1, 0, 2).contiguous()
            return ops.fused_moe(h2, lw.w_up.view(E, 2 * F_, d), lw.w_down_e, w, ids)

        def expert(e: int, rows: torch.Tensor) -> torch.Tensor:
            gu = F.linear(rows, lw.w_up[e * 2 * F_:(e + 1) * 2 * F_])
            u = torch.empty(rows.shape[0], F_, dtype=gu.dtype, device=gu.device)
            sops.swiglu(gu, u)
            return F.linear(u, lw.w_down[:, e * F_:(e + 1) * F_])

        return routed_sorted(h2, ids, w, E, E, expert)

    def forward(self, input_ids: torch.Tensor, batch: AttnBatch, k_caches, v_caches
                ) -> torch.Tensor:
        cfg, dt, dev = self.cfg, self.dtype, self.device
        T, d = input_ids.shape[0], cfg.hidden_size
        eps = cfg.rms_eps
        if self.state is None:
            raise RuntimeError("Sazepel: allocate_state() must run before forward()")
        if batch.tail_slot is None:
            raise RuntimeError("Sazepel: the batch carries no sequence slots")
        seq_slot = batch.tail_slot[:T]
        q_start = batch.q_start if batch.is_prefill else None
        small = (not batch.is_prefill) or T <= MOE_DENSE_ROWS
        e = sops.embed_scaled(input_ids, self.embed, 1.0)
        x = torch.empty_like(e)                                  # fp32 [T, d]: the stream
        h = torch.empty(T, d, dtype=dt, device=dev)
        sops.stream_post_norm_add_norm(x, e, None, None, None, self.embed_norm,
                                       self.layers[self.runs[0]].norm1, eps, h, fresh=True)
        for r, li in enumerate(self.runs):
            lw = self.layers[li]
            a, rs = self._parts(lw.spec)
            nxt = self.layers[self.runs[r + 1]].norm1 if r + 1 < len(self.runs) else self._final_w
            proj = self._linear(h, lw.w_in)
            hd, hv = rs.heads * rs.dim, rs.heads * rs.vdim
            o = lw.ret_off
            ret = torch.empty(T, hv, dtype=dt, device=dev)
            sops.retention(ret, proj, o, o + hd, o + 2 * hd, o + 2 * hd + hv, self.state[r],
                           seq_slot, batch.positions, q_start, lw.cos_sin, lw.log2_decay,
                           rs.heads, rs.dim, rs.vdim, eps)
            y_r = self._linear(ret, lw.w_o)
            y_a = None
            if a is not None:
                att = torch.empty(T, a.heads * a.vdim, dtype=dt, device=dev)
                self._attention(lw, a, proj, batch, k_caches[r], v_caches[r], att)
                y_a = self._linear(att, lw.w_ao)
            h = torch.empty(T, d, dtype=dt, device=dev)
            after = lw.norm2 if lw.spec.mlp is not None else nxt
            if y_a is None:
                sops.stream_post_norm_add_norm(x, y_r, None, None, None, lw.norm1b, after, eps, h)
            else:
                sops.stream_post_norm_add_norm(x, y_a, y_r, lw.out_a, lw.out_r, lw.norm1b, after,
                                               eps, h)
            if lw.spec.mlp is not None:
                y2 = self._routed(lw, h, small)
                h = torch.empty(T, d, dtype=dt, device=dev)
                sops.stream_post_norm_add_norm(x, y2, None, None, None, lw.norm2b, nxt, eps, h)
        return h

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.lm_head)
