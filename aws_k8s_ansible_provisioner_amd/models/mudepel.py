"""Mudepel: a layered decoder over several fp32 residual streams (LayeredConfig, arch "mudepel").

Layers are pre-norm (RMS norm whose weight is stored around zero: rms(x) (1 + w)) and
sequential, mixer then feed-forward.  Instead of one residual there are S streams, all equal to
the embedding at the start: a sublayer reads u = sum_s in[s] x_s, and its output y is written as
x_r <- sum_s mix[s, r] x_s + out[r] y with learned in / mix / out per sublayer; the model's
output norm reads the plain sum of the streams.  Mixers: "attention" -- grouped-query attention
with biased projections, rotate-half rotary positions under YaRN scaling, a sliding window plus
one mean key / mean value for every block of `pool` tokens wholly before the window, and a
constant 1 in the softmax denominator -- or "mamba2", a selective state-space layer (causal
convolution + silu on x, B, C; per-head fp32 state S [state, vdim]; silu gate, grouped RMS
norm).  Feed-forwards: dense gelu-gated, or routed (sigmoid scores, group-limited top-k,
silu-gated experts weighted by their scores, a shared expert).  A span of layers can run
several times with the same weights (own cache and state per pass).  The embedding is the
output head; logits are capped by tanh.

MI355X mapping.  Per sublayer one GEMM in and one GEMM out, through ops.linear like the other
layered models (tuned MFMA kernels for decode-sized batches, hipBLASLt for prompts).  Between
sublayers ONE kernel does the stream write, the next sublayer's read and its norm on the
[T, S, d] fp32 streams (a token's streams are contiguous, read and written once).  Attention:
one kernel adds the biases, rotates and writes q and the paged K / V cache; one small kernel
refreshes the pooled entries of blocks that a token of the step completed (fp32, stored with
the page of the block's first token, so pages and pooled entries are freed together); one
attention kernel walks pooled entries and window tokens in a single online softmax that starts
from the sink.  State space: one kernel for convolution + silu with the last taps - 1 inputs
in the scheduler's sequence slots, one scan kernel with the state in registers (a workgroup
per sequence and head), one kernel for gate and grouped norm.  The routed feed-forward takes
its path by batch size like the framework's other routed models; the shared expert rides in the
same GEMM pair as the routed ones.  Decode steps are sync-free and allocation-stable, so the
runner captures them in hipGraphs.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import stream as sops
from ..parallel.state import ParallelState, get_state
from .config import AttentionSpec, LayeredConfig, LayerSpec, StateSpaceSpec
from .routed import MOE_DENSE_ROWS, routed_sorted
from .transformer import AttnBatch


@dataclasses.dataclass
class HyperWeights:
    """Read / mix / write weights of one sublayer over the streams (fp32)."""
    w_in: torch.Tensor      # [S]
    w_out: torch.Tensor     # [S]
    mix: torch.Tensor       # [S, S], indexed [from, to]


@dataclasses.dataclass
class StreamLayerWeights:
    spec: LayerSpec
    norm1: torch.Tensor                       # fp32 [d], stored around zero
    norm1p: torch.Tensor                      # 1 + norm1
    hc1: HyperWeights
    w_in: torch.Tensor                        # attention [q | k | v, d]; state space [z|x|B|C|dt, d]
    w_o: torch.Tensor                         # [d, H Dv] / [d, inner]
    b_in: Optional[torch.Tensor] = None       # fp32 [rows of w_in]: q / k / v biases
    b_o: Optional[torch.Tensor] = None        # fp32 [d]
    cos_sin: Optional[torch.Tensor] = None
    conv_w: Optional[torch.Tensor] = None     # fp32 [C, taps]
    conv_b: Optional[torch.Tensor] = None     # fp32 [C]
    dt_bias: Optional[torch.Tensor] = None    # fp32 [H]
    a_log: Optional[torch.Tensor] = None
    d_skip: Optional[torch.Tensor] = None
    gnorm: Optional[torch.Tensor] = None      # fp32 [inner]
    norm2: Optional[torch.Tensor] = None
    norm2p: Optional[torch.Tensor] = None
    hc2: Optional[HyperWeights] = None
    w_up: Optional[torch.Tensor] = None       # dense [2 ff, d] = [gate | up]; routed: per expert
    w_down: Optional[torch.Tensor] = None     # [gate | up] then the shared one; [d, sum of ffs]
    router: Optional[torch.Tensor] = None     # fp32 [E, d]
    w_down_e: Optional[torch.Tensor] = None   # [E, d, F]: the routed experts' down-projections,
                                              # made on first use


class MudepelLM:
    """Weights + forward of one replica (same surface as DecoderLM for the model runner)."""

    supports_v_tail = False
    gemm_tunable = True
    gemm_weight_names = ("w_in", "w_o", "w_up", "w_down")
    fused_gemm_chain = False
    dtypes = (torch.bfloat16, torch.float32)
    # convolution inputs and state-space states of a live sequence sit in one of the
    # scheduler's sequence slots: the runner sizes the slot pool and turns prefix caching off
    state_slots = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cpu",
                 dtype: torch.dtype = torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, max_model_len: int = 4096,
                 full_then_shard: bool = False, init_std: float = 0.02):
        if dtype not in self.dtypes:
            raise ValueError(f"Mudepel runs in bfloat16 or float32, not {dtype}")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError("Mudepel: tensor parallelism is not implemented (tp must be 1)")
        if max_model_len > cfg.max_position:
            raise ValueError(f"max_model_len {max_model_len} exceeds max_position "
                             f"{cfg.max_position}")
        self.max_model_len = max_model_len
        self.init_std = init_std
        self.runs = cfg.layer_runs()
        self.S = max(1, cfg.streams)
        self.hq, self.hkv, self.D = cfg.num_heads, max(1, cfg.num_kv_heads), cfg.head_dim
        self.ffn = cfg.intermediate_size
        self.vocab_start, self.vocab_end = 0, cfg.vocab_size
        self._tables: dict = {}
        self.state: Optional[list] = None       # per run: (conv inputs, states) or None
        self.pooled: dict = {}                  # run -> (k_pool, v_pool)
        self._seg_map: dict = {}
        self._init_weights(seed)

    # ------------------------------------------------------------------ weights
    def _table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        key = (rot.dims, rot.base, tuple(sorted((rot.scaling or {}).items())))
        if key not in self._tables:
            self._tables[key] = sops.rotary_table_yarn(max(self.max_model_len, 16), rot.dims,
                                                       rot.base, rot.scaling, device=self.device)
        return self._tables[key]

    @staticmethod
    def _mlp_cols(ml) -> tuple:
        """(rows of w_up, columns of w_down) of a feed-forward."""
        if ml.kind == "dense":
            return 2 * ml.ff, ml.ff
        E = ml.router.experts
        return E * 2 * ml.ff + 2 * ml.shared_ff, E * ml.ff + ml.shared_ff

    def _init_weights(self, seed: int) -> None:
        cfg, d, S = self.cfg, self.cfg.hidden_size, self.S
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        std = self.init_std
        f32 = torch.float32

        def rand(*shape, s=std, mean=0.0, dt=None):
            t = torch.empty(*shape, dtype=f32).normal_(mean, s, generator=g)
            return t.to(torch.bfloat16).to(dt or self.dtype).to(self.device)

        def hyper():
            if cfg.streams <= 0:        # one stream, plain residual sum
                one = torch.ones(1, dtype=f32, device=self.device)
                return HyperWeights(one, one.clone(), one.clone().view(1, 1))
            eye = torch.eye(S) + 0.1 * torch.randn(S, S, generator=g)
            return HyperWeights(rand(S, s=0.2, mean=1.0 / S, dt=f32), rand(S, s=0.2, mean=1.0, dt=f32),
                                eye.to(torch.bfloat16).to(f32).to(self.device))

        self.embed = rand(cfg.vocab_size, d, s=1.0)
        self.layers: list[StreamLayerWeights] = []
        for ls in cfg.layer_specs:
            m = ls.mixer
            if isinstance(m, AttentionSpec):
                n = m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)
                lw = StreamLayerWeights(
                    spec=ls, norm1=rand(d, s=0.1, dt=f32), norm1p=None, hc1=hyper(),
                    w_in=rand(n, d), w_o=rand(d, m.heads * m.vdim),
                    b_in=rand(n, s=0.1, dt=f32) if m.bias else None,
                    b_o=rand(d, s=0.1, dt=f32) if m.bias else None, cos_sin=self._table(m.rot))
            else:
                C = m.conv_channels
                lw = StreamLayerWeights(
                    spec=ls, norm1=rand(d, s=0.1, dt=f32), norm1p=None, hc1=hyper(),
                    w_in=rand(m.proj_rows, d), w_o=rand(d, m.inner),
                    conv_w=rand(C, m.conv, s=0.3, dt=f32), conv_b=rand(C, s=0.1, dt=f32),
                    dt_bias=rand(m.heads, s=0.5, mean=-1.0, dt=f32),
                    a_log=rand(m.heads, s=0.5, mean=0.0, dt=f32),
                    d_skip=rand(m.heads, s=0.2, mean=1.0, dt=f32),
                    gnorm=rand(m.inner, s=0.1, mean=1.0, dt=f32))
            ml = ls.mlp
            if ml is not None:
                up, down = self._mlp_cols(ml)
                lw.norm2, lw.hc2 = rand(d, s=0.1, dt=f32), hyper()
                lw.w_up, lw.w_down = rand(up, d), rand(d, down)
                if ml.kind == "moe":
                    lw.router = rand(ml.router.experts, d, s=4 * std, dt=f32)
            self.layers.append(lw)
        self.final_norm = rand(d, s=0.1, dt=f32)
        self._derive()

    def _derive(self) -> None:
        """What the kernels read instead of the stored tensors: 1 + w of every norm, and the
        read weights of the output norm (the plain sum of the streams)."""
        for lw in self.layers:
            lw.norm1p = lw.norm1 + 1.0
            if lw.norm2 is not None:
                lw.norm2p = lw.norm2 + 1.0
        self._final_p = self.final_norm + 1.0
        self._sum_in = torch.ones(self.S, dtype=torch.float32, device=self.device)

    def _names(self, i: int, lw: StreamLayerWeights):
        """(checkpoint name, destination view) of layer i."""
        p = f"l{i}."
        m = lw.spec.mixer
        out = [(p + "norm1", lw.norm1)]
        hcs = [("hc1", lw.hc1)]
        if isinstance(m, AttentionSpec):
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            out += [(p + "mix.q", lw.w_in[:q]), (p + "mix.k", lw.w_in[q:q + k]),
                    (p + "mix.v", lw.w_in[q + k:q + k + v]), (p + "mix.o", lw.w_o)]
            if m.bias:
                out += [(p + "mix.q.b", lw.b_in[:q]), (p + "mix.k.b", lw.b_in[q:q + k]),
                        (p + "mix.v.b", lw.b_in[q + k:q + k + v]), (p + "mix.o.b", lw.b_o)]
        else:
            out += [(p + "mix.in", lw.w_in), (p + "mix.conv", lw.conv_w),
                    (p + "mix.conv.b", lw.conv_b), (p + "mix.dt_bias", lw.dt_bias),
                    (p + "mix.A_log", lw.a_log), (p + "mix.D", lw.d_skip),
                    (p + "mix.norm", lw.gnorm), (p + "mix.o", lw.w_o)]
        ml = lw.spec.mlp
        if ml is not None:
            out.append((p + "norm2", lw.norm2))
            hcs.append(("hc2", lw.hc2))
            F_ = ml.ff
            if ml.kind == "dense":
                out += [(p + "mlp.gate", lw.w_up[:F_]), (p + "mlp.up", lw.w_up[F_:]),
                        (p + "mlp.down", lw.w_down)]
            else:
                E = ml.router.experts
                out.append((p + "mlp.router", lw.router))
                for e in range(E):
                    out += [(p + f"mlp.e{e}.gate", lw.w_up[e * 2 * F_:e * 2 * F_ + F_]),
                            (p + f"mlp.e{e}.up", lw.w_up[e * 2 * F_ + F_:(e + 1) * 2 * F_]),
                            (p + f"mlp.e{e}.down", lw.w_down[:, e * F_:(e + 1) * F_])]
                if ml.shared_ff:
                    Fs, u0, d0 = ml.shared_ff, E * 2 * F_, E * F_
                    out += [(p + "mlp.shared.gate", lw.w_up[u0:u0 + Fs]),
                            (p + "mlp.shared.up", lw.w_up[u0 + Fs:u0 + 2 * Fs]),
                            (p + "mlp.shared.down", lw.w_down[:, d0:d0 + Fs])]
        if self.cfg.streams > 0:
            for name, hc in hcs:
                out += [(p + name + ".in", hc.w_in), (p + name + ".out", hc.w_out),
                        (p + name + ".mix", hc.mix)]
        return out

    def _all_names(self):
        out = [("embed", self.embed), ("final.norm", self.final_norm)]
        for i, lw in enumerate(self.layers):
            out += self._names(i, lw)
        return out

    def state_dict(self) -> dict:
        """The weights under the checkpoint's names."""
        return {name: t.clone() for name, t in self._all_names()}

    def load_state_dict(self, sd: dict) -> None:
        """Checkpoint tensors (bf16 safetensors) into the fused layout; shapes are checked
        against the config."""
        for name, dst in self._all_names():
            if name not in sd:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            src = sd[name]
            if tuple(src.shape) != tuple(dst.shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(src.shape)} does not fit the "
                                 f"config (wanted {tuple(dst.shape)})")
            dst.copy_(src.to(dst.dtype))
        for lw in self.layers:
            lw.w_down_e = None
        self._derive()

    @property
    def graph_safe(self) -> bool:
        return True

    def weight_bytes(self) -> int:
        skip = ("cos_sin", "norm1p", "norm2p", "spec", "hc1", "hc2", "w_down_e")
        seen = [self.embed, self.final_norm]
        for lw in self.layers:
            seen += [getattr(lw, f.name) for f in dataclasses.fields(lw)
                     if f.name not in skip and isinstance(getattr(lw, f.name), torch.Tensor)]
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
            m = self.cfg.layer_specs[i].mixer
            if isinstance(m, AttentionSpec):
                n += block_size * es * m.kv_heads * (m.dim + m.vdim)
                n += sops.pool_slots(block_size, m.pool) * 4 * m.kv_heads * (m.dim + m.vdim)
        return max(n, es)

    def allocate_kv_segments(self, num_blocks: int, block_size: int, kv_dtype: str = "auto",
                             max_segment_bytes: Optional[int] = None) -> list:
        """Per layer run with an attention: K [NB, G, BS, D] (token-major rows) and V
        [NB, G, BS / 8, Dv, 8] (groups of 8 tokens, dimension-major inside a group: what a
        matrix-core operand contracts over is one 16-byte load) in the model's dtype, and for a
        pooled mask the fp32 entries K [NB, G, n, D],
        V [NB, G, n, Dv] of the blocks that start in each page (n = ceil(BS / pool)), kept by
        the model beside the pages they belong to.  State-space layers cache nothing per
        token."""
        if kv_dtype not in ("auto", "bf16", "bfloat16"):
            raise ValueError("Mudepel: the KV cache is kept in the model's dtype (no fp8)")
        if block_size % 8:
            raise ValueError("Mudepel: the block size must be a multiple of 8")
        segs, self._seg_map, self.pooled = [], {}, {}
        for r, i in enumerate(self.runs):
            m = self.cfg.layer_specs[i].mixer
            if not isinstance(m, AttentionSpec):
                continue
            self._seg_map[r] = len(segs)
            segs.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.dim, dtype=self.dtype,
                                    device=self.device))
            segs.append(torch.zeros(num_blocks, m.kv_heads, block_size // 8, m.vdim, 8,
                                    dtype=self.dtype, device=self.device))
            if m.pool > 0:
                n = sops.pool_slots(block_size, m.pool)
                self.pooled[r] = (
                    torch.zeros(num_blocks, m.kv_heads, n, m.dim, dtype=torch.float32,
                                device=self.device),
                    torch.zeros(num_blocks, m.kv_heads, n, m.vdim, dtype=torch.float32,
                                device=self.device))
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
        """Per state-space layer run and sequence slot: the last taps - 1 convolution inputs
        [slots, taps - 1, C] (activation type) and the states [slots, H, N, V] (fp32)."""
        self.state = []
        n = max(1, num_slots)
        for i in self.runs:
            m = self.cfg.layer_specs[i].mixer
            if not isinstance(m, StateSpaceSpec):
                self.state.append(None)
                continue
            self.state.append((
                torch.zeros(n, max(1, m.conv - 1), m.conv_channels, dtype=self.dtype,
                            device=self.device),
                torch.zeros(n, m.heads, m.state, m.vdim, dtype=torch.float32,
                            device=self.device)))

    def state_bytes_per_slot(self) -> int:
        es = torch.empty(0, dtype=self.dtype).element_size()
        n = 0
        for i in self.runs:
            m = self.cfg.layer_specs[i].mixer
            if isinstance(m, StateSpaceSpec):
                n += 4 * m.state_floats + es * (m.conv - 1) * m.conv_channels
        return n

    # ------------------------------------------------------------------ forward
    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        if self.dtype == torch.bfloat16:
            return ops.linear(x, w)
        return F.linear(x, w)

    def _attention(self, lw: StreamLayerWeights, m: AttentionSpec, h, batch: AttnBatch, r: int,
                   kc, vc, q_start) -> torch.Tensor:
        T = h.shape[0]
        proj = self._linear(h, lw.w_in)
        nq, nk = m.heads * m.dim, m.kv_heads * m.dim
        q = torch.empty(T, m.heads, m.dim, dtype=self.dtype, device=self.device)
        sops.bias_rope_cache(proj, q, kc, vc, batch.positions, batch.slots, lw.cos_sin, lw.b_in,
                             m.heads, m.kv_heads, m.dim, m.vdim, 0, nq, nq + nk)
        kp, vp = self.pooled.get(r, (None, None))
        if kp is not None:
            sops.pool_cache_blocks(kc, vc, kp, vp, batch.positions, batch.slots,
                                   batch.block_tables, q_start, m.pool)
        att = torch.empty(T, m.heads * m.vdim, dtype=self.dtype, device=self.device)
        if batch.is_prefill:
            sops.pooled_window_attention_prefill(
                att, q, kc, vc, kp, vp, batch.block_tables, q_start, batch.positions, batch.slots,
                batch.tile_seq, batch.tile_row, batch.tile_rows, m.scale, m.window, m.pool,
                m.unit_sink, first_seq=batch.num_decode)
        else:
            sops.pooled_window_attention_decode(att, q, kc, vc, kp, vp, batch.block_tables,
                                                batch.positions, batch.slots, m.scale, m.window,
                                                m.pool, m.unit_sink)
        return self._linear(att, lw.w_o)

    def _state_space(self, lw: StreamLayerWeights, m: StateSpaceSpec, h, batch: AttnBatch,
                     r: int, seq_slot, q_start) -> torch.Tensor:
        T = h.shape[0]
        conv_state, states = self.state[r]
        proj = self._linear(h, lw.w_in)                  # [z | x | B | C | dt]
        inner, C = m.inner, m.conv_channels
        xbc = torch.empty(T, C, dtype=torch.float32, device=self.device)
        sops.conv_silu(xbc, proj, inner, lw.conv_w, lw.conv_b, conv_state, seq_slot,
                       batch.positions, q_start)
        y = torch.empty(T, inner, dtype=torch.float32, device=self.device)
        sops.selective_scan(y, xbc, proj, inner + C, lw.dt_bias, lw.a_log, lw.d_skip, states,
                            seq_slot, batch.positions, q_start, m.heads, m.vdim, m.state, m.groups)
        g = torch.empty(T, inner, dtype=self.dtype, device=self.device)
        sops.gate_group_norm(g, y, proj[:, :inner], lw.gnorm, m.norm_groups, self.cfg.rms_eps)
        return self._linear(g, lw.w_o)

    def _grouped_ok(self, h2: torch.Tensor, ff: int) -> bool:
        """Can the core library's grouped expert GEMMs run this layer (bf16 on the GPU, the
        library loaded -- a replay engine that returns logits alone runs without it --, both
        reduction depths multiples of 64)?"""
        return (h2.is_cuda and self.dtype == torch.bfloat16 and ops.native_loaded()
                and h2.shape[1] % 64 == 0 and ff % 64 == 0)

    def _feed_forward(self, lw: StreamLayerWeights, h2: torch.Tensor, small: bool):
        """(output in the activation type or None, fp32 output or None) of the feed-forward."""
        ml = lw.spec.mlp
        T, d = h2.shape
        F_ = ml.ff
        if ml.kind == "dense":
            gu = self._linear(h2, lw.w_up)
            act = torch.empty(T, F_, dtype=gu.dtype, device=gu.device)
            sops.gated_act(gu, act, "gelu_tanh")
            return self._linear(act, lw.w_down), None
        rt = ml.router
        E, Fs = rt.experts, ml.shared_ff
        ids, w = sops.route_sigmoid(h2, lw.router, rt.top, rt.groups, rt.keep, rt.group_top)
        if small:
            # every expert and the shared one as one GEMM pair: the gated activations are
            # scaled by the routing weights (0 for experts not chosen, 1 for the shared one)
            # and summed inside the down-projection's accumulator
            gu = self._linear(h2, lw.w_up)
            act = torch.empty(T, E * F_ + Fs, dtype=gu.dtype, device=gu.device)
            sops.gated_act(gu[:, :E * 2 * F_], act[:, :E * F_], "silu", ids, w, E)
            if Fs:
                sops.gated_act(gu[:, E * 2 * F_:], act[:, E * F_:], "silu")
            return self._linear(act, lw.w_down), None

        def expert(e: int, rows: torch.Tensor) -> torch.Tensor:
            gu = F.linear(rows, lw.w_up[e * 2 * F_:(e + 1) * 2 * F_])
            u = torch.empty(rows.shape[0], F_, dtype=gu.dtype, device=gu.device)
            sops.gated_act(gu, u, "silu")
            return F.linear(u, lw.w_down[:, e * F_:(e + 1) * F_])

        if self._grouped_ok(h2, F_):
            # prompt-sized batches on an engine that has the core library: the framework's
            # grouped expert GEMMs (device-side sort and tile map, silu gate in the epilogue, no
            # host round trip); they take the down-projections per expert, [E, d, F]
            if lw.w_down_e is None:
                lw.w_down_e = lw.w_down[:, :E * F_].reshape(d, E, F_).permute(1, 0, 2).contiguous()
            routed = ops.fused_moe(h2, lw.w_up[:E * 2 * F_].view(E, 2 * F_, d), lw.w_down_e, w,
                                   ids)
        else:
            routed = routed_sorted(h2, ids, w, E, E, expert)
        shared = None
        if Fs:
            gu = self._linear(h2, lw.w_up[E * 2 * F_:])
            u = torch.empty(T, Fs, dtype=gu.dtype, device=gu.device)
            sops.gated_act(gu, u, "silu")
            shared = self._linear(u, lw.w_down[:, E * F_:])
        return shared, routed

    def forward(self, input_ids: torch.Tensor, batch: AttnBatch, k_caches, v_caches
                ) -> torch.Tensor:
        cfg, dt, dev = self.cfg, self.dtype, self.device
        T, d = input_ids.shape[0], cfg.hidden_size
        eps = cfg.rms_eps
        if self.state is None:
            raise RuntimeError("Mudepel: allocate_state() must run before forward()")
        if batch.tail_slot is None:
            raise RuntimeError("Mudepel: the batch carries no sequence slots")
        seq_slot = batch.tail_slot[:T]
        q_start = batch.q_start if batch.is_prefill else None
        small = (not batch.is_prefill) or T <= MOE_DENSE_ROWS
        e = sops.embed_scaled(input_ids, self.embed, 1.0)
        xs = torch.empty(T, self.S, d, dtype=torch.float32, device=dev)     # the streams
        first = self.layers[self.runs[0]]
        h = torch.empty(T, d, dtype=dt, device=dev)
        sops.hyper_step(xs, None, None, None, None, None, first.hc1.w_in, first.norm1p, eps, h,
                        fresh=e)
        for r, li in enumerate(self.runs):
            lw = self.layers[li]
            m = lw.spec.mixer
            if r + 1 < len(self.runs):
                nl = self.layers[self.runs[r + 1]]
                nxt = (nl.hc1.w_in, nl.norm1p)
            else:
                nxt = (self._sum_in, self._final_p)
            if isinstance(m, AttentionSpec):
                y = self._attention(lw, m, h, batch, r, k_caches[r], v_caches[r], q_start)
            else:
                y = self._state_space(lw, m, h, batch, r, seq_slot, q_start)
            after = (lw.hc2.w_in, lw.norm2p) if lw.spec.mlp is not None else nxt
            h = torch.empty(T, d, dtype=dt, device=dev)
            sops.hyper_step(xs, y, None, lw.b_o, lw.hc1.mix, lw.hc1.w_out, after[0], after[1],
                            eps, h)
            if lw.spec.mlp is not None:
                ya, yb = self._feed_forward(lw, h, small)
                h = torch.empty(T, d, dtype=dt, device=dev)
                sops.hyper_step(xs, ya, yb, None, lw.hc2.mix, lw.hc2.w_out, nxt[0], nxt[1], eps, h)
        return h

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        logits = F.linear(h, self.embed)
        if self.cfg.logit_softcap > 0:
            sops.softcap_(logits, self.cfg.logit_softcap)
        return logits
