"""Puputar: a layered decoder over an fp32 residual stream (LayeredConfig, arch "puputar").

The embedding is normed once (RMS norm in groups).  Every layer is PARALLEL with two norms of
the same stream: x <- x + mixer(shift(norm1(x))) + ff(norm2(x)).  The token shift blends each
row of norm1(x) with the previous token's unshifted row (per-channel weights); that previous
row is the only recurrent state of a sequence, one row per layer, kept in the scheduler's
sequence slots.  The mixer is latent attention: queries W_uq rms(W_dq h); ONE cached row per
token, [c | k_rot] = [rms(W_dkv h)[:R] | rot(W_dkv h)[R:]], from which every head's keys
(W_uk c) and values (W_uv c) derive; a sigmoid gate per head or per output entry; a layer may
read an earlier layer's cache instead of projecting a latent of its own.  The feed-forward is
dense (xIELU, biases) or routed (softmax scores, corrected grouped top-k choice, squared-ReLU
experts, identity outputs).

MI355X mapping.  Attention runs in the latent space ("absorbed" form) for prompts and decoding
alike: q_lat = W_uk^T q_unrot (a per-head batched GEMM), scores against the cached rows, the
softmax-weighted sum of cached latents, then W_uv per head (another batched GEMM) -- the cache
is read once for all heads and never expanded.  Everything that reads the shifted mixer input
is one GEMM over [W_dq | W_dkv | W_g]; a dense layer's output projection and down projection
are one GEMM over [gated heads | act(up)] with weight [W_o | W_down], so the two sublayers sum
in its fp32 accumulator.  Routed layers pick their expert path by batch size: small batches
(every decode step, hipGraph-captured) scale the activations of ALL experts by the routing
weights and sum the chosen ones inside one GEMM over the concatenated down-projections (every
expert's weights are streamed regardless; no sort, no host round trip); prompt-sized batches
sort (token, choice) pairs by expert and run each expert's rows through its own GEMMs.  The
residual update, the deferred biases and both norms of the next layer are one kernel.
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
from .config import LatentAttentionSpec, LayeredConfig, LayerSpec
from .routed import MOE_DENSE_ROWS, routed_sorted
from .transformer import AttnBatch


@dataclasses.dataclass
class LatentLayerWeights:
    spec: LayerSpec
    norm1: torch.Tensor                 # fp32 [d]
    norm2: Optional[torch.Tensor]       # fp32 [d] (None: no feed-forward)
    shift: torch.Tensor                 # fp32 [d]
    w_in: torch.Tensor                  # [dq | dkv | g | pad, d]
    kv_off: int                         # -1: the layer reads another layer's cache
    g_off: int
    dq_norm: torch.Tensor               # fp32 [q_rank]
    dkv_norm: Optional[torch.Tensor]    # fp32 [kv_rank]
    w_uq: torch.Tensor                  # [H (D + r), q_rank]
    w_uk: torch.Tensor                  # [H, R, D]: q_lat[h] = q_unrot[h] @ w_uk[h]^T
    w_uv: torch.Tensor                  # [H, V, R]: o[h] = o_lat[h] @ w_uv[h]^T
    w_out: torch.Tensor                 # [d, H V (+ ff)] = [W_o | W_down]
    b_out: Optional[torch.Tensor]       # [d]
    cos_sin: torch.Tensor
    hv: int
    ff: int = 0                         # width of the dense feed-forward fused into w_out
    w_up: Optional[torch.Tensor] = None     # dense [ff, d] | routed [E F, d]
    b_up: Optional[torch.Tensor] = None
    act: Optional[torch.Tensor] = None      # fp32 [2]
    w_down: Optional[torch.Tensor] = None   # routed [d, E F] (experts side by side)
    router: Optional[torch.Tensor] = None   # fp32 [n, d]
    correction: Optional[torch.Tensor] = None


class PuputarLM:
    """Weights + forward of one replica (same surface as DecoderLM for the model runner)."""

    supports_v_tail = False
    gemm_tunable = True
    gemm_weight_names = ("w_in", "w_uq", "w_out")
    fused_gemm_chain = False
    dtypes = (torch.bfloat16, torch.float32)
    # one row of recurrent state per layer and live sequence (the token shift's previous row):
    # the runner sizes the scheduler's sequence-slot pool for it and turns prefix caching off
    state_slots = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cpu",
                 dtype: torch.dtype = torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, max_model_len: int = 4096,
                 full_then_shard: bool = False, init_std: float = 0.02):
        if dtype not in self.dtypes:
            raise ValueError(f"Puputar runs in bfloat16 or float32, not {dtype}")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError("Puputar: tensor parallelism is not implemented (tp must be 1)")
        if max_model_len > cfg.max_position:
            raise ValueError(f"max_model_len {max_model_len} exceeds max_position "
                             f"{cfg.max_position}")
        self.max_model_len = max_model_len
        self.init_std = init_std
        self.runs = cfg.layer_runs()
        self.hq, self.hkv, self.D = cfg.num_heads, 1, cfg.head_dim
        self.ffn = cfg.intermediate_size
        self.vocab_start, self.vocab_end = 0, cfg.vocab_size
        self._tables: dict = {}
        self.state: Optional[torch.Tensor] = None
        self._ws: Optional[tuple] = None
        self._ws_kept: list = []
        self._seg_map: dict = {}
        self._init_weights(seed)

    # ------------------------------------------------------------------ weights
    def _table(self, rot) -> torch.Tensor:
        key = (rot.dims, rot.base)
        if key not in self._tables:
            self._tables[key] = sops.rotary_table(max(self.max_model_len, 16), rot.dims, rot.base,
                                                  None, device=self.device)
        return self._tables[key]

    def _init_weights(self, seed: int) -> None:
        cfg, d = self.cfg, self.cfg.hidden_size
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        std = self.init_std

        def rand(*shape, s=std, mean=0.0, dt=None):
            t = torch.empty(*shape, dtype=torch.float32).normal_(mean, s, generator=g)
            return t.to(torch.bfloat16).to(dt or self.dtype).to(self.device)

        f32 = torch.float32
        self.embed = rand(cfg.vocab_size, d, s=1.0)
        self.embed_norm = rand(d, s=0.1, mean=1.0, dt=f32)
        self.layers: list[LatentLayerWeights] = []
        for ls in cfg.layer_specs:
            m: LatentAttentionSpec = ls.mixer
            own = m.kv_from is None
            n = m.q_rank + (m.cache_dim if own else 0) + m.gate_rows
            npad = -(-n // 256) * 256
            if npad > 1.05 * n:
                npad = -(-n // 8) * 8
            w_in = torch.zeros(npad, d, dtype=self.dtype, device=self.device)
            w_in[:n] = rand(n, d)
            hv = m.heads * m.vdim
            sq, sr = m.q_rank ** -0.5, m.kv_rank ** -0.5
            lw = LatentLayerWeights(
                spec=ls, norm1=rand(d, s=0.1, mean=1.0, dt=f32), norm2=None,
                shift=rand(d, s=0.2, mean=0.5, dt=f32), w_in=w_in,
                kv_off=m.q_rank if own else -1,
                g_off=m.q_rank + (m.cache_dim if own else 0),
                dq_norm=rand(m.q_rank, s=0.1, mean=1.0, dt=f32),
                dkv_norm=rand(m.kv_rank, s=0.1, mean=1.0, dt=f32) if own else None,
                w_uq=rand(m.heads * (m.dim + m.rot_dim), m.q_rank, s=sq),
                w_uk=rand(m.heads, m.kv_rank, m.dim, s=sr),
                w_uv=rand(m.heads, m.vdim, m.kv_rank, s=sr),
                w_out=rand(d, hv), b_out=None, cos_sin=self._table(m.rot), hv=hv)
            ml = ls.mlp
            if ml is not None:
                lw.norm2 = rand(d, s=0.1, mean=1.0, dt=f32)
                if ml.kind == "dense":
                    lw.ff = ml.ff
                    lw.w_out = rand(d, hv + ml.ff)
                    lw.w_up, lw.b_up = rand(ml.ff, d), rand(ml.ff)
                    lw.b_out = rand(d)
                    lw.act = rand(2, s=0.5, dt=f32)
                else:
                    rt = ml.router
                    lw.w_up = rand(rt.experts * ml.ff, d)
                    lw.w_down = rand(d, rt.experts * ml.ff)
                    lw.router = rand(rt.outputs, d, s=4 * std, dt=f32)
                    lw.correction = rand(rt.outputs, s=0.05, dt=f32)
            self.layers.append(lw)
        self.final_norm = rand(d, s=0.1, mean=1.0, dt=f32)
        self.lm_head = rand(cfg.vocab_size, d)

    def _names(self, i: int, lw: LatentLayerWeights):
        """(checkpoint name, destination view, transform of the checkpoint tensor) of layer i."""
        m, p = lw.spec.mixer, f"l{i}."
        H, D, r, V, R = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
        same = lambda t: t  # noqa: E731
        out = [(p + "norm1", lw.norm1, same), (p + "shift", lw.shift, same),
               (p + "mix.dq", lw.w_in[:m.q_rank], same), (p + "mix.dq.norm", lw.dq_norm, same),
               (p + "mix.uq", lw.w_uq, same),
               # [H D, R] -> [H, R, D] and [H V, R] -> [H, V, R]: both contiguous in the index
               # their product contracts over
               (p + "mix.uk", lw.w_uk,
                lambda t: self._want(t, (H * D, R)).reshape(H, D, R).transpose(1, 2)),
               (p + "mix.uv", lw.w_uv, lambda t: self._want(t, (H * V, R)).reshape(H, V, R)),
               (p + "mix.g", lw.w_in[lw.g_off:lw.g_off + m.gate_rows], same),
               (p + "mix.o", lw.w_out[:, :lw.hv], same)]
        if lw.kv_off >= 0:
            out += [(p + "mix.dkv", lw.w_in[lw.kv_off:lw.kv_off + R + r], same),
                    (p + "mix.dkv.norm", lw.dkv_norm, same)]
        ml = lw.spec.mlp
        if ml is None:
            return out
        out.append((p + "norm2", lw.norm2, same))
        if ml.kind == "dense":
            out += [(p + "mlp.up", lw.w_up, same), (p + "mlp.up.b", lw.b_up, same),
                    (p + "mlp.down", lw.w_out[:, lw.hv:], same), (p + "mlp.down.b", lw.b_out, same),
                    (p + "mlp.act", lw.act, same)]
        else:
            F_ = ml.ff
            for e in range(ml.router.experts):
                out += [(p + f"mlp.e{e}.up", lw.w_up[e * F_:(e + 1) * F_], same),
                        (p + f"mlp.e{e}.down", lw.w_down[:, e * F_:(e + 1) * F_], same)]
            out += [(p + "mlp.router", lw.router, same), (p + "mlp.correction", lw.correction, same)]
        return out

    @staticmethod
    def _want(t: torch.Tensor, shape: tuple) -> torch.Tensor:
        if tuple(t.shape) != shape:
            raise ValueError(f"checkpoint shape {tuple(t.shape)} does not fit the config "
                             f"(wanted {shape})")
        return t

    def _all_names(self):
        same = lambda t: t  # noqa: E731
        out = [("embed", self.embed, same), ("embed.norm", self.embed_norm, same),
               ("final.norm", self.final_norm, same), ("head", self.lm_head, same)]
        for i, lw in enumerate(self.layers):
            out += self._names(i, lw)
        return out

    def state_dict(self) -> dict:
        """The weights under the checkpoint's names, un-fusing the per-layer GEMM weights."""
        sd = {}
        for i, lw in enumerate(self.layers):
            m = lw.spec.mixer
            sd[f"l{i}.mix.uk"] = lw.w_uk.transpose(1, 2).reshape(m.heads * m.dim, m.kv_rank).clone()
            sd[f"l{i}.mix.uv"] = lw.w_uv.reshape(m.heads * m.vdim, m.kv_rank).clone()
        for name, t, _ in self._all_names():
            if name not in sd:
                sd[name] = t.clone()
        return sd

    def load_state_dict(self, sd: dict) -> None:
        """Checkpoint tensors (bf16 safetensors) into the fused layout; shapes are checked
        against the config."""
        for name, dst, tf in self._all_names():
            if name not in sd:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            src = tf(sd[name])
            if tuple(src.shape) != tuple(dst.shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(sd[name].shape)} does not fit "
                                 f"the config (wanted {tuple(dst.shape)} after layout)")
            dst.copy_(src.to(dst.dtype))

    @property
    def graph_safe(self) -> bool:
        return True

    def weight_bytes(self) -> int:
        seen = [self.embed, self.embed_norm, self.final_norm, self.lm_head]
        for lw in self.layers:
            seen += [getattr(lw, f.name) for f in dataclasses.fields(lw)
                     if f.name != "cos_sin" and isinstance(getattr(lw, f.name), torch.Tensor)]
        return sum(t.numel() * t.element_size() for t in seen)

    # ------------------------------------------------------------------ cache and state
    def prefill_tile_plan(self) -> tuple:
        """(q rows per token, rows per tile, rows per tile of short steps) of the scheduler's
        prefill tile map (the latent attention kernel takes its grid from the token rows)."""
        return 1, 128, 0

    def _grouped(self, m: LatentAttentionSpec, block_size: int) -> bool:
        """Does the layer keep the grouped second copy of its latents (the operand layout of
        the matrix-core attention kernels: bf16 on the GPU, sizes they are built for)?"""
        if self.device.type != "cuda" or self.dtype != torch.bfloat16 or block_size % 32:
            return False
        sops.load_native(required=True)
        return bool(torch.ops.akap_stream.latent_mfma_supported(m.kv_rank, m.rot_dim))

    def kv_block_bytes(self, block_size: int, kv_dtype: str = "auto") -> int:
        es = torch.empty(0, dtype=self.dtype).element_size()
        n = 0
        for i in self.runs:
            m = self.cfg.layer_specs[i].mixer
            if m.kv_from is None:
                n += block_size * es * (m.cache_dim + (m.kv_rank if self._grouped(m, block_size)
                                                       else 0))
        return n

    def allocate_kv_segments(self, num_blocks: int, block_size: int, kv_dtype: str = "auto",
                             max_segment_bytes: Optional[int] = None) -> list:
        """Per layer that projects its own latent: one allocation [NB, BS, kv_rank + rot_dim]
        (a cached token is ONE row, [latent | rotated key]) and, where the matrix-core kernels
        run, the latents again as [NB, BS / 8, kv_rank, 8].  Zero-filled, the model's dtype."""
        if kv_dtype not in ("auto", "bf16", "bfloat16"):
            raise ValueError("Puputar: the latent cache is kept in the model's dtype (no fp8)")
        segs, self._seg_map = [], {}
        for i in self.runs:
            m = self.cfg.layer_specs[i].mixer
            if m.kv_from is not None:
                continue
            self._seg_map[i] = [len(segs), None]
            segs.append(torch.zeros(num_blocks, block_size, m.cache_dim, dtype=self.dtype,
                                    device=self.device))
            if self._grouped(m, block_size):
                self._seg_map[i][1] = len(segs)
                segs.append(torch.zeros(num_blocks, block_size // 8, m.kv_rank, 8,
                                        dtype=self.dtype, device=self.device))
        return segs

    def allocate_kv_cache(self, num_blocks: int, block_size: int, kv_dtype: str = "auto"):
        return self.allocate_kv_segments(num_blocks, block_size, kv_dtype)

    def cache_views(self, kv, block_size: int):
        """Per layer run: (row caches, grouped copies or None) of its own latents or of the
        layer it reads."""
        segs = list(kv)
        rows, groups = [], []
        for i in self.runs:
            j = self.cfg.layer_specs[i].mixer.kv_from
            a, b = self._seg_map[i if j is None else j]
            rows.append(segs[a])
            groups.append(segs[b] if b is not None else None)
        return rows, groups

    def allocate_state(self, num_slots: int) -> None:
        """The token shift's previous row per layer run and sequence slot."""
        self.state = torch.zeros(len(self.runs), max(1, num_slots), self.cfg.hidden_size,
                                 dtype=self.dtype, device=self.device)

    # ------------------------------------------------------------------ forward
    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        if self.dtype == torch.bfloat16:
            return ops.linear(x, w)
        return F.linear(x, w)

    def _decode_parts(self, rows: int, heads: int) -> int:
        """Key partitions of a decode row: static in the batch size and the model length
        (hipGraph-capturable).  One workgroup per (row, 32 heads, partition); about one
        workgroup per CU measured best (64 rows x 2112 keys, 16 heads, latent 512 + 64: 138 us
        unsplit, 64 us at 4 partitions, 80 at 8, 87 at 16), a partition never under 128 keys."""
        max_parts = max(1, math.ceil(self.max_model_len / 128))
        groups = max(1, rows * math.ceil(heads / 32))
        return min(max_parts, 64, max(1, math.ceil(256 / groups)))

    def _workspace(self, rows: int, heads: int, kv_rank: int, parts: int):
        """Partial softmax state of the split decode: (max, sum) per (row, head, partition) and
        the unnormalised latent output.  Layers differ in heads and latent size, so both
        buffers are checked; a buffer that has to grow (eager steps only: the runner warms a
        bucket before capturing it) is kept alive, since captured graphs may still point at
        it."""
        n_ml, n_o = 2 * rows * heads * parts, rows * heads * parts * kv_rank
        if self._ws is None or self._ws[0].numel() < n_ml or self._ws[1].numel() < n_o:
            if self._ws is not None:
                self._ws_kept.append(self._ws)
                n_ml, n_o = max(n_ml, self._ws[0].numel()), max(n_o, self._ws[1].numel())
            self._ws = (torch.empty(n_ml, dtype=torch.float32, device=self.device),
                        torch.empty(n_o, dtype=torch.float32, device=self.device))
        return self._ws

    def _attention(self, m: LatentAttentionSpec, o_lat, q_lat, q, batch: AttnBatch, cache,
                   groups) -> None:
        T = q.shape[0]
        nd = batch.num_decode if batch.is_prefill else T
        if nd:
            parts, ws = 1, None
            if groups is not None:
                parts = self._decode_parts(nd, m.heads)
                ws = self._workspace(nd, m.heads, m.kv_rank, parts) if parts > 1 else None
            # the leading nd rows are contiguous slices of the head-major buffers only when
            # they are all rows; a mixed step's decode rows go through narrow copies
            if nd == T:
                sops.latent_attention_decode(o_lat, q_lat, q, m.dim, cache, groups,
                                             batch.block_tables[:nd], batch.seq_lens[:nd],
                                             batch.positions[:nd], m.scale, ws, parts)
            else:
                od = torch.empty(m.heads, nd, m.kv_rank, dtype=o_lat.dtype, device=o_lat.device)
                sops.latent_attention_decode(od, q_lat[:, :nd].contiguous(), q[:nd], m.dim, cache,
                                             groups, batch.block_tables[:nd], batch.seq_lens[:nd],
                                             batch.positions[:nd], m.scale, ws, parts)
                o_lat[:, :nd] = od
        if batch.is_prefill:
            sops.latent_attention_prefill(o_lat, q_lat, q, m.dim, cache, groups,
                                          batch.block_tables, batch.seq_lens, batch.q_start,
                                          batch.positions, batch.tile_seq, batch.tile_row,
                                          batch.tile_rows, m.scale, first_seq=nd)

    def _routed(self, lw: LatentLayerWeights, h2: torch.Tensor, small: bool) -> torch.Tensor:
        """The routed feed-forward of h2 [T, d] as fp32 [T, d]."""
        ml = lw.spec.mlp
        rt, F_ = ml.router, ml.ff
        T, d = h2.shape
        E = rt.experts
        ids, w = sops.moe_route(h2, lw.router, lw.correction, rt.top, rt.groups, rt.keep)
        if small:
            out = torch.empty(T, d, dtype=torch.float32, device=h2.device)
            up = self._linear(h2, lw.w_up)                       # every expert: [T, E F]
            act = torch.empty_like(up)
            sops.relu2_routed(up, ids, w, E, act)
            sops.moe_combine(out, self._linear(act, lw.w_down), None, ids, w, h2, E)
            return out

        def expert(e: int, rows: torch.Tensor) -> torch.Tensor:
            u = F.linear(rows, lw.w_up[e * F_:(e + 1) * F_])
            sops.relu2(u, u)
            return F.linear(u, lw.w_down[:, e * F_:(e + 1) * F_])

        return routed_sorted(h2, ids, w, E, rt.outputs, expert)

    def forward(self, input_ids: torch.Tensor, batch: AttnBatch, k_caches, v_caches
                ) -> torch.Tensor:
        cfg, dt, dev = self.cfg, self.dtype, self.device
        T, d = input_ids.shape[0], cfg.hidden_size
        eps, groups = cfg.rms_eps, cfg.norm_groups
        if self.state is None:
            raise RuntimeError("Puputar: allocate_state() must run before forward()")
        seq_slot = batch.tail_slot
        if seq_slot is None:
            raise RuntimeError("Puputar: the batch carries no sequence slots")
        seq_slot = seq_slot[:T]
        small = (not batch.is_prefill) or T <= MOE_DENSE_ROWS
        e = sops.embed_scaled(input_ids, self.embed, 1.0)
        x = torch.empty_like(e)                                  # fp32 [T, d]: the stream
        sops.stream_add_group_norm(e, None, None, None, self.embed_norm, None, groups, eps, x)
        n1 = torch.empty(T, d, dtype=dt, device=dev)
        n2 = torch.empty(T, d, dtype=dt, device=dev)
        h = torch.empty(T, d, dtype=dt, device=dev)
        y = y2 = bias = None
        for r, li in enumerate(self.runs):
            lw = self.layers[li]
            m: LatentAttentionSpec = lw.spec.mixer
            H, D, rd, V, R = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
            if batch.is_prefill:
                sops.stream_add_group_norm(x, y, y2, bias, lw.norm1, lw.norm2, groups, eps, n1,
                                           n2 if lw.norm2 is not None else None)
                sops.token_shift(n1, lw.shift, self.state[r], seq_slot, batch.positions, h)
            else:
                # every row is a sequence of its own: the shift rides in the norm kernel
                sops.stream_add_group_norm(x, y, y2, bias, lw.norm1, lw.norm2, groups, eps, h,
                                           n2 if lw.norm2 is not None else None,
                                           shift=(lw.shift, self.state[r], seq_slot,
                                                  batch.positions))
            proj = self._linear(h, lw.w_in)                      # [T, dq | dkv | g]
            cq = torch.empty(T, m.q_rank, dtype=dt, device=dev)
            sops.latent_prep(proj, cq, k_caches[r] if lw.kv_off >= 0 else None, batch.positions,
                             batch.slots, lw.cos_sin, lw.dq_norm, lw.dkv_norm, m.q_rank, R, rd,
                             0, lw.kv_off, eps, v_caches[r] if lw.kv_off >= 0 else None)
            q = self._linear(cq, lw.w_uq).view(T, H, D + rd)
            sops.rotate_heads_(q, batch.positions, lw.cos_sin, D)
            q_lat = sops.head_matmul(q[:, :, :D].transpose(0, 1), lw.w_uk)    # [H, T, R]
            o_lat = torch.empty(H, T, R, dtype=dt, device=dev)
            self._attention(m, o_lat, q_lat, q, batch, k_caches[r], v_caches[r])
            o = sops.head_matmul(o_lat, lw.w_uv)                               # [H, T, V]
            cat = torch.empty(T, lw.hv + lw.ff, dtype=dt, device=dev)
            sops.head_gate(o, proj[:, lw.g_off:lw.g_off + m.gate_rows], cat[:, :lw.hv])
            ml = lw.spec.mlp
            y2 = None
            if ml is not None and ml.kind == "dense":
                sops.xielu(self._linear(n2, lw.w_up), lw.b_up, lw.act, cat[:, lw.hv:])
            elif ml is not None:
                y2 = self._routed(lw, n2, small)
            y = self._linear(cat, lw.w_out)                      # W_o heads (+ W_down act)
            bias = lw.b_out
        out = torch.empty(T, d, dtype=dt, device=dev)
        sops.stream_add_group_norm(x, y, y2, bias, self.final_norm, None, groups, eps, out)
        return out

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.lm_head)
