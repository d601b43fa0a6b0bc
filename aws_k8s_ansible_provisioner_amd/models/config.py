"""Model architecture configs (random-init friendly: no checkpoint download needed).

The registry holds the exact shapes of the model families the reference stack
serves or the north star names (Qwen3-0.6B is what ``llm-d-deploy.yaml:118`` deploys;
Llama-3-8B / 70B and Mixtral-8x7B are the disaggregated, TP=8 and EP configs of
BASELINE.json), plus tiny variants for CPU tests.  A HF ``config.json`` can also be
loaded (``from_hf_dict``) when real weights are mounted from the model PVC.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Optional


@dataclasses.dataclass
class ModelConfig:
    name: str
    hf_id: str
    arch: str  # "qwen3" | "llama" | "mixtral" | "qwen3_moe" | "bidetar" | "puputar" | "sazepel" (LayeredConfig)
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int = 128
    rms_eps: float = 1e-6
    rope_theta: float = 10000.0
    rope_scaling: Optional[dict] = None
    max_position: int = 32768
    tie_embeddings: bool = False
    qk_norm: bool = False
    num_experts: int = 0
    experts_per_token: int = 0
    moe_renormalize: bool = True  # top-k router weights renormalised to sum 1 (norm_topk_prob)
    bos_id: int = 1
    eos_id: int = 2
    dtype: str = "bfloat16"

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def gqa_group(self) -> int:
        return self.num_heads // self.num_kv_heads

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    def kv_bytes_per_token(self, tp: int = 1) -> int:
        return self.num_layers * 2 * max(1, self.num_kv_heads // tp) * self.head_dim * 2

    def num_params(self) -> int:
        d, f, L = self.hidden_size, self.intermediate_size, self.num_layers
        attn = d * (self.q_size + 2 * self.kv_size) + self.q_size * d
        mlp = 3 * d * f * (self.num_experts if self.is_moe else 1)
        router = d * self.num_experts if self.is_moe else 0
        emb = self.vocab_size * d * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp + router + 2 * d) + emb + d

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_hf_dict(name: str, d: dict) -> "ModelConfig":
        mt = d.get("model_type", "llama")
        arch = {"qwen3": "qwen3", "mixtral": "mixtral", "qwen3_moe": "qwen3_moe"}.get(mt, "llama")
        heads = d["num_attention_heads"]
        moe_ffn = d.get("moe_intermediate_size") if arch == "qwen3_moe" else None
        return ModelConfig(
            name=name, hf_id=name, arch=arch, vocab_size=d["vocab_size"],
            hidden_size=d["hidden_size"], intermediate_size=moe_ffn or d["intermediate_size"],
            num_layers=d["num_hidden_layers"], num_heads=heads,
            num_kv_heads=d.get("num_key_value_heads", heads),
            head_dim=d.get("head_dim") or d["hidden_size"] // heads,
            rms_eps=d.get("rms_norm_eps", 1e-6), rope_theta=d.get("rope_theta", 10000.0),
            rope_scaling=d.get("rope_scaling"),
            max_position=d.get("max_position_embeddings", 32768),
            tie_embeddings=d.get("tie_word_embeddings", False),
            qk_norm=arch in ("qwen3", "qwen3_moe"),
            num_experts=d.get("num_local_experts", d.get("num_experts", 0)),
            experts_per_token=d.get("num_experts_per_tok", 0),
            moe_renormalize=bool(d.get("norm_topk_prob", True)),
            bos_id=d.get("bos_token_id", 1) or 1,
            eos_id=(d.get("eos_token_id", 2) if not isinstance(d.get("eos_token_id"), list)
                    else d["eos_token_id"][0]),
        )


@dataclasses.dataclass
class RotarySpec:
    """Rotary positions on the first `dims` dimensions of every head (pairs (2i, 2i+1)):
    f_i = base^(-2i/dims), optionally rescaled by wavelength (`scaling`: factor, low, high,
    original -- the Llama-3.1 rule)."""
    dims: int
    base: float
    scaling: Optional[dict] = None
    # layout "pairs": entries (2i, 2i+1) turn together; "half": entry i with i + dims/2.
    # scaling with the keys factor / original / fast / slow is the YaRN rule: frequencies whose
    # index lies under that of `fast` turns in `original` positions are kept, over that of
    # `slow` turns divided by factor, blended linearly in the index between, and cos and sin
    # are multiplied by 0.1 ln(factor) + 1
    layout: str = "pairs"


@dataclasses.dataclass
class AttentionSpec:
    """One attention mixer of a layered model: H query heads over G key/value heads of size
    `dim`; chunk > 0 restricts a query to the keys of its own chunk of that many positions
    (window > 0: to the last `window` keys); sink: a learned per-head logit in the softmax
    denominator; gate: a per-head sigmoid gate on the head outputs; shared_kv: the values are
    the key projection itself (before its norm and rotation)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None
    chunk: int = 0
    window: int = 0
    sink: bool = True
    gate: bool = True
    shared_kv: bool = True
    # head_norm: q and k are divided by their root mean square per head (no weights);
    # v_norm: so are the cached values; talk: the heads' softmax weights are mixed by a learned
    # [H, H] matrix before they meet the values; gate_per "element": one sigmoid gate per
    # output entry instead of one per head
    head_norm: bool = False
    v_norm: bool = False
    talk: bool = False
    gate_per: str = "head"
    # pool > 0 (with window > 0): beside the last `window` tokens a query sees one mean key and
    # mean value for every block of `pool` tokens that lies wholly before its window;
    # unit_sink: a constant 1 in the softmax denominator (a sink of score 0 without a tensor);
    # bias: the q / k / v / output projections have biases
    pool: int = 0
    unit_sink: bool = False
    bias: bool = False


@dataclasses.dataclass
class RetentionSpec:
    """Linear attention with a fixed decay per head and no softmax: per head a state
    S [dim, vdim] (fp32, one per live sequence) with S_t = decay_h S_{t-1} + k_t v_t^T and
    o_t = S_t^T q_t; rotary positions on q and k in the rotate-half layout (dimension i pairs
    with i + dims/2); k scaled by dim^-1/2; each head's output divided by its root mean square
    and gated by silu of a projection of the mixer's input."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: Optional[RotarySpec] = None
    # sizing fields shared with AttentionSpec: a retention mixer caches no keys
    kv_heads: int = 0
    chunk: int = 0
    window: int = 0

    @property
    def state_floats(self) -> int:
        return self.heads * self.dim * self.vdim


@dataclasses.dataclass
class StateSpaceSpec:
    """A selective state-space mixer (Mamba-2 form): `heads` heads of `vdim` channels, each with
    an fp32 state S [state, vdim] per live sequence, S_t = exp(-exp(A_h) dt_t) S_(t-1) +
    dt_t B_t x_t^T and y_t = S_t^T C_t + D_h x_t; B and C (`groups` groups of `state` entries,
    shared by neighbouring heads) and x pass a causal per-channel convolution of `conv` taps
    and silu; the output is gated by silu(z) and RMS-normed in `norm_groups` equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1
    # sizing fields shared with AttentionSpec: nothing is cached per token
    kv_heads: int = 0
    chunk: int = 0
    window: int = 0

    @property
    def dim(self) -> int:
        return self.vdim

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def proj_rows(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.state + self.heads

    @property
    def state_floats(self) -> int:
        return self.heads * self.state * self.vdim


@dataclasses.dataclass
class ParallelMixerSpec:
    """Two mixers side by side on the same input; the layer's mixer output is half the sum of
    their outputs, each RMS-normed over the model width with a weight vector of its own."""
    left: AttentionSpec
    right: RetentionSpec

    @property
    def heads(self) -> int:
        return max(self.left.heads, self.right.heads)

    @property
    def kv_heads(self) -> int:
        return self.left.kv_heads

    @property
    def dim(self) -> int:
        return max(self.left.dim, self.left.vdim)


@dataclasses.dataclass
class LatentAttentionSpec:
    """Attention through low-rank latents: queries are W_uq rms(W_dq h) (rank q_rank), keys and
    values are up-projections (W_uk, W_uv, per head) of ONE cached latent c = rms(W_dkv h) of
    size kv_rank, plus a rotated key part of rot_dim dimensions shared by all heads.  A head
    has `dim` unrotated and `rot_dim` rotated query/key dimensions and values of size `vdim`.
    gate: "head" (one sigmoid per head) or "element" (one per output dimension), computed from
    the mixer's input.  kv_from: index of an earlier layer whose cached latent and rotated key
    this layer reads instead of projecting its own."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotarySpec
    gate: str = "head"
    kv_from: Optional[int] = None
    # sizing fields shared with AttentionSpec: one cached "head" of kv_rank + rot_dim entries
    kv_heads: int = 1
    chunk: int = 0
    window: int = 0

    @property
    def cache_dim(self) -> int:
        return self.kv_rank + self.rot_dim

    @property
    def gate_rows(self) -> int:
        return self.heads if self.gate == "head" else self.heads * self.vdim


@dataclasses.dataclass
class RouterSpec:
    """Softmax router over experts + identity outputs (the last `identity` outputs return their
    input).  The choice adds a per-output correction to the scores; outputs form
    `groups` equal groups of neighbours of which only the `keep` best (by their largest
    choice score) may be chosen from; `top` outputs are chosen and their uncorrected scores
    renormalised."""
    experts: int
    top: int
    identity: int = 0
    groups: int = 1
    keep: int = 1
    # "corrected": the rule above.  "logits": the `top` largest of (router h + bias) win and
    # their weights are the softmax over the winners' logits only.  "sigmoid": scores are
    # sigmoid(router h); a group scores the sum of its `group_top` largest scores; the `top`
    # largest scores of the kept groups win and weigh their experts as they are (no
    # renormalisation)
    kind: str = "corrected"
    group_top: int = 1

    @property
    def outputs(self) -> int:
        return self.experts + self.identity


@dataclasses.dataclass
class MlpSpec:
    kind: str   # "dense": down(act(up h)) | "moe": routed experts of that form
    ff: int
    # "relu2" | "xielu" (two learned numbers per layer) | "swiglu" | "geglu" (gated, tanh form
    # of gelu on the gate)
    act: str = "relu2"
    bias: bool = False
    router: Optional[RouterSpec] = None
    shared_ff: int = 0              # > 0: a gated expert of this width that every token uses


@dataclasses.dataclass
class LayerSpec:
    # "attention" | "latent_attention[_2]" | "retention" | "parallel" | "mamba2"
    type: str
    # AttentionSpec | LatentAttentionSpec | RetentionSpec | ParallelMixerSpec | StateSpaceSpec
    mixer: object
    mlp: Optional[MlpSpec] = None   # None: the layer has no feed-forward


@dataclasses.dataclass
class LayeredConfig(ModelConfig):
    """A model given as an explicit list of layers (each with its own mixer and feed-forward
    sizes) over an fp32 residual stream, with an optional loop that runs a span of layers
    several times with the same weights (each pass has its own KV cache).  The ModelConfig
    fields hold the stack's maxima (heads, head size, ffn) for buffer sizing; num_layers is
    the number of layer RUNS (= KV cache layers)."""
    layer_specs: list = dataclasses.field(default_factory=list)
    loop: Optional[tuple] = None    # (start, stop, times)
    embed_scale: float = 1.0
    residual_mult: float = 1.0
    norm_groups: int = 1            # RMS norms of the stream run in this many equal parts
    logit_scale: float = 1.0        # logits = head x * logit_scale
    # > 0: that many residual streams with learned read / mix / write weights per sublayer
    # (hyper-connections) instead of one stream and a plain sum
    streams: int = 0
    logit_softcap: float = 0.0      # > 0: logits <- cap tanh(logits / cap)

    def layer_runs(self) -> list:
        """Indices into layer_specs in execution order."""
        n = len(self.layer_specs)
        if not self.loop:
            return list(range(n))
        a, b, t = self.loop
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    def kv_bytes_per_token(self, tp: int = 1) -> int:
        es = 4 if self.dtype == "float32" else 2
        n = 0
        for i in self.layer_runs():
            m = self.layer_specs[i].mixer
            if isinstance(m, LatentAttentionSpec):
                n += 0 if m.kv_from is not None else m.cache_dim * es
            elif isinstance(m, (RetentionSpec, StateSpaceSpec)):
                pass
            elif isinstance(m, ParallelMixerSpec):
                n += m.left.kv_heads * (m.left.dim + m.left.vdim) * es
            else:
                n += m.kv_heads * (m.dim + m.vdim) * es
                if m.pool > 0:
                    n += -(-m.kv_heads * (m.dim + m.vdim) * 4 // m.pool)
        return n

    def num_params(self) -> int:
        d = self.hidden_size
        n = 2 * self.vocab_size * d + (2 if self.arch == "sazepel" else d)
        if self.arch == "mudepel":
            return self.vocab_size * d + d + sum(_mudepel_layer_params(d, max(self.streams, 0), ls)
                                                 for ls in self.layer_specs)
        for ls in self.layer_specs:
            m = ls.mixer
            if isinstance(m, (RetentionSpec, ParallelMixerSpec)):
                n += _sazepel_layer_params(d, ls)
                continue
            if isinstance(m, LatentAttentionSpec):
                n += 3 * d + m.q_rank * (d + 1) + m.heads * (m.dim + m.rot_dim) * m.q_rank \
                    + m.heads * (m.dim + m.vdim) * m.kv_rank + m.gate_rows * d \
                    + d * m.heads * m.vdim
                if m.kv_from is None:
                    n += m.cache_dim * d + m.kv_rank
                if ls.mlp is not None:
                    e = ls.mlp.router.experts if ls.mlp.router else 1
                    n += 2 * d * ls.mlp.ff * e
                    if ls.mlp.router:
                        n += ls.mlp.router.outputs * (d + 1)
                continue
            n += d + (m.heads + m.kv_heads) * m.dim * (d + 2) + m.heads * (d + 1) \
                + d * (m.heads * m.vdim + 1)
            if ls.mlp is not None:
                n += 2 * d * ls.mlp.ff
        return n


def _sazepel_layer_params(d: int, ls: "LayerSpec") -> int:
    def ret(r):
        return d * r.heads * (2 * r.dim + 3 * r.vdim)

    def att(a):
        return d * (a.heads * (a.dim + 2 * a.vdim) + a.kv_heads * (a.dim + a.vdim)) + a.heads ** 2

    m = ls.mixer
    n = 2 + (ret(m) if isinstance(m, RetentionSpec) else att(m.left) + ret(m.right) + 2 * d)
    if ls.mlp is not None:
        e = ls.mlp.router.experts if ls.mlp.router else 1
        n += 2 + 3 * d * ls.mlp.ff * e + (e * (d + 1) if ls.mlp.router else 0)
    return n


def _mudepel_layer_params(d: int, streams: int, ls: "LayerSpec") -> int:
    m = ls.mixer
    hc = streams * (streams + 2)
    if isinstance(m, StateSpaceSpec):
        n = d * m.proj_rows + m.conv_channels * (m.conv + 1) + 3 * m.heads + m.inner + d * m.inner
    else:
        n = (d + 1) * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + d * (m.heads * m.vdim + 1)
    n += d + hc
    ml = ls.mlp
    if ml is not None:
        e = ml.router.experts if ml.router else 1
        n += d + hc + 3 * d * ml.ff * e + 3 * d * ml.shared_ff + (e * d if ml.router else 0)
    return n


def bidetar_config(name: str, d: dict, max_position: int = 1 << 20) -> LayeredConfig:
    """A Bidetar config.json: parallel layers (one norm feeds the attention mixer and the
    feed-forward) of chunked sink attention with shared key/value projections."""
    specs = []
    for ly in d["layers"]:
        if ly["type"] != "attention":
            raise ValueError(f"Bidetar: unknown mixer type {ly['type']!r}")
        m = ly["mixer"]
        rot = m.get("rot")
        rs = None
        if rot:
            rs = RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling") or None)
        mask = m.get("mask") or {}
        if int(m.get("vdim", m["dim"])) != int(m["dim"]):
            raise ValueError("Bidetar: the values are the key projection, vdim must equal dim")
        mixer = AttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                              dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                              scale=float(m["scale"]), rot=rs, chunk=int(mask.get("size") or 0))
        if mixer.heads % mixer.kv_heads:
            raise ValueError("Bidetar: heads must be a multiple of kv_heads")
        ml = ly.get("mlp")
        mlp = None
        if ml is not None:
            if ml.get("kind", "dense") != "dense":
                raise ValueError(f"Bidetar: unknown feed-forward kind {ml.get('kind')!r}")
            mlp = MlpSpec("dense", int(ml["ff"]))
        specs.append(LayerSpec("attention", mixer, mlp))
    lp = d.get("loop")
    loop = None
    if lp and int(lp.get("times", 1)) != 1 and int(lp["stop"]) > int(lp["start"]):
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(specs)) or loop[2] < 1:
            raise ValueError(f"Bidetar: bad loop {lp}")
    cfg = LayeredConfig(
        name=name, hf_id=name, arch="bidetar", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]),
        intermediate_size=max([ls.mlp.ff for ls in specs if ls.mlp is not None] or [0]),
        num_layers=0, num_heads=max(ls.mixer.heads for ls in specs),
        num_kv_heads=max(ls.mixer.kv_heads for ls in specs),
        head_dim=max(ls.mixer.dim for ls in specs), rms_eps=float(d["norm"]["eps"]),
        max_position=max_position, bos_id=0, eos_id=-1, layer_specs=specs, loop=loop,
        embed_scale=float(d["embedding"]["scale"]), residual_mult=float(d["residual_mult"]))
    cfg.num_layers = len(cfg.layer_runs())
    return cfg


def _puputar_layer(ly: dict) -> LayerSpec:
    kinds = {"latent_attention": "head", "latent_attention_2": "element"}
    if ly["type"] not in kinds:
        raise ValueError(f"Puputar: unknown mixer type {ly['type']!r}")
    m = ly["mixer"]
    rot = m["rot"]
    if int(rot["dims"]) != int(m["rot_dim"]) or int(m["rot_dim"]) % 2:
        raise ValueError("Puputar: the rotated part is rotated whole (rot.dims == rot_dim, even)")
    kv_from = m.get("kv_from")
    mixer = LatentAttentionSpec(
        heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
        kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
        rot=RotarySpec(int(rot["dims"]), float(rot["base"])), gate=kinds[ly["type"]],
        kv_from=None if kv_from is None else int(kv_from))
    ml = ly.get("mlp")
    mlp = None
    if ml is not None:
        if ml["kind"] == "dense":
            mlp = MlpSpec("dense", int(ml["ff"]), act="xielu", bias=True)
        elif ml["kind"] == "moe":
            rt, gr = ml["router"], ml["router"].get("groups") or {}
            router = RouterSpec(experts=int(rt["experts"]), top=int(rt["top"]),
                                identity=int(rt.get("identity") or 0),
                                groups=int(gr.get("count") or 1), keep=int(gr.get("keep") or 1))
            if router.outputs % router.groups or not 1 <= router.keep <= router.groups \
                    or router.top > router.keep * (router.outputs // router.groups):
                raise ValueError(f"Puputar: bad router {rt}")
            mlp = MlpSpec("moe", int(ml["expert"]["ff"]), act="relu2", router=router)
        else:
            raise ValueError(f"Puputar: unknown feed-forward kind {ml['kind']!r}")
    return LayerSpec(ly["type"], mixer, mlp)


def puputar_config(name: str, d: dict, max_position: int = 1 << 20) -> LayeredConfig:
    """A Puputar config.json: parallel layers with two grouped RMS norms (one feeds the mixer
    through a token shift, one the feed-forward), latent attention mixers (per-head or
    per-element output gate, optionally reading an earlier layer's cached latent) and dense
    xIELU or routed squared-ReLU feed-forwards."""
    specs = [_puputar_layer(ly) for ly in d["layers"]]
    for i, ls in enumerate(specs):
        j = ls.mixer.kv_from
        if j is None:
            continue
        if not 0 <= j < i or specs[j].mixer.kv_from is not None:
            raise ValueError(f"Puputar: layer {i} reads the cache of layer {j}, which must be an "
                             "earlier layer with a cache of its own")
        a, b = ls.mixer, specs[j].mixer
        if (a.kv_rank, a.rot_dim, a.rot.base) != (b.kv_rank, b.rot_dim, b.rot.base):
            raise ValueError(f"Puputar: layers {i} and {j} share a cache of unequal shape")
    width, groups = int(d["width"]), int(d["norm"].get("groups") or 1)
    if width % groups:
        raise ValueError("Puputar: width must be a multiple of norm.groups")
    cfg = LayeredConfig(
        name=name, hf_id=name, arch="puputar", vocab_size=int(d["vocab"]), hidden_size=width,
        intermediate_size=max([ls.mlp.ff for ls in specs if ls.mlp is not None] or [0]),
        num_layers=len(specs), num_heads=max(ls.mixer.heads for ls in specs), num_kv_heads=1,
        head_dim=max(ls.mixer.cache_dim for ls in specs), rms_eps=float(d["norm"]["eps"]),
        max_position=max_position, bos_id=0, eos_id=-1, layer_specs=specs, norm_groups=groups)
    return cfg


def _sazepel_retention(m: dict) -> RetentionSpec:
    rot = m.get("rot")
    rs = RotarySpec(int(rot["dims"]), float(rot["base"])) if rot and int(rot["dims"]) > 0 else None
    spec = RetentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                         decay=tuple(float(g) for g in m["decay"]), rot=rs)
    if len(spec.decay) != spec.heads or not all(0.0 < g <= 1.0 for g in spec.decay):
        raise ValueError("Sazepel: one decay in (0, 1] per retention head")
    if rs is not None and (rs.dims % 2 or rs.dims > spec.dim):
        raise ValueError("Sazepel: rot.dims must be even and at most dim")
    return spec


def _sazepel_attention(m: dict) -> AttentionSpec:
    spec = AttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                         vdim=int(m["vdim"]), scale=float(m["scale"]), rot=None, sink=False,
                         gate=True, shared_kv=False, head_norm=True, v_norm=True, talk=True,
                         gate_per="element")
    if spec.heads % spec.kv_heads:
        raise ValueError("Sazepel: heads must be a multiple of kv_heads")
    return spec


def sazepel_config(name: str, d: dict, max_position: int = 1 << 20) -> LayeredConfig:
    """A Sazepel config.json: sequential layers (a norm before and after each sublayer, every
    norm weight one number), mixers "retention" (decayed linear attention with a recurrent
    state) or "parallel" (a softmax attention with head-mixed weights beside a retention),
    routed SwiGLU feed-forwards (or none), scaled logits."""
    specs = []
    for ly in d["layers"]:
        if ly["type"] == "retention":
            mixer = _sazepel_retention(ly["mixer"])
        elif ly["type"] == "parallel":
            mixer = ParallelMixerSpec(_sazepel_attention(ly["mixer"]["left"]),
                                      _sazepel_retention(ly["mixer"]["right"]))
        else:
            raise ValueError(f"Sazepel: unknown mixer type {ly['type']!r}")
        ml = ly.get("mlp")
        mlp = None
        if ml is not None:
            if ml.get("kind") != "moe":
                raise ValueError(f"Sazepel: unknown feed-forward kind {ml.get('kind')!r}")
            rt = ml["router"]
            router = RouterSpec(experts=int(rt["experts"]), top=int(rt["top"]), kind="logits")
            if not 1 <= router.top <= router.experts:
                raise ValueError(f"Sazepel: bad router {rt}")
            mlp = MlpSpec("moe", int(ml["expert"]["ff"]), act="swiglu", router=router)
        specs.append(LayerSpec(ly["type"], mixer, mlp))
    cfg = LayeredConfig(
        name=name, hf_id=name, arch="sazepel", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]),
        intermediate_size=max([ls.mlp.ff for ls in specs if ls.mlp is not None] or [0]),
        num_layers=len(specs), num_heads=max(ls.mixer.heads for ls in specs),
        num_kv_heads=max([ls.mixer.kv_heads for ls in specs] + [1]),
        head_dim=max(ls.mixer.dim for ls in specs), rms_eps=float(d["norm"]["eps"]),
        max_position=max_position, bos_id=0, eos_id=-1, layer_specs=specs,
        logit_scale=float(d.get("logit_scale", 1.0)))
    return cfg


def sazepel_dict(width: int, layers: list, vocab: int = 32000, eps: float = 1e-6,
                 logit_scale: float = 1.0) -> dict:
    """A Sazepel config.json dictionary from short layer dicts (random-init benchmarks and
    tests).  A layer gives `ret` = (heads, dim, vdim) and optionally `att` = (heads, kv_heads,
    dim, vdim) (then the layer is "parallel"), `experts` / `expert_ff` / `top` (else no
    feed-forward), and optional decay (list), rot_dims, base, scale."""
    out = []
    for ly in layers:
        H, D, V = ly["ret"]
        decay = ly.get("decay") or [1.0 - 2.0 ** (-5.0 - 5.0 * h / max(1, H - 1)) for h in range(H)]
        ret = {"heads": H, "dim": D, "vdim": V, "decay": [float(g) for g in decay],
               "rot": {"base": float(ly.get("base", 10000.0)), "dims": int(ly.get("rot_dims", D))}}
        if "att" in ly:
            h, g, dd, vv = ly["att"]
            mixer = {"left": {"heads": h, "kv_heads": g, "dim": dd, "vdim": vv,
                              "scale": float(ly.get("scale", dd ** -0.5))}, "right": ret}
            kind = "parallel"
        else:
            mixer, kind = ret, "retention"
        mlp = None
        if ly.get("experts"):
            mlp = {"kind": "moe", "expert": {"ff": ly["expert_ff"]},
                   "router": {"experts": ly["experts"], "top": ly["top"]}}
        out.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Sazepel", "layers": out, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def puputar_dict(width: int, layers: list, vocab: int = 32000, eps: float = 1e-6,
                 norm_groups: int = 1) -> dict:
    """A Puputar config.json dictionary from short layer tuples (random-init benchmarks and
    tests): each layer is a dict with heads, dim, rot_dim, vdim, kv_rank, q_rank and optional
    base, scale, gate ("head" | "element"), kv_from, and ff (dense), or experts / expert_ff /
    top / identity / groups / keep (routed), or neither (no feed-forward)."""
    out = []
    for ly in layers:
        m = {"heads": ly["heads"], "dim": ly["dim"], "rot_dim": ly["rot_dim"], "vdim": ly["vdim"],
             "kv_rank": ly["kv_rank"], "q_rank": ly["q_rank"],
             "rot": {"base": float(ly.get("base", 10000.0)), "dims": ly["rot_dim"]},
             "scale": float(ly.get("scale", (ly["dim"] + ly["rot_dim"]) ** -0.5))}
        if ly.get("kv_from") is not None:
            m["kv_from"] = ly["kv_from"]
        if "experts" in ly:
            mlp = {"kind": "moe", "expert": {"ff": ly["expert_ff"]},
                   "router": {"experts": ly["experts"], "top": ly["top"],
                              "identity": ly.get("identity", 0),
                              "groups": {"count": ly.get("groups", 1), "keep": ly.get("keep", 1)}}}
        elif ly.get("ff"):
            mlp = {"kind": "dense", "ff": ly["ff"]}
        else:
            mlp = None
        out.append({"type": "latent_attention_2" if ly.get("gate") == "element"
                    else "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Puputar", "layers": out, "norm": {"eps": eps, "groups": norm_groups},
            "vocab": vocab, "width": width}


def _mudepel_attention(m: dict) -> AttentionSpec:
    rot = m.get("rot")
    rs = None
    if rot and int(rot.get("dims") or 0) > 0:
        rs = RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling") or None,
                        layout="half")
        if rs.dims % 2 or rs.dims > int(m["dim"]):
            raise ValueError("Mudepel: rot.dims must be even and at most dim")
        if rs.scaling is not None and not all(k in rs.scaling for k in
                                              ("factor", "original", "fast", "slow")):
            raise ValueError("Mudepel: rot.scaling needs factor, original, fast and slow")
    mask = m.get("mask") or {}
    spec = AttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                         vdim=int(m["vdim"]), scale=float(m["scale"]), rot=rs,
                         window=int(mask.get("size") or 0), sink=False, gate=False,
                         shared_kv=False, pool=int(mask.get("pool") or 0), unit_sink=True,
                         bias=True)
    if spec.heads % spec.kv_heads:
        raise ValueError("Mudepel: heads must be a multiple of kv_heads")
    if spec.window <= 0:
        spec.pool = 0
    return spec


def _mudepel_state_space(m: dict) -> StateSpaceSpec:
    spec = StateSpaceSpec(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                          groups=int(m["groups"]), conv=int(m["conv"]),
                          norm_groups=int(m.get("norm_groups") or 1))
    if spec.heads % spec.groups or spec.inner % spec.norm_groups or spec.conv < 1:
        raise ValueError("Mudepel: heads must be a multiple of groups, heads x vdim of "
                         "norm_groups, and conv at least 1")
    return spec


def mudepel_config(name: str, d: dict, max_position: int = 1 << 20) -> LayeredConfig:
    """A Mudepel config.json: pre-norm layers (norm weights stored around zero) over several
    residual streams with learned read / mix / write weights, mixers "attention" (biased
    projections, rotate-half positions with YaRN scaling, a sliding window plus mean-pooled
    blocks before it, a constant 1 in the softmax denominator) or "mamba2" (selective
    state-space), feed-forwards "dense" (gelu-gated) or "moe" (sigmoid router over expert
    groups, silu-gated experts, optional shared expert), an optional loop over a span of
    layers, tied embeddings and a tanh cap on the logits."""
    specs = []
    for ly in d["layers"]:
        if ly["type"] == "attention":
            mixer = _mudepel_attention(ly["mixer"])
        elif ly["type"] == "mamba2":
            mixer = _mudepel_state_space(ly["mixer"])
        else:
            raise ValueError(f"Mudepel: unknown mixer type {ly['type']!r}")
        ml = ly.get("mlp")
        mlp = None
        if ml is not None:
            if ml.get("kind") == "dense":
                mlp = MlpSpec("dense", int(ml["ff"]), act="geglu")
            elif ml.get("kind") == "moe":
                rt, gr = ml["router"], ml["router"].get("groups") or {}
                router = RouterSpec(experts=int(rt["experts"]), top=int(rt["top"]),
                                    groups=int(gr.get("count") or 1), keep=int(gr.get("keep") or 1),
                                    kind="sigmoid", group_top=2)
                if router.experts % router.groups or not 1 <= router.keep <= router.groups \
                        or not 1 <= router.top <= router.keep * (router.experts // router.groups):
                    raise ValueError(f"Mudepel: bad router {rt}")
                sh = ml.get("shared")
                mlp = MlpSpec("moe", int(ml["expert"]["ff"]), act="swiglu", router=router,
                              shared_ff=int(sh["ff"]) if sh else 0)
            else:
                raise ValueError(f"Mudepel: unknown feed-forward kind {ml.get('kind')!r}")
        specs.append(LayerSpec(ly["type"], mixer, mlp))
    lp = d.get("loop")
    loop = None
    if lp and int(lp.get("times", 1)) != 1 and int(lp["stop"]) > int(lp["start"]):
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(specs)) or loop[2] < 1:
            raise ValueError(f"Mudepel: bad loop {lp}")
    att = [ls.mixer for ls in specs if isinstance(ls.mixer, AttentionSpec)]
    cfg = LayeredConfig(
        name=name, hf_id=name, arch="mudepel", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]),
        intermediate_size=max([ls.mlp.ff for ls in specs if ls.mlp is not None] or [0]),
        num_layers=0, num_heads=max(ls.mixer.heads for ls in specs),
        num_kv_heads=max([a.kv_heads for a in att] + [1]),
        head_dim=max([max(a.dim, a.vdim) for a in att] + [ls.mixer.dim for ls in specs]),
        rms_eps=float(d["norm"]["eps"]), max_position=max_position, bos_id=0, eos_id=-1,
        tie_embeddings=True, layer_specs=specs, loop=loop, streams=int(d.get("streams") or 0),
        logit_softcap=float(d.get("logit_softcap") or 0.0))
    cfg.num_layers = len(cfg.layer_runs())
    return cfg


def mudepel_dict(width: int, layers: list, vocab: int = 32000, eps: float = 1e-6,
                 streams: int = 2, logit_softcap: float = 30.0, loop: Optional[tuple] = None
                 ) -> dict:
    """A Mudepel config.json dictionary from short layer dicts (random-init benchmarks and
    tests).  A layer gives either `att` = (heads, kv_heads, dim, vdim) with optional window,
    pool, rot_dims, base, yarn (a scaling dict), scale, or `ssm` = (heads, vdim, state, groups)
    with optional conv, norm_groups; and `ff` (dense), or experts / expert_ff / top / groups /
    keep / shared_ff (routed), or neither."""
    out = []
    for ly in layers:
        if "att" in ly:
            h, g, dd, vv = ly["att"]
            m = {"heads": h, "kv_heads": g, "dim": dd, "vdim": vv,
                 "scale": float(ly.get("scale", dd ** -0.5)),
                 "rot": {"base": float(ly.get("base", 10000.0)),
                         "dims": int(ly.get("rot_dims", dd)), "scaling": ly.get("yarn")}}
            if ly.get("window"):
                m["mask"] = {"size": int(ly["window"]), "pool": int(ly.get("pool") or 0)}
            kind = "attention"
        else:
            h, vv, n, g = ly["ssm"]
            m = {"heads": h, "vdim": vv, "state": n, "groups": g, "conv": int(ly.get("conv", 4)),
                 "norm_groups": int(ly.get("norm_groups", 1))}
            kind = "mamba2"
        if ly.get("experts"):
            mlp = {"kind": "moe", "expert": {"ff": ly["expert_ff"]},
                   "router": {"experts": ly["experts"], "top": ly["top"],
                              "groups": {"count": ly.get("groups", 1), "keep": ly.get("keep", 1)}}}
            if ly.get("shared_ff"):
                mlp["shared"] = {"ff": ly["shared_ff"]}
        elif ly.get("ff"):
            mlp = {"kind": "dense", "ff": ly["ff"]}
        else:
            mlp = None
        out.append({"type": kind, "mixer": m, "mlp": mlp})
    d = {"architecture": "Mudepel", "layers": out, "logit_softcap": logit_softcap,
         "norm": {"eps": eps}, "streams": streams, "vocab": vocab, "width": width}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


# config.json readers of designs that do not use the HF key set, by their "architecture" value
_NATIVE_READERS = {"Bidetar": bidetar_config, "Puputar": puputar_config,
                   "Sazepel": sazepel_config, "Mudepel": mudepel_config}

_REGISTRY: dict[str, ModelConfig] = {}


def register(cfg: ModelConfig) -> ModelConfig:
    _REGISTRY[cfg.name] = cfg
    _REGISTRY[cfg.hf_id.lower()] = cfg
    return cfg


# Qwen3-0.6B -- the model the reference deploys (llm-d-deploy.yaml:118, llm-d-test.yaml:7)
QWEN3_0_6B = register(ModelConfig(
    name="qwen3-0.6b", hf_id="Qwen/Qwen3-0.6B", arch="qwen3", vocab_size=151936,
    hidden_size=1024, intermediate_size=3072, num_layers=28, num_heads=16, num_kv_heads=8,
    head_dim=128, rms_eps=1e-6, rope_theta=1_000_000.0, max_position=40960,
    tie_embeddings=True, qk_norm=True, bos_id=151643, eos_id=151645))

LLAMA3_8B = register(ModelConfig(
    name="llama-3-8b", hf_id="meta-llama/Meta-Llama-3-8B-Instruct", arch="llama",
    vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_layers=32,
    num_heads=32, num_kv_heads=8, head_dim=128, rms_eps=1e-5, rope_theta=500000.0,
    max_position=8192, bos_id=128000, eos_id=128009))

LLAMA3_70B = register(ModelConfig(
    name="llama-3-70b", hf_id="meta-llama/Meta-Llama-3-70B-Instruct", arch="llama",
    vocab_size=128256, hidden_size=8192, intermediate_size=28672, num_layers=80,
    num_heads=64, num_kv_heads=8, head_dim=128, rms_eps=1e-5, rope_theta=500000.0,
    max_position=8192, bos_id=128000, eos_id=128009))

# Llama-3-70B's real layer widths (d 8192, 64/8 heads, ffn 28672, vocab 128256) at 4 layers:
# the TP=4 / TP=8 decode collectives at their production message sizes (B=256 x 8192 bf16 =
# 4 MiB per all-reduce) on one GPU, multi-process
LLAMA3_70B_L4 = register(ModelConfig(
    name="llama-3-70b-l4", hf_id="test/llama-3-70b-l4", arch="llama",
    vocab_size=128256, hidden_size=8192, intermediate_size=28672, num_layers=4,
    num_heads=64, num_kv_heads=8, head_dim=128, rms_eps=1e-5, rope_theta=500000.0,
    max_position=8192, bos_id=128000, eos_id=128009))

MIXTRAL_8X7B = register(ModelConfig(
    name="mixtral-8x7b", hf_id="mistralai/Mixtral-8x7B-Instruct-v0.1", arch="mixtral",
    vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_layers=32,
    num_heads=32, num_kv_heads=8, head_dim=128, rms_eps=1e-5, rope_theta=1_000_000.0,
    max_position=32768, num_experts=8, experts_per_token=2, bos_id=1, eos_id=2))

# Qwen3 mixture-of-experts: 128 fine-grained experts, 8 per token (3.3B of 30.5B parameters
# active); every layer MoE, q/k RMSNorm like the dense Qwen3
QWEN3_30B_A3B = register(ModelConfig(
    name="qwen3-30b-a3b", hf_id="Qwen/Qwen3-30B-A3B", arch="qwen3_moe", vocab_size=151936,
    hidden_size=2048, intermediate_size=768, num_layers=48, num_heads=32, num_kv_heads=4,
    head_dim=128, rms_eps=1e-6, rope_theta=1_000_000.0, max_position=40960, qk_norm=True,
    num_experts=128, experts_per_token=8, bos_id=151643, eos_id=151645))

# tiny shapes for CPU tests / smoke (same code paths, seconds to run)
TINY_QWEN3 = register(ModelConfig(
    name="tiny-qwen3", hf_id="test/tiny-qwen3", arch="qwen3", vocab_size=512,
    hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4, num_kv_heads=2,
    head_dim=128, rope_theta=1_000_000.0, max_position=4096, tie_embeddings=True,
    qk_norm=True, bos_id=1, eos_id=2))

TINY_LLAMA = register(ModelConfig(
    name="tiny-llama", hf_id="test/tiny-llama", arch="llama", vocab_size=512,
    hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4, num_kv_heads=2,
    head_dim=128, rope_theta=500000.0, max_position=4096, bos_id=1, eos_id=2))

TINY_MIXTRAL = register(ModelConfig(
    name="tiny-mixtral", hf_id="test/tiny-mixtral", arch="mixtral", vocab_size=512,
    hidden_size=256, intermediate_size=256, num_layers=2, num_heads=4, num_kv_heads=2,
    head_dim=128, rope_theta=1_000_000.0, max_position=4096, num_experts=4,
    experts_per_token=2, bos_id=1, eos_id=2))


TINY_QWEN3_MOE = register(ModelConfig(
    name="tiny-qwen3-moe", hf_id="test/tiny-qwen3-moe", arch="qwen3_moe", vocab_size=512,
    hidden_size=256, intermediate_size=256, num_layers=2, num_heads=4, num_kv_heads=2,
    head_dim=128, rope_theta=1_000_000.0, max_position=4096, qk_norm=True, num_experts=16,
    experts_per_token=4, bos_id=1, eos_id=2))


# the real multi-GPU layouts at world size 8: Llama-3-70B's 8 KV heads (one per TP rank, GQA
# 8) and Mixtral's 8 experts (one per EP rank)
TINY_LLAMA_KV8 = register(ModelConfig(
    name="tiny-llama-kv8", hf_id="test/tiny-llama-kv8", arch="llama", vocab_size=512,
    hidden_size=256, intermediate_size=512, num_layers=2, num_heads=16, num_kv_heads=8,
    head_dim=128, rope_theta=500000.0, max_position=4096, bos_id=1, eos_id=2))

TINY_MIXTRAL8 = register(ModelConfig(
    name="tiny-mixtral8", hf_id="test/tiny-mixtral8", arch="mixtral", vocab_size=512,
    hidden_size=256, intermediate_size=256, num_layers=2, num_heads=16, num_kv_heads=8,
    head_dim=128, rope_theta=1_000_000.0, max_position=4096, num_experts=8,
    experts_per_token=2, bos_id=1, eos_id=2))


def layered_config(name: str, width: int, num_layers: int, heads: int, kv_heads: int, dim: int,
                   ff: int, chunk: int, vocab: int = 32000, loop: Optional[tuple] = None,
                   rot_dims: Optional[int] = None, rot_base: float = 500000.0,
                   rot_scaling: Optional[dict] = None, residual_mult: float = 1.0,
                   embed_scale: float = 1.0, eps: float = 1e-5) -> LayeredConfig:
    """A Bidetar-design config with `num_layers` equal layers (random-init benchmarks, tests)."""
    spec = LayerSpec("attention",
                     AttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim,
                                   scale=dim ** -0.5,
                                   rot=RotarySpec(rot_dims or dim, rot_base, rot_scaling),
                                   chunk=chunk),
                     MlpSpec("dense", ff) if ff else None)
    cfg = LayeredConfig(name=name, hf_id="test/" + name, arch="bidetar", vocab_size=vocab,
                        hidden_size=width, intermediate_size=ff, num_layers=0, num_heads=heads,
                        num_kv_heads=kv_heads, head_dim=dim, rms_eps=eps, max_position=1 << 20,
                        bos_id=0, eos_id=-1, layer_specs=[spec] * num_layers, loop=loop,
                        embed_scale=embed_scale, residual_mult=residual_mult)
    cfg.num_layers = len(cfg.layer_runs())
    return cfg


_LLAMA31_SCALING = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}

# Bidetar at layer sizes of real models (random weights; bench.py --compare-design), each
# beside a Llama-style dense model of the same width, heads, depth and feed-forward FLOPs
# (SwiGLU's three matrices at 2/3 of the squared-ReLU feed-forward's width)
BIDETAR_W2048 = register(layered_config(
    "bidetar-w2048", width=2048, num_layers=16, heads=16, kv_heads=4, dim=128, ff=8192,
    chunk=8192, rot_scaling=_LLAMA31_SCALING, residual_mult=0.5))
LLAMA_W2048 = register(ModelConfig(
    name="llama-w2048", hf_id="test/llama-w2048", arch="llama", vocab_size=32000,
    hidden_size=2048, intermediate_size=5632, num_layers=16, num_heads=16, num_kv_heads=4,
    head_dim=128, rms_eps=1e-5, rope_theta=500000.0, max_position=1 << 17, bos_id=1, eos_id=2))
BIDETAR_W4096 = register(layered_config(
    "bidetar-w4096", width=4096, num_layers=8, heads=32, kv_heads=8, dim=128, ff=21504,
    chunk=8192, rot_scaling=_LLAMA31_SCALING, residual_mult=0.5))
LLAMA_W4096 = register(ModelConfig(
    name="llama-w4096", hf_id="test/llama-w4096", arch="llama", vocab_size=32000,
    hidden_size=4096, intermediate_size=14336, num_layers=8, num_heads=32, num_kv_heads=8,
    head_dim=128, rms_eps=1e-5, rope_theta=500000.0, max_position=1 << 17, bos_id=1, eos_id=2))
# 64-wide heads, short chunks, a looped span (no D = 128-only model to set beside it)
BIDETAR_W1536 = register(layered_config(
    "bidetar-w1536-d64", width=1536, num_layers=8, heads=24, kv_heads=8, dim=64, ff=6144,
    chunk=1024, loop=(2, 6, 3), rot_dims=32, residual_mult=0.5))
TINY_BIDETAR = register(layered_config(
    "tiny-bidetar", width=128, num_layers=3, heads=4, kv_heads=2, dim=32, ff=256, chunk=48,
    vocab=512, loop=(1, 3, 2), rot_dims=16, residual_mult=0.7, embed_scale=4.0))


def _puputar_stack(name: str, width: int, n: int, heads: int, dim: int, rot_dim: int, vdim: int,
                   kv_rank: int, q_rank: int, ff: int, experts: int = 0, expert_ff: int = 0,
                   top: int = 0, identity: int = 0, groups: int = 1, keep: int = 1,
                   vocab: int = 32000, norm_groups: int = 1) -> LayeredConfig:
    """n layers; every second one after the first has a routed feed-forward (when experts > 0),
    every third gates per element, and the last of those reads the first one's cache."""
    layers, first_el = [], None
    for i in range(n):
        ly = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                  q_rank=q_rank)
        if i % 3 == 1:
            ly["gate"] = "element"
            if first_el is None:
                first_el = i
            elif i + 3 >= n:
                ly["kv_from"] = first_el
        if experts and i and i % 2 == 0:
            ly.update(experts=experts, expert_ff=expert_ff, top=top, identity=identity,
                      groups=groups, keep=keep)
        else:
            ly["ff"] = ff
        layers.append(ly)
    cfg = puputar_config(name, puputar_dict(width, layers, vocab=vocab, norm_groups=norm_groups))
    cfg.hf_id = "test/" + name
    return cfg


# Puputar at layer sizes of real models (random weights; bench.py --compare-design puputar):
# 128 + 64 query/key dimensions per head over a 512 + 64 latent cache
PUPUTAR_W2048 = register(_puputar_stack(
    "puputar-w2048", width=2048, n=16, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512,
    q_rank=768, ff=8192))
PUPUTAR_W2048_MOE = register(_puputar_stack(
    "puputar-w2048-moe", width=2048, n=16, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512,
    q_rank=768, ff=8192, experts=14, expert_ff=2048, top=4, identity=2, groups=4, keep=2))
PUPUTAR_W4096 = register(_puputar_stack(
    "puputar-w4096", width=4096, n=8, heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=512,
    q_rank=1536, ff=21504, norm_groups=4))
TINY_PUPUTAR = register(_puputar_stack(
    "tiny-puputar", width=128, n=6, heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=48,
    ff=192, experts=6, expert_ff=64, top=3, identity=2, groups=4, keep=2, vocab=512,
    norm_groups=4))


def _sazepel_stack(name: str, width: int, n: int, att: tuple, ret: tuple, experts: int,
                   expert_ff: int, top: int, vocab: int = 32000, rot_dims: Optional[int] = None,
                   logit_scale: float = 1.0) -> LayeredConfig:
    """n layers; every third one (from the second) is a retention alone, the others put an
    attention beside it; the last layer has no feed-forward."""
    layers = []
    for i in range(n):
        ly = dict(ret=ret, base=500000.0)
        if rot_dims is not None:
            ly["rot_dims"] = rot_dims
        if i % 3 != 1:
            ly["att"] = att
        if i + 1 < n:
            ly.update(experts=experts, expert_ff=expert_ff, top=top)
        layers.append(ly)
    cfg = sazepel_config(name, sazepel_dict(width, layers, vocab=vocab, logit_scale=logit_scale))
    cfg.hf_id = "test/" + name
    return cfg


# Sazepel at layer sizes of real models (random weights; bench.py --compare-design sazepel):
# 16 / 4 attention heads of 128 beside 8 retention heads with 128 x 128 states, 8 experts of
# which 2 per token
SAZEPEL_W2048 = register(_sazepel_stack(
    "sazepel-w2048", width=2048, n=16, att=(16, 4, 128, 128), ret=(8, 128, 128), experts=8,
    expert_ff=1408, top=2, rot_dims=64))
SAZEPEL_W4096 = register(_sazepel_stack(
    "sazepel-w4096", width=4096, n=8, att=(32, 8, 128, 128), ret=(16, 128, 128), experts=8,
    expert_ff=3584, top=2, rot_dims=64))
TINY_SAZEPEL = register(_sazepel_stack(
    "tiny-sazepel", width=128, n=4, att=(4, 2, 32, 16), ret=(2, 16, 32), experts=6, expert_ff=64,
    top=2, vocab=512, rot_dims=8, logit_scale=1.5))


def _mudepel_stack(name: str, width: int, n: int, att: tuple, ssm: tuple, ff: int, experts: int,
                   expert_ff: int, top: int, window: int, pool: int, vocab: int = 32000,
                   streams: int = 4, groups: int = 1, keep: int = 1, norm_groups: int = 1,
                   loop: Optional[tuple] = None, rot_dims: Optional[int] = None,
                   yarn: Optional[dict] = None) -> LayeredConfig:
    """n layers alternating state-space (dense gelu-gated feed-forward) and windowed attention
    with pooled blocks (routed feed-forward with a shared expert)."""
    layers = []
    for i in range(n):
        if i % 2 == 0:
            layers.append(dict(ssm=ssm, norm_groups=norm_groups, ff=ff))
        else:
            ly = dict(att=att, window=window, pool=pool, base=500000.0, yarn=yarn,
                      experts=experts, expert_ff=expert_ff, top=top, groups=groups, keep=keep,
                      shared_ff=expert_ff)
            if rot_dims is not None:
                ly["rot_dims"] = rot_dims
            layers.append(ly)
    cfg = mudepel_config(name, mudepel_dict(width, layers, vocab=vocab, streams=streams,
                                            loop=loop))
    cfg.hf_id = "test/" + name
    return cfg


# Mudepel at layer sizes of real models (random weights; bench.py --compare-design mudepel):
# state-space layers of width / 32 heads x 64 channels with 128-entry states, attention layers
# of 16 / 4 heads of 128 over a 1024-token window and 64-token pooled blocks, 8 experts of
# which 2 per token beside a shared one
_YARN = {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}
MUDEPEL_W2048 = register(_mudepel_stack(
    "mudepel-w2048", width=2048, n=16, att=(16, 4, 128, 128), ssm=(64, 64, 128, 1), ff=5632,
    experts=8, expert_ff=1408, top=2, window=1024, pool=64, yarn=_YARN))
MUDEPEL_W4096 = register(_mudepel_stack(
    "mudepel-w4096", width=4096, n=8, att=(32, 8, 128, 128), ssm=(128, 64, 128, 8), ff=11008,
    experts=8, expert_ff=3584, top=2, window=1024, pool=64, norm_groups=8, yarn=_YARN))
TINY_MUDEPEL = register(_mudepel_stack(
    "tiny-mudepel", width=128, n=4, att=(4, 2, 32, 16), ssm=(4, 16, 16, 2), ff=192, experts=6,
    expert_ff=64, top=2, window=24, pool=8, vocab=512, streams=3, groups=3, keep=2,
    norm_groups=2, loop=(1, 3, 2), rot_dims=16,
    yarn={"factor": 2.0, "original": 64, "fast": 8.0, "slow": 1.0}))


def get_config(name: str) -> ModelConfig:
    """Resolve a registry name, HF id, or a directory holding a HF config.json."""
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        with open(os.path.join(name, "config.json")) as f:
            d = json.load(f)
        reader = _NATIVE_READERS.get(d.get("architecture"))
        if reader is not None:
            return reader(name, d)
        return ModelConfig.from_hf_dict(name, d)
    key = name.lower()
    if key in _REGISTRY:
        return _REGISTRY[key]
    raise KeyError(f"unknown model {name!r}; known: {sorted(set(c.name for c in _REGISTRY.values()))}")


def list_models() -> list[str]:
    return sorted(set(c.name for c in _REGISTRY.values()))
