"""Float64 oracle of the Sazepel design, written from its equations: one function per
mechanism, whole sequences at once, sharing no code with the package.

Notation: x [T, d] is the residual stream of one sequence, positions count from 0.
rms(v) = v / sqrt(mean(v^2) + eps) over the last axis.
"""
import math

import torch

F64 = torch.float64


def rms(v, eps):
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number."""
    return rms(x, eps) * g.to(F64).reshape(())


def rotate_half(x, dims, base):
    """x [T, H, D]: the first `dims` entries of every head, entry i paired with i + dims/2,
    turned by the angle position * base^(-2i/dims)."""
    if not dims:
        return x
    T = x.shape[0]
    half = dims // 2
    out = x.clone()
    for t in range(T):
        for i in range(half):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def retain(q, k, v, decay):
    """The recurrence alone, token by token: q, k [T, H, D] (already rotated and scaled),
    v [T, H, V]; S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Returns o [T, H, V] and the
    last state [H, D, V]."""
    T, H, D = q.shape
    V = v.shape[2]
    o = torch.zeros(T, H, V, dtype=F64)
    last = torch.zeros(H, D, V, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = decay[hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
        last[hd] = S
    return o, last


def retention(h, w, m, eps):
    """h [T, d]; w: q, k, v, g, o matrices ([out, in]); m: heads, dim, vdim, decay, rot."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_half((h @ w["q"].T).view(T, H, D), rot["dims"], rot["base"])
    k = rotate_half((h @ w["k"].T).view(T, H, D), rot["dims"], rot["base"]) * D ** -0.5
    o, _ = retain(q, k, (h @ w["v"].T).view(T, H, V), m["decay"])
    g = h @ w["g"].T
    return (rms(o, eps).reshape(T, H * V) * g * torch.sigmoid(g)) @ w["o"].T


def retention_closed_form(h, w, m, eps):
    """The same mixer without a state: o_t = sum_{j <= t} decay^(t - j) (q_t . k_j) v_j."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_half((h @ w["q"].T).view(T, H, D), rot["dims"], rot["base"])
    k = rotate_half((h @ w["k"].T).view(T, H, D), rot["dims"], rot["base"]) * D ** -0.5
    v = (h @ w["v"].T).view(T, H, V)
    i = torch.arange(T)
    lag = (i[:, None] - i[None, :]).clamp(min=0).to(F64)
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        wgt = torch.tril((q[:, hd] @ k[:, hd].T) * m["decay"][hd] ** lag)
        o[:, hd] = wgt @ v[:, hd]
    g = h @ w["g"].T
    return (rms(o, eps).reshape(T, H * V) * g * torch.sigmoid(g)) @ w["o"].T


def mix_heads_attend(q, k, v, scale, talk, first=0):
    """q [n, H, D] are the queries of positions first .. first + n - 1; k [T, G, D], v [T, G, V]
    all keys and values.  Causal softmax per query head over its key head, the heads' weights
    mixed by talk [H, H] (None: not mixed), each head's mixed weights applied to the values of
    its own key/value head.  Returns [n, H, V]."""
    n, H, _ = q.shape
    T, G, V = v.shape
    rep = H // G
    P = torch.zeros(H, n, T, dtype=F64)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // rep].T) * scale
        for t in range(n):
            P[hd, t, :first + t + 1] = torch.softmax(s[t, :first + t + 1], dim=0)
    out = torch.zeros(n, H, V, dtype=F64)
    for hd in range(H):
        mixed = P[hd] if talk is None else sum(talk[hd, g] * P[g] for g in range(H))
        out[:, hd] = mixed @ v[:, hd // rep]
    return out


def mixed_head_attention(h, w, m, eps):
    """Softmax attention without positions: per-head unit-rms q, k and v, mixed head weights,
    a sigmoid gate per entry."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms((h @ w["q"].T).view(T, H, D), eps)
    k = rms((h @ w["k"].T).view(T, G, D), eps)
    v = rms((h @ w["v"].T).view(T, G, V), eps)
    out = mix_heads_attend(q, k, v, m["scale"], w["talk"])
    return (out.reshape(T, H * V) * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def parallel_mixer(h, wl, wr, out_l, out_r, m, eps):
    a = mixed_head_attention(h, wl, m["left"], eps)
    b = retention(h, wr, m["right"], eps)
    return 0.5 * (rms(a, eps) * out_l + rms(b, eps) * out_r)


def routed_experts(h, w, ml):
    """w: router [E, d], router.b [E], e<i>.gate / up / down."""
    E, top = ml["router"]["experts"], ml["router"]["top"]
    z = h @ w["router"].T + w["router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        zs = torch.stack([z[t, e] for e in order])
        p = torch.exp(zs - zs.max())
        p = p / p.sum()
        for pe, e in zip(p, order):
            a = w[f"e{e}.gate"] @ h[t]
            out[t] += pe * (w[f"e{e}.down"] @ (a * torch.sigmoid(a) * (w[f"e{e}.up"] @ h[t])))
    return out


def sub(sd, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in sd.items() if k.startswith(prefix)}


def forward(cfg, sd, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence."""
    eps = cfg["norm"]["eps"]
    x = scalar_norm(sd["embed"].to(F64)[torch.tensor(tokens)], sd["embed.norm"], eps)
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, sd[p + "norm1"], eps)
        if ly["type"] == "retention":
            y = retention(h, sub(sd, p + "mix."), ly["mixer"], eps)
        else:
            y = parallel_mixer(h, sub(sd, p + "mix.left."), sub(sd, p + "mix.right."),
                               sd[p + "mix.left.out"].to(F64), sd[p + "mix.right.out"].to(F64),
                               ly["mixer"], eps)
        x = x + scalar_norm(y, sd[p + "norm1b"], eps)
        if ly["mlp"] is not None:
            h = scalar_norm(x, sd[p + "norm2"], eps)
            x = x + scalar_norm(routed_experts(h, sub(sd, p + "mlp."), ly["mlp"]), sd[p + "norm2b"],
                                eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (scalar_norm(x, sd["final.norm"], eps) @ sd["head"].to(F64).T) * cfg["logit_scale"]


def random_weights(cfg, seed, scale=1.0):
    """bf16-representable random weights under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else scale * i ** -0.5)
                ).to(torch.bfloat16)

    def num():
        return (1 + 0.2 * torch.randn((), generator=g)).to(torch.bfloat16)

    def ret(p, m):
        hd, hv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
        return {p + "q": mat(hd, d), p + "k": mat(hd, d), p + "v": mat(hv, d), p + "g": mat(hv, d),
                p + "o": mat(d, hv)}

    sd = {"embed": mat(cfg["vocab"], d, 1.0), "embed.norm": num(), "final.norm": num(),
          "head": mat(cfg["vocab"], d)}
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        sd[p + "norm1"], sd[p + "norm1b"] = num(), num()
        if ly["type"] == "retention":
            sd.update(ret(p + "mix.", ly["mixer"]))
        else:
            a = ly["mixer"]["left"]
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            sd.update({q + "q": mat(H * D, d), q + "k": mat(G * D, d), q + "v": mat(G * V, d),
                       q + "g": mat(H * V, d), q + "o": mat(d, H * V),
                       q + "talk": (torch.eye(H) + 0.4 * torch.randn(H, H, generator=g)
                                    ).to(torch.bfloat16),
                       p + "mix.left.out": (1 + 0.3 * torch.randn(d, generator=g)).to(torch.bfloat16),
                       p + "mix.right.out": (1 + 0.3 * torch.randn(d, generator=g)).to(torch.bfloat16)})
            sd.update(ret(p + "mix.right.", ly["mixer"]["right"]))
        ml = ly["mlp"]
        if ml is not None:
            sd[p + "norm2"], sd[p + "norm2b"] = num(), num()
            E, F_ = ml["router"]["experts"], ml["expert"]["ff"]
            sd[p + "mlp.router"] = mat(E, d, 1.0)
            sd[p + "mlp.router.b"] = torch.randn(E, generator=g).to(torch.bfloat16)
            for e in range(E):
                sd[p + f"mlp.e{e}.gate"], sd[p + f"mlp.e{e}.up"] = mat(F_, d), mat(F_, d)
                sd[p + f"mlp.e{e}.down"] = mat(d, F_)
    return sd


def make_config(width, vocab, layers, eps=1e-5, logit_scale=1.0):
    return {"architecture": "Sazepel", "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def ret_spec(heads, dim, vdim, rot_dims=None, base=10000.0, decay=None):
    decay = decay or [1.0 - 0.3 * 0.4 ** h for h in range(heads)]
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
            "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims}}


def make_layer(ret, att=None, moe=None):
    """ret: ret_spec(...); att: (heads, kv_heads, dim, vdim, scale) makes the layer parallel;
    moe: (experts, top, ff) or None."""
    if att is None:
        kind, mixer = "retention", ret
    else:
        kind = "parallel"
        mixer = {"left": {"heads": att[0], "kv_heads": att[1], "dim": att[2], "vdim": att[3],
                          "scale": att[4]}, "right": ret}
    mlp = None
    if moe is not None:
        mlp = {"kind": "moe", "expert": {"ff": moe[2]}, "router": {"experts": moe[0], "top": moe[1]}}
    return {"type": kind, "mixer": mixer, "mlp": mlp}
