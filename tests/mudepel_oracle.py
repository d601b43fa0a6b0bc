"""Float64 oracle of the Mudepel design, written from its equations: one function per
mechanism, whole sequences at once, token by token where the design is a recurrence, sharing no
code with the package.

Notation: positions count from 0; rms(v) = v / sqrt(mean(v^2) + eps) over the last axis; linear
weights are [out, in].  A model is (cfg, w): the config.json dictionary and a dictionary of
float64 tensors under the checkpoint's names.
"""
import math

import torch

F64 = torch.float64


def rms(v, eps):
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def norm1p(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ----------------------------------------------------------------------------- rotary
def yarn_frequencies(dims, base, scaling):
    """(frequencies [dims / 2], factor on cos and sin)."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def where(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [T, H, D]: the first rot.dims entries of every head, entry i paired with i + dims/2."""
    if not rot or not rot.get("dims"):
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, m = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    out = x.clone()
    for t, p in enumerate(positions):
        for i in range(half):
            a = p * f[i]
            c, s = math.cos(a) * m, math.sin(a) * m
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


# ----------------------------------------------------------------------------- attention
def pooled_window_weights(s_tok, s_blk, i, size, pool):
    """Softmax weights of query position i: s_tok [n] are the scores of the keys 0 .. n-1
    (n > i is allowed, later ones are not seen), s_blk [nb] of the pooled blocks.  One is added
    to the denominator.  Returns (token weights, block weights), zeros where nothing is seen."""
    n, nb = s_tok.shape[0], s_blk.shape[0]
    tok = torch.zeros(n, dtype=F64)
    blk = torch.zeros(nb, dtype=F64)
    seen_t = [j for j in range(n) if 0 <= i - j and (size <= 0 or i - j < size)]
    seen_b = [b for b in range(nb) if pool > 0 and size > 0 and b * pool + pool - 1 <= i - size]
    den = 1.0
    for j in seen_t:
        den = den + math.exp(float(s_tok[j]))
    for b in seen_b:
        den = den + math.exp(float(s_blk[b]))
    for j in seen_t:
        tok[j] = math.exp(float(s_tok[j])) / den
    for b in seen_b:
        blk[b] = math.exp(float(s_blk[b])) / den
    return tok, blk


def pooled_window_attention(q, k, v, scale, size, pool, store=None):
    """q [T, H, D], k [T, G, D] (rotated), v [T, G, Dv] of one sequence from position 0.  A
    query sees the last `size` tokens (itself included) and, for every block of `pool` tokens
    that lies wholly before that window, the mean key and mean value of the block.  store: what
    the cache does to a key or value before it is averaged (rounding), identity by default."""
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    if store is not None:
        k, v = store(k), store(v)
    nb = T // pool if pool > 0 else 0
    kb = torch.zeros(nb, G, D, dtype=F64)
    vb = torch.zeros(nb, G, Dv, dtype=F64)
    for b in range(nb):
        kb[b] = k[b * pool:(b + 1) * pool].mean(dim=0)
        vb[b] = v[b * pool:(b + 1) * pool].mean(dim=0)
    out = torch.zeros(T, H, Dv, dtype=F64)
    rep = H // G
    for h in range(H):
        g = h // rep
        for i in range(T):
            s_tok = (k[:, g] @ q[i, h]) * scale
            s_blk = (kb[:, g] @ q[i, h]) * scale if nb else torch.zeros(0, dtype=F64)
            pt, pb = pooled_window_weights(s_tok, s_blk, i, size, pool)
            out[i, h] = pt @ v[:, g] + (pb @ vb[:, g] if nb else 0.0)
    return out


def attention(h, w, p, m, store=None):
    """The attention mixer on h [T, d]; w: the checkpoint, p the layer's prefix ('l3.'),
    m the mixer's config."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[p + "mix.q"].T + w[p + "mix.q.b"]).view(T, H, D)
    k = (h @ w[p + "mix.k"].T + w[p + "mix.k.b"]).view(T, G, D)
    v = (h @ w[p + "mix.v"].T + w[p + "mix.v.b"]).view(T, G, Dv)
    pos = list(range(T))
    q, k = rotate_half(q, pos, m.get("rot")), rotate_half(k, pos, m.get("rot"))
    mask = m.get("mask") or {}
    o = pooled_window_attention(q, k, v, float(m["scale"]), int(mask.get("size") or 0),
                                int(mask.get("pool") or 0), store)
    return o.reshape(T, H * Dv) @ w[p + "mix.o"].T + w[p + "mix.o.b"]


# ----------------------------------------------------------------------------- state-space mixer
def causal_conv(u, cw, cb):
    """u [T, C]; cw [C, taps] whose last column weighs the current token; zeros before the
    start."""
    T, C = u.shape
    taps = cw.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = cb.clone()
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                acc = acc + cw[:, j] * u[src]
        out[t] = acc
    return out


def selective_scan(x, B, C, dt, A_log, D, groups):
    """x [T, H, V], B and C [T, groups, N], dt [T, H] (after softplus).  Per head
    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T (S is N x V), y_t = S_t^T C_t + D x_t.
    Returns y [T, H, V] and the last states [H, N, V]."""
    T, H, V = x.shape
    N = B.shape[2]
    per = H // groups
    y = torch.zeros(T, H, V, dtype=F64)
    last = torch.zeros(H, N, V, dtype=F64)
    for h in range(H):
        g = h // per
        S = torch.zeros(N, V, dtype=F64)
        for t in range(T):
            a = math.exp(-math.exp(float(A_log[h])) * float(dt[t, h]))
            S = a * S + float(dt[t, h]) * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
        last[h] = S
    return y, last


def grouped_rms(y, parts, eps):
    T, n = y.shape
    return rms(y.view(T, parts, n // parts), eps).reshape(T, n)


def mamba2(h, w, p, m, eps):
    T = h.shape[0]
    H, V, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * V
    zx = h @ w[p + "mix.in"].T
    z = zx[:, :inner]
    xbc = zx[:, inner:2 * inner + 2 * G * N]
    dt = zx[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "mix.conv"], w[p + "mix.conv.b"]))
    x = xbc[:, :inner].reshape(T, H, V)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "mix.dt_bias"])
    y, _ = selective_scan(x, B, C, dt, w[p + "mix.A_log"], w[p + "mix.D"], G)
    y = y.reshape(T, inner) * silu(z)
    y = grouped_rms(y, int(m["norm_groups"]), eps) * w[p + "mix.norm"]
    return y @ w[p + "mix.o"].T


# ----------------------------------------------------------------------------- feed-forward
def gated(h, w, p, act):
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(scores, top, count, keep):
    """scores [E] of one token -> the chosen experts (a set)."""
    E = scores.shape[0]
    per = E // count
    gs = []
    for g in range(count):
        part = sorted((float(s) for s in scores[g * per:(g + 1) * per]), reverse=True)
        gs.append(sum(part[:2]))
    best = sorted(range(count), key=lambda g: (-gs[g], g))[:keep]
    allowed = [e for e in range(E) if e // per in best]
    return sorted(allowed, key=lambda e: (-float(scores[e]), e))[:top]


def moe(h, w, p, ml):
    rt = ml["router"]
    gr = rt.get("groups") or {}
    T = h.shape[0]
    s = torch.sigmoid(h @ w[p + "mlp.router"].T)
    out = torch.zeros(T, h.shape[1], dtype=F64)
    for t in range(T):
        for e in route(s[t], int(rt["top"]), int(gr.get("count") or 1), int(gr.get("keep") or 1)):
            out[t] += s[t, e] * gated(h[t:t + 1], w, p + f"mlp.e{e}.", silu)[0]
    if ml.get("shared"):
        out = out + gated(h, w, p + "mlp.shared.", silu)
    return out


def feed_forward(h, w, p, ml):
    if ml["kind"] == "dense":
        return gated(h, w, p + "mlp.", gelu_tanh)
    return moe(h, w, p, ml)


# ----------------------------------------------------------------------------- streams
def hyper_read(xs, w_in):
    """xs [S, T, d] -> the sublayer's input before its norm."""
    return torch.einsum("s,std->td", w_in, xs)


def hyper_write(xs, y, mix, w_out):
    """All streams at once from the old ones: x_t <- sum_s mix[s, t] x_s + out[t] y."""
    return torch.einsum("sr,std->rtd", mix, xs) + w_out[:, None, None] * y[None]


# ----------------------------------------------------------------------------- the model
def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, t = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def forward(cfg, w, tokens, store=None):
    """Logits [T, vocab] of one sequence and the sum of the streams after every layer run."""
    eps = float(cfg["norm"]["eps"])
    S = int(cfg.get("streams") or 0)
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = x[None].repeat(max(S, 1), 1, 1)
    after = []
    for li in layer_runs(cfg):
        ly = cfg["layers"][li]
        p = f"l{li}."
        for q, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and ly.get("mlp") is None:
                continue
            u = hyper_read(xs, w[p + f"hc{q}.in"]) if S else xs[0]
            hn = norm1p(u, w[p + f"norm{q}"], eps)
            if sub == "mlp":
                y = feed_forward(hn, w, p, ly["mlp"])
            elif ly["type"] == "attention":
                y = attention(hn, w, p, ly["mixer"], store)
            else:
                y = mamba2(hn, w, p, ly["mixer"], eps)
            xs = hyper_write(xs, y, w[p + f"hc{q}.mix"], w[p + f"hc{q}.out"]) if S \
                else xs + y[None]
        after.append(xs.sum(dim=0))
    hn = norm1p(xs.sum(dim=0), w["final.norm"], eps)
    logits = hn @ w["embed"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)


# ----------------------------------------------------------------------------- test models
def random_weights(cfg, seed=0):
    """Random weights under the checkpoint's names, values a bf16 file can hold (bf16 tensors).
    Norm weights sit around zero, stream weights around an identity, decays and step sizes in a
    range where the state neither dies at once nor stays for ever."""
    g = torch.Generator().manual_seed(seed)
    d, S = int(cfg["width"]), int(cfg.get("streams") or 0)

    def rnd(*shape, s=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * s + mean).to(torch.bfloat16)

    w = {"embed": rnd(int(cfg["vocab"]), d), "final.norm": rnd(d, s=0.2)}
    for i, ly in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = ly["mixer"]
        w[p + "norm1"] = rnd(d, s=0.2)
        subs = ["hc1"]
        if ly["type"] == "attention":
            H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
            for name, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                w[p + "mix." + name] = rnd(rows, d, s=d ** -0.5)
                w[p + "mix." + name + ".b"] = rnd(rows, s=0.3)
            w[p + "mix.o"] = rnd(d, H * Dv, s=(H * Dv) ** -0.5)
            w[p + "mix.o.b"] = rnd(d, s=0.3)
        else:
            H, V, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
            inner, C = H * V, H * V + 2 * G * N
            w[p + "mix.in"] = rnd(2 * inner + 2 * G * N + H, d, s=d ** -0.5)
            w[p + "mix.conv"] = rnd(C, int(m["conv"]), s=0.5)
            w[p + "mix.conv.b"] = rnd(C, s=0.2)
            w[p + "mix.dt_bias"] = rnd(H, s=1.0, mean=-1.0)
            w[p + "mix.A_log"] = rnd(H, s=0.7, mean=-0.5)
            w[p + "mix.D"] = rnd(H, s=0.3, mean=1.0)
            w[p + "mix.norm"] = rnd(inner, s=0.2, mean=1.0)
            w[p + "mix.o"] = rnd(d, inner, s=inner ** -0.5)
        ml = ly.get("mlp")
        if ml is not None:
            w[p + "norm2"] = rnd(d, s=0.2)
            subs.append("hc2")

            def gated_w(q, ff):
                w[q + "gate"] = rnd(ff, d, s=d ** -0.5)
                w[q + "up"] = rnd(ff, d, s=d ** -0.5)
                w[q + "down"] = rnd(d, ff, s=ff ** -0.5)

            if ml["kind"] == "dense":
                gated_w(p + "mlp.", int(ml["ff"]))
            else:
                w[p + "mlp.router"] = rnd(int(ml["router"]["experts"]), d, s=2 * d ** -0.5)
                for e in range(int(ml["router"]["experts"])):
                    gated_w(p + f"mlp.e{e}.", int(ml["expert"]["ff"]))
                if ml.get("shared"):
                    gated_w(p + "mlp.shared.", int(ml["shared"]["ff"]))
        if S:
            for name in subs:
                w[p + name + ".in"] = rnd(S, s=0.3, mean=1.0 / S)
                w[p + name + ".out"] = rnd(S, s=0.3, mean=0.8)
                w[p + name + ".mix"] = (torch.eye(S) + 0.15 * torch.randn(S, S, generator=g)
                                        ).to(torch.bfloat16)
    return w


def as_f64(weights):
    return {k: v.to(F64) for k, v in weights.items()}


def att_layer(heads, kv_heads, dim, vdim, scale, window=0, pool=0, rot_dims=None, base=100.0,
              yarn=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base, "scaling": yarn}}
    if window:
        m["mask"] = {"size": window, "pool": pool}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def ssm_layer(heads, vdim, state, groups, conv=4, norm_groups=1, mlp=None):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                      "norm_groups": norm_groups}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def routed(experts, top, ff, count=1, keep=1, shared=0):
    ml = {"kind": "moe", "expert": {"ff": ff},
          "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}
    if shared:
        ml["shared"] = {"ff": shared}
    return ml


def make_config(width, vocab, layers, streams=2, eps=1e-5, softcap=12.0, loop=None):
    cfg = {"architecture": "Mudepel", "layers": layers, "norm": {"eps": eps}, "vocab": vocab,
           "width": width}
    if streams:
        cfg["streams"] = streams
    if softcap:
        cfg["logit_softcap"] = softcap
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg
