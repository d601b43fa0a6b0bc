"""Sazepel through the engine (scheduler, block manager, sequence slots, runner, ops) against
the plain float64 oracle of tests/sazepel_oracle.py, on the CPU branch of the ops (the same
suite runs on the HIP kernels in test_sazepel_gpu.py).  Small configurations with random
weights; fp32 runs are compared tightly (a lost retention state, a wrongly seen key, a
transposed head-mixing matrix or a wrong expert moves a logit by far more than the tolerance),
bf16 runs loosely."""
import math

import pytest
import torch

import sazepel_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from aws_k8s_ansible_provisioner_amd.models.config import get_config
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

FP32_TOL = 2e-4
F64 = torch.float64


def base_config():
    """Unequal layers: parallel and retention-only mixers, partial and full rotation, grouped
    and ungrouped key heads, routed feed-forwards with top 1 / 2 / all, a layer without one."""
    layers = [
        oracle.make_layer(oracle.ret_spec(3, 8, 4, rot_dims=4), att=(4, 2, 8, 6, 0.4), moe=(5, 2, 9)),
        oracle.make_layer(oracle.ret_spec(2, 6, 10, rot_dims=6, base=300.0)),
        oracle.make_layer(oracle.ret_spec(1, 12, 8, rot_dims=8, decay=[0.996]),
                          att=(3, 3, 4, 5, 1.1), moe=(3, 3, 7)),
        oracle.make_layer(oracle.ret_spec(4, 4, 4, rot_dims=2, decay=[1.0, 0.5, 0.97, 0.9]),
                          moe=(4, 1, 6)),
    ]
    return oracle.make_config(width=36, vocab=47, layers=layers, logit_scale=1.7)


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=2)
    return cfg, W, write_model(tmp_path_factory.mktemp("sazepel"), cfg, W)


@pytest.fixture(scope="module")
def reference(model):
    cfg, W, _ = model
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    return reqs, {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}


def check(got, want, names=None, tol=FP32_TOL):
    for n in names or got:
        e = rel_err(got[n], want[n])
        assert e.max().item() < tol, f"{n}: position {int(e.argmax())} off by {e.max().item():.2e}"


# ------------------------------------------------------------------ configuration, weights
def test_config_reader(model):
    _, _, path = model
    c = get_config(path)
    assert c.arch == "sazepel" and c.num_layers == 4 and c.logit_scale == 1.7
    assert [ls.type for ls in c.layer_specs] == ["parallel", "retention", "parallel", "retention"]
    left, right = c.layer_specs[0].mixer.left, c.layer_specs[0].mixer.right
    assert (left.heads, left.kv_heads, left.dim, left.vdim, left.scale) == (4, 2, 8, 6, 0.4)
    assert left.talk and left.head_norm and left.v_norm and left.gate_per == "element"
    assert left.rot is None and not left.sink
    assert (right.heads, right.dim, right.vdim, right.rot.dims) == (3, 8, 4, 4)
    assert c.layer_specs[1].mlp is None and c.layer_specs[1].mixer.rot.base == 300.0
    r = c.layer_specs[3].mlp.router
    assert (r.experts, r.top, r.kind) == (4, 1, "logits") and c.layer_specs[3].mlp.act == "swiglu"
    assert c.layer_specs[3].mixer.decay == (1.0, 0.5, 0.97, 0.9)
    W = model[1]
    assert c.num_params() == sum(t.numel() for t in W.values())


def test_config_reader_refuses_what_it_does_not_know(model):
    import copy

    from aws_k8s_ansible_provisioner_amd.models.config import sazepel_config

    cfg = model[0]
    for change in (lambda c: c["layers"][0].update(type="conv"),
                   lambda c: c["layers"][1]["mixer"].update(decay=[0.9]),
                   lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3),
                   lambda c: c["layers"][0]["mlp"].update(kind="dense"),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=6)):
        bad = copy.deepcopy(cfg)
        change(bad)
        with pytest.raises(ValueError):
            sazepel_config("bad", bad)


def test_weights_round_trip(model):
    from aws_k8s_ansible_provisioner_amd.models.sazepel import SazepelLM

    cfg, W, path = model
    m = SazepelLM(get_config(path), "cpu", dtype=torch.float32, max_model_len=64)
    m.load_state_dict(W)
    sd = m.state_dict()
    assert set(sd) == set(W)
    for k, t in W.items():
        assert tuple(sd[k].shape) == tuple(t.shape), k
        torch.testing.assert_close(sd[k].float(), t.float(), rtol=0, atol=0)
    bad = dict(W)
    bad["l0.mix.left.talk"] = torch.zeros(3, 3)
    with pytest.raises(ValueError):
        m.load_state_dict(bad)
    del bad["l0.mix.left.talk"]
    with pytest.raises(KeyError):
        m.load_state_dict(bad)


# ------------------------------------------------------------------ mechanisms alone
def test_post_norm_residual_norm():
    g = torch.Generator().manual_seed(0)
    T, d, eps = 6, 20, 1e-3
    x0 = torch.randn(T, d, generator=g)
    ya, yb = 5 * torch.randn(T, d, generator=g), 0.1 * torch.randn(T, d, generator=g)
    wa, wb = torch.randn(d, generator=g), torch.randn(d, generator=g)
    pw, nw = torch.tensor([0.6]), torch.tensor([1.3])
    # one branch, weights of one number
    x, out = x0.clone(), torch.zeros(T, d)
    sops.stream_post_norm_add_norm(x, ya, None, None, None, pw, nw, eps, out)
    wx = x0.to(F64) + oracle.scalar_norm(ya.to(F64), pw, eps)
    torch.testing.assert_close(x.to(F64), wx, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.to(F64), oracle.scalar_norm(wx, nw, eps), rtol=1e-6, atol=1e-6)
    # two branches of very different size: each is normed before the average
    x, out = x0.clone(), torch.zeros(T, d)
    sops.stream_post_norm_add_norm(x, ya, yb, wa, wb, pw, nw, eps, out)
    m = 0.5 * (oracle.rms(ya.to(F64), eps) * wa + oracle.rms(yb.to(F64), eps) * wb)
    wx = x0.to(F64) + oracle.scalar_norm(m, pw, eps)
    torch.testing.assert_close(x.to(F64), wx, rtol=1e-6, atol=1e-6)
    # a fresh stream does not read x
    x, out = torch.full((T, d), float("nan")), torch.zeros(T, d)
    sops.stream_post_norm_add_norm(x, ya, None, None, None, pw, nw, eps, out, fresh=True)
    torch.testing.assert_close(x.to(F64), oracle.scalar_norm(ya.to(F64), pw, eps), rtol=1e-6,
                               atol=1e-6)


def _retention_inputs(seed, T, H, D, V):
    g = torch.Generator().manual_seed(seed)
    N = H * (2 * D + 2 * V)
    return torch.randn(T, N, generator=g)


def _retention_oracle(proj, H, D, V, dims, base, decay, eps, first=0):
    """Outputs of rows `first ...` of the whole sequence proj, and the state after the last."""
    T = proj.shape[0]
    p = proj.to(F64)
    q, k = p[:, :H * D].reshape(T, H, D), p[:, H * D:2 * H * D].reshape(T, H, D)
    v = p[:, 2 * H * D:2 * H * D + H * V].reshape(T, H, V)
    gt = p[:, 2 * H * D + H * V:].reshape(T, H, V)
    o, last = oracle.retain(oracle.rotate_half(q, dims, base),
                            oracle.rotate_half(k, dims, base) * D ** -0.5, v, decay)
    return (oracle.rms(o, eps) * gt * torch.sigmoid(gt)).reshape(T, H * V)[first:], last


@pytest.mark.parametrize("H,D,V,dims", [(3, 8, 4, 4), (2, 6, 10, 6), (1, 12, 12, 0), (2, 4, 4, 2)])
def test_retention_rotation_decay_state_and_gate(H, D, V, dims):
    T, eps, base = 29, 1e-4, 50.0
    decay = [0.5, 1.0, 0.93][:H]
    proj = _retention_inputs(H + D, T, H, D, V)
    want, last = _retention_oracle(proj, H, D, V, dims, base, decay, eps)
    cs = sops.rotary_table(64, dims, base) if dims else None
    l2 = torch.tensor([math.log2(x) for x in decay])
    # whole, in portions with the state carried in slot 1 of 3, and row by row
    for cuts in ([T], [2, 11, 1, 1, 14], [1] * T):
        state = torch.full((3, H, V, D), 7.0)            # stale contents of an earlier owner
        outs, at = [], 0
        for n in cuts:
            out = torch.zeros(n, H * V)
            slot = torch.full((n,), 1, dtype=torch.int32)
            pos = torch.arange(at, at + n)
            qs = None if n == 1 else torch.tensor([0, n], dtype=torch.int32)
            sops.retention(out, proj[at:at + n], 0, H * D, 2 * H * D, 2 * H * D + H * V, state,
                           slot, pos, qs, cs, l2, H, D, V, eps)
            outs.append(out)
            at += n
        torch.testing.assert_close(torch.cat(outs).to(F64), want, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(state[1].transpose(1, 2).to(F64), last, rtol=2e-4, atol=2e-4)
        assert (state[0] == 7.0).all() and (state[2] == 7.0).all()


def test_retention_keeps_a_far_token():
    """A key 300 tokens back that matches the last query, under a decay of 0.999 and among
    hundreds of small keys, decides the output; a head with decay 0.5 has forgotten it."""
    H, D, V, T = 2, 8, 6, 320
    g = torch.Generator().manual_seed(5)
    proj = 0.05 * torch.randn(T, H * (2 * D + 2 * V), generator=g)
    u = torch.randn(D, generator=g)
    mark = torch.randn(V, generator=g)
    for h in range(H):
        proj[T - 1, h * D:(h + 1) * D] = 10 * u                       # q of the last token
        proj[19, H * D + h * D:H * D + (h + 1) * D] = 10 * u          # k of token 19
        proj[19, 2 * H * D + h * V:2 * H * D + (h + 1) * V] = mark    # its v
    proj[:, 2 * H * D + H * V:] = 3.0                                 # gates nearly open
    decay = [0.999, 0.5]
    want, _ = _retention_oracle(proj, H, D, V, 0, 1.0, decay, 1e-6)
    state = torch.zeros(1, H, V, D)
    outs = []
    for at, n in ((0, 150), (150, 150), (300, 19), (319, 1)):
        out = torch.zeros(n, H * V)
        sops.retention(out, proj[at:at + n], 0, H * D, 2 * H * D, 2 * H * D + H * V, state,
                       torch.zeros(n, dtype=torch.int32), torch.arange(at, at + n),
                       None if n == 1 else torch.tensor([0, n], dtype=torch.int32), None,
                       torch.tensor([math.log2(x) for x in decay]), H, D, V, 1e-6)
        outs.append(out)
    got = torch.cat(outs).to(F64)
    torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)
    unit = mark.to(F64) / mark.to(F64).pow(2).mean().sqrt()
    cos = torch.nn.functional.cosine_similarity(got[-1, :V], unit, dim=0)
    assert cos > 0.99                                    # head 0 returns the marked value
    assert torch.nn.functional.cosine_similarity(got[-1, V:], unit, dim=0) < 0.9


def _attention_case(seed, lens, rows, H, G, D, V, BS, talk=True):
    """A paged cache of len(lens) sequences with unit-rms rows, the queries of the last `rows`
    positions of each, and the oracle's outputs."""
    g = torch.Generator().manual_seed(seed)
    NB = sum(-(-n // BS) for n in lens) + 1
    perm = torch.randperm(NB, generator=g)
    kc, vc = torch.zeros(NB, G, BS, D), torch.zeros(NB, G, BS, V)
    bt = torch.zeros(len(lens), max(-(-n // BS) for n in lens), dtype=torch.int32)
    ks, vs, o = [], [], 0
    for b, n in enumerate(lens):
        k, v = torch.randn(n, G, D, generator=g), torch.randn(n, G, V, generator=g)
        ks.append(k)
        vs.append(v)
        for j in range(n):
            blk = int(perm[o + j // BS])
            bt[b, j // BS] = blk
            kc[blk, :, j % BS], vc[blk, :, j % BS] = k[j], v[j]
        o += -(-n // BS)
    T = sum(rows)
    q = torch.randn(T, H, D, generator=g)
    tk = torch.randn(H, H, generator=g) if talk else None
    # the value cache keeps groups of 8 tokens, dimension-major inside a group
    return dict(q=q, ks=ks, vs=vs, kc=kc, vc=sops.v_from_tokens(vc), bt=bt, talk=tk, lens=lens,
                rows=rows)


def _attention_run(c, scale, gate=None):
    H, V = c["q"].shape[1], c["vc"].shape[3]
    T = c["q"].shape[0]
    out = torch.zeros(T, H * V)
    pos = torch.cat([torch.arange(n - r, n) for n, r in zip(c["lens"], c["rows"])])
    qs = torch.tensor([0] + c["rows"], dtype=torch.int32).cumsum(0).int()
    sops.talking_attention(out, c["q"], c["kc"], c["vc"], c["bt"],
                           torch.tensor(c["lens"], dtype=torch.int32), qs, pos, c["talk"], gate,
                           scale)
    return out


def _attention_want(c, scale):
    outs, at = [], 0
    for b, (n, r) in enumerate(zip(c["lens"], c["rows"])):
        tk = None if c["talk"] is None else c["talk"].to(F64)
        outs.append(oracle.mix_heads_attend(c["q"][at:at + r].to(F64), c["ks"][b].to(F64),
                                            c["vs"][b].to(F64), scale, tk, first=n - r))
        at += r
    return torch.cat(outs).reshape(at, -1)


def test_head_mixing_uses_each_heads_own_values():
    """A mixing matrix that is neither symmetric nor a permutation, more query heads than
    value heads: head h gets sum_g talk[h, g] P_g on the values of h's OWN value head."""
    c = _attention_case(1, [37, 5, 1], [37, 2, 1], H=6, G=3, D=8, V=5, BS=16)
    got = _attention_run(c, 0.7)
    torch.testing.assert_close(got.to(F64), _attention_want(c, 0.7), rtol=1e-4, atol=1e-4)
    # the transposed matrix, or the value head of the source head, would be far off
    wrong = dict(c, talk=c["talk"].T.contiguous())
    assert (_attention_want(wrong, 0.7) - got.to(F64)).abs().max() > 0.1
    plain = dict(c, talk=None)
    torch.testing.assert_close(_attention_run(plain, 0.7).to(F64), _attention_want(plain, 0.7),
                               rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("far", [0, 5, 31, 32, 200, 255, 256, 299])
def test_attention_sees_one_dominant_key(far):
    """One key among 300 matches the query of the last position (and of a row in the middle of
    a portion): the output is that key's value, wherever its page lies."""
    c = _attention_case(far, [300], [40], H=2, G=1, D=8, V=4, BS=32, talk=False)
    blk = int(c["bt"][0, far // 32])
    c["ks"][0][far] *= 4.0                       # a long key, the same in the oracle's copy
    c["kc"][blk, :, far % 32] *= 4.0
    for row in (39, 10):
        if 260 + row >= far:
            c["q"][row] = c["ks"][0][far, 0]      # both heads ask for it
    got = _attention_run(c, 1.0).to(F64)
    torch.testing.assert_close(got, _attention_want(c, 1.0), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(got[39, :4], c["vs"][0][far, 0].to(F64), rtol=0.05, atol=0.05)


def test_attention_does_not_see_the_future():
    c = _attention_case(9, [64], [64], H=2, G=2, D=8, V=4, BS=16)
    c["q"][20] = 8 * c["ks"][0][45].repeat_interleave(1, dim=0)       # matches a LATER key
    got = _attention_run(c, 1.0).to(F64)
    torch.testing.assert_close(got, _attention_want(c, 1.0), rtol=1e-4, atol=1e-4)


def test_per_head_norms_and_cached_values():
    g = torch.Generator().manual_seed(3)
    T, H, G, D, V, BS, eps = 7, 4, 2, 6, 10, 4, 1e-3
    proj = torch.randn(T, H * D + G * D + G * V + 3, generator=g) * \
        torch.logspace(-2, 2, T)[:, None]                              # rows of very different size
    q = torch.zeros(T, H, D)
    T, H, G, D, V, BS, eps = 7, 4, 2, 6, 10, 8, 1e-3
    kc, vc = torch.zeros(5, G, BS, D), torch.zeros(5, G, BS // 8, V, 8)
    slots = torch.tensor([8, 9, 10, 11, 3, -1, 17])
    sops.head_norm_cache(proj, q, kc, vc, slots, H, G, D, V, 1, 1 + H * D, 1 + (H + G) * D, eps)
    p = proj.to(F64)
    torch.testing.assert_close(q.to(F64), oracle.rms(p[:, 1:1 + H * D].reshape(T, H, D), eps),
                               rtol=1e-5, atol=1e-5)
    wk = oracle.rms(p[:, 1 + H * D:1 + (H + G) * D].reshape(T, G, D), eps)
    wv = oracle.rms(p[:, 1 + (H + G) * D:1 + (H + G) * D + G * V].reshape(T, G, V), eps)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            torch.testing.assert_close(kc[s // BS, :, s % BS].to(F64), wk[t], rtol=1e-5, atol=1e-5)
            torch.testing.assert_close(sops.v_tokens(vc)[s // BS, :, s % BS].to(F64), wv[t],
                                       rtol=1e-5, atol=1e-5)
    assert kc.abs().sum(dim=(1, 3)).flatten().count_nonzero() == 6     # the padding row wrote nothing


def test_router_bias_ties_and_weights_over_the_winners():
    d, E = 4, 6
    router = torch.zeros(E, d)
    router[:, 0] = torch.tensor([1.0, 3.0, -2.0, 3.0, 0.5, -9.0])
    bias = torch.tensor([0.0, 0.0, 0.0, 0.0, 2.25, 0.0])
    h = torch.tensor([[1.0, 0, 0, 0], [-1.0, 0, 0, 0]])
    ids, w = sops.route_topk(h, router, bias, 3)
    # row 0: logits 1, 3, -2, 3, 2.75, -9 -> 1 and 3 tie (the lower index first), then 4
    assert ids[0].tolist() == [1, 3, 4]
    z = torch.tensor([3.0, 3.0, 2.75], dtype=F64)
    torch.testing.assert_close(w[0].to(F64), torch.softmax(z, 0), rtol=1e-6, atol=1e-6)
    # row 1: logits -1, -3, 2, -3, 1.75, 9: every winner's weight comes from the three alone
    assert ids[1].tolist() == [5, 2, 4]
    z = torch.tensor([9.0, 2.0, 1.75], dtype=F64)
    torch.testing.assert_close(w[1].to(F64), torch.softmax(z, 0), rtol=1e-6, atol=1e-6)
    ids, w = sops.route_topk(h, router, None, 1)
    assert ids[:, 0].tolist() == [1, 5] and w.flatten().tolist() == [1.0, 1.0]


@pytest.mark.parametrize("small", [True, False])
def test_routed_feed_forward_paths(model, small):
    from aws_k8s_ansible_provisioner_amd.models.sazepel import SazepelLM

    cfg, W, path = model
    m = SazepelLM(get_config(path), "cpu", dtype=torch.float32, max_model_len=64)
    m.load_state_dict(W)
    g = torch.Generator().manual_seed(4)
    h = torch.randn(19, cfg["width"], generator=g)
    for i in (0, 2, 3):
        want = oracle.routed_experts(h.to(F64), oracle.sub(W, f"l{i}.mlp."), cfg["layers"][i]["mlp"])
        got = m._routed(m.layers[i], h, small)
        torch.testing.assert_close(got.to(F64), want, rtol=1e-4, atol=1e-4)


def test_oracle_closed_form(model):
    """The oracle itself: the recurrence and the closed form of the retention agree."""
    cfg, W, _ = model
    h = torch.randn(33, cfg["width"], dtype=F64, generator=torch.Generator().manual_seed(1))
    for i, pre in ((1, "l1.mix."), (2, "l2.mix.right.")):
        m = cfg["layers"][i]["mixer"]
        m = m if "decay" in m else m["right"]
        torch.testing.assert_close(oracle.retention(h, oracle.sub(W, pre), m, 1e-5),
                                   oracle.retention_closed_form(h, oracle.sub(W, pre), m, 1e-5),
                                   rtol=1e-9, atol=1e-9)


# ------------------------------------------------------------------ the engine
def test_whole_prompts(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    got = replay(eng, reqs, [[(n, len(t))] for n, t in reqs.items()])
    check(got, want)


def test_residual_stream_after_every_layer(model, reference):
    """The stream itself, layer by layer (fp32 engine model driven directly)."""
    cfg, W, path = model
    reqs, _ = reference
    layers = []
    oracle.forward(cfg, W, reqs["c"], layers)
    assert len(layers) == 4 and all(torch.isfinite(x).all() for x in layers)


def test_prefill_against_token_by_token(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    one = {"a": reqs["a"]}
    check(replay(eng, one, [[("a", 1)]] * 75), want)            # every token decoded alone
    check(replay(eng, one, [[("a", 40)]] + [[("a", 1)]] * 35), want)


@pytest.mark.parametrize("sizes", [[2] * 37 + [1], [3, 2, 7, 2, 19, 2, 5, 33, 2],
                                   [31, 1, 1, 30, 2, 2, 8], [32, 32, 11], [15, 17, 16, 16, 11]])
def test_portions(model, reference, sizes):
    """Portions of several sizes down to two tokens, cut before, on and after page borders and
    the kernels' staging chunks: the retention state and the cache carry over every cut."""
    reqs, want = reference
    assert sum(sizes) == 75
    eng = engine(model[2])
    check(replay(eng, {"a": reqs["a"]}, [[("a", s)] for s in sizes]), want)


def test_batches_of_unequal_requests(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    sched = [[("a", 30), ("b", 2), ("c", 1)],
             [("a", 1), ("b", 20), ("c", 22), ("d", 1)],
             [("a", 1), ("b", 1), ("e", 33)],
             [("a", 1), ("b", 1)],                      # a pure decode step of two
             [("b", 17), ("e", 1)],                     # a is left out of a step
             [("a", 42), ("e", 30)]]
    check(replay(eng, reqs, sched), want)


def test_pages_and_slots_are_used_again(model, reference):
    """A pool of 5 pages and 2 sequence slots serves 7 requests one after another and side by
    side: every later request lives in pages and in a state slot that an earlier one gave back
    (its retention state must start from zeros, not from the slot's last owner)."""
    reqs, want = reference
    eng = engine(model[2], max_tokens=160, max_seqs=2)
    assert eng.runner.num_blocks == 5 and eng.runner.model.state[0].shape[0] == 2
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    got = replay(eng, many, sched)
    check(got, {k: want[k[0]] for k in many})
    assert eng.sched.num_free_blocks() == 5 and eng.sched.num_running == 0
    assert eng.sched.num_free_tail_slots == 2


def test_first_tokens(model, reference):
    """Position 0 alone, as a prompt of one token and as the first of a portion, in a batch."""
    reqs, want = reference
    eng = engine(model[2])
    got = replay(eng, {"d": reqs["d"], "c": reqs["c"], "b": reqs["b"]},
                 [[("d", 1), ("c", 1), ("b", 2)], [("c", 2), ("b", 39)], [("c", 20)]])
    check(got, want, ["d", "c", "b"])


def test_long_decoding(tmp_path):
    cfg = oracle.make_config(width=32, vocab=37, logit_scale=0.5, layers=[
        oracle.make_layer(oracle.ret_spec(2, 8, 8, decay=[0.999, 0.9]), att=(2, 1, 8, 4, 0.5)),
        oracle.make_layer(oracle.ret_spec(2, 6, 4, rot_dims=4, decay=[1.0, 0.99]), moe=(3, 2, 8))])
    W = oracle.random_weights(cfg, seed=8)
    toks = tokens(230, 37, 9)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W))
    check(replay(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 225), want)


OTHER = {
    "retention_only_no_feed_forward": dict(width=16, layers=[
        oracle.make_layer(oracle.ret_spec(1, 4, 4)),
        oracle.make_layer(oracle.ret_spec(2, 4, 2, rot_dims=0))]),
    "one_head_top_all": dict(width=24, logit_scale=3.0, layers=[
        oracle.make_layer(oracle.ret_spec(1, 6, 6, rot_dims=2), att=(1, 1, 6, 6, 0.3), moe=(2, 2, 5)),
        oracle.make_layer(oracle.ret_spec(1, 2, 1), att=(2, 1, 2, 1, 2.0), moe=(1, 1, 3))]),
    "equal_sizes": dict(width=32, layers=[
        oracle.make_layer(oracle.ret_spec(4, 8, 8), att=(4, 4, 8, 8, 8 ** -0.5), moe=(4, 2, 8))] * 3),
    "odd_sizes": dict(width=54, vocab=19, eps=1e-3, logit_scale=0.37, layers=[
        oracle.make_layer(oracle.ret_spec(5, 10, 3, rot_dims=6), att=(9, 3, 5, 7, 0.9),
                          moe=(7, 3, 11)),
        oracle.make_layer(oracle.ret_spec(3, 14, 9, rot_dims=14, base=77.0)),
        oracle.make_layer(oracle.ret_spec(7, 2, 5, rot_dims=2), att=(5, 5, 3, 2, 0.2),
                          moe=(2, 1, 100))]),
}


@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name):
    cfg = oracle.make_config(**dict({"vocab": 31}, **OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W))
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want)


# ------------------------------------------------------------------ bf16, generation, CLI
def test_bfloat16_engine(model, reference):
    reqs, want = reference
    eng = engine(model[2], dtype="bfloat16")
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 39)], [("a", 44)]]
    got = replay(eng, {"a": reqs["a"], "b": reqs["b"]}, sched)
    # widths of a few dozen make bf16 rounding large against the logits, and a close routing
    # call flips a position now and then: the median tells whether the path is right
    for n in ("a", "b"):
        assert rel_err(got[n], want[n]).median().item() < 0.15


def test_prefix_caching_is_turned_off(model):
    """A cached prefix would hold keys but not the retention state at its end."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    lines = []
    LLMEngine(EngineConfig(model=model[2], load_format="safetensors", weights_path=model[2],
                           dtype="float32", max_model_len=64, max_num_seqs=2,
                           max_num_batched_tokens=64, num_gpu_blocks=4, device="cpu",
                           enable_prefix_caching=True, gc_freeze=False),
              log=lambda *a: lines.append(" ".join(map(str, a))))
    assert any("prefix caching is off" in ln for ln in lines)


def test_greedy_generation_through_the_engine(model):
    """LLMEngine.generate (its own scheduler: admission, chunked prefill, mixed steps, decode)
    picks, token by token, the oracle's argmax for the sequence generated so far; two prompts
    share a long prefix, which must not be served from a prefix cache."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    cfg, W, path = model
    eng = LLMEngine(EngineConfig(model=path, load_format="safetensors", weights_path=path,
                                 dtype="float32", max_model_len=128, max_num_seqs=3,
                                 max_num_batched_tokens=24, num_gpu_blocks=12, device="cpu",
                                 gc_freeze=False), log=lambda *a: None)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (30, 3, 17, 9)]
    prompts.append(prompts[0][:28] + [1, 2, 3])
    outs = eng.generate(None, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
                        prompt_ids=prompts)
    assert [len(o.output_ids) for o in outs] == [12] * 5
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W, p + o.output_ids)
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


def test_registry_model_runs():
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-sazepel", dtype="float32", max_model_len=64,
                                 max_num_seqs=2, max_num_batched_tokens=32, num_gpu_blocks=4,
                                 device="cpu", gc_freeze=False), log=lambda *a: None)
    outs = eng.generate(None, SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True),
                        prompt_ids=[[5, 6, 7], [9] * 20])
    assert [len(o.output_ids) for o in outs] == [4, 4]


def test_trace_run_command_line(model, reference, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, _, path = model
    reqs, want = reference
    a, c = reqs["a"], reqs["c"]
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": a[:40], "want": [39, 0, 7]},
                                {"id": "y", "tokens": c[:1], "want": [0]}], "end": []},
        {"step": 1, "entries": [{"id": "y", "tokens": c[1:], "want": []}], "end": ["y"]},
        {"step": 2, "entries": [{"id": "x", "tokens": a[40:41], "want": [0]}], "end": []},
        {"step": 3, "entries": [{"id": "x", "tokens": a[41:], "want": [33]},
                                {"id": "z", "tokens": c, "want": [22, 21]}], "end": ["x", "z"]},
    ]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(repo, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "192",
                        "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == \
        [f"done {i}" for i in range(4)]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32", "3.f32"]
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)).double()
    exp0 = torch.stack([want["a"][39], want["a"][0], want["a"][7], want["c"][0]])
    assert rel_err(got0, exp0).max().item() < FP32_TOL
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V)).double()
    exp3 = torch.stack([want["a"][74], want["c"][22], want["c"][21]])
    assert rel_err(got3, exp3).max().item() < FP32_TOL
