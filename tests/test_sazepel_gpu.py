"""Sazepel on the HIP kernels: every new kernel against the PyTorch version of the same op (fp32
and bf16 storage, odd sizes), then the engine -- mixed steps, hipGraph decode, a small page and
slot pool -- against the float64 oracle (tests/sazepel_oracle.py), and greedy generation
through LLMEngine.generate."""
import pytest
import torch

import sazepel_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from test_sazepel import OTHER, base_config
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-4, "bfloat16": 0.3}


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close(a, b, dtype, scale=1.0):
    tol = 3e-5 if dtype == "float32" else 2e-2
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=tol, atol=tol * scale)


# ------------------------------------------------------------------ kernels against their ops
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [24, 200, 2048, 4100, 8192])
def test_post_norm_add_norm_kernel(dtype, d):
    g, dt = gen(d), DT[dtype]
    T = 5
    x = torch.randn(T, d, generator=g)
    ya = torch.randn(T, d + 8, generator=g).to(dt)[:, :d]
    yb = (3 * torch.randn(T, d, generator=g)).to(dt)
    y32 = torch.randn(T, d, generator=g)
    wa, wb = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    one, vec = torch.tensor([0.7]), 1 + 0.3 * torch.randn(d, generator=g)
    cases = [(ya, None, None, None, one, one, False), (ya, yb, wa, wb, one, vec, False),
             (y32, None, None, None, vec, one, False), (ya, None, None, None, one, one, True),
             (ya, yb, one, one, vec, vec, True)]
    for a, b, u, v, pw, nw, fresh in cases:
        res = []
        for dev in ("cpu", "cuda"):
            mv = lambda t: None if t is None else t.to(dev)  # noqa: E731
            xx = x.clone().to(dev) if not fresh else torch.full((T, d), 9.0, device=dev)
            o = torch.zeros(T, d, dtype=dt, device=dev)
            sops.stream_post_norm_add_norm(xx, mv(a), mv(b), mv(u), mv(v), mv(pw), mv(nw), 1e-6, o,
                                           fresh=fresh)
            res.append((xx, o))
        close(res[1][0], res[0][0], "float32")
        close(res[1][1], res[0][1], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,Dv", [(6, 2, 80, 96), (4, 1, 20, 36), (8, 8, 128, 64), (3, 3, 7, 5)])
def test_head_norm_cache_kernel(dtype, H, G, D, Dv):
    g, dt = gen(H * D), DT[dtype]
    T, NB, BS = 9, 4, 16
    N = H * D + G * (D + Dv) + 11
    proj = torch.randn(T, N, generator=g).to(dt)
    slots = torch.tensor([5, 17, 63, 0, -1, 33, 16, 15, 48])
    res = []
    for dev in ("cpu", "cuda"):
        for nq, nv in ((True, True), (False, True), (True, False)):
            q = torch.zeros(T, H, D, dtype=dt, device=dev)
            kc = torch.zeros(NB, G, BS, D, dtype=dt, device=dev)
            vc = torch.zeros(NB, G, BS // 8, Dv, 8, dtype=dt, device=dev)
            sops.head_norm_cache(proj.to(dev), q, kc, vc, slots.to(dev), H, G, D, Dv, 3, 3 + H * D,
                                 3 + H * D + G * D, 1e-6, nq, nv)
            res.append((q, kc, vc))
    n = len(res) // 2
    for i in range(n):
        for a, b in zip(res[i], res[n + i]):
            close(b, a, dtype)


def _retention_case(dtype, H, D, V, rot, dev, steps, g, slots=3):
    """Run `steps` (each a list of (slot, first position, rows)) through the op; returns the
    outputs of all steps and the final state."""
    dt = DT[dtype]
    N = H * (2 * D + 2 * V) + 5
    state = torch.zeros(slots, H, V, D, device=dev)
    decay = torch.log2(torch.tensor([0.9 + 0.099 * h / max(1, H - 1) for h in range(H)]))
    cs = sops.rotary_table(1024, rot, 10000.0) if rot else None
    outs = []
    for step in steps:
        T = sum(n for _, _, n in step)
        proj = torch.randn(T, N, generator=g).to(dt)
        slot = torch.cat([torch.full((n,), s, dtype=torch.int32) for s, _, n in step])
        pos = torch.cat([torch.arange(p, p + n) for _, p, n in step])
        qs = torch.tensor([0] + [n for _, _, n in step], dtype=torch.int32).cumsum(0).int()
        single = all(n == 1 for _, _, n in step)
        out = torch.zeros(T, H * V + 3, dtype=dt, device=dev)
        sops.retention(out[:, :H * V], proj.to(dev), 2, 2 + H * D, 2 + 2 * H * D,
                       2 + 2 * H * D + H * V, state, slot.to(dev), pos.to(dev),
                       None if single else qs.to(dev), cs.to(dev) if rot else None,
                       decay.to(dev), H, D, V, 1e-6)
        outs.append(out)
    return outs, state


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,V,rot", [(3, 64, 64, 32), (5, 64, 32, 64), (2, 128, 128, 64),
                                       (3, 24, 40, 8), (2, 80, 96, 0), (1, 256, 256, 128),
                                       (2, 16, 8, 16)])
def test_retention_kernel(dtype, H, D, V, rot):
    # portions of several sequences, a sequence continued from its slot, single rows, a slot
    # started again at position 0 over what an earlier sequence left, a padding row
    steps = [[(0, 0, 37), (2, 0, 3)], [(0, 37, 1), (2, 3, 1)], [(2, 4, 18), (0, 38, 2), (-1, 0, 1)],
             [(1, 0, 1), (0, 40, 1)], [(2, 0, 5)]]
    res = [_retention_case(dtype, H, D, V, rot, dev, steps, gen(7)) for dev in ("cpu", "cuda")]
    for a, b in zip(res[0][0], res[1][0]):
        close(b, a, dtype, scale=3.0)
    close(res[1][1], res[0][1], "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,V,rot", [(3, 64, 32, 16), (2, 128, 128, 64), (2, 24, 40, 8)])
def test_retention_kernel_in_segments(dtype, H, D, V, rot):
    """A step long enough for the segmented form: sequences of many segments, one that goes on
    from its slot's state, a single row and a padding row among them; then single rows that
    continue from the states the segmented step left."""
    steps = [[(2, 0, 10)], [(0, 0, 700), (2, 10, 600), (1, 0, 1), (-1, 0, 3), (3, 0, 257)],
             [(0, 700, 1), (2, 610, 1), (3, 257, 1)]]
    assert sum(n for _, _, n in steps[1]) >= sops.RETENTION_SEGMENTED_ROWS
    res = [_retention_case(dtype, H, D, V, rot, dev, steps, gen(9), slots=4) for dev in ("cpu", "cuda")]
    for a, b in zip(res[0][0], res[1][0]):
        close(b, a, dtype, scale=10.0)
    torch.testing.assert_close(res[1][1].cpu(), res[0][1], rtol=2e-4, atol=2e-3)


def _attention_case(dtype, H, G, D, Dv, dev, g, parts, talk=True, gate=True, BS=16):
    dt = DT[dtype]
    lens = [70, 1, 33, 130]                     # cached keys per sequence
    rows = [5, 1, 33, 1]                        # rows of this step (the last positions)
    NB = sum(-(-n // BS) for n in lens) + 2
    kc = torch.randn(NB, G, BS, D, generator=g).to(dt)
    vc = torch.randn(NB, G, BS // 8, Dv, 8, generator=g).to(dt)
    perm = torch.randperm(NB, generator=g).int()
    mb = max(-(-n // BS) for n in lens)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    o = 0
    for b, n in enumerate(lens):
        nb = -(-n // BS)
        bt[b, :nb] = perm[o:o + nb]
        o += nb
    T = sum(rows)
    q = torch.randn(T, H, D, generator=g).to(dt)
    pos = torch.cat([torch.arange(n - r, n) for n, r in zip(lens, rows)])
    qs = torch.tensor([0] + rows, dtype=torch.int32).cumsum(0).int()
    tk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)) if talk else None
    gt = torch.randn(T, H * Dv + 4, generator=g).to(dt)[:, 2:2 + H * Dv] if gate else None
    out = torch.zeros(T, H * Dv + 8, dtype=dt, device=dev)
    mv = lambda t: None if t is None else t.to(dev)  # noqa: E731
    ws = sops.talking_attention_workspace(T, H, G, Dv, parts, dev) if parts > 1 else None
    sops.talking_attention(out[:, :H * Dv], mv(q), mv(kc), mv(vc), mv(bt),
                           torch.tensor(lens, dtype=torch.int32, device=dev), mv(qs), mv(pos),
                           mv(tk), mv(gt), 0.3, ws, parts)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,Dv", [(6, 2, 80, 96), (4, 1, 20, 36), (8, 8, 32, 64),
                                      (16, 4, 128, 128), (5, 5, 8, 200)])
def test_talking_attention_kernel(dtype, H, G, D, Dv):
    want = _attention_case(dtype, H, G, D, Dv, "cpu", gen(3), 1)
    for parts in (1, 2, 5):
        close(_attention_case(dtype, H, G, D, Dv, "cuda", gen(3), parts), want, dtype)
    want = _attention_case(dtype, H, G, D, Dv, "cpu", gen(4), 1, talk=False, gate=False)
    close(_attention_case(dtype, H, G, D, Dv, "cuda", gen(4), 3, talk=False, gate=False), want,
          dtype)


def test_talking_attention_decode_rows_without_sequence_starts():
    # one row per sequence (a decode step), a padding sequence among them
    g = gen(11)
    H, G, D, Dv, BS = 4, 2, 32, 16, 32
    lens = torch.tensor([40, 0, 200, 1], dtype=torch.int32)
    NB = 12
    kc, vc = torch.randn(NB, G, BS, D, generator=g), torch.randn(NB, G, BS // 8, Dv, 8, generator=g)
    bt = torch.tensor([[0, 1, 0, 0, 0, 0, 0], [0] * 7, [2, 3, 4, 5, 6, 7, 8], [9, 0, 0, 0, 0, 0, 0]],
                      dtype=torch.int32)
    q = torch.randn(4, H, D, generator=g)
    pos = (lens - 1).clamp(min=0).long()
    tk, gt = torch.randn(H, H, generator=g), torch.randn(4, H * Dv, generator=g)
    outs = []
    for dev, parts in (("cpu", 1), ("cuda", 1), ("cuda", 4)):
        out = torch.full((4, H * Dv), 7.0, device=dev)
        ws = sops.talking_attention_workspace(4, H, G, Dv, parts, dev) if parts > 1 else None
        sops.talking_attention(out, q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), lens.to(dev),
                               None, pos.to(dev), tk.to(dev), gt.to(dev), 0.2, ws, parts)
        outs.append(out)
    assert (outs[0][1] == 7.0).all() and (outs[1][1] == 7.0).all() and (outs[2][1] == 7.0).all()
    close(outs[1], outs[0], "float32")
    close(outs[2], outs[0], "float32")


def _tile_map(q_start, first_seq, tile_rows):
    """The scheduler's prefill tile map: (sequence, first chunk row) per tile of tile_rows."""
    seqs, rows = [], []
    for b in range(first_seq, len(q_start) - 1):
        for r in range(0, q_start[b + 1] - q_start[b], tile_rows):
            seqs.append(b)
            rows.append(r)
    return (torch.tensor(seqs, dtype=torch.int32, device="cuda"),
            torch.tensor(rows, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("H,G,D,Dv,BS", [(6, 2, 80, 96, 32), (4, 1, 16, 32, 16), (8, 8, 32, 64, 32),
                                         (16, 4, 128, 128, 32), (2, 2, 48, 160, 16),
                                         (32, 8, 64, 128, 32)])
def test_talking_attention_matrix_core_kernel(H, G, D, Dv, BS):
    """Prompt chunks on the matrix cores against the op on the CPU: chunks that start at 0 and
    in the middle of a sequence, tiles cut by a chunk's end, single rows that lead the step."""
    g = gen(H + D)
    lens = [9, 301, 140, 33, 700]               # cached keys per sequence after this step
    rows = [1, 1, 140, 20, 333]                 # two single-token sequences lead
    NB = sum(-(-n // BS) for n in lens) + 2
    kc = torch.randn(NB, G, BS, D, generator=g).bfloat16()
    vc = torch.randn(NB, G, BS // 8, Dv, 8, generator=g).bfloat16()
    perm = torch.randperm(NB, generator=g).int()
    bt = torch.zeros(len(lens), max(-(-n // BS) for n in lens), dtype=torch.int32)
    o = 0
    for b, n in enumerate(lens):
        nb = -(-n // BS)
        bt[b, :nb] = perm[o:o + nb]
        o += nb
    T = sum(rows)
    q = (0.5 * torch.randn(T, H, D, generator=g)).bfloat16()
    pos = torch.cat([torch.arange(n - r, n) for n, r in zip(lens, rows)])
    qs = torch.tensor([0] + rows, dtype=torch.int32).cumsum(0).int()
    tk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    gt = torch.randn(T, H * Dv, generator=g).bfloat16()
    sl = torch.tensor(lens, dtype=torch.int32)
    want = torch.zeros(T, H * Dv, dtype=torch.bfloat16)
    sops.talking_attention(want, q, kc, vc, bt, sl, qs, pos, tk, gt, 0.3)
    for tile_rows in (128, 32):
        ts, tr = _tile_map(qs.tolist(), 2, tile_rows)
        out = torch.zeros(T, H * Dv + 8, dtype=torch.bfloat16, device="cuda")
        sops.talking_attention_prefill(out[:, :H * Dv], q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(),
                                       sl.cuda(), qs.cuda(), pos.cuda(), ts, tr, tile_rows,
                                       tk.cuda(), gt.cuda(), 0.3, first_seq=2)
        close(out[:, :H * Dv], want, "bfloat16")
        assert (out[:, H * Dv:] == 0).all()


@pytest.mark.parametrize("H,G,D,Dv,BS", [(6, 2, 80, 96, 32), (4, 1, 16, 32, 16), (8, 8, 32, 64, 32),
                                         (16, 4, 128, 128, 32), (2, 2, 48, 160, 16),
                                         (32, 8, 64, 128, 32)])
def test_talking_attention_matrix_core_decode_kernel(H, G, D, Dv, BS):
    """One query per sequence on the matrix cores (heads as columns), several partition counts,
    sequences of 1 key, of a few and of many steps, a padding row."""
    g = gen(H * D + 1)
    lens = [1, 700, 0, 129, 128, 333, 64]
    NB = sum(-(-n // BS) for n in lens) + 2
    kc = torch.randn(NB, G, BS, D, generator=g).bfloat16()
    vc = torch.randn(NB, G, BS // 8, Dv, 8, generator=g).bfloat16()
    perm = torch.randperm(NB, generator=g).int()
    bt = torch.zeros(len(lens), max(-(-n // BS) for n in lens), dtype=torch.int32)
    o = 0
    for b, n in enumerate(lens):
        nb = -(-n // BS)
        bt[b, :nb] = perm[o:o + nb]
        o += nb
    T = len(lens)
    q = (0.5 * torch.randn(T, H, D, generator=g)).bfloat16()
    sl = torch.tensor(lens, dtype=torch.int32)
    pos = (sl - 1).clamp(min=0).long()
    tk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    gt = torch.randn(T, H * Dv, generator=g).bfloat16()
    want = torch.full((T, H * Dv), 3.0, dtype=torch.bfloat16)
    sops.talking_attention(want, q, kc, vc, bt, sl, None, pos, tk, gt, 0.3)
    for parts in (1, 3, 8):
        out = torch.full((T, H * Dv), 3.0, dtype=torch.bfloat16, device="cuda")
        ws = sops.talking_attention_workspace(T, H, G, Dv, parts, "cuda")
        sops.talking_attention_decode(out, q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), sl.cuda(),
                                      pos.cuda(), tk.cuda(), gt.cuda(), 0.3, ws, parts)
        close(out, want, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("E,top,F_,d", [(12, 3, 80, 160), (5, 5, 7, 40), (8, 1, 64, 256), (3, 2, 8, 24)])
def test_routing_and_gated_activation_kernels(dtype, E, top, F_, d):
    g, dt = gen(E * d), DT[dtype]
    T = 13
    h = torch.randn(T, d, generator=g).to(dt)
    router, bias = torch.randn(E, d, generator=g), torch.randn(E, generator=g)
    ids_c, w_c = sops.route_topk(h, router, bias, top)
    ids_g, w_g = sops.route_topk(h.cuda(), router.cuda(), bias.cuda(), top)
    assert (ids_g.cpu() == ids_c).all()
    close(w_g, w_c, "float32")
    ids_n, w_n = sops.route_topk(h.cuda(), router.cuda(), None, top)
    want = sops.route_topk(h, router, None, top)
    assert (ids_n.cpu() == want[0]).all()
    gu = torch.randn(T, E * 2 * F_ + 8, generator=g).to(dt)[:, :E * 2 * F_]
    a_c = torch.zeros(T, E * F_, dtype=dt)
    a_g = torch.zeros(T, E * F_, dtype=dt, device="cuda")
    sops.swiglu_routed(gu, ids_c, w_c, E, a_c)
    sops.swiglu_routed(gu.cuda(), ids_g, w_g, E, a_g)
    close(a_g, a_c, dtype)
    s_c, s_g = torch.zeros(T, E * F_, dtype=dt), torch.zeros(T, E * F_, dtype=dt, device="cuda")
    sops.swiglu(gu[:, :2 * E * F_], s_c)
    sops.swiglu(gu.cuda()[:, :2 * E * F_], s_g)
    close(s_g, s_c, dtype)


# ------------------------------------------------------------------ the engine on the GPU
@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=2)
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    return cfg, W, write_model(tmp_path_factory.mktemp("sazepel_gpu"), cfg, W), reqs, want


def check(got, want, dtype):
    for n in got:
        e = rel_err(got[n], want[n])
        if dtype == "bfloat16":
            # widths of a few dozen make bf16 rounding large against the logits and a close
            # routing choice can flip: the bulk of the positions must be close
            assert e.median().item() < 0.15, f"{n}: median {e.median():.2e}, worst {e.max():.2e}"
        else:
            assert e.max().item() < TOL[dtype], f"{n}: position {int(e.argmax())} off by {e.max():.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("eager", [False, True])
def test_schedules(model, dtype, eager):
    _, _, path, reqs, want = model
    eng = engine(path, dtype=dtype, device="cuda", eager=eager)
    assert eager or eng.runner.graphs, "decode hipGraphs were not captured"
    one = {"a": reqs["a"]}
    check(replay(eng, reqs, [[(n, len(t))] for n, t in reqs.items()]), want, dtype)
    check(replay(eng, one, [[("a", 40)]] + [[("a", 1)]] * 35), want, dtype)
    check(replay(eng, one, [[("a", s)] for s in [3, 2, 7, 2, 19, 2, 5, 33, 2]]), want, dtype)
    sched = [[("a", 30), ("b", 2), ("c", 1)],
             [("a", 1), ("b", 20), ("c", 22), ("d", 1)],
             [("a", 1), ("b", 1), ("e", 33)],
             [("a", 1), ("b", 1)],
             [("b", 17), ("e", 1)],
             [("a", 42), ("e", 30)]]
    check(replay(eng, reqs, sched), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pool_is_used_again(model, dtype):
    _, _, path, reqs, want = model
    eng = engine(path, dtype=dtype, max_tokens=160, max_seqs=2, device="cuda")
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    for _ in range(2):  # graphs replayed again over pages and slots that changed owners
        check(replay(eng, many, sched), {k: want[k[0]] for k in many}, dtype)
    assert eng.sched.num_free_blocks() == 5 and eng.sched.num_free_tail_slots == 2


def test_long_decode_through_graphs(tmp_path):
    """Decoding far past the first key partition of the split attention, the retention state
    carried by the captured graphs."""
    cfg = oracle.make_config(width=64, vocab=37, logit_scale=0.8, layers=[
        oracle.make_layer(oracle.ret_spec(2, 16, 16, rot_dims=8, decay=[0.999, 0.97]),
                          att=(4, 2, 16, 8, 0.25), moe=(6, 2, 16)),
        oracle.make_layer(oracle.ret_spec(4, 8, 12, decay=[1.0, 0.995, 0.9, 0.6]))])
    W = oracle.random_weights(cfg, seed=5)
    toks = tokens(700, 37, 6)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=704, device="cuda")
    assert eng.runner.graphs
    check(replay(eng, {"a": toks}, [[("a", 500)]] + [[("a", 1)]] * 200), want, "float32")


def test_large_prompt_takes_the_sorted_expert_path(tmp_path):
    """A prompt portion over the small-batch threshold of the routed feed-forward."""
    from aws_k8s_ansible_provisioner_amd.models import sazepel

    cfg = oracle.make_config(width=32, vocab=37, layers=[
        oracle.make_layer(oracle.ret_spec(2, 8, 8, rot_dims=4), att=(2, 1, 8, 8, 0.4),
                          moe=(5, 2, 16))])
    W = oracle.random_weights(cfg, seed=6)
    toks = tokens(sazepel.MOE_DENSE_ROWS + 70, 37, 7)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=512, device="cuda")
    n = sazepel.MOE_DENSE_ROWS + 40
    check(replay(eng, {"a": toks}, [[("a", n)], [("a", 30)]]), want, "float32")


def test_greedy_generation(model):
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    cfg, W, path, _, _ = model
    eng = LLMEngine(EngineConfig(model=path, load_format="safetensors", weights_path=path,
                                 dtype="float32", max_model_len=128, max_num_seqs=4,
                                 max_num_batched_tokens=24, num_gpu_blocks=16, device="cuda",
                                 gc_freeze=False), log=lambda *a: None)
    assert eng.runner.graphs
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (30, 3, 17, 9)]
    outs = eng.generate(None, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
                        prompt_ids=prompts)
    assert [len(o.output_ids) for o in outs] == [12] * 4
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W, p + o.output_ids)
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name, dtype):
    cfg = oracle.make_config(**dict({"vocab": 31}, **OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W), dtype=dtype, device="cuda")
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want, dtype)


def test_registry_model_generates_with_sampling():
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-sazepel", dtype="bfloat16", max_model_len=256,
                                 max_num_seqs=4, max_num_batched_tokens=64, num_gpu_blocks=32,
                                 device="cuda", gc_freeze=False), log=lambda *a: None)
    outs = eng.generate(None, SamplingParams(max_tokens=20, temperature=0.8, top_p=0.9, seed=3,
                                             ignore_eos=True),
                        prompt_ids=[[5, 6, 7], [9] * 70, [1, 2], [3] * 33, [4] * 5])
    assert [len(o.output_ids) for o in outs] == [20] * 5


def test_large_batches_take_the_grouped_expert_gemms():
    """With the core library loaded, prompt-sized batches of a routed layer run the framework's
    grouped expert GEMMs (no host round trip); same result as the oracle's experts."""
    from aws_k8s_ansible_provisioner_amd import ops
    from aws_k8s_ansible_provisioner_amd.models.config import sazepel_config
    from aws_k8s_ansible_provisioner_amd.models.sazepel import SazepelLM

    ops.load_native(required=True)
    cfg = oracle.make_config(width=128, vocab=37, layers=[
        oracle.make_layer(oracle.ret_spec(2, 16, 16), moe=(6, 2, 64))])
    W = oracle.random_weights(cfg, seed=3)
    m = SazepelLM(sazepel_config("g", cfg), "cuda", dtype=torch.bfloat16, max_model_len=64)
    m.load_state_dict(W)
    h = torch.randn(300, 128, generator=gen(5)).bfloat16()
    assert m._grouped_ok(h.cuda(), 64)
    got = m._routed(m.layers[0], h.cuda(), small=False)
    want = oracle.routed_experts(h.double(), oracle.sub(W, "l0.mlp."), cfg["layers"][0]["mlp"])
    torch.testing.assert_close(got.double().cpu(), want, rtol=3e-2, atol=3e-2)
    dense = m._routed(m.layers[0], h.cuda(), small=True)
    torch.testing.assert_close(dense.double().cpu(), want, rtol=3e-2, atol=3e-2)
