"""Mudepel on the HIP kernels: every new kernel against the PyTorch version of the same op (fp32
and bf16 storage, odd sizes), then the engine -- mixed steps, hipGraph decode, a small page and
slot pool -- against the float64 oracle (tests/mudepel_oracle.py), and greedy generation
through LLMEngine.generate."""
import pytest
import torch

import mudepel_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-4, "bfloat16": 0.3}


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close(a, b, dtype, scale=1.0):
    tol = 3e-5 if dtype == "float32" else 2e-2
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=tol, atol=tol * scale)


def both(fn):
    """fn(device) on the CPU and on the GPU; returns the two results."""
    return fn("cpu"), fn("cuda")


# ------------------------------------------------------------------ kernels against their ops
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("S,d", [(1, 24), (3, 200), (4, 2048), (8, 514), (2, 8192)])
def test_hyper_step_kernel(dtype, S, d):
    g, dt = gen(S * d), DT[dtype]
    T = 5
    xs0 = torch.randn(T, S, d, generator=g)
    ya = torch.randn(T, d + 8, generator=g).to(dt)[:, :d]
    yb = torch.randn(T, d, generator=g)
    bias = torch.randn(d, generator=g)
    mix = torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)
    wo, wi = torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = 1 + 0.3 * torch.randn(d, generator=g)
    e = torch.randn(T, d, generator=g)
    for a, b, bb, fresh in ((ya, None, None, None), (ya, yb, bias, None), (None, yb, None, None),
                            (None, None, None, e)):
        def run(dev):
            mv = lambda t: None if t is None else t.to(dev)  # noqa: E731
            xs = xs0.clone().to(dev)
            o = torch.zeros(T, d, dtype=dt, device=dev)
            sops.hyper_step(xs, mv(a), mv(b), mv(bb), mv(mix), mv(wo), mv(wi), mv(nw), 1e-6, o,
                            fresh=mv(fresh))
            return xs, o
        c, n = both(run)
        close(n[0], c[0], "float32", scale=4.0)
        close(n[1], c[1], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_softcap_and_gated_act_kernels(dtype):
    g, dt = gen(3), DT[dtype]
    x = (20 * torch.randn(7, 333, generator=g)).to(dt)
    c, n = both(lambda dev: sops.softcap_(x.clone().to(dev), 12.5))
    close(n, c, dtype, scale=12.5)
    E, F_, T = 5, 24, 9
    gu = (2 * torch.randn(T, E * 2 * F_ + 6, generator=g)).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:2] for _ in range(T)]).int()
    w = torch.rand(T, 2, generator=g)
    for act in ("silu", "gelu_tanh"):
        def run(dev):
            o = torch.zeros(T, E * F_ + 4, dtype=dt, device=dev)
            sops.gated_act(gu.to(dev)[:, :E * 2 * F_], o[:, :E * F_], act, ids.to(dev), w.to(dev), E)
            o2 = torch.zeros(T, E * F_, dtype=dt, device=dev)
            sops.gated_act(gu.to(dev)[:, :E * 2 * F_], o2, act, None, None, E)
            return o, o2
        c, n = both(run)
        close(n[0], c[0], dtype, scale=4.0)
        close(n[1], c[1], dtype, scale=4.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,groups", [(48, 3), (512, 1), (640, 5), (4096, 8)])
def test_gate_group_norm_kernel(dtype, n, groups):
    g, dt = gen(n), DT[dtype]
    T = 6
    y = 3 * torch.randn(T, n, generator=g)
    gate = torch.randn(T, n + 16, generator=g).to(dt)
    w = 1 + 0.2 * torch.randn(n, generator=g)

    def run(dev):
        o = torch.zeros(T, n, dtype=dt, device=dev)
        sops.gate_group_norm(o, y.to(dev), gate.to(dev)[:, 8:8 + n], w.to(dev), groups, 1e-5)
        return o
    c, nn = both(run)
    close(nn, c, dtype, scale=3.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("E,top,groups,keep,d", [(16, 4, 4, 2, 160), (6, 2, 3, 2, 40),
                                                 (8, 8, 1, 1, 64), (12, 4, 4, 2, 1024),
                                                 (5, 1, 5, 3, 33), (64, 6, 8, 4, 256)])
def test_route_sigmoid_kernel(dtype, E, top, groups, keep, d):
    g, dt = gen(E * d), DT[dtype]
    T = 40
    h = torch.randn(T, d, generator=g).to(dt)
    router = (torch.randn(E, d, generator=g) * 2 * d ** -0.5)
    (ci, cw), (ni, nw) = both(lambda dev: sops.route_sigmoid(h.to(dev), router.to(dev), top, groups,
                                                            keep, 2))
    # a choice may differ only where two scores are within rounding of each other
    same = (ci == ni.cpu()).all(dim=1)
    assert same.float().mean() > 0.9
    close(nw[same], cw[same], "float32")


def _conv_scan_case(dtype, H, V, N, G, taps, dev, steps, g, slots=3):
    """Run `steps` (each a list of (slot, first position, rows)) through convolution, scan and
    gate; returns the outputs of all steps and the final states."""
    dt = DT[dtype]
    inner, C = H * V, H * V + 2 * G * N
    rows = 2 * inner + 2 * G * N + H + 5
    cw = (0.5 * torch.randn(C, taps, generator=g)).to(dev)
    cb = (0.2 * torch.randn(C, generator=g)).to(dev)
    dtb = (torch.randn(H, generator=g) - 1).to(dev)
    alog = (0.7 * torch.randn(H, generator=g) - 0.5).to(dev)
    dsk = (1 + 0.3 * torch.randn(H, generator=g)).to(dev)
    cst = torch.full((slots, max(1, taps - 1), C), 7.0, dtype=dt, device=dev)   # stale contents
    st = torch.full((slots, H, N, V), 7.0, device=dev)
    outs = []
    for step in steps:
        T = sum(n for _, _, n in step)
        proj = torch.randn(T, rows, generator=g).to(dt).to(dev)
        slot = torch.cat([torch.full((n,), s, dtype=torch.int32) for s, _, n in step]).to(dev)
        pos = torch.cat([torch.arange(p, p + n) for _, p, n in step]).to(dev)
        single = all(n == 1 for _, _, n in step)
        qs = None
        if not single:
            qs = torch.tensor([0] + [n for _, _, n in step]).cumsum(0).int().to(dev)
        xbc = torch.zeros(T, C, device=dev)
        sops.conv_silu(xbc, proj, inner, cw, cb, cst, slot, pos, qs)
        y = torch.zeros(T, inner, device=dev)
        sops.selective_scan(y, xbc, proj, inner + C, dtb, alog, dsk, st, slot, pos, qs, H, V, N, G)
        outs += [xbc, y]
    return outs, cst, st


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,V,N,G,taps", [(4, 32, 16, 4, 3), (3, 16, 8, 1, 2), (2, 64, 128, 2, 4),
                                          (6, 48, 20, 3, 3), (1, 128, 64, 1, 1), (8, 8, 16, 8, 5),
                                          (3, 5, 3, 1, 3), (2, 128, 256, 1, 4), (2, 64, 256, 2, 2)])
def test_conv_and_scan_kernels(dtype, H, V, N, G, taps):
    # a prompt in portions (one shorter than the taps), a mixed step, single rows, a slot used
    # again from position 0 on top of stale contents, a padding row (slot -1)
    steps = [[(0, 0, 37), (1, 0, 2)], [(1, 2, 1), (0, 37, 1)], [(0, 38, 19), (1, 3, 2), (2, 0, 1)],
             [(2, 1, 1), (-1, 0, 1), (1, 5, 1)], [(1, 0, 21)]]
    c = _conv_scan_case(dtype, H, V, N, G, taps, "cpu", steps, gen(H * V + N))
    n = _conv_scan_case(dtype, H, V, N, G, taps, "cuda", steps, gen(H * V + N))
    for i, (a, b) in enumerate(zip(c[0], n[0])):
        if i // 2 == 3:          # the padding row is left unwritten
            a, b = a[[0, 2]], b[[0, 2]]
        close(b, a, "float32", scale=8.0)
    close(n[1], c[1], dtype)
    close(n[2], c[2], "float32", scale=8.0)


def _attention_case(dtype, H, G, D, Dv, rot, window, pool, BS, dev, steps, g, sink=True):
    dt = DT[dtype]
    NB = 24
    N = H * D + G * (D + Dv) + 3
    kc = torch.zeros(NB, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(NB, G, BS // 8, Dv, 8, dtype=dt, device=dev)
    PS = sops.pool_slots(BS, pool)
    kp = torch.full((NB, G, max(PS, 1), D), 5.0, device=dev) if pool else None
    vp = torch.full((NB, G, max(PS, 1), Dv), 5.0, device=dev) if pool else None
    cs = sops.rotary_table_yarn(512, rot, 1000.0, {"factor": 4.0, "original": 64, "fast": 8.0,
                                                   "slow": 1.0}).to(dev) if rot else None
    bias = (0.3 * torch.randn(N, generator=g)).to(dev)
    # two sequences on interleaved pages in a scrambled order
    perm = torch.randperm(NB, generator=g).int()
    bt_all = torch.stack([perm[:NB // 2], perm[NB // 2:]])
    outs = []
    for step in steps:
        T = sum(n for _, _, n in step)
        proj = torch.randn(T, N, generator=g).to(dt).to(dev)
        seqs = [s for s, _, _ in step]
        pos = torch.cat([torch.arange(p, p + n) for _, p, n in step])
        sq = torch.cat([torch.full((n,), s) for s, _, n in step])
        slots = torch.where(sq >= 0, bt_all[sq.clamp(min=0), pos // BS].long() * BS + pos % BS,
                            torch.tensor(-1))
        bt = bt_all[torch.tensor(seqs).clamp(min=0)].to(dev)
        single = all(n == 1 for _, _, n in step)
        qs = None if single else torch.tensor([0] + [n for _, _, n in step]).cumsum(0).int().to(dev)
        q = torch.zeros(T, H, D, dtype=dt, device=dev)
        sops.bias_rope_cache(proj, q, kc, vc, pos.to(dev), slots.to(dev), cs, bias, H, G, D, Dv,
                             0, H * D, H * D + G * D)
        if pool:
            sops.pool_cache_blocks(kc, vc, kp, vp, pos.to(dev), slots.to(dev), bt, qs, pool)
        o = torch.zeros(T, H * Dv + 2, dtype=dt, device=dev)
        sops.pooled_window_attention(o, q, kc, vc, kp, vp, bt, qs, pos.to(dev), slots.to(dev),
                                     0.3, window, pool, sink)
        keep = (slots >= 0)
        outs += [q[keep.to(dev)], o[keep.to(dev)]]
    return outs, kc, vc


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,Dv,rot,window,pool,BS", [
    (6, 3, 64, 64, 32, 44, 12, 32), (4, 2, 32, 16, 16, 24, 8, 32), (3, 1, 20, 36, 8, 10, 3, 16),
    (8, 2, 128, 128, 64, 50, 48, 32), (2, 2, 8, 8, 0, 0, 0, 32), (4, 4, 16, 24, 16, 33, 0, 32),
    (5, 5, 12, 7, 12, 7, 20, 16), (40, 2, 16, 8, 8, 9, 4, 16), (2, 1, 24, 300, 0, 12, 6, 16)])
def test_attention_kernels(dtype, H, G, D, Dv, rot, window, pool, BS):
    # prompts in portions across pages and pooled blocks, a mixed step, single rows, a padding row
    steps = [[(0, 0, 70), (1, 0, 3)], [(1, 3, 1), (0, 70, 1)], [(0, 71, 59), (1, 4, 30)],
             [(0, 130, 1), (-1, 0, 1), (1, 34, 1)], [(1, 35, 61)], [(0, 131, 1), (1, 96, 1)]]
    for sink in (True, False):
        c = _attention_case(dtype, H, G, D, Dv, rot, window, pool, BS, "cpu", steps, gen(H * D),
                            sink)
        n = _attention_case(dtype, H, G, D, Dv, rot, window, pool, BS, "cuda", steps, gen(H * D),
                            sink)
        for a, b in zip(c[0], n[0]):
            close(b, a, dtype, scale=2.0)
        close(n[1], c[1], dtype, scale=2.0)
        close(n[2], c[2], dtype, scale=2.0)


# ------------------------------------------------------------------ the engine on the GPU
from test_mudepel import OTHER, base_config  # noqa: E402


def check(got, want, dtype, names=None):
    for n in names or got:
        e = rel_err(got[n], want[n])
        if dtype == "float32":
            assert e.max().item() < TOL[dtype], \
                f"{n}: position {int(e.argmax())} off by {e.max().item():.2e}"
        else:   # small widths: bf16 rounding is large and a close routing call flips a position
            assert e.median().item() < 0.15, f"{n}: median error {e.median().item():.2e}"


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=2)
    W64 = oracle.as_f64(W)
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    want = {n: oracle.forward(cfg, W64, t)[0] for n, t in reqs.items()}
    return cfg, W, write_model(tmp_path_factory.mktemp("mudepel_gpu"), cfg, W), reqs, want


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
    """Decoding while the window and its pooled blocks pass over decoded tokens, the states and
    convolution inputs carried by the captured graphs."""
    cfg = oracle.make_config(width=64, vocab=37, streams=2, layers=[
        oracle.ssm_layer(4, 16, 16, 2, conv=4, norm_groups=2, mlp=oracle.dense(48)),
        oracle.att_layer(4, 2, 16, 8, 0.25, window=36, pool=12, rot_dims=8,
                         mlp=oracle.routed(6, 2, 16, count=2, keep=1, shared=16))])
    W = oracle.random_weights(cfg, seed=5)
    toks = tokens(400, 37, 6)
    want = {"a": oracle.forward(cfg, oracle.as_f64(W), toks)[0]}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=416, device="cuda")
    assert eng.runner.graphs
    check(replay(eng, {"a": toks}, [[("a", 250)]] + [[("a", 1)]] * 150), want, "float32")


def test_large_prompt_takes_the_sorted_expert_path(tmp_path):
    """A prompt portion over the small-batch threshold of the routed feed-forward."""
    from aws_k8s_ansible_provisioner_amd.models import mudepel

    cfg = oracle.make_config(width=32, vocab=37, layers=[
        oracle.att_layer(2, 1, 8, 8, 0.4, window=30, pool=10, rot_dims=4,
                         mlp=oracle.routed(5, 2, 16, shared=8))])
    W = oracle.random_weights(cfg, seed=6)
    toks = tokens(mudepel.MOE_DENSE_ROWS + 70, 37, 7)
    want = {"a": oracle.forward(cfg, oracle.as_f64(W), toks)[0]}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=512, device="cuda")
    n = mudepel.MOE_DENSE_ROWS + 40
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
    W64 = oracle.as_f64(W)
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W64, p + o.output_ids)[0]
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name, dtype):
    cfg = oracle.make_config(**dict({"vocab": 31}, **OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    W64 = oracle.as_f64(W)
    want = {n: oracle.forward(cfg, W64, t)[0] for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W), dtype=dtype, device="cuda")
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want, dtype)


def test_registry_model_generates_with_sampling():
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-mudepel", dtype="bfloat16", max_model_len=256,
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
    from aws_k8s_ansible_provisioner_amd.models.config import mudepel_config
    from aws_k8s_ansible_provisioner_amd.models.mudepel import MudepelLM

    ops.load_native(required=True)
    cfg = oracle.make_config(width=128, vocab=37, layers=[
        oracle.ssm_layer(2, 16, 16, 1, mlp=oracle.routed(6, 2, 64, count=3, keep=2, shared=64))])
    W = oracle.random_weights(cfg, seed=3)
    m = MudepelLM(mudepel_config("g", cfg), "cuda", dtype=torch.bfloat16, max_model_len=64)
    m.load_state_dict(W)
    h = torch.randn(300, 128, generator=gen(5)).bfloat16()
    assert m._grouped_ok(h.cuda(), 64)
    want = oracle.moe(h.double(), oracle.as_f64(W), "l0.", cfg["layers"][0]["mlp"])
    for small in (False, True):
        ya, yb = m._feed_forward(m.layers[0], h.cuda(), small)
        got = sum(t.double().cpu() for t in (ya, yb) if t is not None)
        torch.testing.assert_close(got, want, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("H,G,D,Dv,rot,window,pool,BS", [
    (6, 3, 64, 64, 32, 44, 12, 32), (4, 2, 32, 32, 16, 24, 8, 32), (8, 2, 128, 128, 64, 100, 48, 32),
    (2, 1, 16, 256, 0, 0, 0, 16), (4, 4, 80, 64, 16, 33, 0, 8), (3, 1, 48, 32, 48, 7, 5, 16),
    (4, 1, 128, 128, 128, 200, 4, 32)])
def test_attention_matrix_core_kernel(H, G, D, Dv, rot, window, pool, BS):
    """Prompt chunks on the matrix cores against the row ops on the CPU: chunks that start in
    the middle of a sequence, tiles cut by a chunk's end, more than one tile per chunk, leading
    single rows of a mixed step, windows and pooled blocks that start inside a 32-key step."""
    g = gen(H * D + window)
    dt = torch.bfloat16
    lens = [(400, 1), (77, 1), (300, 300), (391, 150), (33, 33), (260, 129)]   # (cached, rows)
    nd = 2
    NB = sum(-(-n // BS) for n, _ in lens) + 1
    perm = torch.randperm(NB, generator=g).int()
    mb = max(-(-n // BS) for n, _ in lens)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    kc = torch.zeros(NB, G, BS, D, dtype=dt)
    vc = torch.zeros(NB, G, BS // 8, Dv, 8, dtype=dt)
    PS = sops.pool_slots(BS, pool)
    kp = torch.zeros(NB, G, max(PS, 1), D) if pool else None
    vp = torch.zeros(NB, G, max(PS, 1), Dv) if pool else None
    cs = sops.rotary_table_yarn(512, rot, 1000.0, None) if rot else None
    N = H * D + G * (D + Dv)
    o = 0
    for b, (n, _) in enumerate(lens):       # fill the cache of every sequence from position 0
        nbk = -(-n // BS)
        bt[b, :nbk] = perm[o:o + nbk]
        o += nbk
        pos = torch.arange(n)
        slots = bt[b][pos // BS].long() * BS + pos % BS
        proj = torch.randn(n, N, generator=g).to(dt)
        sops.bias_rope_cache(proj, torch.zeros(n, H, D, dtype=dt), kc, vc, pos, slots, cs, None,
                             H, G, D, Dv, 0, H * D, H * D + G * D)
        if pool:
            sops.pool_cache_blocks(kc, vc, kp, vp, pos, slots, bt[b:b + 1],
                                   torch.tensor([0, n], dtype=torch.int32), pool)
    rows = [r for _, r in lens]
    T = sum(rows)
    q = torch.randn(T, H, D, generator=g).to(dt)
    qs = torch.tensor([0] + rows).cumsum(0).int()
    pos = torch.cat([torch.arange(n - r, n) for n, r in lens])
    slots = torch.cat([bt[b][torch.arange(n - r, n) // BS].long() * BS + torch.arange(n - r, n) % BS
                       for b, (n, r) in enumerate(lens)])
    tiles = sorted((min(r - r0, 128) + n - r + r0, b, r0) for b, (n, r) in enumerate(lens)
                   if b >= nd for r0 in range(0, r, 128))
    tile_seq = torch.tensor([t[1] for t in tiles], dtype=torch.int32)
    tile_row = torch.tensor([t[2] for t in tiles], dtype=torch.int32)
    want = torch.zeros(T, H * Dv, dtype=dt)
    sops.pooled_window_attention(want, q, kc, vc, kp, vp, bt, qs, pos, slots, 0.2, window, pool, True)
    mv = lambda t: None if t is None else t.cuda()  # noqa: E731
    got = torch.zeros(T, H * Dv, dtype=dt, device="cuda")
    assert sops.pooled_mfma_ok(q.cuda(), kc.cuda(), vc.cuda())
    sops.pooled_window_attention_prefill(got, q.cuda(), kc.cuda(), vc.cuda(), mv(kp), mv(vp),
                                         bt.cuda(), qs.cuda(), pos.cuda(), slots.cuda(),
                                         tile_seq.cuda(), tile_row.cuda(), 128, 0.2, window, pool,
                                         True, first_seq=nd)
    close(got, want, "bfloat16", scale=2.0)
    # one query per sequence (the last position of each) plus a padding row, heads as columns
    last = torch.tensor([r - 1 for r in torch.tensor(rows).cumsum(0).tolist()])
    B = len(lens)
    qd = torch.cat([q[last], torch.zeros(1, H, D, dtype=dt)])
    posd = torch.cat([pos[last], torch.zeros(1, dtype=torch.long)])
    slotd = torch.cat([slots[last], torch.tensor([-1])])
    btd = torch.cat([bt, bt[:1]])
    got = torch.full((B + 1, H * Dv), 3.0, dtype=dt, device="cuda")
    sops.pooled_window_attention_decode(got, qd.cuda(), kc.cuda(), vc.cuda(), mv(kp), mv(vp),
                                        btd.cuda(), posd.cuda(), slotd.cuda(), 0.2, window, pool,
                                        True)
    close(got[:B], want[last], "bfloat16", scale=2.0)
    assert (got[B] == 3.0).all()                     # the padding row is left unwritten


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mid_size_engine_against_the_cpu_ops(tmp_path, dtype):
    """Sizes between the tiny oracle models and the benchmark's (matrix-core attention, the
    four-column scan, 16-byte paths everywhere): the engine on the GPU against the same engine
    on the CPU ops, over a mixed schedule with a looped span."""
    yarn = {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 2.0}
    cfg = oracle.make_config(width=256, vocab=301, streams=2, loop=(1, 3, 2), layers=[
        oracle.att_layer(8, 2, 64, 32, 0.11, window=96, pool=24, rot_dims=32, yarn=yarn,
                         mlp=oracle.routed(8, 2, 96, count=4, keep=2, shared=64)),
        oracle.ssm_layer(8, 32, 64, 2, conv=4, norm_groups=4, mlp=oracle.dense(320)),
        oracle.att_layer(4, 4, 32, 64, 0.2, window=50, pool=7, base=5000.0,
                         mlp=oracle.routed(6, 3, 40)),
        oracle.ssm_layer(4, 64, 16, 1, conv=3, mlp=None)])
    W = oracle.random_weights(cfg, seed=11)
    path = write_model(tmp_path, cfg, W)
    reqs = {"a": tokens(330, 301, 1), "b": tokens(140, 301, 2), "c": tokens(61, 301, 3)}
    sched = [[("a", 200), ("b", 3)], [("a", 1), ("b", 100), ("c", 60)], [("a", 1), ("b", 1)],
             [("a", 128), ("b", 36), ("c", 1)]]
    want = replay(engine(path, dtype="float32", max_tokens=640, device="cpu"), reqs, sched)
    got = replay(engine(path, dtype=dtype, max_tokens=640, device="cuda"), reqs, sched)
    for n in reqs:
        e = rel_err(got[n], want[n])
        if dtype == "float32":
            assert e.max().item() < 1e-4, f"{n}: position {int(e.argmax())} off by {e.max().item():.2e}"
        else:
            assert e.median().item() < 0.05 and e.max().item() < 0.5, (n, e.median().item(),
                                                                       e.max().item())
