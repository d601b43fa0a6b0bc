"""Ops of models that keep an fp32 residual stream (``_C_stream.so``, csrc/stream/).

Same dispatch rule as the rest of ``ops``: GPU tensors run the hand-written HIP kernel (and
raise if the library is missing), CPU tensors a plain PyTorch version of the same op.  The
kernels are templated on the activation type (bf16 or fp32) and take every size at run time
(any head size, head count and GQA ratio), so a model's weights and KV cache may be bf16 or
fp32; norms, rotary angles, attention scores and weights and the residual sum are fp32 in both.

KV cache layout of these ops: K [num_blocks, G, block_size, D] (token-major rows) and
V [num_blocks, G, block_size / 8, D, 8] (groups of 8 tokens, dimension-major inside a group: the
8 keys a matrix-core operand contracts over, or a decode lane accumulates, are one 16-byte load).
"""
from __future__ import annotations

import os
from typing import Optional

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB = os.path.join(_PKG, "_C_stream.so")
_loaded = False
_load_error: Optional[str] = None


def load_native(required: bool = False) -> bool:
    """Load ``_C_stream.so`` (torch.ops.akap_stream), building it on first use."""
    global _loaded, _load_error
    if _loaded:
        return True
    from .. import build_ext

    try:
        if os.path.exists(build_ext.STREAM_SRC):
            have = build_ext.library_hash(_LIB, "akap_stream_build_hash")
            if have != build_ext.stream_tree_hash():
                if os.environ.get("AKAP_ALLOW_STALE_NATIVE") == "1" and have:
                    pass
                else:
                    build_ext.build_stream()
        torch.ops.load_library(_LIB)
        _loaded = True
    except Exception as e:  # pragma: no cover - depends on the box
        _load_error = repr(e)
    if required and not _loaded:
        raise RuntimeError("stream HIP kernels unavailable: " + str(_load_error))
    return _loaded


def _native(t: torch.Tensor) -> bool:
    if t.is_cuda:
        load_native(required=True)
        return True
    return False


# ----------------------------------------------------------------------------- embedding, norms
def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t] = table[ids[t]] * scale as fp32 (the residual stream)."""
    if out is None:
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
    if _native(table):
        torch.ops.akap_stream.embed_scaled(out, ids, table, float(scale))
        return out
    out.copy_(table[ids.long()].float() * scale)
    return out


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def stream_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype: torch.dtype,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of the fp32 stream x [T, d] with fp32 weights w, result in out_dtype."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if _native(x):
        torch.ops.akap_stream.add_norm(out, x, None, 0.0, w, float(eps))
        return out
    out.copy_((_rms(x.float(), eps) * w.float()).to(out.dtype))
    return out


def stream_add_norm(x: torch.Tensor, y: torch.Tensor, mult: float, w: torch.Tensor, eps: float,
                    out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
                    bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += mult * (y + bias) in place (fp32 sum), then the RMS norm of the new x as out_dtype:
    the residual update of one layer fused with the norm that feeds the next.  bias [d] (y's
    dtype): the bias of the projection that produced y, when its GEMM has no bias epilogue."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if _native(x):
        torch.ops.akap_stream.add_norm(out, x, y, float(mult), w, float(eps), bias)
        return out
    x.add_((y.float() + (bias.float() if bias is not None else 0.0)) * mult)
    out.copy_((_rms(x, eps) * w.float()).to(out.dtype))
    return out


def relu2(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = relu(x)^2; x and out are [T, F] views that may be column slices of wider rows."""
    if _native(x):
        torch.ops.akap_stream.relu2(out, x)
        return out
    r = torch.relu(x.float())
    out.copy_((r * r).to(out.dtype))
    return out


# ----------------------------------------------------------------------------- rotary, cache
def rotary_table(max_pos: int, dims: int, base: float, scaling: Optional[dict] = None,
                 device=None) -> torch.Tensor:
    """fp32 [max_pos, dims] = [cos | sin] of angle p * f_i, f_i = base^(-2i/dims), with the
    wavelength rule of `scaling` = {factor, low, high, original}: frequencies whose wavelength
    is under original/high are kept, over original/low divided by factor, and blended linearly
    (in original/wavelength) between.  Angles are formed in fp64 and rounded once."""
    from . import reference as ref

    sc = None
    if scaling:
        sc = {"rope_type": "llama3", "factor": float(scaling["factor"]),
              "low_freq_factor": float(scaling["low"]), "high_freq_factor": float(scaling["high"]),
              "original_max_position_embeddings": scaling["original"]}
    return ref.rope_cos_sin(max_pos, dims, base, sc, device=device)


def proj_norm_rope_cache(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                         v_cache: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                         cos_sin: Optional[torch.Tensor], q_w: torch.Tensor, k_w: torch.Tensor,
                         H: int, G: int, D: int, q_off: int, k_off: int, eps: float,
                         q_b: Optional[torch.Tensor] = None,
                         k_b: Optional[torch.Tensor] = None) -> None:
    """Per token t of the fused projection proj [T, N]: q = proj[t, q_off : q_off + H D] and
    k = proj[t, k_off : k_off + G D] are each RMS-normalised over their WHOLE length (one
    mean over all heads) with weights q_w / k_w, then rotated per head on the first
    cos_sin.shape[1] dimensions, interleaved pairs (2i, 2i+1), by the angle row of
    positions[t].  q goes to q_out [T, H, D]; k to k_cache at slots[t]; the raw k (before norm
    and rotation) to v_cache at the same slot: the values are the keys' projection.  Slot -1
    writes nothing.  k_cache [NB, G, BS, D], v_cache [NB, G, BS/8, D, 8].  q_b / k_b (proj's
    dtype): the projection's biases, added to the slices first when its GEMM did not."""
    if _native(proj):
        torch.ops.akap_stream.proj_norm_rope_cache(proj, q_out, k_cache, v_cache, positions, slots,
                                                   cos_sin, q_w, k_w, H, G, D, q_off, k_off,
                                                   float(eps), q_b, k_b)
        return
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * D].float()
    k = proj[:, k_off:k_off + G * D].float()
    if q_b is not None:
        q = q + q_b.float()
    if k_b is not None:
        k = k + k_b.float()
    qn = (_rms(q, eps) * q_w.float()).view(T, H, D)
    kn = (_rms(k, eps) * k_w.float()).view(T, G, D)
    if cos_sin is not None:
        rd = cos_sin.shape[1]
        cs = cos_sin[positions.long()]
        c, s = cs[:, None, :rd // 2], cs[:, None, rd // 2:]

        def rot(x):
            u, v = x[..., 0:rd:2], x[..., 1:rd:2]
            o = x.clone()
            o[..., 0:rd:2] = u * c - v * s
            o[..., 1:rd:2] = v * c + u * s
            return o

        qn, kn = rot(qn), rot(kn)
    q_out.copy_(qn.to(q_out.dtype))
    BS = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // BS, :, sl % BS] = kn[ok].to(k_cache.dtype)
    v_cache[sl // BS, :, (sl % BS) // 8, :, sl % 8] = k.view(T, G, D)[ok].to(v_cache.dtype)


def v_tokens(v_cache: torch.Tensor) -> torch.Tensor:
    """The V cache [NB, G, BS/8, D, 8] as token-major rows [NB, G, BS, D] (a copy)."""
    NB, G, NG, D, _ = v_cache.shape
    return v_cache.permute(0, 1, 2, 4, 3).reshape(NB, G, NG * 8, D)


def v_from_tokens(v: torch.Tensor) -> torch.Tensor:
    """Token-major values [NB, G, BS, D] in the V cache layout [NB, G, BS/8, D, 8]."""
    NB, G, BS, D = v.shape
    return v.view(NB, G, BS // 8, 8, D).permute(0, 1, 2, 4, 3).contiguous()


# ----------------------------------------------------------------------------- attention
def _attend_rows(out, q, k_cache, v_cache, bt_row, kv_len: int, pos0: int, rows: slice,
                 gate, sink, scale: float, chunk: int, window: int) -> None:
    """CPU: the queries `rows` of one sequence (positions pos0 ...) against its cached keys."""
    n = rows.stop - rows.start
    H, D = q.shape[1], q.shape[2]
    G, BS = k_cache.shape[1], k_cache.shape[2]
    nb = -(-kv_len // BS)
    blocks = bt_row[:nb].long()
    K = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :kv_len].float()
    V = v_tokens(v_cache[blocks]).permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :kv_len].float()
    i = torch.arange(pos0, pos0 + n)[:, None]
    j = torch.arange(kv_len)[None, :]
    ok = j <= i
    if chunk > 0:
        ok &= (i // chunk) == (j // chunk)
    if window > 0:
        ok &= j > i - window
    qf = q[rows].float()
    rep = H // G
    for h in range(H):
        s = (qf[:, h] @ K[h // rep].T) * scale
        s = s.masked_fill(~ok, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].float())
        e = torch.exp(s - m)
        den = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h].float() - m)
        o = (e / den) @ V[h // rep]
        if gate is not None:
            o = o * torch.sigmoid(gate[rows, h].float())[:, None]
        out[rows, h * D:(h + 1) * D] = o.to(out.dtype)


def sink_attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, block_tables: torch.Tensor,
                           seq_lens: torch.Tensor, q_start: torch.Tensor, tile_seq: torch.Tensor,
                           tile_row: torch.Tensor, tile_rows: int, gate: Optional[torch.Tensor],
                           sink: Optional[torch.Tensor], scale: float, chunk: int = 0,
                           window: int = 0, first_seq: int = 0) -> torch.Tensor:
    """Paged causal attention of prompt chunks.  Sequence b's chunk is rows
    [q_start[b], q_start[b+1]) of q [T, H, D]; its keys are positions [0, seq_lens[b]) of its
    block-table row, the chunk's tokens being the last ones.  A query at position i sees key
    j <= i, and only if floor(i / chunk) == floor(j / chunk) (chunk > 0; chunks count from
    position 0 of the sequence) and j > i - window (window > 0).  sink [H] (fp32): exp(sink_h)
    is added to the softmax denominator (no key, no value, unscaled).  gate [T, H] (a column
    slice of the projection): head h's output is multiplied by sigmoid(gate[t, h]).  Scores,
    softmax and the gate are fp32.  out [T, >= H D] (rows may be wider: a slice of the buffer
    the output projection reads).  The tile map (tile_seq, tile_row: a sequence and the first
    chunk row of a tile of tile_rows tokens) drives the GPU grid; sequences before first_seq
    (the decode rows of a mixed step) are not in it."""
    if _native(q):
        torch.ops.akap_stream.sink_attention_prefill(out, q, k_cache, v_cache, block_tables,
                                                     seq_lens, q_start, tile_seq, tile_row,
                                                     tile_rows, gate, sink, float(scale), chunk,
                                                     window)
        return out
    B = seq_lens.numel()
    for b in range(first_seq, B):
        r0, r1 = int(q_start[b]), int(q_start[b + 1])
        if r1 > r0:
            kv = int(seq_lens[b])
            _attend_rows(out, q, k_cache, v_cache, block_tables[b], kv, kv - (r1 - r0),
                         slice(r0, r1), gate, sink, scale, chunk, window)
    return out


# fewest keys worth a decode partition of their own
DECODE_PART = 128


def decode_workspace(max_seqs: int, max_heads: int, max_dim: int, max_parts: int, device):
    """Partial softmax state of the split decode kernel: (max, sum) and the unnormalised
    output per (sequence, head, partition), fp32."""
    n = max(1, max_seqs * max_heads * max_parts)
    return (torch.empty(n * 2, dtype=torch.float32, device=device),
            torch.empty(n * max_dim, dtype=torch.float32, device=device))


def sink_attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                          v_cache: torch.Tensor, block_tables: torch.Tensor,
                          seq_lens: torch.Tensor, gate: Optional[torch.Tensor],
                          sink: Optional[torch.Tensor], scale: float, chunk: int = 0,
                          window: int = 0, workspace=None, num_parts: int = 1) -> torch.Tensor:
    """One query per sequence, at position seq_lens[b] - 1 (seq_lens 0: a padding row, left
    unwritten); same mask, sink and gate as sink_attention_prefill.  num_parts > 1 (GPU): the
    visible key range is cut into num_parts equal partitions (whole 32- or 64-key pieces), one
    workgroup each, merged by a second launch (workspace from decode_workspace)."""
    if _native(q):
        ws_ml, ws_o = workspace if (workspace is not None and num_parts > 1) else (None, None)
        torch.ops.akap_stream.sink_attention_decode(out, q, k_cache, v_cache, block_tables,
                                                    seq_lens, gate, sink, float(scale), chunk,
                                                    window, ws_ml, ws_o, num_parts)
        return out
    for b in range(seq_lens.numel()):
        kv = int(seq_lens[b])
        if kv > 0:
            _attend_rows(out, q, k_cache, v_cache, block_tables[b], kv, kv - 1, slice(b, b + 1),
                         gate, sink, scale, chunk, window)
    return out


# ----------------------------------------------------------------------------- grouped norms
def _group_rms(x: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    T, d = x.shape
    return _rms(x.view(T, groups, d // groups), eps).view(T, d)


def stream_add_group_norm(x: torch.Tensor, y: Optional[torch.Tensor], y2: Optional[torch.Tensor],
                          bias: Optional[torch.Tensor], w1: torch.Tensor,
                          w2: Optional[torch.Tensor], groups: int, eps: float,
                          out1: torch.Tensor, out2: Optional[torch.Tensor] = None,
                          shift: Optional[tuple] = None) -> None:
    """x += y + bias + y2 in place (fp32 stream; y [T, d] and bias [d] in the activation type,
    y2 [T, d] fp32; each may be None), then the RMS norm of the new x in `groups` equal
    consecutive parts (each divided by its own root mean square), written twice: out1 with the
    weights w1 and out2 with w2 (None: one output).  One pass over the row serves the residual
    update and both norms of a layer whose mixer and feed-forward read differently-weighted
    norms of the same stream.  shift = (mu, state, seq_slot, positions): out1 additionally goes
    through token_shift(single=True) inside the same kernel (batches whose every row is a
    sequence of its own: decode steps)."""
    if _native(x):
        torch.ops.akap_stream.add_group_norm(out1, out2, x, y, y2, bias, w1, w2, int(groups),
                                             float(eps), *(shift or (None, None, None, None)))
        return
    if y is not None:
        x.add_(y.float())
    if bias is not None:
        x.add_(bias.float())
    if y2 is not None:
        x.add_(y2)
    n = _group_rms(x, groups, eps)
    if shift is None:
        out1.copy_((n * w1.float()).to(out1.dtype))
    else:
        mu, state, seq_slot, positions = shift
        token_shift((n * w1.float()).to(out1.dtype), mu, state, seq_slot, positions, out1,
                    single=True)
    if out2 is not None:
        out2.copy_((n * w2.float()).to(out2.dtype))


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, seq_slot: torch.Tensor,
                positions: torch.Tensor, out: torch.Tensor, single: bool = False) -> None:
    """out[t] = h[t] + (prev_t - h[t]) * mu, where prev_t is the UNSHIFTED row of the token
    before t in its sequence: row t-1 when that row is the same sequence's previous position
    (equal seq_slot, positions[t-1] + 1 == positions[t]), zeros at position 0, else what an
    earlier step left in state[seq_slot[t]].  Then state[seq_slot[t]] = h[t] for the last row of
    every sequence in the batch.  state [slots, d] (h's type), mu [d] fp32, seq_slot int32
    (-1: a padding row, no state read or written).  single: the caller guarantees that every
    row is a sequence of its own with a distinct slot (a decode step), which lets the GPU read
    and replace the state in one launch."""
    if _native(h):
        torch.ops.akap_stream.token_shift(out, h, mu, state, seq_slot, positions, bool(single))
        return
    T = h.shape[0]
    slot, pos = seq_slot.long(), positions.long()
    cont = torch.zeros(T, dtype=torch.bool)
    cont[1:] = (slot[1:] == slot[:-1]) & (pos[1:] == pos[:-1] + 1) & (slot[1:] >= 0)
    prev = torch.zeros(T, h.shape[1], dtype=torch.float32)
    prev[1:][cont[1:]] = h[:-1][cont[1:]].float()
    old = ~cont & (pos > 0) & (slot >= 0)
    prev[old] = state[slot[old]].float()
    last = torch.ones(T, dtype=torch.bool)
    last[:-1] = ~cont[1:]
    last &= slot >= 0
    hf = h.float()
    new_state = h[last].clone()
    out.copy_((hf + (prev - hf) * mu.float()).to(out.dtype))
    state[slot[last]] = new_state


# ----------------------------------------------------------------------------- latent attention
def _rotate_pairs(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [T, ..., dims] rotated in interleaved pairs by the table rows cs [T, dims]."""
    dims = cs.shape[1]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = cs[:, :dims // 2].reshape(shape), cs[:, dims // 2:].reshape(shape)
    u, v = x[..., 0::2], x[..., 1::2]
    o = torch.empty_like(x)
    o[..., 0::2] = u * c - v * s
    o[..., 1::2] = v * c + u * s
    return o


def latent_prep(proj: torch.Tensor, cq_out: torch.Tensor, cache: Optional[torch.Tensor],
                positions: torch.Tensor, slots: torch.Tensor, cos_sin: torch.Tensor,
                q_w: torch.Tensor, kv_w: Optional[torch.Tensor], q_rank: int, kv_rank: int,
                rot_dim: int, q_off: int, kv_off: int, eps: float,
                vgroups: Optional[torch.Tensor] = None) -> None:
    """Per token t of the fused down-projection proj [T, N]: the query latent
    proj[t, q_off : q_off + q_rank] is RMS-normalised (weights q_w, fp32) into cq_out
    [T, q_rank]; the key/value latent proj[t, kv_off : kv_off + kv_rank] is RMS-normalised
    (kv_w) and the next rot_dim entries rotated in interleaved pairs by the angle row of
    positions[t], and both are written as one row [kv_rank + rot_dim] of the paged latent
    cache [NB, BS, kv_rank + rot_dim] at slots[t] (-1: nothing).  cache None: the layer reads
    another layer's cache and projects no latent of its own.  vgroups
    [NB, BS / 8, kv_rank, 8]: the normed latent once more, in groups of 8 tokens
    (dimension-major inside a group: the operand layout of the matrix-core attention)."""
    if _native(proj):
        torch.ops.akap_stream.latent_prep(proj, cq_out, cache, positions, slots, cos_sin, q_w,
                                          kv_w, q_rank, kv_rank, rot_dim, q_off, kv_off,
                                          float(eps), vgroups)
        return
    cq = _rms(proj[:, q_off:q_off + q_rank].float(), eps) * q_w.float()
    cq_out.copy_(cq.to(cq_out.dtype))
    if cache is None:
        return
    c = _rms(proj[:, kv_off:kv_off + kv_rank].float(), eps) * kv_w.float()
    kr = _rotate_pairs(proj[:, kv_off + kv_rank:kv_off + kv_rank + rot_dim].float(),
                       cos_sin[positions.long()])
    BS = cache.shape[1]
    ok = slots >= 0
    sl = slots[ok].long()
    cache[sl // BS, sl % BS] = torch.cat([c, kr], dim=1)[ok].to(cache.dtype)
    if vgroups is not None:
        vgroups[sl // BS, (sl % BS) // 8, :, sl % 8] = c[ok].to(vgroups.dtype)


def rotate_heads_(q: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor,
                  offset: int) -> None:
    """In place: the cos_sin.shape[1] entries from `offset` of every head of q [T, H, n] are
    rotated in interleaved pairs by the angle row of positions[t] (fp32 arithmetic)."""
    if _native(q):
        torch.ops.akap_stream.rotate_heads(q, positions, cos_sin, int(offset))
        return
    dims = cos_sin.shape[1]
    part = q[:, :, offset:offset + dims].float()
    q[:, :, offset:offset + dims] = _rotate_pairs(part, cos_sin[positions.long()]).to(q.dtype)


def latent_attention(out: torch.Tensor, q_lat: torch.Tensor, q: torch.Tensor, rot_off: int,
                     cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                     q_start: Optional[torch.Tensor], positions: torch.Tensor,
                     scale: float) -> None:
    """Causal softmax attention of every head against ONE cached row per key: the score of
    query (t, h) and key j is (q_lat[h, t] . cache[j, :R] + q[t, h, rot_off:rot_off + r] .
    cache[j, R:R + r]) * scale, where q_lat [H, T, R] is the unrotated query already multiplied
    into the latent space (W_uk^T q), and out[h, t] = sum_j softmax_j(score) cache[j, :R]
    (still latent: the caller applies W_uv per head).  The keys of token t are positions
    0 .. positions[t] of its sequence's block-table row; its sequence is b with
    q_start[b] <= t < q_start[b+1] (q_start None: row t is sequence t, one query each).
    Sequences with seq_lens[b] == 0 are padding.  Scores and softmax are fp32."""
    if _native(q):
        torch.ops.akap_stream.latent_attention(out, q_lat, q, int(rot_off), cache, block_tables,
                                               seq_lens, q_start, positions, float(scale))
        return
    H, T, R = q_lat.shape
    BS, r = cache.shape[1], cache.shape[2] - R
    B = seq_lens.numel()
    for b in range(B):
        kv = int(seq_lens[b])
        if kv == 0:
            continue
        r0, r1 = (b, b + 1) if q_start is None else (int(q_start[b]), int(q_start[b + 1]))
        if r1 <= r0:
            continue
        nb = -(-kv // BS)
        rows = cache[block_tables[b, :nb].long()].reshape(nb * BS, R + r)[:kv].float()
        pos = positions[r0:r1].long()
        ok = torch.arange(kv)[None, :] <= pos[:, None]
        s = torch.einsum("htr,jr->htj", q_lat[:, r0:r1].float(), rows[:, :R]) + \
            torch.einsum("thr,jr->htj", q[r0:r1, :, rot_off:rot_off + r].float(), rows[:, R:])
        s = (s * scale).masked_fill(~ok[None], float("-inf"))
        out[:, r0:r1] = torch.einsum("htj,jr->htr", torch.softmax(s, dim=-1),
                                     rows[:, :R]).to(out.dtype)


def latent_mfma_ok(cache: torch.Tensor, vgroups: Optional[torch.Tensor], kv_rank: int,
                   q: torch.Tensor, rot_off: int, scale: float, max_blocks: int = 0) -> bool:
    """The matrix-core kernels take a bf16 GPU cache with its grouped copy, latent / rotated
    sizes they were built for, 32-token-aligned blocks and 16-byte-aligned query rows."""
    if vgroups is None or not cache.is_cuda or cache.dtype != torch.bfloat16:
        return False
    load_native(required=True)
    return (torch.ops.akap_stream.latent_mfma_supported(kv_rank, cache.shape[2] - kv_rank)
            and cache.shape[1] % 32 == 0 and rot_off % 8 == 0 and q.shape[2] % 8 == 0
            and scale > 0 and max_blocks * (cache.shape[1] // 32) <= 16384)


def latent_attention_prefill(out: torch.Tensor, q_lat: torch.Tensor, q: torch.Tensor,
                             rot_off: int, cache: torch.Tensor, vgroups: Optional[torch.Tensor],
                             block_tables: torch.Tensor, seq_lens: torch.Tensor,
                             q_start: torch.Tensor, positions: torch.Tensor, tile_seq, tile_row,
                             tile_rows: int, scale: float, first_seq: int = 0) -> None:
    """latent_attention for the prompt chunks of a step (sequences from first_seq on; the rows
    before q_start[first_seq] belong to single-token sequences and are left alone): on the
    matrix cores when latent_mfma_ok, driven by the scheduler's tile map (tile_seq / tile_row:
    sequence and first chunk row of a tile of tile_rows tokens), else the row kernel."""
    if latent_mfma_ok(cache, vgroups, q_lat.shape[2], q, rot_off, scale, block_tables.shape[1]):
        torch.ops.akap_stream.latent_attention_prefill_mfma(
            out, q_lat, q, rot_off, cache, vgroups, block_tables, seq_lens, q_start, tile_seq,
            tile_row, tile_rows, float(scale))
        return
    if first_seq:
        # the leading rows were handled as decode rows: hide their sequences from this pass
        seq_lens = seq_lens.clone()
        seq_lens[:first_seq] = 0
    latent_attention(out, q_lat, q, rot_off, cache, block_tables, seq_lens, q_start, positions,
                     scale)


def latent_decode_workspace(rows: int, heads: int, kv_rank: int, parts: int, device):
    n = max(1, rows * heads * parts)
    return (torch.empty(n * 2, dtype=torch.float32, device=device),
            torch.empty(n * kv_rank, dtype=torch.float32, device=device))


def latent_attention_decode(out: torch.Tensor, q_lat: torch.Tensor, q: torch.Tensor, rot_off: int,
                            cache: torch.Tensor, vgroups: Optional[torch.Tensor],
                            block_tables: torch.Tensor, seq_lens: torch.Tensor,
                            positions: torch.Tensor, scale: float, workspace=None,
                            num_parts: int = 1) -> None:
    """latent_attention with one query per sequence, at position seq_lens[b] - 1 (0: a padding
    row, left unwritten).  On the matrix cores (latent_mfma_ok) the heads of a token are the
    columns of one tile and the keys are cut into num_parts partitions of whole 32-key blocks,
    one wave each, merged by a second launch (workspace from latent_decode_workspace)."""
    if latent_mfma_ok(cache, vgroups, q_lat.shape[2], q, rot_off, scale, block_tables.shape[1]):
        ws_ml, ws_o = workspace if (workspace is not None and num_parts > 1) else (None, None)
        torch.ops.akap_stream.latent_attention_decode_mfma(
            out, q_lat, q, rot_off, cache, vgroups, block_tables, seq_lens, float(scale), ws_ml,
            ws_o, num_parts if ws_ml is not None else 1)
        return
    latent_attention(out, q_lat, q, rot_off, cache, block_tables, seq_lens, None, positions, scale)


# rows up to which the per-head products take the one-wave-per-tile kernel
HEAD_MATMUL_ROWS = 256


def head_matmul(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out[h] = a[h] @ w[h]^T for every head: a [H, T, K] (any head / row strides, unit stride in
    k: a view of [T, H, n] rows is fine), w [H, N, K].  A few rows of bf16 on the GPU (decode
    steps) run a small matrix-core kernel; everything else the library's batched GEMM."""
    H, T, K = a.shape
    N = w.shape[1]
    if (a.is_cuda and a.dtype == torch.bfloat16 and 0 < T <= HEAD_MATMUL_ROWS and K % 16 == 0
            and N % 32 == 0 and a.stride(2) == 1 and a.stride(0) % 8 == 0 and a.stride(1) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.is_contiguous()):
        load_native(required=True)
        out = torch.empty(H, T, N, dtype=a.dtype, device=a.device)
        torch.ops.akap_stream.head_matmul(out, a, w)
        return out
    return torch.bmm(a, w.transpose(1, 2))


def head_gate(o: torch.Tensor, gate: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, h V + j] = o[h, t, j] * sigmoid(g), g = gate[t, h] when gate has H columns (one
    gate per head) or gate[t, h V + j] when it has H V (one per output entry).  o [H, T, V]
    (head-major, as the per-head up-projection leaves it), gate and out are [T, .] views that
    may be column slices of wider rows.  The sigmoid and the product are fp32."""
    if _native(o):
        torch.ops.akap_stream.head_gate(out, o, gate)
        return
    H, T, V = o.shape
    g = torch.sigmoid(gate.float())
    g = g[:, :, None] if gate.shape[1] == H else g.view(T, H, V)
    out.copy_((o.float().permute(1, 0, 2) * g).reshape(T, H * V).to(out.dtype))


def xielu(x: torch.Tensor, bias: Optional[torch.Tensor], act: torch.Tensor,
          out: torch.Tensor) -> None:
    """out = f(x + bias), f(z) = softplus(p) z^2 + z / 2 for z > 0 and
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 otherwise, (p, q) = act (fp32 [2], read on
    the device).  x and out are [T, F] views that may be column slices of wider rows."""
    if _native(x):
        torch.ops.akap_stream.xielu(out, x, bias, act)
        return
    z = x.float()
    if bias is not None:
        z = z + bias.float()
    ap, aq = torch.nn.functional.softplus(act.float()[0]), torch.nn.functional.softplus(act.float()[1])
    neg = torch.clamp(z, max=0.0)
    out.copy_(torch.where(z > 0, ap * z * z + z / 2,
                          (0.5 + aq) * (torch.expm1(neg) - neg) + z / 2).to(out.dtype))


# ----------------------------------------------------------------------------- routed experts
def moe_route(h: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor],
              top: int, groups: int = 1, keep: int = 1):
    """Grouped top-k routing: scores s = softmax(router h) over all n router outputs (fp32
    logits from h's stored values); the choice uses s + correction; outputs form `groups` equal
    groups of neighbours, a group scores its largest choice value, and only outputs of the
    `keep` best groups can be chosen; the `top` largest allowed choice values win (ties: the
    lower index).  Returns ids int32 [T, top] and weights fp32 [T, top] = the winners' s
    divided by their sum (+ 1e-20).  router fp32 [n, d], correction fp32 [n]."""
    T, n = h.shape[0], router.shape[0]
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    w = torch.empty(T, top, dtype=torch.float32, device=h.device)
    if _native(h):
        torch.ops.akap_stream.moe_route(ids, w, h, router, correction, int(groups), int(keep))
        return ids, w
    s = torch.softmax(h.float() @ router.float().T, dim=-1)
    choice = s + correction.float() if correction is not None else s.clone()
    per = n // groups
    if groups > 1:
        gs = choice.view(T, groups, per).max(dim=-1).values
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        choice = choice.masked_fill(~allowed[:, :, None].expand(T, groups, per).reshape(T, n),
                                    float("-inf"))
    idx = choice.topk(top, dim=-1).indices
    sel = s.gather(1, idx)
    ids.copy_(idx)
    w.copy_(sel / (sel.sum(dim=-1, keepdim=True) + 1e-20))
    return ids, w


def relu2_routed(up: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, experts: int,
                 out: torch.Tensor) -> None:
    """out[t, e F + f] = w_e(t) relu(up[t, e F + f])^2, w_e(t) the routing weight of expert e for
    token t (0 when it was not chosen): the activation of EVERY expert's up-projection scaled so
    that one GEMM with the concatenated down-projections [d, E F] sums the chosen experts
    (small batches, where all expert weights are streamed anyway).  ids [T, top] >= experts are
    identity outputs and scale nothing here."""
    if _native(up):
        torch.ops.akap_stream.relu2_routed(out, up, ids, w, int(experts))
        return
    T = up.shape[0]
    F_ = up.shape[1] // experts
    full = torch.zeros(T, experts + 1, dtype=torch.float32)
    full.scatter_(1, ids.long().clamp(max=experts), w)
    r = torch.relu(up.float()).view(T, experts, F_)
    out.copy_((r * r * full[:, :experts, None]).view(T, experts * F_).to(out.dtype))


def moe_combine(out: torch.Tensor, y: torch.Tensor, inv: Optional[torch.Tensor],
                ids: torch.Tensor, w: torch.Tensor, h: torch.Tensor, experts: int) -> None:
    """out (fp32 [T, d]) = the routed feed-forward's output.  inv None: y [T, d] already holds
    the weighted sum over the chosen experts.  inv int32 [T, top]: y [T top, d] are expert
    outputs in expert-sorted row order, inv[t, k] the row of choice k of token t, and
    out[t] = sum_k w[t, k] y[inv[t, k]].  Either way choices with ids >= experts (identity
    outputs) add w[t, k] h[t]."""
    if _native(y):
        torch.ops.akap_stream.moe_combine(out, y, inv, ids, w, h, int(experts))
        return
    ident = (w * (ids >= experts)).sum(dim=1, keepdim=True)
    if inv is None:
        acc = y.float()
    else:
        real = (w * (ids < experts))[:, :, None]
        acc = (y.float()[inv.long().clamp(min=0, max=y.shape[0] - 1)] * real).sum(dim=1)
    out.copy_(acc + ident * h.float())


# ----------------------------------------------------------------------------- sandwich norms
def _w(w: torch.Tensor) -> torch.Tensor:
    return w.float()


def stream_post_norm_add_norm(x: torch.Tensor, ya: torch.Tensor, yb: Optional[torch.Tensor],
                              wa: Optional[torch.Tensor], wb: Optional[torch.Tensor],
                              post_w: torch.Tensor, next_w: torch.Tensor, eps: float,
                              out: torch.Tensor, fresh: bool = False) -> None:
    """The residual update of a sublayer whose OUTPUT is normed, fused with the norm that feeds
    the next sublayer:  m = ya, or with two branches m = (rms(ya) wa + rms(yb) wb) / 2;
    x <- x + rms(m) post_w (fresh: x <- rms(m) post_w, x is not read);  out = rms(x) next_w.
    rms(v) = v / sqrt(mean(v^2) + eps) over the row.  x fp32 [T, d] (the stream, updated in
    place); ya / yb [T, d] in the activation type or fp32; every weight is fp32 with d entries
    or ONE (a single number for all coordinates).  All arithmetic is fp32; out is rounded
    once."""
    if _native(x):
        torch.ops.akap_stream.post_norm_add_norm(out, x, ya, yb, wa, wb, post_w, next_w,
                                                 float(eps), bool(fresh))
        return
    m = ya.float()
    if yb is not None:
        m = 0.5 * (_rms(m, eps) * _w(wa) + _rms(yb.float(), eps) * _w(wb))
    upd = _rms(m, eps) * _w(post_w)
    if fresh:
        x.copy_(upd)
    else:
        x.add_(upd)
    out.copy_((_rms(x, eps) * _w(next_w)).to(out.dtype))


# ----------------------------------------------------------------------------- head-mixed attention
def head_norm_cache(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, slots: torch.Tensor, H: int, G: int, D: int, Dv: int,
                    q_off: int, k_off: int, v_off: int, eps: float, norm_qk: bool = True,
                    norm_v: bool = True) -> None:
    """Per token t of the fused projection proj [T, N]: the H query heads
    proj[t, q_off : q_off + H D] go to q_out [T, H, D], the G key heads (from k_off) to k_cache
    [NB, G, BS, D] and the G value heads (from v_off, size Dv) to v_cache [NB, G, BS / 8, Dv, 8]
    (groups of 8 tokens, dimension-major inside a group) at slots[t] (-1: nothing is cached).  norm_qk / norm_v: each head is first divided by its own
    root mean square (fp32, eps inside the root, no weights)."""
    if _native(proj):
        torch.ops.akap_stream.head_norm_cache(proj, q_out, k_cache, v_cache, slots, H, G, D, Dv,
                                              q_off, k_off, v_off, float(eps), bool(norm_qk),
                                              bool(norm_v))
        return
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * D].float().view(T, H, D)
    k = proj[:, k_off:k_off + G * D].float().view(T, G, D)
    v = proj[:, v_off:v_off + G * Dv].float().view(T, G, Dv)
    if norm_qk:
        q, k = _rms(q, eps), _rms(k, eps)
    if norm_v:
        v = _rms(v, eps)
    q_out.copy_(q.to(q_out.dtype))
    BS = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // BS, :, sl % BS] = k[ok].to(k_cache.dtype)
    v_cache[sl // BS, :, (sl % BS) // 8, :, sl % 8] = v[ok].to(v_cache.dtype)


def talking_attention_parts(rows: int, kv_heads: int, max_len: int) -> int:
    """Key partitions of a decode row of talking_attention: static in the batch size and the
    model length (hipGraph-capturable); one workgroup per (row, partition), about two per CU,
    a partition never under 128 keys."""
    max_parts = max(1, -(-max_len // 128))
    return max(1, min(max_parts, 32, -(-512 // max(1, rows))))


def talking_attention_workspace(rows: int, H: int, G: int, Dv: int, parts: int, device):
    """Partial state of the split form: (max, sum) per (row, partition, head) and the
    unnormalised outputs of every (head, value head) pair, fp32."""
    n = max(1, rows * parts)
    return (torch.empty(n * H * 2, dtype=torch.float32, device=device),
            torch.empty(n * H * G * Dv, dtype=torch.float32, device=device))


def talking_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                      q_start: Optional[torch.Tensor], positions: torch.Tensor,
                      talk: Optional[torch.Tensor], gate: Optional[torch.Tensor], scale: float,
                      workspace=None, num_parts: int = 1) -> None:
    """Causal softmax attention whose heads exchange their weights AFTER the softmax: with
    P_g(t, j) = softmax_j(q[t, g] . k[j, g // (H / G)] * scale) over the keys j <= positions[t]
    of row t's sequence, head h uses P'_h = sum_g talk[h, g] P_g on the values of ITS OWN
    key/value head:  out[t, h Dv : (h + 1) Dv] = sum_j P'_h(t, j) v[j, h // (H / G)], times
    sigmoid(gate[t, h Dv + i]) per entry when gate is given.  talk None: no mixing.
    Row t belongs to sequence b with q_start[b] <= t < q_start[b + 1] (q_start None: row t is
    sequence t); sequences with seq_lens[b] == 0 are padding and their rows are left unwritten.
    q [T, H, D]; k_cache [NB, G, BS, D]; v_cache [NB, G, BS / 8, Dv, 8]; talk fp32 [H, H]; gate and
    out are [T, H Dv] views that may be column slices of wider rows.  Scores, softmax, the
    mixing and the gate are fp32.
    The GPU kernel forms, for every head g, the unnormalised sums of ALL G value heads under
    its weights (one pass over the keys with a running maximum), and mixes them at the end;
    num_parts > 1 cuts the keys of a row into that many partitions, one workgroup each, merged,
    mixed and gated by a second launch (workspace from talking_attention_workspace)."""
    if _native(q):
        ws_ml, ws_o = workspace if (workspace is not None and num_parts > 1) else (None, None)
        torch.ops.akap_stream.talking_attention(out, q, k_cache, v_cache, block_tables, seq_lens,
                                                q_start, positions, talk, gate, float(scale),
                                                ws_ml, ws_o, num_parts if ws_ml is not None else 1)
        return
    T, H, D = q.shape
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    B = seq_lens.numel() if q_start is None else min(seq_lens.numel(), q_start.numel() - 1)
    for b in range(min(B, T) if q_start is None else B):
        kv = int(seq_lens[b])
        r0, r1 = (b, b + 1) if q_start is None else (int(q_start[b]), int(q_start[b + 1]))
        if kv == 0 or r1 <= r0:
            continue
        nb = -(-kv // BS)
        blocks = block_tables[b, :nb].long()
        K = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :kv].float()
        V = v_tokens(v_cache[blocks]).permute(1, 0, 2, 3).reshape(G, nb * BS, Dv)[:, :kv].float()
        pos = positions[r0:r1].long()
        ok = torch.arange(kv)[None, :] <= pos[:, None]
        s = torch.einsum("thd,hjd->htj", q[r0:r1].float(), K.repeat_interleave(rep, dim=0)) * scale
        P = torch.softmax(s.masked_fill(~ok[None], float("-inf")), dim=-1)
        if talk is not None:
            P = torch.einsum("hg,gtj->htj", talk.float(), P)
        o = torch.einsum("htj,hjv->thv", P, V.repeat_interleave(rep, dim=0)).reshape(r1 - r0, H * Dv)
        if gate is not None:
            o = o * torch.sigmoid(gate[r0:r1].float())
        out[r0:r1] = o.to(out.dtype)


def talking_attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                             v_cache: torch.Tensor, block_tables: torch.Tensor,
                             seq_lens: torch.Tensor, positions: torch.Tensor,
                             talk: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                             scale: float, workspace=None, num_parts: int = 1) -> None:
    """talking_attention with one query per sequence (row t is sequence t; seq_lens 0: a
    padding row, left unwritten).  On the GPU in bf16, at sizes the matrix-core kernel takes and
    with a workspace (talking_attention_workspace), the heads of a token are the columns of one
    matrix tile and every cached key and value is read once per row; the keys are cut into
    num_parts partitions, one workgroup each, merged, mixed and gated by a second launch."""
    H, D = q.shape[1], q.shape[2]
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    if (q.is_cuda and q.dtype == torch.bfloat16 and workspace is not None
            and load_native(required=True)
            and torch.ops.akap_stream.talking_mfma_supported(H, G, D, Dv, BS)):
        torch.ops.akap_stream.talking_attention_decode_mfma(
            out, q, k_cache, v_cache, block_tables, seq_lens, positions, talk, gate, float(scale),
            workspace[0], workspace[1], int(num_parts))
        return
    talking_attention(out, q, k_cache, v_cache, block_tables, seq_lens, None, positions, talk,
                      gate, scale, workspace, num_parts)


def talking_attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                              v_cache: torch.Tensor, block_tables: torch.Tensor,
                              seq_lens: torch.Tensor, q_start: torch.Tensor,
                              positions: torch.Tensor, tile_seq, tile_row, tile_rows: int,
                              talk: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                              scale: float, first_seq: int = 0) -> None:
    """talking_attention for a step with prompt chunks.  The rows of the sequences before
    first_seq (single-token sequences that lead a mixed step, one row each) go through the row
    kernel; the chunks, on the GPU in bf16 and at sizes the matrix-core kernel takes, run on
    the matrix cores, driven by the scheduler's tile map (tile_seq / tile_row: sequence and
    first chunk row of a tile of tile_rows tokens): per query head the unnormalised sums of all
    value heads, then one launch that normalises, mixes the heads and gates."""
    H, D = q.shape[1], q.shape[2]
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    T = q.shape[0]
    if (q.is_cuda and q.dtype == torch.bfloat16 and tile_seq is not None and tile_rows % 32 == 0
            and load_native(required=True)
            and torch.ops.akap_stream.talking_mfma_supported(H, G, D, Dv, BS)):
        nd = first_seq
        if nd:
            talking_attention(out[:nd], q[:nd], k_cache, v_cache, block_tables[:nd], seq_lens[:nd],
                              None, positions[:nd], talk, gate[:nd] if gate is not None else None,
                              scale)
        if T > nd:
            ws_ml = torch.empty(T * H * 2, dtype=torch.float32, device=q.device)
            ws_o = torch.empty(T * H * G * Dv, dtype=torch.float32, device=q.device)
            torch.ops.akap_stream.talking_attention_prefill_mfma(
                out, q, k_cache, v_cache, block_tables, seq_lens, q_start, positions, tile_seq,
                tile_row, int(tile_rows), int(nd), talk, gate, float(scale), ws_ml, ws_o)
        return
    talking_attention(out, q, k_cache, v_cache, block_tables, seq_lens, q_start, positions, talk,
                      gate, scale)


# ----------------------------------------------------------------------------- retention
def rotate_half_(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [T, H, D] (fp32) with its first cs.shape[1] dimensions rotated, dimension i paired
    with i + dims/2, by the table rows cs [T, dims] = [cos | sin]."""
    dims = cs.shape[1]
    half = dims // 2
    c, s = cs[:, None, :half], cs[:, None, half:]
    u, v = x[..., :half].clone(), x[..., half:dims].clone()
    x[..., :half] = u * c - v * s
    x[..., half:dims] = v * c + u * s
    return x


# steps of at least this many rows run the retention in segments of RETENTION_SEGMENT rows
RETENTION_SEGMENTED_ROWS = 1024
RETENTION_SEGMENT = 256


def retention(out: torch.Tensor, proj: torch.Tensor, q_off: int, k_off: int, v_off: int,
              g_off: int, state: torch.Tensor, seq_slot: torch.Tensor, positions: torch.Tensor,
              q_start: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
              log2_decay: torch.Tensor, H: int, D: int, V: int, eps: float) -> None:
    """Decayed linear attention with a recurrent state, for the token rows of a step.  Per
    token t and head h, from the fused projection proj [T, N]: q, k = proj[t, q_off / k_off +
    h D ...] (D entries), v = proj[t, v_off + h V ...], g = proj[t, g_off + h V ...] (V
    entries).  q and k are rotated on their first cos_sin.shape[1] dimensions in the rotate-half
    layout (i pairs with i + dims/2) by the angle row of positions[t]; k is scaled by D^-1/2;
    S <- decay_h S + k v^T and o = S^T q with decay_h = 2^log2_decay[h]; o is divided by its
    root mean square over V (eps inside the root) and multiplied by silu(g):
    out[t, h V : (h + 1) V].  The state of a sequence lives TRANSPOSED in state[slot, h]
    (fp32 [V, D] = S^T: the D entries a GPU thread keeps in registers are contiguous): the rows of sequence b are [q_start[b], q_start[b + 1]) (q_start None: row
    t is a sequence of its own), its slot is seq_slot of its first row (-1: padding, nothing
    is read or written); it starts from zeros when its first row has position 0, else from
    what an earlier step left in the slot, and the state after its last row is written back.
    Rotation, decay, state, the output norm and the gate are fp32.  out may be a column slice
    of wider rows."""
    if _native(proj):
        seg_buf, T = None, proj.shape[0]
        if q_start is not None and T >= RETENTION_SEGMENTED_ROWS:
            # long prompt chunks: the segments of a sequence run side by side (each leaves its
            # own state, a scan turns these into the state before each segment, a second pass
            # produces the outputs); the buffer is sized from the step's shape alone
            n = (T // RETENTION_SEGMENT + q_start.numel() - 1) * H * V * D
            seg_buf = torch.empty(n, dtype=torch.float32, device=proj.device)
        torch.ops.akap_stream.retention(out, proj, q_off, k_off, v_off, g_off, state, seq_slot,
                                        positions, q_start, cos_sin, log2_decay, H, D, V,
                                        float(eps), seg_buf, RETENTION_SEGMENT)
        return
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * D].float().reshape(T, H, D).clone()
    k = proj[:, k_off:k_off + H * D].float().reshape(T, H, D).clone()
    v = proj[:, v_off:v_off + H * V].float().reshape(T, H, V)
    g = proj[:, g_off:g_off + H * V].float().reshape(T, H, V)
    if cos_sin is not None:
        cs = cos_sin[positions.long()]
        rotate_half_(q, cs)
        rotate_half_(k, cs)
    k = k * (D ** -0.5)
    decay = torch.exp2(log2_decay.float())[:, None, None]
    B = T if q_start is None else q_start.numel() - 1
    o = torch.zeros(T, H, V, dtype=torch.float32)
    for b in range(B):
        r0, r1 = (b, b + 1) if q_start is None else (int(q_start[b]), int(q_start[b + 1]))
        if r1 <= r0 or int(seq_slot[r0]) < 0:
            continue
        slot = int(seq_slot[r0])
        S = state[slot].float().transpose(1, 2).clone() if int(positions[r0]) > 0 else \
            torch.zeros(H, D, V, dtype=torch.float32)
        for t in range(r0, r1):
            S = decay * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S.transpose(1, 2)
        on = _rms(o[r0:r1], eps) * torch.nn.functional.silu(g[r0:r1])
        out[r0:r1] = on.reshape(r1 - r0, H * V).to(out.dtype)


# ----------------------------------------------------------------------------- logit-top-k routing
def route_topk(h: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int):
    """Routing by the largest logits: z = router h + bias (fp32, from h's stored values); the
    `top` largest z win (ties: the lower index) and their weights are the softmax over the
    winners' logits only.  Returns ids int32 [T, top] (by falling logit) and weights fp32
    [T, top].  router fp32 [E, d], bias fp32 [E]."""
    T = h.shape[0]
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    w = torch.empty(T, top, dtype=torch.float32, device=h.device)
    if _native(h):
        torch.ops.akap_stream.route_topk(ids, w, h, router, bias)
        return ids, w
    z = h.float() @ router.float().T
    if bias is not None:
        z = z + bias.float()
    val, idx = z.topk(top, dim=-1)
    ids.copy_(idx)
    w.copy_(torch.softmax(val, dim=-1))
    return ids, w


def swiglu(gu: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, f] = silu(gu[t, f]) gu[t, F + f] for gu [T, 2 F] = [gate | up] (fp32 arithmetic);
    both may be column slices of wider rows."""
    if _native(gu):
        torch.ops.akap_stream.swiglu_routed(out, gu, None, None, 1)
        return
    F_ = gu.shape[1] // 2
    out.copy_((torch.nn.functional.silu(gu[:, :F_].float()) * gu[:, F_:].float()).to(out.dtype))


def swiglu_routed(gu: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, experts: int,
                  out: torch.Tensor) -> None:
    """out[t, e F + f] = w_e(t) silu(gu[t, e 2F + f]) gu[t, e 2F + F + f], with w_e(t) the
    routing weight of expert e for token t (0 when it was not chosen): the gated activation of
    EVERY expert's [gate | up] projection, scaled so that one GEMM with the side-by-side
    down-projections [d, E F] sums the chosen experts (small batches, where all expert weights
    are streamed anyway)."""
    if _native(gu):
        torch.ops.akap_stream.swiglu_routed(out, gu, ids, w, int(experts))
        return
    T = gu.shape[0]
    F_ = gu.shape[1] // (2 * experts)
    full = torch.zeros(T, experts, dtype=torch.float32)
    full.scatter_(1, ids.long(), w)
    g3 = gu.float().view(T, experts, 2, F_)
    act = torch.nn.functional.silu(g3[:, :, 0]) * g3[:, :, 1] * full[:, :, None]
    out.copy_(act.view(T, experts * F_).to(out.dtype))


# ----------------------------------------------------------------------------- residual streams
def hyper_step(xs: torch.Tensor, ya: Optional[torch.Tensor], yb: Optional[torch.Tensor],
               bias: Optional[torch.Tensor], mix: Optional[torch.Tensor],
               w_out: Optional[torch.Tensor], w_in: torch.Tensor, norm_w: torch.Tensor,
               eps: float, out: torch.Tensor, fresh: Optional[torch.Tensor] = None) -> None:
    """One step of a model with S residual streams xs [T, S, d] (fp32, updated in place): the
    write of a sublayer's output fused with the read and norm that feed the next sublayer.
    With y = ya + yb + bias (each may be None; [T, d] in the activation type or fp32, bias [d]):
    every stream at once from the old ones, xs[:, r] <- sum_s mix[s, r] xs[:, s] + w_out[r] y;
    then u = sum_s w_in[s] xs[:, s] and out = u / sqrt(mean(u^2) + eps) * norm_w.  fresh [T, d]
    (fp32): instead of an update every stream is set to it (the start of the stack).  mix
    [S, S] (indexed [from, to]), w_out, w_in [S] and norm_w [d] are fp32; S = 1 with ones is a
    plain residual sum.  All arithmetic is fp32; out is rounded once."""
    if _native(xs):
        torch.ops.akap_stream.hyper_step(out, xs, ya, yb, bias, mix, w_out, w_in, norm_w,
                                         float(eps), fresh)
        return
    if fresh is not None:
        xs.copy_(fresh.float()[:, None, :].expand_as(xs))
    else:
        y = torch.zeros(xs.shape[0], xs.shape[2], dtype=torch.float32)
        for t in (ya, yb, bias):
            if t is not None:
                y = y + t.float()
        xs.copy_(torch.einsum("sr,tsd->trd", mix.float(), xs) + w_out.float()[None, :, None]
                 * y[:, None, :])
    u = torch.einsum("s,tsd->td", w_in.float(), xs)
    out.copy_((_rms(u, eps) * norm_w.float()).to(out.dtype))


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap tanh(logits / cap) in place (fp32 arithmetic)."""
    if _native(logits):
        torch.ops.akap_stream.softcap_(logits, float(cap))
        return logits
    logits.copy_((cap * torch.tanh(logits.float() / cap)).to(logits.dtype))
    return logits


# ----------------------------------------------------------------------------- windowed attention with pooled blocks
def rotary_table_yarn(max_pos: int, dims: int, base: float, scaling: Optional[dict],
                      device=None) -> torch.Tensor:
    """fp32 [max_pos, dims] = [cos | sin] of the angle p f_i, f_i = base^(-2i/dims), i <
    dims / 2, under the YaRN rule of scaling = {factor, original, fast, slow}: with
    at(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(at(fast)), 0),
    hi = min(ceil(at(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    the frequency is f_i / factor r_i + f_i (1 - r_i), and cos and sin carry the factor
    0.1 ln(factor) + 1.  Angles are formed in fp64 and rounded once."""
    import math

    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    m = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def at(turns: float) -> float:
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(at(float(scaling["fast"]))), 0)
        hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
        r = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * r + f * (1.0 - r)
        m = 0.1 * math.log(factor) + 1.0
    a = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None, :]
    t = torch.cat([torch.cos(a) * m, torch.sin(a) * m], dim=1).to(torch.float32)
    return t.to(device) if device is not None else t


def pool_slots(block_size: int, pool: int) -> int:
    """Pooled entries a cache page holds: a block of `pool` tokens is stored with the page of
    its first token, at index (first token's offset in the page) // pool."""
    return -(-block_size // pool) if pool > 0 else 0


def bias_rope_cache(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                    cos_sin: Optional[torch.Tensor], bias: Optional[torch.Tensor], H: int, G: int,
                    D: int, Dv: int, q_off: int, k_off: int, v_off: int) -> None:
    """Per token t of the fused projection proj [T, N]: q = proj[t, q_off : q_off + H D],
    k = proj[t, k_off : k_off + G D], v = proj[t, v_off : v_off + G Dv], each plus its slice of
    bias (fp32 [N], laid out like proj's columns; None: no biases); q and k are rotated per head
    on their first cos_sin.shape[1] dimensions in the rotate-half layout (entry i with
    i + dims/2) by the table row of positions[t] (fp32).  q goes to q_out [T, H, D]; k to
    k_cache [NB, G, BS, D] and v to v_cache [NB, G, BS / 8, Dv, 8] at slots[t]; slot -1 writes
    nothing."""
    if _native(proj):
        torch.ops.akap_stream.bias_rope_cache(proj, q_out, k_cache, v_cache, positions, slots,
                                              cos_sin, bias, H, G, D, Dv, q_off, k_off, v_off)
        return
    T = proj.shape[0]
    b = bias.float() if bias is not None else torch.zeros(proj.shape[1])
    q = (proj[:, q_off:q_off + H * D].float() + b[q_off:q_off + H * D]).view(T, H, D).clone()
    k = (proj[:, k_off:k_off + G * D].float() + b[k_off:k_off + G * D]).view(T, G, D).clone()
    v = (proj[:, v_off:v_off + G * Dv].float() + b[v_off:v_off + G * Dv]).view(T, G, Dv)
    if cos_sin is not None:
        cs = cos_sin[positions.long()]
        rotate_half_(q, cs)
        rotate_half_(k, cs)
    q_out.copy_(q.to(q_out.dtype))
    BS = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // BS, :, sl % BS] = k[ok].to(k_cache.dtype)
    v_cache[sl // BS, :, (sl % BS) // 8, :, sl % 8] = v[ok].to(v_cache.dtype)


def _row_sequences(T: int, q_start: Optional[torch.Tensor]):
    """(first row, end row) per sequence of a step: from q_start, or one row each."""
    if q_start is None:
        return [(t, t + 1) for t in range(T)]
    qs = q_start.tolist()
    return [(qs[b], qs[b + 1]) for b in range(len(qs) - 1)]


def pool_cache_blocks(k_cache: torch.Tensor, v_cache: torch.Tensor, k_pool: torch.Tensor,
                      v_pool: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                      block_tables: torch.Tensor, q_start: Optional[torch.Tensor],
                      pool: int) -> None:
    """For every token row whose position p ends a block of `pool` positions ((p + 1) % pool ==
    0, slot >= 0): the mean (fp32 sum) of the block's `pool` cached keys, as the cache holds
    them, goes to k_pool [NB, G, pool_slots, D] (fp32) and the mean of its values to v_pool, at
    the page of the block's first token, index (its offset in the page) // pool.  Runs after the
    step's cache write.  The rows of sequence b are [q_start[b], q_start[b + 1]) (None: row t is
    sequence t); its pages are block_tables[b]."""
    if _native(k_cache):
        torch.ops.akap_stream.pool_cache_blocks(k_cache, v_cache, k_pool, v_pool, positions, slots,
                                                block_tables, q_start, int(pool))
        return
    BS = k_cache.shape[2]
    for b, (r0, r1) in enumerate(_row_sequences(positions.shape[0], q_start)):
        for t in range(r0, r1):
            p = int(positions[t])
            if int(slots[t]) < 0 or (p + 1) % pool:
                continue
            first = p + 1 - pool
            pos = torch.arange(first, p + 1)
            pages = block_tables[b][pos // BS].long()
            kk = k_cache[pages, :, pos % BS].float().mean(dim=0)
            vv = v_cache[pages, :, (pos % BS) // 8, :, pos % 8].float().mean(dim=0)
            page, idx = int(block_tables[b][first // BS]), (first % BS) // pool
            k_pool[page, :, idx] = kk
            v_pool[page, :, idx] = vv


def pooled_window_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                            v_cache: torch.Tensor, k_pool: Optional[torch.Tensor],
                            v_pool: Optional[torch.Tensor], block_tables: torch.Tensor,
                            q_start: Optional[torch.Tensor], positions: torch.Tensor,
                            slots: torch.Tensor, scale: float, window: int, pool: int,
                            unit_sink: bool, first_seq: int = 0) -> None:
    """Paged attention of the token rows of a step.  The query at position i of sequence b
    (rows by q_start as in pool_cache_blocks) sees the cached tokens j <= i with i - j < window
    (window 0: all) and, with pool > 0, the pooled entry of every block c with
    c pool + pool - 1 <= i - window (pool_cache_blocks' layout); tokens and blocks share one
    softmax over scale q.k, with 1 added to its denominator when unit_sink.  Query head h reads
    key/value head h // (H / G).  Scores, softmax and the weighted sums are fp32.  Rows with
    slot -1 are padding and left unwritten.  out [T, >= H Dv].  K [NB, G, BS, D] token-major,
    V [NB, G, BS / 8, Dv, 8].  first_seq (CPU tensors): sequences before it are skipped."""
    if _native(q):
        torch.ops.akap_stream.pooled_window_attention(out, q, k_cache, v_cache, k_pool, v_pool,
                                                      block_tables, q_start, positions, slots,
                                                      float(scale), int(window), int(pool),
                                                      bool(unit_sink))
        return
    T, H, D = q.shape
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    for b, (r0, r1) in enumerate(_row_sequences(T, q_start)):
        if b < first_seq:
            continue
        for t in range(r0, r1):
            if int(slots[t]) < 0:
                continue
            i = int(positions[t])
            lo = max(0, i - window + 1) if window > 0 else 0
            pos = torch.arange(lo, i + 1)
            pages = block_tables[b][pos // BS].long()
            K = k_cache[pages, :, pos % BS].float()            # [n, G, D]
            V = v_cache[pages, :, (pos % BS) // 8, :, pos % 8].float()
            nb = (i - window + 1) // pool if (pool > 0 and window > 0 and i - window + 1 > 0) \
                else 0
            if nb > 0:
                first = torch.arange(nb) * pool
                pg = block_tables[b][first // BS].long()
                K = torch.cat([k_pool[pg, :, (first % BS) // pool].float(), K])
                V = torch.cat([v_pool[pg, :, (first % BS) // pool].float(), V])
            for h in range(H):
                s = (K[:, h // rep] @ q[t, h].float()) * scale
                m = s.max()
                if unit_sink:
                    m = torch.clamp(m, min=0.0)
                e = torch.exp(s - m)
                den = e.sum() + (torch.exp(-m) if unit_sink else 0.0)
                out[t, h * Dv:(h + 1) * Dv] = ((e / den) @ V[:, h // rep]).to(out.dtype)


def pooled_mfma_ok(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> bool:
    """Can the matrix-core kernel take these prompt chunks (bf16 on the GPU, head size a
    multiple of 16, value size 32 / 64 / 128 / 256)?"""
    if not (q.is_cuda and q.dtype == torch.bfloat16):
        return False
    load_native(required=True)
    return bool(torch.ops.akap_stream.pooled_mfma_supported(
        q.shape[1], k_cache.shape[1], q.shape[2], v_cache.shape[3], k_cache.shape[2]))


def pooled_window_attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                                   v_cache: torch.Tensor, k_pool: Optional[torch.Tensor],
                                   v_pool: Optional[torch.Tensor], block_tables: torch.Tensor,
                                   positions: torch.Tensor, slots: torch.Tensor, scale: float,
                                   window: int, pool: int, unit_sink: bool) -> None:
    """pooled_window_attention for one query per sequence (row t is sequence t).  bf16 rows with
    matrix-core sizes run on the matrix cores: the query heads of a key/value head are the
    columns of a tile, so a group reads its keys once, and the key range is split over the
    waves of a workgroup; everything else on the row kernel."""
    if pooled_mfma_ok(q, k_cache, v_cache) and q.shape[1] // k_cache.shape[1] <= 32:
        torch.ops.akap_stream.pooled_window_attention_decode_mfma(
            out, q, k_cache, v_cache, k_pool, v_pool, block_tables, positions, slots,
            float(scale), int(window), int(pool), bool(unit_sink))
        return
    pooled_window_attention(out, q, k_cache, v_cache, k_pool, v_pool, block_tables, None,
                            positions, slots, scale, window, pool, unit_sink)


def pooled_window_attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                                    v_cache: torch.Tensor, k_pool: Optional[torch.Tensor],
                                    v_pool: Optional[torch.Tensor], block_tables: torch.Tensor,
                                    q_start: torch.Tensor, positions: torch.Tensor,
                                    slots: torch.Tensor, tile_seq: torch.Tensor,
                                    tile_row: torch.Tensor, tile_rows: int, scale: float,
                                    window: int, pool: int, unit_sink: bool,
                                    first_seq: int = 0) -> None:
    """pooled_window_attention for a step with prompt chunks.  The tile map (tile_seq, tile_row:
    a sequence and the first chunk row of a tile of tile_rows tokens) covers the sequences from
    first_seq on; the sequences before it are the single rows of a mixed step.  bf16 chunks with
    matrix-core sizes run on the matrix cores (pooled entries rounded to bf16 operands), the
    leading single rows and everything else on the row kernel."""
    if pooled_mfma_ok(q, k_cache, v_cache) and tile_rows == 128 and out.stride(0) % 4 == 0:
        nd = first_seq
        if nd:
            pooled_window_attention_decode(out[:nd], q[:nd], k_cache, v_cache, k_pool, v_pool,
                                           block_tables, positions[:nd], slots[:nd], scale,
                                           window, pool, unit_sink)
        torch.ops.akap_stream.pooled_window_attention_prefill_mfma(
            out, q, k_cache, v_cache, k_pool, v_pool, block_tables, q_start, positions, slots,
            tile_seq, tile_row, int(tile_rows), float(scale), int(window), int(pool),
            bool(unit_sink))
        return
    pooled_window_attention(out, q, k_cache, v_cache, k_pool, v_pool, block_tables, q_start,
                            positions, slots, scale, window, pool, unit_sink)


# ----------------------------------------------------------------------------- selective state space
def conv_silu(out: torch.Tensor, proj: torch.Tensor, off: int, conv_w: torch.Tensor,
              conv_b: torch.Tensor, state: torch.Tensor, seq_slot: torch.Tensor,
              positions: torch.Tensor, q_start: Optional[torch.Tensor]) -> None:
    """Causal per-channel convolution + silu over the columns [off, off + C) of proj [T, N]:
    out[t, c] = silu(conv_b[c] + sum_j conv_w[c, j] u[t - (taps - 1 - j), c]) (fp32 [T, C]),
    u the column of the sequence's earlier tokens: rows of this step, before them what an
    earlier step left in state[slot] ([slots, taps - 1, C], proj's type, oldest first), zeros
    before position 0.  After the step state[slot] holds the sequence's last taps - 1 inputs.
    Sequences as in `retention`: rows [q_start[b], q_start[b + 1]) (None: one row each), slot =
    seq_slot of the first row (-1: padding), fresh when that row has position 0.  conv_w
    [C, taps], conv_b [C] fp32."""
    if _native(proj):
        torch.ops.akap_stream.conv_silu(out, proj, int(off), conv_w, conv_b, state, seq_slot,
                                        positions, q_start)
        return
    C, taps = conv_w.shape
    for r0, r1 in _row_sequences(proj.shape[0], q_start):
        if r1 <= r0 or int(seq_slot[r0]) < 0:
            continue
        slot = int(seq_slot[r0])
        prev = state[slot, :taps - 1].float() if int(positions[r0]) > 0 \
            else torch.zeros(taps - 1, C)
        u = torch.cat([prev, proj[r0:r1, off:off + C].float()])      # [taps - 1 + n, C]
        acc = conv_b.float()[None, :].repeat(r1 - r0, 1)
        for j in range(taps):
            acc = acc + conv_w[:, j].float()[None, :] * u[j:j + r1 - r0]
        out[r0:r1] = torch.nn.functional.silu(acc)
        if taps > 1:
            state[slot, :taps - 1] = u[-(taps - 1):].to(state.dtype)


def selective_scan(y: torch.Tensor, xbc: torch.Tensor, proj: torch.Tensor, dt_off: int,
                   dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
                   state: torch.Tensor, seq_slot: torch.Tensor, positions: torch.Tensor,
                   q_start: Optional[torch.Tensor], H: int, V: int, N: int, G: int) -> None:
    """The state-space recurrence for the token rows of a step, fp32 throughout.  xbc [T, H V +
    2 G N] (fp32) = [x | B | C]; dt_t,h = softplus(proj[t, dt_off + h] + dt_bias[h]) (no
    clamp).  Per head h with group g = h // (H / G):  S <- exp(-exp(a_log[h]) dt) S + dt B_g
    x_h^T (S is [N, V]),  y[t, h V : (h + 1) V] = S^T C_g + d_skip[h] x_h.  The state of a
    sequence lives in state[slot, h] (fp32 [N, V]); sequences, slots and fresh starts as in
    `retention`."""
    if _native(xbc):
        torch.ops.akap_stream.selective_scan(y, xbc, proj, int(dt_off), dt_bias, a_log, d_skip,
                                             state, seq_slot, positions, q_start, H, V, N, G)
        return
    T = xbc.shape[0]
    inner = H * V
    x = xbc[:, :inner].float().view(T, H, V)
    Bm = xbc[:, inner:inner + G * N].float().view(T, G, N).repeat_interleave(H // G, dim=1)
    Cm = xbc[:, inner + G * N:inner + 2 * G * N].float().view(T, G, N).repeat_interleave(
        H // G, dim=1)
    dt = torch.nn.functional.softplus(proj[:, dt_off:dt_off + H].float() + dt_bias.float(),
                                      threshold=30.0)
    decay = torch.exp(-torch.exp(a_log.float())[None, :] * dt)            # [T, H]
    for r0, r1 in _row_sequences(T, q_start):
        if r1 <= r0 or int(seq_slot[r0]) < 0:
            continue
        slot = int(seq_slot[r0])
        S = state[slot].clone() if int(positions[r0]) > 0 else torch.zeros(H, N, V)
        for t in range(r0, r1):
            S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bm[t][:, :, None] \
                * x[t][:, None, :]
            y[t] = (torch.einsum("hnv,hn->hv", S, Cm[t]) + d_skip.float()[:, None] * x[t]
                    ).reshape(inner)
        state[slot] = S


def gate_group_norm(out: torch.Tensor, y: torch.Tensor, gate: torch.Tensor, w: torch.Tensor,
                    groups: int, eps: float) -> None:
    """out = gnorm(y silu(gate)) w: y [T, n] fp32, gate [T, n] (a column slice of a projection),
    the product RMS-normed in `groups` equal consecutive parts (each by its own root mean
    square), times the fp32 weights w [n].  The gate comes before the norm.  fp32 arithmetic."""
    if _native(y):
        torch.ops.akap_stream.gate_group_norm(out, y, gate, w, int(groups), float(eps))
        return
    g = y.float() * torch.nn.functional.silu(gate.float())
    out.copy_((_group_rms(g, groups, eps) * w.float()).to(out.dtype))


# ----------------------------------------------------------------------------- sigmoid group routing
def route_sigmoid(h: torch.Tensor, router: torch.Tensor, top: int, groups: int = 1,
                  keep: int = 1, group_top: int = 2):
    """Routing by sigmoid scores: s = sigmoid(router h) (fp32, from h's stored values); experts
    form `groups` equal groups of neighbours, a group scores the sum of its `group_top` largest
    s, only experts of the `keep` best groups can be chosen (ties: the lower index); the `top`
    largest s among them win (ties: the lower index) and weigh their experts as they are.
    Returns ids int32 [T, top] (by falling score) and weights fp32 [T, top].  router fp32
    [E, d]."""
    T, E = h.shape[0], router.shape[0]
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    w = torch.empty(T, top, dtype=torch.float32, device=h.device)
    if _native(h):
        torch.ops.akap_stream.route_sigmoid(ids, w, h, router, int(groups), int(keep),
                                            int(group_top))
        return ids, w
    s = torch.sigmoid(h.float() @ router.float().T)
    choice = s.clone()
    per = E // groups
    if groups > 1:
        gs = s.view(T, groups, per).topk(min(group_top, per), dim=-1).values.sum(dim=-1)
        best = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        allowed = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        choice = choice.masked_fill(~allowed[:, :, None].expand(T, groups, per).reshape(T, E),
                                    -1.0)
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    ids.copy_(idx)
    w.copy_(s.gather(1, idx))
    return ids, w


def gated_act(gu: torch.Tensor, out: torch.Tensor, act: str = "silu",
              ids: Optional[torch.Tensor] = None, w: Optional[torch.Tensor] = None,
              experts: int = 1) -> None:
    """out[t, e F + f] = w_e(t) act(gu[t, e 2F + f]) gu[t, e 2F + F + f] for gu [T, E 2F] = per
    expert [gate | up]; act "silu" or "gelu_tanh" (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715
    z^3)))); ids / w None: one plain gated layer (weight 1), else the routing weights as in
    swiglu_routed.  fp32 arithmetic; both tensors may be column slices of wider rows."""
    if act not in ("silu", "gelu_tanh"):
        raise ValueError(f"gated_act: unknown activation {act!r}")
    if _native(gu):
        torch.ops.akap_stream.swiglu_routed(out, gu, ids, w, int(experts),
                                            1 if act == "gelu_tanh" else 0)
        return
    T = gu.shape[0]
    F_ = gu.shape[1] // (2 * experts)
    g3 = gu.float().view(T, experts, 2, F_) if gu.is_contiguous() else \
        gu.float().reshape(T, experts, 2, F_)
    a = torch.nn.functional.silu(g3[:, :, 0]) if act == "silu" else \
        torch.nn.functional.gelu(g3[:, :, 0], approximate="tanh")
    r = a * g3[:, :, 1]
    if ids is not None:
        full = torch.zeros(T, experts, dtype=torch.float32)
        full.scatter_(1, ids.long(), w)
        r = r * full[:, :, None]
    out.copy_(r.reshape(T, experts * F_).to(out.dtype))
