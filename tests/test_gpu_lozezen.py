"""The Lozezen design on the GPU against the plain implementation of ``plain_lozezen.py``: every mechanism's kernels
alone, then whole models through the engine's own step function, cache manager and scheduler, cut and batched in every
way that must not change a token's logits."""
from __future__ import annotations

import math
import random

import numpy as np
import pytest
import torch

import plain_lozezen as P
from lozezen_common import (CONFIGS, assert_close, chunk_attention, config, dense, make_folder, parallel, plain_logits, random_weights,
                            retention, tokens_of, window_attention)

pytestmark = pytest.mark.gpu
F64 = torch.float64
TYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL = {"float32": 3e-4, "bfloat16": 6e-2}         # of the largest expected value
SAME = {"float32": 2e-5, "bfloat16": 2.5e-2}      # between two runs of the engine that cut or batch the same tokens differently


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def i32(v):
    return torch.tensor(v, dtype=torch.int32).cuda()


def hand_step(q_lens, ctx_lens, slots, block_table=None, slot_map=None):
    """A step made by hand: requests that feed ``q_lens`` tokens and then hold ``ctx_lens``, in state ``slots``."""
    from llama_cu_amd.engine.batch import StepContext
    n = sum(q_lens)
    starts = [0]
    for x in q_lens:
        starts.append(starts[-1] + x)
    pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
    return StepContext(n=n, n_req=len(q_lens), tokens=i32([0] * n), positions=i32(pos),
                       req_of_token=i32([r for r, x in enumerate(q_lens) for _ in range(x)]), q_start=i32(starts),
                       ctx_len=i32(ctx_lens), state_slot=i32(slots), logit_rows=i32([]), n_logits=0,
                       block_tables=[block_table] if block_table is not None else [],
                       slot_maps=[slot_map] if slot_map is not None else [], q_lens=list(q_lens), ctx_lens=list(ctx_lens),
                       state_slots=list(slots))


# ------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [72, 2048 + 520])
def test_norm_behind_a_sublayer_the_sum_and_the_next_norm(dtype, d):
    from llama_cu_amd.kernels import ops
    n, e1, e2 = 5, 1e-3, 1e-5
    x, a = rnd(n, d, seed=1, std=3.0), rnd(n, d, seed=2, std=0.01).to(TYPES[dtype])       # (a small: the eps counts)
    w1, w2 = rnd(d, seed=3, std=0.2) + 1, rnd(d, seed=4, std=0.2) + 1
    s = x.double().numpy() + P.unit_rms(a.double().numpy(), e1) * w1.double().numpy()
    xg = x.clone().cuda()
    h = ops.norm_post(xg, a.cuda(), w1.cuda(), e1, w2.cuda(), e2, out_dtype=TYPES[dtype])
    assert_close(xg, s, 1e-6, "the stream")
    assert_close(h, P.unit_rms(s, e2) * w2.double().numpy(), 1e-5 if dtype == "float32" else 1e-2, "the next norm")
    xg = x.clone().cuda()
    assert ops.norm_post(xg, a.cuda(), w1.cuda(), e1) is None
    assert_close(xg, s, 1e-6, "the stream alone")


def paged(lens, page, seed):
    """Block tables of shuffled pages for requests of ``lens`` tokens, with pages between them that nobody owns."""
    rng = random.Random(seed)
    need = [(n + page - 1) // page for n in lens]
    order = list(range(sum(need) + 4))
    rng.shuffle(order)
    tables, at = [], 0
    for k in need:
        tables.append(order[at:at + k])
        at += k
    bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
    for r, t in enumerate(tables):
        bt[r, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return tables, bt.cuda(), len(order)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,dv,rot,inter,factor,window,chunk,norm,page", [
    (6, 2, 24, 40, 10, True, 2.5, 19, 0, False, 8),       # a rotation of 10 of 24 dims, neighbours paired, values wider than keys
    (4, 1, 20, 12, 6, False, 1.0, 7, 0, False, 16),       # a head size that is filled up with zeros; halves paired
    (3, 3, 12, 20, 0, False, 1.0, 0, 11, True, 16),       # chunks, a norm per head, no rotation
    (4, 4, 64, 64, 64, True, 8.0, 33, 0, False, 16),      # whole heads rotated
    (2, 1, 32, 32, 0, False, 1.0, 0, 16, True, 16),       # chunks of one page
])
def test_bias_head_norm_rotation_and_attention_within_windows_and_chunks(dtype, nh, nkv, dh, dv, rot, inter, factor, window, chunk, norm, page):
    """Two requests whose keys lie in shuffled pages among pages of NaN, the second fed in three steps (a portion, a
    portion beside a single token of the first, single tokens); the scale is large, so that the softmax is peaked and a
    key that is wrongly seen or wrongly hidden at a window's or a chunk's edge moves the output."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.base import BuildContext
    from llama_cu_amd.parts.position import Rotary
    tdt, eps, scale = TYPES[dtype], 1e-4, 1.7
    lens, cut = [45, 70], 37
    tables, bt, n_pages = paged(lens, page, 5)
    dhp = (dh + 7) // 8 * 8
    cache = torch.full((n_pages, 1, nkv * (dhp + dv) * page), float("nan"), dtype=tdt, device="cuda")
    width = nh * dh + nkv * (dh + dv) + 3                 # (three more columns, as a gate's would be)
    offs = (0, nh * dh, (nh + nkv) * dh)
    bias = rnd(width, seed=1, std=0.3)
    qn, kn = (rnd(dh, seed=2, std=0.2) + 1, rnd(dh, seed=3, std=0.2) + 1) if norm else (None, None)
    cos = sin = None
    if rot:
        part = Rotary(dh, 300.0, 128, interleaved=inter, rot_dim=rot, scaling_factor=factor)
        part.load({}, BuildContext(tdt, torch.device("cuda"), 128, page))
        cos, sin, _, pairing = part.rotary_tables()
    rows = [rnd(n, width, seed=20 + r) for r, n in enumerate(lens)]
    gpu = lambda t: None if t is None else t.cuda()

    def run(q_lens, ctx_lens, chunks):
        pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
        req = [r for r, x in enumerate(q_lens) for _ in range(x)]
        slot = [tables[r][p // page] * page + p % page for r, p in zip(req, pos)]
        step = hand_step(q_lens, ctx_lens, [0, 1], bt, i32(slot))
        q = ops.qkv_prepare(torch.cat(chunks).contiguous().cuda(), offs, nh, nkv, dh, dv, dhp, dv, tdt, positions=step.positions,
                            bias=bias.cuda(), q_norm=gpu(qn), k_norm=gpu(kn), eps=eps, cos=cos, sin=sin, rot_dim=rot,
                            pairing=1 if inter else 0, cache=cache, slots=step.slots(0), page_size=page)
        out = torch.empty(sum(q_lens), nh * dv, dtype=tdt, device="cuda")
        ops.paged_attention(q, out, cache, step, 0, nh, nkv, dhp, page, scale, window, value_dim=dv, chunk=chunk)
        return out.float().cpu()

    a = run([lens[0], cut], [lens[0], cut], [rows[0], rows[1][:cut]])
    b = run([1, lens[1] - cut - 2], [lens[0], lens[1] - 2], [rows[0][-1:], rows[1][cut:-2]])      # request 0's last token once more
    c = run([1, 1], [lens[0], lens[1] - 1], [rows[0][-1:], rows[1][-2:-1]])
    d = run([1, 1], [lens[0], lens[1]], [rows[0][-1:], rows[1][-1:]])
    got = [a[:lens[0]], torch.cat([a[lens[0]:], b[1:], c[1:], d[1:]])]
    for r, x in enumerate(rows):
        T = lens[r]
        x = x.double().numpy() + bias.double().numpy()
        q, k = x[:, :nh * dh].reshape(T, nh, dh), x[:, offs[1]:offs[1] + nkv * dh].reshape(T, nkv, dh)
        v = x[:, offs[2]:offs[2] + nkv * dv].reshape(T, nkv, dv)
        if norm:
            q, k = P.unit_rms(q, eps) * qn.double().numpy(), P.unit_rms(k, eps) * kn.double().numpy()
        if rot:
            q, k = (P.rotate(t, np.arange(T), rot, 300.0, factor, interleaved=inter) for t in (q, k))
        if dtype == "bfloat16":                  # what the cache and the queries hold is rounded
            q, k, v = (torch.from_numpy(t).to(tdt).double().numpy() for t in (q, k, v))
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        visible = (j <= i) & ((i // chunk == j // chunk) if chunk else (i - j < window))
        want = P.masked_softmax_attention(q, k, v, scale, visible)
        assert_close(got[r], want.reshape(T, -1), 1e-4 if dtype == "float32" else 2e-2, f"request {r}")
    # (in bfloat16 the matrix-core kernels for portions and for single tokens round differently)
    assert_close(b[:1], a[lens[0] - 1:lens[0]], 1e-6 if dtype == "float32" else 1e-2, "the same token in another batch")
    assert torch.isnan(cache.float()).any(), "the pages that nobody owns were written"


def test_a_gate_per_head():
    from llama_cu_amd.kernels import ops
    n, nh, dv = 7, 5, 12
    out, gates = rnd(n, nh * dv, seed=1), rnd(n, 9, seed=2, std=2.0)
    got = ops.head_gate(out.clone().cuda(), gates.cuda(), 3, nh, dv)
    want = out.view(n, nh, dv).double() * torch.sigmoid(gates[:, 3:3 + nh].double())[:, :, None]
    assert_close(got, want.view(n, -1), 1e-6)


def cut_runs(T, other_T):
    """Steps that feed one request in portions of 1, 2, 7, ... tokens, a second request beside it from its third step on."""
    done, o_done, portion, k, steps = 0, 0, [1, 2, 7, 1, 3, 16, 1, 2, 4], 0, []
    while done < T:
        take = min(portion[k % len(portion)], T - done)
        o_take = min(3, other_T - o_done) if done >= 3 else 0
        steps.append((done, take, o_done, o_take))
        done, o_done, k = done + take, o_done + o_take, k + 1
    return steps


@pytest.mark.parametrize("dtype,heads,d,dv,rot,inter", [("float32", 3, 24, 16, 12, False), ("float32", 2, 20, 12, 20, False),
                                                       ("float32", 1, 64, 64, 64, False), ("bfloat16", 2, 64, 40, 32, True),
                                                       ("float32", 2, 128, 72, 0, False), ("float32", 1, 136, 8, 8, False)])
def test_retention_against_the_recurrence_in_any_cut(dtype, heads, d, dv, rot, inter):
    """The kernels against the recurrence written out token by token; then the same tokens in portions down to one
    token, beside another request, from slots that held another state: the same outputs and the same last state."""
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.base import BuildContext
    from llama_cu_amd.parts.position import Rotary
    T, eps, tdt = 41, 1e-4, TYPES[dtype]
    hk, hv = heads * d, heads * dv
    off = {"q": 0, "k": hk, "v": 2 * hk, "g": 2 * hk + hv}
    proj, other = rnd(T, 2 * hk + 2 * hv, seed=1), rnd(11, 2 * hk + 2 * hv, seed=2)
    decay = [0.9, 0.999, 0.5][:heads]
    cos = sin = None
    if rot:
        part = Rotary(d, 1000.0, 64, interleaved=inter, rot_dim=rot)
        part.load({}, BuildContext(tdt, torch.device("cuda"), 64, 16))
        cos, sin, _, _ = part.rotary_tables()
    kw = dict(cos=cos, sin=sin, rot_dim=rot, pairing=1 if inter else 0)

    x = proj.double().numpy()
    q, k = x[:, :hk].reshape(T, heads, d), x[:, hk:2 * hk].reshape(T, heads, d)
    v, g = x[:, 2 * hk:2 * hk + hv].reshape(T, heads, dv), x[:, 2 * hk + hv:]
    if rot:
        q, k = (P.rotate(t, np.arange(T), rot, 1000.0, interleaved=inter) for t in (q, k))
    k = k * 0.3
    o, S = np.zeros((T, heads, dv)), np.zeros((heads, d, dv))
    for t in range(T):
        for h in range(heads):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    want = P.unit_rms(o, eps).reshape(T, hv) * P.silu(g)

    rel = 2e-4 if dtype == "float32" else 2e-2
    dec = torch.tensor(decay, dtype=torch.float32).cuda()
    state = torch.full((3, heads, d, dv), 5.0, device="cuda")
    whole = ops.retention(proj.cuda(), off, dec, state, hand_step([T], [T], [1]), heads, d, dv, 0.3, eps, tdt, **kw)
    assert_close(whole, want, rel, "whole")
    assert_close(state[1], S, 2e-4, "state after the whole")
    assert (state[0] == 5.0).all() and (state[2] == 5.0).all()
    state = torch.full((3, heads, d, dv), -3.0, device="cuda")
    got = torch.zeros(T, hv)
    for done, take, o_done, o_take in cut_runs(T, 11):
        rows, q_lens, ctx, slots = [proj[done:done + take]], [take], [done + take], [2]
        if o_take:
            rows.insert(0, other[o_done:o_done + o_take])
            q_lens.insert(0, o_take); ctx.insert(0, o_done + o_take); slots.insert(0, 0)
        out = ops.retention(torch.cat(rows).contiguous().cuda(), off, dec, state, hand_step(q_lens, ctx, slots), heads, d, dv, 0.3, eps, tdt, **kw)
        got[done:done + take] = out[-take:].float().cpu()
    assert_close(got, want, rel, "portions")
    assert_close(state[2], S, 2e-4, "state after the portions")
    assert torch.equal(got, whole.float().cpu()), "a cut changed the bits"


@pytest.mark.parametrize("dtype,width,blocks,taps", [("float32", 72, 3, 3), ("float32", 40, 5, 1), ("float32", 96, 2, 2),
                                                    ("bfloat16", 128, 1, 4), ("float32", 320, 1, 7)])
def test_the_recurrent_unit_against_the_recurrence_in_any_cut(dtype, width, blocks, taps):
    """Convolution, gates, decay and recurrence against the plain mixer's inner part; then in portions down to one
    token (shorter than the convolution), beside another request, from slots that held other rows."""
    from llama_cu_amd.kernels import ops
    T, tdt, bs = 41, TYPES[dtype], width // blocks
    rows, other = rnd(T, 2 * width + 5, seed=1), rnd(11, 2 * width + 5, seed=2)
    bias = rnd(2 * width + 5, seed=3, std=0.3)
    conv_w, conv_b = rnd(width, taps, seed=4, std=0.5), rnd(width, seed=5, std=0.3)
    wa, wi = rnd(blocks, bs, bs, seed=6, std=2 / math.sqrt(bs)), rnd(blocks, bs, bs, seed=7, std=2 / math.sqrt(bs))
    ba, bi, lam = rnd(width, seed=8), rnd(width, seed=9), rnd(width, seed=10, std=1.5) - 2.0
    y_off, x_off = 3, width + 5

    x = rows.double().numpy() + bias.double().numpy()
    y = P.gelu_tanh(x[:, y_off:y_off + width])
    u = P.causal_conv(x[:, x_off:x_off + width], conv_w.double().numpy(), conv_b.double().numpy())
    ub = u.reshape(T, blocks, bs)
    r = P.sigmoid(np.einsum("tbi,boi->tbo", ub, wa.double().numpy()).reshape(T, width) + ba.double().numpy())
    g = P.sigmoid(np.einsum("tbi,boi->tbo", ub, wi.double().numpy()).reshape(T, width) + bi.double().numpy())
    a = np.exp(-8.0 * r * P.softplus(lam.double().numpy()))
    S, want = np.zeros(width), np.zeros((T, width))
    for t in range(T):
        S = a[t] * S + np.sqrt(1 - a[t] ** 2) * g[t] * u[t]
        want[t] = S * y[t]

    args = (y_off, x_off, bias.cuda(), conv_w.cuda(), conv_b.cuda(), wa.transpose(1, 2).contiguous().cuda(),
            wi.transpose(1, 2).contiguous().cuda(), ba.cuda(), bi.cuda(), lam.cuda(), 8.0)
    rel = 2e-4 if dtype == "float32" else 2e-2
    state = torch.full((3, taps, width), 5.0, device="cuda")
    whole = ops.rglru(rows.cuda(), *args, state, hand_step([T], [T], [1]), tdt)
    assert_close(whole, want, rel, "whole")
    assert_close(state[1, taps - 1], S, 2e-4, "the recurrence's state after the whole")
    if taps > 1:
        assert_close(state[1, :taps - 1], x[T - taps + 1:, x_off:x_off + width], 1e-6, "the convolution's last inputs")
    assert (state[0] == 5.0).all() and (state[2] == 5.0).all()
    state = torch.full((3, taps, width), -3.0, device="cuda")
    got = torch.zeros(T, width)
    for done, take, o_done, o_take in cut_runs(T, 11):
        part, q_lens, ctx, slots = [rows[done:done + take]], [take], [done + take], [2]
        if o_take:
            part.insert(0, other[o_done:o_done + o_take])
            q_lens.insert(0, o_take); ctx.insert(0, o_done + o_take); slots.insert(0, 0)
        out = ops.rglru(torch.cat(part).contiguous().cuda(), *args, state, hand_step(q_lens, ctx, slots), tdt)
        got[done:done + take] = out[-take:].float().cpu()
    assert_close(got, want, rel, "portions")
    assert_close(state[2, taps - 1], S, 2e-4, "state after the portions")
    assert torch.equal(got, whole.float().cpu()), "a cut changed the bits"


def test_retention_over_a_long_prompt_cut_into_runs():
    """A request that feeds many tokens is walked in several runs at once, each first from zeros, then from the state
    that the runs before it leave: against the recurrence token by token, beside a short request in the same step, and
    against the same tokens fed in two steps (the second from a state that is not zero)."""
    from llama_cu_amd.kernels import ops
    T, heads, d, dv, eps = 1100, 2, 24, 40, 1e-5
    hk, hv = heads * d, heads * dv
    off = {"q": 0, "k": hk, "v": 2 * hk, "g": 2 * hk + hv}
    proj, short = rnd(T, 2 * hk + 2 * hv, seed=1), rnd(5, 2 * hk + 2 * hv, seed=2)
    decay = [0.97, 0.9995]
    x = proj.double().numpy()
    q, k = x[:, :hk].reshape(T, heads, d), x[:, hk:2 * hk].reshape(T, heads, d) * 0.2
    v, g = x[:, 2 * hk:2 * hk + hv].reshape(T, heads, dv), x[:, 2 * hk + hv:]
    o, S = np.zeros((T, heads, dv)), np.zeros((heads, d, dv))
    for t in range(T):
        for h in range(heads):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    want = P.unit_rms(o, eps).reshape(T, hv) * P.silu(g)
    dec = torch.tensor(decay, dtype=torch.float32).cuda()
    state = torch.full((2, heads, d, dv), 7.0, device="cuda")
    both = ops.retention(torch.cat([short, proj]).cuda(), off, dec, state, hand_step([5, T], [5, T], [0, 1]), heads, d, dv, 0.2, eps, torch.float32)
    assert_close(both[5:], want, 2e-4, "the long request")
    assert_close(state[1], S, 2e-4, "its state")
    state2 = torch.full((2, heads, d, dv), -1.0, device="cuda")
    first = ops.retention(proj[:520].contiguous().cuda(), off, dec, state2, hand_step([520], [520], [1]), heads, d, dv, 0.2, eps, torch.float32)
    second = ops.retention(proj[520:].contiguous().cuda(), off, dec, state2, hand_step([T - 520], [T], [1]), heads, d, dv, 0.2, eps, torch.float32)
    assert_close(torch.cat([first, second]), both[5:], 1e-5, "two steps against one")
    assert_close(state2[1], state[1], 1e-5, "the states after them")


@pytest.mark.parametrize("width,blocks,taps", [(72, 3, 3), (128, 2, 4), (320, 1, 2)])
def test_the_recurrent_unit_over_a_long_prompt_cut_into_runs(width, blocks, taps):
    """A request that feeds many tokens is scanned in several runs at once whose effects are chained: against the
    recurrence token by token, beside a short request in the same step, and against the same tokens fed in two steps.
    (Blocks of 24, 64 and 320 channels: the last are more than a workgroup's threads.)"""
    from llama_cu_amd.kernels import ops
    T = 1100
    bs = width // blocks
    rows, short = rnd(T, 2 * width, seed=1), rnd(5, 2 * width, seed=2)
    bias = rnd(2 * width, seed=3, std=0.3)
    conv_w, conv_b = rnd(width, taps, seed=4, std=0.5), rnd(width, seed=5, std=0.3)
    wa, wi = rnd(blocks, bs, bs, seed=6, std=2 / math.sqrt(bs)), rnd(blocks, bs, bs, seed=7, std=2 / math.sqrt(bs))
    ba, bi, lam = rnd(width, seed=8), rnd(width, seed=9), rnd(width, seed=10, std=1.5) - 4.0       # (decays close to 1: a long memory)
    names = {"y": "y", "x": "x", "conv": "conv", "ra": "ra", "ri": "ri", "lam": "lam", "o": "o"}
    w = {"y": torch.eye(2 * width)[:width], "y.b": bias[:width], "x": torch.eye(2 * width)[width:], "x.b": bias[width:], "conv": conv_w,
         "conv.b": conv_b, "ra": wa, "ra.b": ba.view(blocks, bs), "ri": wi, "ri.b": bi.view(blocks, bs), "lam": lam, "o": torch.eye(width)}
    w = {k: v.double().numpy() for k, v in w.items()}
    want = P.rglru(rows.double().numpy(), w, "", {"width": width, "blocks": blocks})
    args = (0, width, bias.cuda(), conv_w.cuda(), conv_b.cuda(), wa.transpose(1, 2).contiguous().cuda(),
            wi.transpose(1, 2).contiguous().cuda(), ba.cuda(), bi.cuda(), lam.cuda(), 8.0)
    state = torch.full((2, taps, width), 7.0, device="cuda")
    both = ops.rglru(torch.cat([short, rows]).cuda(), *args, state, hand_step([5, T], [5, T], [0, 1]), torch.float32)
    assert_close(both[5:], want, 2e-4, "the long request")
    state2 = torch.full((2, taps, width), -1.0, device="cuda")
    first = ops.rglru(rows[:600].contiguous().cuda(), *args, state2, hand_step([600], [600], [1]), torch.float32)
    second = ops.rglru(rows[600:].contiguous().cuda(), *args, state2, hand_step([T - 600], [T], [1]), torch.float32)
    assert_close(torch.cat([first, second]), both[5:], 1e-5, "two steps against one")
    assert_close(state2[1], state[1], 1e-5, "the states after them")


# ------------------------------------------------------------------ whole models through the engine


_made = {}


def model(name, sharp=1.0):
    """(configuration, weights, folder) of a test model, made once."""
    key = (name, sharp)
    if key not in _made:
        cfg = CONFIGS[name]
        w = random_weights(cfg, 1 + sorted(CONFIGS).index(name), sharp_keys=sharp)
        _made[key] = (cfg, w, make_folder(cfg, w))
    return _made[key]


def runner_for(folder, dtype, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    args = dict(dtype=dtype, page_size=16, max_tokens=1024, max_seqs=4, max_batch_tokens=1024)
    args.update(kw)
    return ModelRunner.from_folder(folder, **args)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16"), ("C", "float32"),
                                        ("C", "bfloat16"), ("D", "float32"), ("E", "float32")])
def test_a_whole_prompt_against_the_plain_model(name, dtype):
    cfg, w, folder = model(name)
    toks = tokens_of(cfg["vocab"], 100, 1)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, dtype)
    got = r.step([0], [toks], [list(range(len(toks)))])
    assert_close(got, want, REL[dtype], f"model {name} in {dtype}")
    r.end(0)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("D", "float32"), ("E", "float32"), ("E", "bfloat16"), ("C", "float32")])
def test_models_of_one_kind_of_mixer_and_the_first_tokens_of_a_sequence(name, dtype):
    """Recurrent layers alone (no pages at all) and attention alone (no state): a prompt in portions, then tokens one by
    one, a second request beside the first that starts with portions of one and two tokens, a slot used again."""
    cfg, w, folder = model(name)
    a, b = tokens_of(cfg["vocab"], 40, 50), tokens_of(cfg["vocab"], 21, 51)
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    r = runner_for(folder, dtype, max_seqs=2, max_tokens=128)
    got_a = [r.step([0], [a[:17]], [list(range(17))]).clone()]
    out = r.step([0, 1], [a[17:30], b[:1]], [list(range(13)), [0]]).clone()
    got_a.append(out[:13])
    got_b = [out[13:]]
    out = r.step([1, 0], [b[1:3], a[30:31]], [[0, 1], [0]]).clone()
    got_b.append(out[:2]); got_a.append(out[2:])
    got_b.append(r.step([1], [b[3:]], [list(range(18))]).clone())
    r.end(1)
    got_a += [r.step([0], [[t]], [[0]]).clone() for t in a[31:]]
    assert_close(torch.cat(got_a), wa, REL[dtype], "first request")
    assert_close(torch.cat(got_b), wb, REL[dtype], "second request")
    again = r.step([2], [b], [list(range(21))])          # in the slot (and pages) that the second request held
    assert_close(again, wb, REL[dtype], "the slot used again")
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32")])
def test_prefill_against_token_by_token_decoding_and_portions_down_to_two_tokens(name, dtype):
    cfg, w, folder = model(name)
    toks = tokens_of(cfg["vocab"], 90, 2)
    r = runner_for(folder, dtype)
    whole = r.step([0], [toks], [list(range(len(toks)))]).clone()
    want = plain_logits(cfg, w, toks)
    # one token at a time from the first (long enough for captured graphs to replay)
    single = torch.cat([r.step([1], [[t]], [[0]]).clone() for t in toks])
    assert_close(single, want, REL[dtype], "token by token")
    sizes, at, parts = [2, 3, 5, 1, 17, 2, 31, 4, 2, 1, 64], 0, []
    for k in range(100):
        if at >= len(toks):
            break
        take = toks[at:at + sizes[k % len(sizes)]]
        parts.append(r.step([2], [take], [list(range(len(take)))]).clone())
        at += len(take)
    portions = torch.cat(parts)
    assert_close(portions, want, REL[dtype], "portions")
    assert_close(single, whole, SAME[dtype], "token by token against the whole prompt")
    assert_close(portions, whole, SAME[dtype], "portions against the whole prompt")
    if r.use_graphs:
        assert sum(r.graph_replays.values()) > 50, "decoding was not replayed from captured graphs"
    for i in range(3):
        r.end(i)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_batches_of_unequal_requests_and_slots_and_pages_used_again(name, dtype):
    """Seven requests of unequal lengths through an engine with three slots and a pool that holds only what is live:
    portions of some beside single tokens of others; finished requests give their pages and slots to new ones
    (pages that change hands are filled with NaN first).  Every request's logits equal those it gets alone."""
    cfg, w, folder = model(name, sharp=4.0)
    lens = [70, 33, 1, 48, 19, 90, 7]
    reqs = [tokens_of(cfg["vocab"], n, 10 + i) for i, n in enumerate(lens)]
    r = runner_for(folder, dtype, max_seqs=3, max_tokens=3 * 96, max_batch_tokens=256, poison_freed=True)
    if dtype == "float32":
        want = [plain_logits(cfg, w, t) for t in reqs]
    else:       # each alone through the engine: with keys this sharp a bfloat16 run is compared with another of its own
        want = []
        for i, t in enumerate(reqs):
            want.append(r.step([100 + i], [t], [list(range(len(t)))]).clone())
            r.end(100 + i)
    rng = random.Random(3)
    waiting, live, done = list(range(len(reqs))), {}, {i: [] for i in range(len(reqs))}
    slots_seen = {}
    while waiting or live:
        while waiting and len(live) < 3:
            live[waiting.pop(0)] = 0
        ids, toks = [], []
        for i, at in live.items():
            left = len(reqs[i]) - at
            take = 1 if (left <= 12 or rng.random() < 0.3) else min(left - 12, rng.choice([2, 3, 9, 16, 25]))
            ids.append(i); toks.append(reqs[i][at:at + take])
        out = r.step(ids, toks, [list(range(len(t))) for t in toks]).clone()
        at = 0
        for i, t in zip(ids, toks):
            slots_seen.setdefault(r.cache.slot(i), set()).add(i)
            done[i].append(out[at:at + len(t)])
            at += len(t)
            live[i] += len(t)
            if live[i] == len(reqs[i]):
                del live[i]
                r.end(i)
        r.cache.check()
    assert max(len(v) for v in slots_seen.values()) >= 2, "no slot was used again"
    for i in range(len(reqs)):
        assert_close(torch.cat(done[i]), want[i], REL[dtype] if dtype == "float32" else SAME[dtype], f"request {i} of {lens[i]} tokens")


@pytest.mark.parametrize("name", ["A", "B"])
def test_keys_far_back_at_page_borders_and_at_the_edges_of_windows_and_chunks(name):
    """Sharp keys make single keys carry an output, so one that is lost, or seen from outside its window or chunk,
    shows; 330 tokens over pages of 16 (windows and chunks that are whole pages in B, odd sizes in A), cut inside pages,
    windows and chunks, the last 70 decoded one by one: every position's logits against the plain model, in 32-bit."""
    cfg, w, folder = model(name, sharp=6.0)
    toks = tokens_of(cfg["vocab"], 330, 7)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, "float32")
    parts = [r.step([0], [toks[:127]], [list(range(127))]).clone(), r.step([0], [toks[127:260]], [list(range(133))]).clone()]
    parts += [r.step([0], [[t]], [[0]]).clone() for t in toks[260:]]
    assert_close(torch.cat(parts), want, REL["float32"], "far keys")
    r.end(0)
    r.cache.check()


def test_long_decoding_in_bfloat16():
    cfg, w, folder = model("B")
    toks = tokens_of(cfg["vocab"], 260, 8)
    r = runner_for(folder, "bfloat16")
    want = r.step([1], [toks], [list(range(260))]).clone()
    got = [r.step([0], [toks[:20]], [list(range(20))]).clone()] + [r.step([0], [[t]], [[0]]).clone() for t in toks[20:]]
    assert_close(torch.cat(got), want, SAME["bfloat16"], "long decoding against the whole prompt")
    assert_close(want, plain_logits(cfg, w, toks), REL["bfloat16"], "the whole prompt against the plain model")
    assert sum(r.graph_replays.values()) > 100, "decoding was not replayed from captured graphs"


def test_logits_do_not_depend_on_the_cut_or_the_batch_in_32_bit():
    cfg, w, folder = model("A")
    a, b = tokens_of(cfg["vocab"], 60, 20), tokens_of(cfg["vocab"], 41, 21)
    r = runner_for(folder, "float32")
    alone = r.step([0], [a], [list(range(60))]).clone()
    r.step([1], [b[:30]], [[]])
    p1 = r.step([2, 1], [a[:17], b[30:31]], [list(range(17)), [0]]).clone()
    p2 = r.step([1, 2], [b[31:], a[17:]], [[], list(range(43))]).clone()
    assert_close(torch.cat([p1[:17], p2]), alone, 2e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine_and_its_scheduler(dtype):
    """The framework's entry point: prompts of unequal lengths, more than run at a time, prefilled in portions; the
    generated tokens equal the plain model's arg-max continuation."""
    from llama_cu_amd.engine.engine import Engine
    cfg, w, folder = model("B")
    prompts = [tokens_of(cfg["vocab"], n, 30 + i) for i, n in enumerate([21, 5, 40, 2, 13])]
    steps = 12
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=512, max_seqs=3, prefill_chunk=16)
    got = engine.generate(prompts, max_steps=steps, ignore_eos=True)
    for k, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == steps
        seq = list(p) + list(g)
        logits = plain_logits(cfg, w, seq)[list(range(len(p) - 1, len(seq) - 1))]
        if dtype == "float32":
            assert torch.argmax(logits, -1).tolist() == list(g), f"prompt {k}"
        else:               # a close call may fall the other way
            for j, tok in enumerate(g):
                assert logits[j].max() - logits[j, tok] <= 0.06 * logits[j].abs().max(), f"prompt {k}, token {j}: {tok} is not the best"
    engine.runner.cache.check()


def test_trace_replay_of_the_design(tmp_path):
    """The replay program's own path: steps as JSON objects, logits as arrays; four state slots and a pool for what is
    live, so that slots and pages change hands."""
    from llama_cu_amd.engine.trace import TraceReplayer
    cfg, w, folder = model("A")
    seqs = {n: tokens_of(cfg["vocab"], k, 40 + i) for i, (n, k) in enumerate([("x", 50), ("y", 30), ("z", 64), ("u", 9), ("v", 40)])}
    rep = TraceReplayer.open(folder, "float32", 256, max_live=4)
    out0 = rep.step({"step": 0, "entries": [{"id": "x", "tokens": seqs["x"][:33], "want": [0, 32]}], "end": []})
    out1 = rep.step({"step": 1, "entries": [{"id": "x", "tokens": seqs["x"][33:], "want": [16]}, {"id": "y", "tokens": seqs["y"], "want": [29]},
                                            {"id": "z", "tokens": seqs["z"], "want": [63]}, {"id": "u", "tokens": seqs["u"][:2], "want": []}],
                     "end": ["x", "y"]})
    out2 = rep.step({"step": 2, "entries": [{"id": "u", "tokens": seqs["u"][2:], "want": [6]}, {"id": "v", "tokens": seqs["v"], "want": [0, 39]}],
                     "end": ["u", "v", "z"]})
    want = {n: plain_logits(cfg, w, t) for n, t in seqs.items()}
    assert_close(out0, want["x"][[0, 32]], REL["float32"])
    assert_close(out1, torch.stack([want["x"][49], want["y"][29], want["z"][63]]), REL["float32"])
    assert_close(out2, torch.stack([want["u"][8], want["v"][0], want["v"][39]]), REL["float32"])


def test_the_command_line_writes_a_random_model_generates_from_it_and_replays_a_trace(tmp_path):
    """``random-model`` writes a folder of the design from a configuration; ``generate`` continues a prompt from it;
    ``bin/trace_run`` (the program itself, steps on its standard input) gives the plain model's logits for the folder's
    weights."""
    import json
    import os
    import subprocess

    from llama_cu_amd.weights import open_safetensors
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = config(288, 96, [
        {"type": "rglru", "mixer": {"width": 96, "blocks": 2, "conv": 3}, "mlp": None},
        {"type": "parallel", "mixer": parallel(chunk_attention(4, 2, 16, 16, 0.25, 24), retention(2, 32, 24, [0.9, 0.99], 16), 0.8, 1.1),
         "mlp": dense(48)},
        {"type": "attention", "mixer": window_attention(4, 2, 32, 24, 0.2, 20, 16, factor=2.0), "mlp": dense(64)},
    ], eps=1e-5, scale=4.0)
    cfg_path, folder, out = str(tmp_path / "c.json"), str(tmp_path / "m"), str(tmp_path / "out")
    with open(cfg_path, "w") as f:
        json.dump(cfg, f)
    tool = os.path.join(root, "bin", "llama.cu_amd")
    p = subprocess.run([tool, "random-model", cfg_path, folder, "--seed", "3", "--std", "0.1"], capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    p = subprocess.run([tool, "generate", folder, "--max-steps", "6", "-p", "Hi", "--dtype", "float32", "--max-tokens", "256",
                        "--max-seqs", "2"], capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    assert p.stdout.startswith(b"Hi") and b"n toks = 6" in p.stderr
    files = open_safetensors(folder)
    w = {n: f.tensor(n).float() for f in files for n in f.names()}
    a, b = tokens_of(288, 30, 60), tokens_of(288, 12, 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:19], "want": [18]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[19:], "want": [0, 10]}, {"id": "b", "tokens": b, "want": [11]}], "end": ["a"]},
             {"step": 2, "entries": [{"id": "b", "tokens": [5], "want": [0]}], "end": ["b"]}]
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps).encode(), capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    assert [l for l in p.stdout.decode().splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b + [5])
    got = [torch.from_numpy(np.fromfile(os.path.join(out, f"{k}.f32"), dtype="<f4").reshape(-1, 288)) for k in range(3)]
    assert_close(got[0], wa[[18]], REL["float32"])
    assert_close(got[1], torch.stack([wa[19], wa[29], wb[11]]), REL["float32"])
    assert_close(got[2], wb[[12]], REL["float32"])
