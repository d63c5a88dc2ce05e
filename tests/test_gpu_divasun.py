"""The Divasun design on the GPU against the plain implementation of ``plain_divasun.py``: every mechanism's
kernels alone, then whole models through the engine's own step function, cache manager and scheduler, cut and
batched in every way that must not change a token's logits."""
from __future__ import annotations

import math
import random

import pytest
import torch

import plain_divasun as P
from divasun_common import (CFG_A, CFG_B, CFG_C1, CFG_C2, CFG_D, CFG_E, CFG_F, RANKS_A, RANKS_B, RANKS_C, RANKS_D, assert_close, make_folder,
                            plain_logits, random_weights, safe_tokens, tokens_of)

pytestmark = pytest.mark.gpu
F64 = torch.float64
TYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL = {"float32": 3e-4, "bfloat16": 6e-2}         # of the largest expected value
SAME = {"float32": 2e-5, "bfloat16": 2e-2}        # between two runs of the engine that cut or batch the same tokens differently


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def hand_step(q_lens, ctx_lens, slots):
    """A step made by hand: requests that feed ``q_lens`` tokens and then hold ``ctx_lens``, in state ``slots``."""
    from llama_cu_amd.engine.batch import StepContext
    n = sum(q_lens)
    starts = [0]
    for x in q_lens:
        starts.append(starts[-1] + x)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
    pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
    return StepContext(n=n, n_req=len(q_lens), tokens=i32([0] * n), positions=i32(pos),
                       req_of_token=i32([r for r, x in enumerate(q_lens) for _ in range(x)]), q_start=i32(starts),
                       ctx_len=i32(ctx_lens), state_slot=i32(slots), logit_rows=i32([]), n_logits=0, block_tables=[],
                       slot_maps=[], q_lens=list(q_lens), ctx_lens=list(ctx_lens), state_slots=list(slots))


# ------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_norm_adds_the_branch_and_norms_twice(dtype):
    from llama_cu_amd.kernels import ops
    n, d, eps = 5, 88, 1e-3
    x, delta = rnd(n, d, seed=1, std=3.0) + 2.0, rnd(2, n, d, seed=2)
    w1, b1, w2, b2 = rnd(d, seed=3) + 1, rnd(d, seed=4), rnd(d, seed=5) + 1, rnd(d, seed=6)
    xg = x.clone().cuda()
    o1 = torch.empty(n, d, dtype=TYPES[dtype], device="cuda")
    o2 = torch.empty_like(o1)
    ops.layernorm(xg, w1.cuda(), b1.cuda(), eps, o1, delta=delta.cuda(), weight2=w2.cuda(), bias2=b2.cuda(), out2=o2)
    s = (x + delta[0] + delta[1]).to(F64)
    assert_close(xg, s, 1e-6, "residual sum")
    assert_close(o1, P.layer_norm(s, w1.to(F64), b1.to(F64), eps), 1e-5 if dtype == "float32" else 1e-2, "first norm")
    assert_close(o2, P.layer_norm(s, w2.to(F64), b2.to(F64), eps), 1e-5 if dtype == "float32" else 1e-2, "second norm")
    # a row of equal values has no variance: the bias alone comes out
    flat = torch.full((1, d), 7.0).cuda()
    o = torch.empty(1, d, dtype=torch.float32, device="cuda")
    ops.layernorm(flat, w1.cuda(), b1.cuda(), eps, o)
    assert_close(o, b1[None].to(F64), 1e-5, "no variance")


def test_scaled_embedding():
    from llama_cu_amd.kernels import ops
    table = rnd(11, 24, seed=1).to(torch.bfloat16)
    ids = torch.tensor([3, 0, 10], dtype=torch.int32).cuda()
    out = torch.empty(3, 24, dtype=torch.float32, device="cuda")
    ops.embedding_gather(table.cuda(), ids, out, 2.5)
    assert_close(out, table[[3, 0, 10]].to(F64) * 2.5, 1e-6)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_convolution_carries_its_inputs_over_any_cut(taps):
    """Two requests in slots that held other requests' rows, fed in portions of 1, 2, 3, ... tokens: every output
    equals the convolution over the whole sequence, the first tokens (zeros before the start) included."""
    from llama_cu_amd.kernels import ops
    d, sets, lens = 40, 2, [23, 9]
    h = [rnd(sets, n, d, seed=10 + i) for i, n in enumerate(lens)]
    w = rnd(sets, d, taps, seed=3, std=0.5)
    want = [torch.stack([P.short_conv(x[s].to(F64), w[s].to(F64)) for s in range(sets)]) for x in h]
    state = torch.full((3, sets, max(taps - 1, 0), d), float("nan"), device="cuda") if taps > 1 else torch.empty(3, sets, 0, d, device="cuda")
    if taps > 1:
        state[:] = 99.0                       # what an earlier owner of the slots left
    done, portion = [0, 0], 1
    got = [torch.zeros(sets, n, d) for n in lens]
    while any(a < n for a, n in zip(done, lens)):
        take = [min(portion, n - a) for a, n in zip(done, lens)]
        live = [r for r in range(2) if take[r] > 0]
        step = hand_step([take[r] for r in live], [done[r] + take[r] for r in live], [2 - r for r in live])
        rows = torch.cat([h[r][:, done[r]:done[r] + take[r]] for r in live], dim=1).contiguous().cuda()
        out = ops.short_conv(rows, w.cuda(), state, torch.empty_like(rows), step).cpu()
        at = 0
        for r in live:
            got[r][:, done[r]:done[r] + take[r]] = out[:, at:at + take[r]]
            at += take[r]
            done[r] += take[r]
        portion = portion % 5 + 1
    for r in range(2):
        assert_close(got[r], want[r], 1e-5, f"request {r}")


@pytest.mark.parametrize("dtype,heads,dim,rank", [("float32", 3, 32, 5), ("float32", 2, 20, 3), ("float32", 1, 64, 8),
                                                  ("bfloat16", 2, 64, 4), ("float32", 2, 128, 2), ("float32", 1, 72, 1)])
def test_delta_rule_against_the_recurrence_in_any_cut(dtype, heads, dim, rank):
    """The kernels against the recurrence written out token by token; then the same tokens in portions down to one
    token, beside another request, from slots that held another state: the same outputs and the same last state."""
    from llama_cu_amd.kernels import ops
    T, hd, eps = 37, heads * dim, 1e-4
    tdt = TYPES[dtype]
    cols = 5 * hd + rank
    proj = rnd(T, cols, seed=1).to(tdt)
    other = rnd(11, cols, seed=2).to(tdt)
    w2, w0, ab, nw = rnd(hd, rank, seed=3), rnd(hd, seed=4), rnd(hd, seed=5), rnd(hd, seed=6) + 1
    off = {"r": 0, "k": hd, "v": 2 * hd, "g": 3 * hd, "a": 4 * hd, "l": 5 * hd}

    def plain(rows):
        x = rows.to(F64)
        r, k, v, g, a, l = [x[:, off[c]:off[c] + (rank if c == "l" else hd)] for c in ("r", "k", "v", "g", "a", "l")]
        k3, v3, r3 = k.view(-1, heads, dim), v.view(-1, heads, dim), r.view(-1, heads, dim)
        decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(l) @ w2.to(F64).T + w0.to(F64))).view(-1, heads, dim)
        rate = torch.sigmoid(a + ab.to(F64)).view(-1, heads, dim)
        unit = k3 / torch.sqrt((k3 * k3).sum(-1, keepdim=True) + 1e-6)
        S = torch.zeros(heads, dim, dim, dtype=F64)
        outs = []
        for t in range(x.shape[0]):
            seen = torch.einsum("hi,hij->hj", unit[t], S)
            S = decay[t][:, :, None] * S - (rate[t] * unit[t])[:, :, None] * seen[:, None, :] + k3[t][:, :, None] * v3[t][:, None, :]
            outs.append(torch.einsum("hij,hi->hj", S, r3[t]))
        o = P.rms_unit(torch.stack(outs), eps).reshape(-1, hd) * nw.to(F64) * torch.sigmoid(g)
        return o, S

    want, want_state = plain(proj)
    args = (off, w2.t().contiguous().cuda(), w0.cuda(), ab.cuda(), nw.cuda())
    rel = 2e-4 if dtype == "float32" else 2e-2
    state = torch.full((3, heads, dim, dim), 5.0, device="cuda")
    whole = ops.delta_rule(proj.cuda(), *args, state, hand_step([T], [T], [1]), heads, dim, dim, eps)
    assert_close(whole, want, rel, "whole")
    assert_close(state[1], want_state, rel, "state after the whole")
    assert (state[0] == 5.0).all() and (state[2] == 5.0).all()
    # in portions, beside another request that starts later and ends earlier
    state = torch.full((3, heads, dim, dim), -3.0, device="cuda")
    got = torch.zeros(T, hd)
    done, o_done, portion, k = 0, 0, [1, 2, 7, 1, 3, 16, 1, 2, 4], 0
    while done < T:
        take = min(portion[k % len(portion)], T - done)
        o_take = min(3, 11 - o_done) if done >= 3 else 0
        rows, q_lens, ctx, slots = [proj[done:done + take]], [take], [done + take], [2]
        if o_take:
            rows.insert(0, other[o_done:o_done + o_take])
            q_lens.insert(0, o_take); ctx.insert(0, o_done + o_take); slots.insert(0, 0)
        out = ops.delta_rule(torch.cat(rows).contiguous().cuda(), *args, state, hand_step(q_lens, ctx, slots), heads, dim, dim, eps)
        got[done:done + take] = out[-take:].float().cpu()
        done, o_done, k = done + take, o_done + o_take, k + 1
    assert_close(got, want, rel, "portions")
    assert_close(state[2], want_state, rel, "state after the portions")
    if dtype == "float32":
        assert torch.equal(got, whole.float().cpu()), "a cut changed the bits"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,top,ff,n", [(5, 2, 40, 33), (12, 1, 24, 150), (3, 3, 16, 1), (9, 4, 72, 70), (4, 2, 136, 300), (3, 1, 200, 260)])
def test_mixture_of_experts(dtype, experts, top, ff, n):
    from llama_cu_amd.kernels import ops
    d, tdt = 72, TYPES[dtype]
    h = rnd(n, d, seed=1).to(tdt)
    w = {"router": rnd(experts, d, seed=2, std=0.5)}
    for e in range(experts):
        w[f"e{e}.up"] = rnd(ff, d, seed=10 + e, std=d ** -0.5).to(tdt).float()
        w[f"e{e}.down"] = rnd(d, ff, seed=50 + e, std=ff ** -0.5).to(tdt).float()
    base = rnd(n, d, seed=3)
    want = base.to(F64) + P.moe(h.to(F64), {k: v.to(F64) for k, v in w.items()}, experts, top)
    ids, wts = ops.moe_route(h.cuda(), w["router"].cuda(), top)
    s = torch.sigmoid(h.to(F64) @ w["router"].to(F64).T)
    order = torch.argsort(-s, dim=-1, stable=True)[:, :top]
    assert torch.equal(ids.cpu().long(), order), "chosen experts"
    assert_close(wts, torch.gather(s, 1, order), 1e-5, "weights")
    up = torch.stack([w[f"e{e}.up"] for e in range(experts)]).to(tdt).cuda()
    down = torch.stack([w[f"e{e}.down"] for e in range(experts)]).to(tdt).cuda()
    out = base.clone().cuda()
    ops.moe_experts(h.cuda(), ids, wts, up, down, out)
    assert_close(out, want, 1e-4 if dtype == "float32" else 3e-2, "output")
    # a row's result does not depend on what else is in the batch
    one = base[:1].clone().cuda()
    i1, w1 = ops.moe_route(h[:1].cuda(), w["router"].cuda(), top)
    ops.moe_experts(h[:1].cuda(), i1, w1, up, down, one)
    assert torch.equal(one[0], out[0]), "the batch changed a row's bits"


def test_router_ties_go_to_the_lower_index_and_the_weight_multiplies_the_input():
    from llama_cu_amd.kernels import ops
    d = 8
    h = torch.ones(1, d).cuda()
    router = torch.zeros(4, d)
    router[1] = router[3] = 0.25                       # experts 1 and 3 tie at logit 2
    ids, wts = ops.moe_route(h, router.cuda(), 1)
    assert ids.item() == 1 and abs(wts.item() - 1 / (1 + math.exp(-2.0))) < 1e-6
    # gelu is not linear: weight * gelu(up h) would differ from gelu(up (weight * h))
    up = torch.zeros(4, 4, d)
    up[1, :, 0] = 3.0
    down = torch.ones(4, d, 4)
    out = torch.zeros(1, d).cuda()
    ops.moe_experts(h, ids, wts, up.cuda(), down.cuda(), out)
    z = 3.0 * wts.item()
    want = 4 * 0.5 * z * (1 + math.erf(z / math.sqrt(2)))
    assert abs(out[0, 0].item() - want) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,dv,page", [(6, 2, 24, 16, 8), (4, 1, 64, 64, 16), (2, 2, 16, 40, 16)])
def test_attention_norm_temperature_bias_and_values_of_their_own_size(dtype, nh, nkv, dh, dv, page):
    """Two requests whose keys lie in shuffled pages among pages of NaN, the second fed in two steps; one key far
    back is made to stand out for the last query of every head."""
    from llama_cu_amd.engine.batch import StepContext
    from llama_cu_amd.kernels import ops
    from llama_cu_amd.parts.position import DistanceBias
    tdt, eps, scale, coef, every = TYPES[dtype], 1e-4, 0.3, 0.4, 5
    lens, cut = [45, 70], 50
    rng = random.Random(5)
    need = [(n + page - 1) // page for n in lens]
    order = list(range(sum(need) + 4))
    rng.shuffle(order)
    tables = [order[:need[0]], order[need[0]:need[0] + need[1]]]
    cache = torch.full((len(order), 1, nkv * (dh + dv) * page), float("nan"), dtype=tdt, device="cuda")
    qw, kw = rnd(nh * dh, seed=1) + 1, (rnd(nkv * dh, seed=2) + 1) * 3
    slopes = torch.tensor(DistanceBias(nh).host_slopes()).cuda()
    assert abs(slopes[0].item() - 2 ** (-8 / nh)) < 1e-7 and abs(slopes[-1].item() - 2 ** -8) < 1e-9
    rows = [rnd(n, nh * dh + nkv * (dh + dv), seed=20 + r).to(tdt) for r, n in enumerate(lens)]
    for r, x in enumerate(rows):                  # key 2 of every group points where the last query of its first head points
        for g in range(nkv):
            x[2, nh * dh + g * dh:nh * dh + (g + 1) * dh] = x[-1, g * (nh // nkv) * dh:(g * (nh // nkv) + 1) * dh] * 2
    max_pages = max(need)
    bt = torch.zeros(2, max_pages, dtype=torch.int32)
    for r, t in enumerate(tables):
        bt[r, :len(t)] = torch.tensor(t, dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32).cuda()

    def run(q_lens, ctx_lens, chunks):
        n = sum(q_lens)
        pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
        req = [r for r, x in enumerate(q_lens) for _ in range(x)]
        slot = [tables[r][p // page] * page + p % page for r, p in zip(req, pos)]
        starts = [0, q_lens[0], n]
        step = StepContext(n=n, n_req=2, tokens=i32([0] * n), positions=i32(pos), req_of_token=i32(req), q_start=i32(starts),
                           ctx_len=i32(ctx_lens), state_slot=i32([0, 1]), logit_rows=i32([]), n_logits=0,
                           block_tables=[bt.cuda()], slot_maps=[i32(slot)], q_lens=q_lens, ctx_lens=ctx_lens)
        qkv = torch.cat(chunks).contiguous().cuda()
        ops.qk_norm_store(qkv, step.positions, nh, nkv, dh, dv, qw.cuda(), kw.cuda(), eps, coef, every, cache, step.slots(0), page)
        out = torch.empty(n, nh * dv, dtype=tdt, device="cuda")
        ops.paged_attention(qkv, out, cache, step, 0, nh, nkv, dh, page, scale, head_slopes=slopes, value_dim=dv)
        return out.float().cpu()

    a = run([lens[0], cut], [lens[0], cut], [rows[0], rows[1][:cut]])
    b = run([1, lens[1] - cut - 1], [lens[0], lens[1] - 1], [rows[0][-1:], rows[1][cut:-1]])      # request 0's last token once more
    c = run([1, 1], [lens[0], lens[1]], [rows[0][-1:], rows[1][-1:]])
    got = [a[:lens[0]], torch.cat([a[lens[0]:], b[1:], c[1:]])]
    for r, x in enumerate(rows):
        x = x.to(F64)
        q = P.rms_unit(x[:, :nh * dh], eps) * qw.to(F64)
        pos = torch.arange(lens[r])
        q = (q * (1 + coef * torch.log(torch.floor((pos + 1).to(F64) / every) + 1))[:, None]).view(-1, nh, dh)
        k = (P.rms_unit(x[:, nh * dh:(nh + nkv) * dh], eps) * kw.to(F64)).view(-1, nkv, dh)
        v = x[:, (nh + nkv) * dh:].view(-1, nkv, dv)
        if dtype == "bfloat16":                  # what the cache and the queries hold is rounded
            q, k = q.to(tdt).to(F64), k.to(tdt).to(F64)
        want = torch.zeros(lens[r], nh, dv, dtype=F64)
        for hd in range(nh):
            g = hd // (nh // nkv)
            s = (q[:, hd] @ k[:, g].T) * scale - (2.0 ** (-8.0 * (hd + 1) / nh)) * (pos[:, None] - pos[None, :]).to(F64)
            s = s.masked_fill(pos[None, :] > pos[:, None], float("-inf"))
            want[:, hd] = torch.softmax(s, -1) @ v[:, g]
        assert_close(got[r], want.reshape(lens[r], -1), 1e-4 if dtype == "float32" else 2e-2, f"request {r}")
    assert_close(b[:1], a[lens[0] - 1:lens[0]], 1e-6, "the same token in another batch")


# ------------------------------------------------------------------ whole models through the engine


_made = {}


def model(name, sharp=1.0):
    """(configuration, weights, folder) of a test model, made once."""
    key = (name, sharp)
    if key not in _made:
        cfg, ranks, seed = {"A": (CFG_A, RANKS_A, 1), "B": (CFG_B, RANKS_B, 2), "C1": (CFG_C1, RANKS_C, 3), "C2": (CFG_C2, RANKS_C, 4),
                            "D": (CFG_D, RANKS_D, 5), "E": (CFG_E, {}, 6), "F": (CFG_F, {}, 7)}[name]
        w = random_weights(cfg, ranks, seed, sharp_keys=sharp)
        _made[key] = (cfg, w, make_folder(cfg, w))
    return _made[key]


def runner_for(folder, dtype, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    args = dict(dtype=dtype, page_size=16, max_tokens=1024, max_seqs=4, max_batch_tokens=1024)
    args.update(kw)
    return ModelRunner.from_folder(folder, **args)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16"), ("C1", "float32"), ("C2", "float32")])
def test_a_whole_prompt_against_the_plain_model(name, dtype):
    cfg, w, folder = model(name)
    toks = safe_tokens(cfg, w, 50, 1) if dtype == "bfloat16" else tokens_of(cfg["vocab"], 75, 1)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, dtype)
    got = r.step([0], [toks], [list(range(len(toks)))])
    assert_close(got, want, REL[dtype], f"model {name} in {dtype}")
    r.end(0)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("D", "float32"), ("E", "float32"), ("F", "float32"), ("F", "bfloat16")])
def test_models_of_one_kind_of_mixer_only_and_head_sizes_that_are_filled_up(name, dtype):
    """Recurrent layers alone (no pages at all) and attention alone (no mixer state): a prompt in portions, then
    tokens one by one, a second request beside the first, a slot used again."""
    cfg, w, folder = model(name)
    make = (lambda n, seed: safe_tokens(cfg, w, n, seed)) if dtype == "bfloat16" else (lambda n, seed: tokens_of(cfg["vocab"], n, seed))
    a, b = make(40, 50), make(21, 51)
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    r = runner_for(folder, dtype, max_seqs=2, max_tokens=128)
    got_a = [r.step([0], [a[:17]], [list(range(17))]).clone()]
    out = r.step([0, 1], [a[17:30], b[:20]], [list(range(13)), list(range(20))]).clone()
    got_a.append(out[:13])
    got_b = [out[13:]]
    out = r.step([1, 0], [b[20:], a[30:31]], [[0], [0]]).clone()
    got_b.append(out[:1]); got_a.append(out[1:])
    r.end(1)
    got_a += [r.step([0], [[t]], [[0]]).clone() for t in a[31:]]
    assert_close(torch.cat(got_a), wa, REL[dtype], "first request")
    assert_close(torch.cat(got_b), wb, REL[dtype], "second request")
    again = r.step([2], [b], [list(range(21))])          # in the slot (and pages) that the second request held
    assert_close(again, wb, REL[dtype], "the slot used again")
    r.cache.check()


def test_the_rank_of_the_decay_comes_from_the_tensor_and_tensors_are_checked():
    from llama_cu_amd.weights.loader import WeightError
    cfg, w, folder = model("A")
    r = runner_for(folder, "float32")
    assert [l.decay_rank for l in r.config.layers] == [None, 5, None, 3]
    bad = dict(w)
    del bad["l0.mix.q.norm"]
    bad["l2.mix.k"] = torch.zeros(48, 72)          # a layer that reads another's keys has none of its own
    with pytest.raises(WeightError) as e:
        runner_for(make_folder(cfg, bad), "float32")
    assert "l0.mix.q.norm" in str(e.value) and "l2.mix.k" in str(e.value)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16")])
def test_prefill_against_token_by_token_decoding_and_portions_down_to_two_tokens(name, dtype):
    cfg, w, folder = model(name)
    toks = tokens_of(cfg["vocab"], 90, 2)
    r = runner_for(folder, dtype)
    whole = r.step([0], [toks], [list(range(len(toks)))]).clone()
    # against the plain model in 32-bit; a bfloat16 run is compared with the engine's own whole prompt (which a test of
    # its own compares with the plain model on a sequence without close calls of the routers)
    want = plain_logits(cfg, w, toks) if dtype == "float32" else whole
    # one token at a time from the first (long enough for captured graphs to replay)
    single = torch.cat([r.step([1], [[t]], [[0]]).clone() for t in toks])
    assert_close(single, want, REL[dtype] if dtype == "float32" else SAME[dtype], "token by token")
    # portions of 2, 3, 5, 1, 17, ... tokens
    sizes, at, parts = [2, 3, 5, 1, 17, 2, 31, 4, 2, 1, 64], 0, []
    for k in range(100):
        if at >= len(toks):
            break
        take = toks[at:at + sizes[k % len(sizes)]]
        parts.append(r.step([2], [take], [list(range(len(take)))]).clone())
        at += len(take)
    portions = torch.cat(parts)
    assert_close(portions, want, REL[dtype] if dtype == "float32" else SAME[dtype], "portions")
    assert_close(single, whole, SAME[dtype], "token by token against the whole prompt")
    assert_close(portions, whole, SAME[dtype], "portions against the whole prompt")
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
    else:       # each alone through the engine (long bfloat16 runs are not compared with the plain model: see safe_tokens)
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


def test_keys_far_back_and_at_page_borders_in_prompts_and_in_decoding():
    """Sharp keys (their norm's weight times 6) make single keys carry an output; 330 tokens over pages of 16, the last
    40 decoded one by one: every position's logits against the plain model, in 32-bit."""
    cfg, w, folder = model("A", sharp=6.0)
    toks = tokens_of(cfg["vocab"], 330, 7)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, "float32")
    parts = [r.step([0], [toks[:127]], [list(range(127))]).clone(), r.step([0], [toks[127:290]], [list(range(163))]).clone()]
    parts += [r.step([0], [[t]], [[0]]).clone() for t in toks[290:]]
    assert_close(torch.cat(parts), want, REL["float32"], "far keys")
    # the temperature's step: positions 5, 6 and 7 differ by it (floor((p + 1) / 7) becomes 1 at p = 6)
    assert CFG_A["layers"][0]["mixer"]["q_temp"]["every"] == 7


def test_long_decoding_in_bfloat16():
    cfg, w, folder = model("B")
    toks = tokens_of(cfg["vocab"], 200, 8)
    r = runner_for(folder, "bfloat16")
    want = r.step([1], [toks], [list(range(200))]).clone()
    got = [r.step([0], [toks[:20]], [list(range(20))]).clone()] + [r.step([0], [[t]], [[0]]).clone() for t in toks[20:]]
    assert_close(torch.cat(got), want, SAME["bfloat16"], "long decoding against the whole prompt")
    assert sum(r.graph_replays.values()) > 100, "decoding was not replayed from captured graphs"


def test_logits_do_not_depend_on_the_cut_or_the_batch_bit_for_bit_in_32_bit():
    cfg, w, folder = model("B")
    a, b = tokens_of(cfg["vocab"], 60, 20), tokens_of(cfg["vocab"], 41, 21)
    r = runner_for(folder, "float32")
    alone = r.step([0], [a], [list(range(60))]).clone()
    r.step([1], [b[:30]], [[]])
    p1 = r.step([2, 1], [a[:17], b[30:31]], [list(range(17)), [0]]).clone()
    p2 = r.step([1, 2], [b[31:], a[17:]], [[], list(range(43))]).clone()
    assert torch.equal(torch.cat([p1[:17], p2]), alone)


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
        places = list(range(len(p) - 1, len(seq) - 1))
        if dtype == "float32":
            logits = plain_logits(cfg, w, seq)[places]
            assert torch.argmax(logits, -1).tolist() == list(g), f"prompt {k}"
        else:
            # in bfloat16 against the engine's own logits for prompt and continuation fed as one prompt (a long bfloat16
            # run is not compared with the plain model: see safe_tokens); a close call may fall the other way
            logits = engine.runner.step([900 + k], [seq], [places]).double().cpu()
            engine.runner.end(900 + k)
            for j, tok in enumerate(g):
                assert logits[j].max() - logits[j, tok] <= 0.02 * logits[j].abs().max(), f"prompt {k}, token {j}: {tok} is not the best"
    engine.runner.cache.check()


def test_trace_replay_of_the_design(tmp_path):
    """The replay program's own path: steps as JSON objects, logits as files."""
    from llama_cu_amd.engine.trace import TraceReplayer
    cfg, w, folder = model("A")
    a, b = tokens_of(cfg["vocab"], 50, 40), tokens_of(cfg["vocab"], 30, 41)
    rep = TraceReplayer.open(folder, "float32", 128, max_live=2)
    out0 = rep.step({"step": 0, "entries": [{"id": "x", "tokens": a[:33], "want": [0, 32]}], "end": []})
    out1 = rep.step({"step": 1, "entries": [{"id": "x", "tokens": a[33:], "want": [16]}, {"id": "y", "tokens": b, "want": [29]}], "end": ["x", "y"]})
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    assert_close(torch.from_numpy(out0), wa[[0, 32]], REL["float32"])
    assert_close(torch.from_numpy(out1), torch.stack([wa[49], wb[29]]), REL["float32"])


def test_the_command_line_writes_a_random_model_generates_from_it_and_replays_a_trace(tmp_path):
    """``random-model`` writes a folder of the design from a configuration that names the decay's rank; ``generate``
    continues a prompt from it; ``bin/trace_run`` (the program itself, steps on its standard input) gives the plain
    model's logits for the folder's weights."""
    import json
    import os
    import subprocess

    import numpy as np
    from llama_cu_amd.weights import open_safetensors
    from divasun_common import attention, config, moe
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = config(288, 96, [
        {"type": "general_delta", "mixer": {"heads": 2, "dim": 32, "decay_rank": 7}, "mlp": moe(4, 2, 48)},
        {"type": "attention", "mixer": attention(4, 2, 32, 32, 0.2, q_temp=(0.3, 9)), "mlp": moe(4, 1, 48)},
    ], taps=3, eps=1e-5, scale=4.0)
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
