"""The Lozezen design without a GPU: its configuration reader, the layout's tensor names and shapes, cache needs, and
the plain implementation's own consistency."""
from __future__ import annotations

import copy

import numpy as np
import pytest
import torch

import plain_lozezen as P
from lozezen_common import CFG_A, CFG_B, CFG_C, CFG_D, CFG_E, CONFIGS, as_numpy, random_weights, tokens_of


def spec_of(cfg):
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd.config import architecture_of
    arch = architecture_of(cfg)
    typed = arch.config_from_dict(cfg)
    return typed, arch.build_spec(typed)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_layout_expects_exactly_the_tensors_of_the_design(name):
    from llama_cu_amd.parts import DecoderModel
    cfg = CONFIGS[name]
    _, spec = spec_of(cfg)
    expected = {k: tuple(v.shape) for k, v in DecoderModel(spec).tensors().items()}
    made = {k: tuple(v.shape) for k, v in random_weights(cfg, 1).items()}
    assert expected == made


def test_the_configuration_reads_back_and_keeps_every_constant():
    from llama_cu_amd.config.lozezen import LozezenConfig
    for cfg in CONFIGS.values():
        typed = LozezenConfig.from_dict(cfg)
        assert LozezenConfig.from_dict(typed.to_dict()) == typed
    a = LozezenConfig.from_dict(CFG_A)
    assert [l.type for l in a.layers] == ["rglru", "attention", "parallel", "rglru"]
    att = a.layers[1].mixer
    assert (att.heads, att.kv_heads, att.dim, att.vdim, att.mask, att.rot.dims, att.rot.base, att.rot.factor) == (6, 2, 24, 40, 19, 10, 500.0, 2.5)
    par = a.layers[2].mixer
    assert (par.left.mask, par.left.rot, par.right.decay, par.right.rot.dims, par.left_scale, par.right_scale) == (11, None, (0.9, 0.97, 0.995), 12, 0.7, 1.3)
    assert a.layers[1].ff is None and a.layers[0].ff == 40 and a.layers[3].mixer.conv == 2


@pytest.mark.parametrize("change,key", [
    (lambda c: c["layers"][1].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][1]["mixer"].pop("rot"), "rot"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=26), "dims"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(decay=[0.9]), "decay"),
    (lambda c: c["layers"][2]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mixer"].update(blocks=5), "blocks"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("vocab"), "vocab"),
])
def test_errors_name_their_key(change, key):
    from llama_cu_amd.config import ConfigError
    from llama_cu_amd.config.lozezen import LozezenConfig
    cfg = copy.deepcopy(CFG_A)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        LozezenConfig.from_dict(cfg)
    assert key in str(e.value)


def test_cache_needs_follow_the_mixers():
    from llama_cu_amd.parts import DecoderModel, PagedKV, SeveralNeeds, SlotState
    _, spec = spec_of(CFG_A)
    needs = DecoderModel(spec).cache_needs()
    assert needs[0] == SlotState((3, 72), torch.float32) and needs[3] == SlotState((2, 96), torch.float32)
    assert isinstance(needs[1], PagedKV) and (needs[1].kv_heads, needs[1].window) == (2, 19)
    assert isinstance(needs[2], SeveralNeeds) and needs[2].pool() == (11, 0) and not needs[2].can_truncate
    assert needs[2].needs[1] == SlotState((3, 24, 16), torch.float32)
    _, spec = spec_of(CFG_E)
    assert all(isinstance(n, PagedKV) for n in DecoderModel(spec).cache_needs())


def test_the_plain_model_is_causal_and_its_masks_end_where_they_should():
    """Changing a token changes no earlier logit; a token outside every window and chunk, with no recurrent layer in
    between, changes no later one."""
    w = as_numpy(random_weights(CFG_E, 3))
    toks = tokens_of(CFG_E["vocab"], 60, 1)
    base = P.forward(CFG_E, w, toks)
    other = list(toks)
    other[30] = (other[30] + 1) % CFG_E["vocab"]
    moved = P.forward(CFG_E, w, other)
    assert np.array_equal(base[:30], moved[:30]) and not np.allclose(base[30], moved[30])
    # one layer with a window of 25: position 30 is seen up to position 54 and no further
    one = dict(CFG_E, layers=CFG_E["layers"][:1])
    a, b = P.forward(one, w, toks), P.forward(one, w, other)
    assert not np.allclose(a[54], b[54]) and np.array_equal(a[55:], b[55:])


def test_plain_mechanisms_one_by_one():
    rng = np.random.default_rng(0)
    # a rotation keeps lengths, turns only the first dims, and position 0 is the identity; the two pairings differ
    x = rng.standard_normal((5, 2, 12))
    for inter in (False, True):
        y = P.rotate(x, np.arange(5), 8, 100.0, 2.0, interleaved=inter)
        assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1))
        assert np.array_equal(y[..., 8:], x[..., 8:]) and np.allclose(y[0], x[0]) and not np.allclose(y[3], x[3])
    assert not np.allclose(P.rotate(x, np.arange(5), 8, 100.0), P.rotate(x, np.arange(5), 8, 100.0, interleaved=True))
    # scaling by f is the rotation at position p / f
    assert np.allclose(P.rotate(x, np.arange(5) * 4, 8, 100.0, 4.0), P.rotate(x, np.arange(5), 8, 100.0))
    # the convolution's last column is the current token's
    cw = np.array([[0.0, 0.0, 1.0]])
    seq = rng.standard_normal((6, 1))
    assert np.allclose(P.causal_conv(seq, cw, np.zeros(1)), seq)
    assert np.allclose(P.causal_conv(seq, np.array([[1.0, 0.0, 0.0]]), np.zeros(1))[2:], seq[:-2])
    assert np.isclose(P.gelu_tanh(np.array(1.0)), 0.841192, atol=1e-6) and np.isclose(P.softplus(np.array(0.0)), np.log(2.0))
    # retention of one head with decay 1, keys and queries e_0 (times 1 / sqrt(dim) on the keys): o_t is the running sum
    # of the values, and its norm and gate follow
    d, T = 4, 5
    h = rng.standard_normal((T, d))
    w = {"q": np.zeros((d, d)), "k": np.zeros((d, d)), "v": np.eye(d), "g": np.eye(d), "o": np.eye(d)}
    w["q"][0], w["k"][0] = np.ones(d), np.ones(d)                      # q_0 = k_0 = sum of the input, the other channels zero
    m = {"heads": 1, "dim": d, "vdim": d, "decay": [1.0]}
    s = h.sum(1)
    o = np.cumsum((s * d ** -0.5)[:, None] * h, axis=0) * s[:, None]
    assert np.allclose(P.retention(h, w, "", m, 1e-9), P.unit_rms(o, 1e-9) * P.silu(h))


def test_several_needs_join_pages_and_states_and_refuse_two_kinds_of_pages():
    from llama_cu_amd.parts import PagedKV, SeveralNeeds, SlotState
    both = SeveralNeeds((SlotState((2, 3), torch.float32), PagedKV(2, 16, window=9), SlotState((5,), torch.float32)))
    assert both.pool() == (9, 0) and not both.can_truncate and both.page_bytes(16, 2) == 2 * 32 * 16 * 2
    made = both.allocate(0, 4, 16, 3, torch.bfloat16, "cpu")
    assert made.pages.shape == (4, 2, 2 * 16 * 16) and made.state.shape == (3, 2, 3)
    assert made.more["state0"].shape == (3, 2, 3) and made.more["state2"].shape == (3, 5)
    with pytest.raises(ValueError):
        SeveralNeeds((PagedKV(1, 8), PagedKV(1, 8, window=4)))
