"""The Divasun configuration reader and the layout of the model out of parts (no GPU)."""
from __future__ import annotations

import copy

import pytest
import torch

import plain_divasun as P
from divasun_common import CFG_A, CFG_B, RANKS_A, random_weights, tokens_of


def _spec(cfg, ranks):
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd import models  # noqa: F401
    from llama_cu_amd.config import architecture_of
    arch = architecture_of(cfg)
    shapes = {f"l{i}.mix.w1": (r, cfg["width"]) for i, r in ranks.items()}
    typed = arch.complete_config(arch.config_from_dict(cfg), shapes)
    return arch, typed, arch.build_spec(typed)


def test_the_architecture_is_found_and_its_tensors_are_the_files():
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights.loader import check_tensors
    arch, typed, spec = _spec(CFG_A, RANKS_A)
    assert arch.name == "Divasun"
    w = random_weights(CFG_A, RANKS_A, 1)
    expected = DecoderModel(spec).tensors()
    check_tensors(expected, {k: tuple(v.shape) for k, v in w.items()}, arch.ignored_tensors)
    assert set(expected) == set(w)
    # a layer without feed-forward may still carry its second norm and convolution in a file
    extra = dict({k: tuple(v.shape) for k, v in w.items()}, **{"l1.norm2": (72,), "l1.norm2.b": (72,), "l1.canon2": (72, 3)})
    check_tensors(expected, extra, arch.ignored_tensors)


def test_the_run_order_shares_keys_and_values_and_every_size_is_the_configurations():
    _, typed, spec = _spec(CFG_A, RANKS_A)
    assert [(e.layer, e.cache_of) for e in spec.run_order] == [(0, None), (1, None), (2, 0), (3, None)]
    att, delta = spec.layers[0].params, spec.layers[1].params
    m = att["mixer"].params
    assert (m["heads"], m["kv_heads"], m["head_dim"], m["value_dim"], m["scale"]) == (6, 2, 24, 16, 0.31)
    assert m["query_temperature"] == (0.5, 7) and m["projection_norm_eps"] == 1e-4 and not m["shares_kv"]
    assert spec.layers[2].params["mixer"].params["shares_kv"] and spec.layers[2].params["mixer"].params["query_temperature"] is None
    assert delta["mixer"].params["decay_rank"] == 5 and "ffn" not in delta and delta["conv_taps"] == 3
    f = att["ffn"].params
    assert (f["experts"], f["top"], f["expert_size"]) == (5, 2, 40)
    assert spec.embedding.params["scale"] == 3.0 and spec.vocab_size == 131 and spec.hidden_size == 72


def test_the_configuration_reads_back_and_errors_name_their_key():
    from llama_cu_amd.config import ConfigError, DivasunConfig
    _, typed, _ = _spec(CFG_B, {0: 8, 2: 4})
    assert DivasunConfig.from_dict(typed.to_dict()) == typed
    for path, value, word in [(("layers", 0, "type"), "mamba", "type"), (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 3, "mixer", "kv_from"), 3, "kv_from"), (("layers", 3, "mixer", "kv_from"), 0, "kv_from"),
                              (("layers", 0, "mlp", "kind"), "dense", "kind"), (("layers", 1, "mlp", "router", "top"), 9, "top"),
                              (("norm",), None, "norm"), (("width",), -4, "width")]:
        bad = copy.deepcopy(CFG_B)
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError) as e:
            DivasunConfig.from_dict(bad)
        assert word in str(e.value), f"{path}: {e.value}"


def test_a_missing_rank_is_said_when_the_model_is_laid_out():
    import llama_cu_amd  # noqa: F401
    from llama_cu_amd import models  # noqa: F401
    from llama_cu_amd.config import ConfigError, architecture_of
    arch = architecture_of(CFG_A)
    with pytest.raises(ConfigError) as e:
        arch.build_spec(arch.config_from_dict(CFG_A))
    assert "l1.mix.w1" in str(e.value)


def test_the_plain_model_is_causal_and_its_convolution_and_state_can_be_cut():
    """The oracle's own consistency: a longer sequence does not change earlier logits; the delta rule run in two
    halves with the state handed over equals one run; the convolution of a sequence equals that of its pieces
    with the last inputs carried."""
    w = random_weights(CFG_A, RANKS_A, 5)
    toks = tokens_of(CFG_A["vocab"], 24, 1)
    full, part = P.forward(CFG_A, w, toks), P.forward(CFG_A, w, toks[:15])
    assert torch.allclose(full[:15], part, atol=1e-9)
    W = {k[len("l1.mix."):]: v.double() for k, v in w.items() if k.startswith("l1.mix.")}
    h = torch.randn(20, 72, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    whole, s_whole = P.general_delta(h, W, 3, 32, 1e-4)
    a, s = P.general_delta(h[:9], W, 3, 32, 1e-4)
    b, s2 = P.general_delta(h[9:], W, 3, 32, 1e-4, state=s)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-10) and torch.allclose(s2, s_whole, atol=1e-10)
    cw = w["l0.canon1"].double()
    y = P.short_conv(h, cw)
    assert torch.allclose(y[0], h[0] * (1 + cw[:, -1]))         # the first token sees zeros before it
    tail = P.short_conv(torch.cat([h[7:9], h[9:]]), cw)[2:]    # taps - 1 = 2 carried inputs
    assert torch.allclose(tail, y[9:], atol=1e-12)
