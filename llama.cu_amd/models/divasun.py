"""The Divasun decoder laid out of parts.

Every layer is a parallel block: two layer norms (weight and bias) of the same residual stream, a short causal
convolution in front of each sublayer, a mixer (the generalised delta rule, or attention without a rotation: a
norm over the whole query and key projections, a query temperature that grows with the logarithm of the position,
a bias on the distance inside the scores; a layer may read an earlier layer's keys and values) and a mixture of
experts with sigmoid scores.  The embedding is scaled; the final norm is a layer norm; the output matrix is its own.
Everything here is data: which parts, with which sizes and constants from the configuration, under which tensor
names, in which order.
"""
from __future__ import annotations

from ..config import ConfigError, register_architecture
from ..config.divasun import DivasunConfig
from ..parts import ModelSpec, PartSpec, RunEntry

# the exponent of the distance bias's slopes, 2^(-8 (h + 1) / heads): the design fixes it
BIAS_EXPONENT = 8.0


def divasun_spec(cfg: DivasunConfig) -> ModelSpec:
    d = cfg.width

    def norm(tensor: str) -> PartSpec:
        return PartSpec("layernorm", {"size": d, "eps": cfg.norm_eps, "tensor": tensor, "bias_tensor": tensor + ".b"}, "")

    layers, order, entry_of = [], [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.type == "general_delta":
            if layer.decay_rank is None:
                raise ConfigError(f"layers[{i}]: the low rank of the delta rule's decay is neither in the configuration "
                                  f"('mixer.decay_rank') nor given by the shape of the tensor 'l{i}.mix.w1'")
            mixer = PartSpec("general_delta", {"hidden_size": d, "heads": layer.heads, "head_dim": layer.dim,
                                               "decay_rank": layer.decay_rank, "norm_eps": cfg.norm_eps}, "mix")
        else:
            position = PartSpec("distance_bias", {"heads": layer.heads, "exponent": BIAS_EXPONENT})
            mixer = PartSpec("attention", {"hidden_size": d, "heads": layer.heads, "kv_heads": layer.kv_heads,
                                           "head_dim": layer.dim, "value_dim": layer.vdim, "scale": layer.scale,
                                           "position": position, "shares_kv": layer.kv_from is not None,
                                           "projection_norm_eps": cfg.norm_eps, "query_temperature": layer.q_temp,
                                           "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm",
                                                     "k_norm": "k.norm"}}, "mix")
        params = {"hidden_size": d, "norm1": norm("norm1"), "mixer": mixer, "conv_taps": cfg.taps,
                  "conv_tensors": ("canon1", "canon2")}
        if layer.mlp is not None:
            params["norm2"] = norm("norm2")
            params["ffn"] = PartSpec("sigmoid_moe", {"hidden_size": d, "expert_size": layer.mlp.expert_size,
                                                     "experts": layer.mlp.experts, "top": layer.mlp.top}, "mlp")
        layers.append(PartSpec("parallel", params, f"l{i}"))
        entry_of[i] = len(order)
        order.append(RunEntry(i, cache_of=entry_of[layer.kv_from] if layer.kv_from is not None else None))
    return ModelSpec(
        hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale,
                                      "tensor": "embed"}, ""),
        layers=layers, run_order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": False, "tensor": "head"}, ""),
        eos_token_ids=cfg.eos_token_ids)


# a file may hold the second norm and its convolution also for a layer that has no feed-forward to read them
register_architecture("Divasun", DivasunConfig.from_dict, divasun_spec, ignored_tensors=[r"l\d+\.(norm2|norm2\.b|canon2)$"],
                      complete_config=lambda cfg, shapes: cfg.complete_from_shapes(shapes))
