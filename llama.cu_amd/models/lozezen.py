"""The Lozezen decoder laid out of parts.

Every layer is a sandwich block: an RMS norm in front of and behind each sublayer, the weights stored around zero.
Three mixers: softmax attention with biases, a rotation of the first dims of neighbouring pairs with scaled-down
frequencies and a sliding window; a recurrent block with a real-gated linear recurrent unit; and two mixers side by
side, softmax attention within chunks (biases, a norm per head on queries and keys, a gate per head) beside retention
(a rotation of half-split pairs, a fixed decay per head).  The feed-forward is the dense gated one, or missing.
Everything here is data: which parts, with which sizes and constants from the configuration, under which tensor
names, in which order.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.lozezen import LozezenConfig
from ..parts import ModelSpec, PartSpec, RunEntry

# the factor in the recurrent unit's decay, a = exp(-8 r softplus(lam)): the design fixes it
RGLRU_DECAY_EXPONENT = 8.0

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                   "q_head_norm": "q.norm", "k_head_norm": "k.norm", "g": "g"}


def lozezen_spec(cfg: LozezenConfig) -> ModelSpec:
    d = cfg.width

    def norm(tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps, "tensor": tensor, "one_plus": True}, "")

    def rotary(rot, head_dim: int, interleaved: bool):
        if rot is None:
            return None
        return PartSpec("rotary", {"head_dim": head_dim, "theta": rot.base, "max_positions": cfg.max_positions,
                                   "interleaved": interleaved, "rot_dim": rot.dims, "scaling_factor": rot.factor})

    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "attention":
            mixer = PartSpec("attention", {"hidden_size": d, "heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim,
                                           "value_dim": m.vdim, "scale": m.scale, "window": m.mask, "bias": True,
                                           "position": rotary(m.rot, m.dim, True), "names": ATTENTION_NAMES}, "mix")
        elif layer.type == "rglru":
            mixer = PartSpec("rglru", {"hidden_size": d, "width": m.width, "blocks": m.blocks, "taps": m.conv,
                                       "decay_exponent": RGLRU_DECAY_EXPONENT}, "mix")
        else:
            left = PartSpec("attention", {"hidden_size": d, "heads": m.left.heads, "kv_heads": m.left.kv_heads,
                                          "head_dim": m.left.dim, "value_dim": m.left.vdim, "scale": m.left.scale,
                                          "chunk": m.left.mask, "bias": True, "head_norm_eps": cfg.norm_eps, "head_gate": True,
                                          "position": rotary(m.left.rot, m.left.dim, True), "names": ATTENTION_NAMES}, "left")
            right = PartSpec("retention", {"hidden_size": d, "heads": m.right.heads, "head_dim": m.right.dim,
                                           "value_dim": m.right.vdim, "decay": list(m.right.decay), "norm_eps": cfg.norm_eps,
                                           "position": rotary(m.right.rot, m.right.dim, False)}, "right")
            mixer = PartSpec("side_by_side", {"mixers": [left, right], "scales": [m.left_scale, m.right_scale]}, "mix")
        params = {"norm1": norm("norm1"), "mixer": mixer, "post1": norm("norm1b")}
        if layer.ff is not None:
            params.update(norm2=norm("norm2"), post2=norm("norm2b"),
                          ffn=PartSpec("swiglu", {"hidden_size": d, "intermediate_size": layer.ff,
                                                  "names": {"gate": "gate", "up": "up", "down": "down"}}, "mlp"))
        layers.append(PartSpec("sandwich", params, f"l{i}"))
    return ModelSpec(
        hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab, "hidden_size": d, "scale": cfg.embedding_scale,
                                      "tensor": "embed"}, ""),
        layers=layers, run_order=[RunEntry(i) for i in range(len(layers))], final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": False, "tensor": "head"}, ""),
        eos_token_ids=cfg.eos_token_ids)


register_architecture("Lozezen", LozezenConfig.from_dict, lozezen_spec)
