"""The configuration of the Divasun decoder.

config.json names the design with ``"architecture": "Divasun"`` and lists its layers: every entry of ``layers``
has a ``type`` (which mixer: ``general_delta`` or ``attention``), the mixer's sizes (``mixer``) and its
feed-forward (``mlp``, or null for none).  Beside them: ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` (the
taps of the convolution in front of every sublayer) and ``embedding.scale``.  One size is no key of config.json:
the low rank of the delta rule's decay, which the shape of the tensor ``<layer>.mix.w1`` gives
(``complete_from_shapes``); a configuration written by this package holds it as ``mixer.decay_rank``.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class DivasunMoE:
    experts: int
    top: int
    expert_size: int


@dataclass(frozen=True)
class DivasunLayer:
    type: str                               # "general_delta" or "attention"
    heads: int
    dim: int                                # per-head size of queries and keys (of everything, for the delta rule)
    kv_heads: int = 0                       # attention only from here on
    vdim: int = 0
    scale: float = 0.0
    q_temp: Optional[Tuple[float, int]] = None      # (coef, every)
    kv_from: Optional[int] = None
    decay_rank: Optional[int] = None        # general_delta: None until the tensors' shapes have given it
    mlp: Optional[DivasunMoE] = None


MIXERS = ("general_delta", "attention")


def _section(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = data.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: required key {key!r} is missing or no object")
    return v


@dataclass(frozen=True)
class DivasunConfig:
    vocab: int
    width: int
    layers: Tuple[DivasunLayer, ...]
    norm_eps: float
    taps: int
    embedding_scale: float
    max_positions: int = 1 << 17            # the design has no table of positions: this bounds a request's block table only
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Divasun"

    @staticmethod
    def from_dict(data: Dict[str, Any], where: str = "config.json") -> "DivasunConfig":
        r = KeyReader(data, where)
        layers = data.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: required key 'layers' is missing or holds no layer")
        out = []
        for i, entry in enumerate(layers):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{at} is no object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{at}: 'type' = {kind!r} is no mixer of this design; known: {list(MIXERS)}")
            m = KeyReader(_section(entry, "mixer", at), at + ".mixer")
            fields: Dict[str, Any] = dict(type=kind, heads=m.integer("heads"), dim=m.integer("dim"))
            if kind == "attention":
                fields["kv_heads"] = m.integer("kv_heads", default=fields["heads"])
                if fields["heads"] % fields["kv_heads"]:
                    raise ConfigError(f"{at}.mixer: 'heads' {fields['heads']} is no multiple of 'kv_heads' {fields['kv_heads']}")
                fields["vdim"] = m.integer("vdim", default=fields["dim"])
                fields["scale"] = m.number("scale")
                qt = m.data.get("q_temp")
                if qt is not None:
                    t = KeyReader(_section(m.data, "q_temp", at + ".mixer"), at + ".mixer.q_temp")
                    fields["q_temp"] = (t.number("coef", positive=False), t.integer("every"))
                src = m.data.get("kv_from")
                if src is not None:
                    if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                        raise ConfigError(f"{at}.mixer: 'kv_from' = {src!r} must name an earlier layer")
                    if out[src].type != "attention" or out[src].kv_from is not None:
                        raise ConfigError(f"{at}.mixer: 'kv_from' = {src} names a layer without keys and values of its own")
                    if (out[src].kv_heads, out[src].dim, out[src].vdim) != (fields["kv_heads"], fields["dim"], fields["vdim"]):
                        raise ConfigError(f"{at}.mixer: layer {src}'s keys and values have other sizes than this layer's")
                    fields["kv_from"] = src
            else:
                fields["decay_rank"] = m.integer("decay_rank", default=None)
            mlp = entry.get("mlp")
            if mlp is not None:
                f = KeyReader(_section(entry, "mlp", at), at + ".mlp")
                if f.data.get("kind") != "moe":
                    raise ConfigError(f"{at}.mlp: 'kind' = {f.data.get('kind')!r} is no feed-forward of this design; known: ['moe']")
                router = KeyReader(_section(f.data, "router", at + ".mlp"), at + ".mlp.router")
                expert = KeyReader(_section(f.data, "expert", at + ".mlp"), at + ".mlp.expert")
                moe = DivasunMoE(router.integer("experts"), router.integer("top"), expert.integer("ff"))
                if moe.top > moe.experts:
                    raise ConfigError(f"{at}.mlp.router: 'top' {moe.top} exceeds 'experts' {moe.experts}")
                fields["mlp"] = moe
            out.append(DivasunLayer(**fields))
        norm = KeyReader(_section(data, "norm", where), where + ": norm")
        canon = data.get("canon")
        taps = KeyReader(canon, where + ": canon").integer("taps") if isinstance(canon, dict) else 0
        emb = data.get("embedding")
        scale = KeyReader(emb, where + ": embedding").number("scale", default=1.0) if isinstance(emb, dict) else 1.0
        return DivasunConfig(vocab=r.integer("vocab"), width=r.integer("width"), layers=tuple(out), norm_eps=norm.number("eps"),
                             taps=taps, embedding_scale=scale, max_positions=r.integer("max_positions", default=1 << 17),
                             eos_token_ids=r.token_ids("eos_token_id"))

    def complete_from_shapes(self, shapes: Dict[str, Tuple[int, ...]]) -> "DivasunConfig":
        """The configuration with every delta layer's ``decay_rank`` taken from the shape of its ``mix.w1``
        (where config.json did not give it and the tensor is there)."""
        layers = []
        for i, layer in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.w1")
            if layer.type == "general_delta" and layer.decay_rank is None and shape is not None and len(shape) == 2:
                layer = dataclasses.replace(layer, decay_rank=int(shape[0]))
            layers.append(layer)
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        layers = []
        for layer in self.layers:
            m: Dict[str, Any] = {"heads": layer.heads, "dim": layer.dim}
            if layer.type == "attention":
                m.update(kv_heads=layer.kv_heads, vdim=layer.vdim, scale=layer.scale)
                if layer.q_temp is not None:
                    m["q_temp"] = {"coef": layer.q_temp[0], "every": layer.q_temp[1]}
                if layer.kv_from is not None:
                    m["kv_from"] = layer.kv_from
            elif layer.decay_rank is not None:
                m["decay_rank"] = layer.decay_rank
            mlp = None
            if layer.mlp is not None:
                mlp = {"kind": "moe", "router": {"experts": layer.mlp.experts, "top": layer.mlp.top},
                       "expert": {"ff": layer.mlp.expert_size}}
            layers.append({"type": layer.type, "mixer": m, "mlp": mlp})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "canon": {"taps": self.taps}, "embedding": {"scale": self.embedding_scale},
             "max_positions": self.max_positions}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
