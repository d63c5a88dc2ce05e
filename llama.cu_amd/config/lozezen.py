"""The configuration of the Lozezen decoder.

config.json names the design with ``"architecture": "Lozezen"`` and lists its layers: every entry of ``layers`` has a
``type`` (which mixer: ``attention``, ``rglru`` or ``parallel``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: ``{"kind": "dense", "ff": n}``, or null for none).  Beside them: ``vocab``, ``width``,
``norm.eps`` and ``embedding.scale``.  Every size and constant is read from here; nothing is assumed equal to
anything else (heads and groups, key and value sizes, rotated dims, windows and chunks differ from layer to layer).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader

MIXERS = ("attention", "rglru", "parallel")


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    factor: float = 1.0           # linear scaling: the frequencies are divided by it


@dataclass(frozen=True)
class SoftmaxAttention:
    """Grouped-query softmax attention: the mixer ``attention`` (rotation and window) and the left half of
    ``parallel`` (chunks, no rotation)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask: int                     # the window's or the chunk's size
    rot: Optional[Rotation] = None


@dataclass(frozen=True)
class RetentionHalf:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation] = None


@dataclass(frozen=True)
class ParallelMixer:
    left: SoftmaxAttention
    right: RetentionHalf
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class RecurrentUnit:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class LozezenLayer:
    type: str
    mixer: Any                    # SoftmaxAttention, RecurrentUnit or ParallelMixer
    ff: Optional[int] = None      # the dense feed-forward's inner size; None: the layer has no feed-forward


def _section(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = data.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: required key {key!r} is missing or no object")
    return v


def _rotation(m: KeyReader, required: bool) -> Optional[Rotation]:
    if m.data.get("rot") is None:
        if required:
            raise ConfigError(f"{m.where}: required key 'rot' is missing")
        return None
    r = KeyReader(_section(m.data, "rot", m.where), m.where + ".rot")
    dims = r.integer("dims", minimum=2)
    if dims % 2:
        raise ConfigError(f"{r.where}: key 'dims' must be even, got {dims}")
    factor = 1.0
    if r.data.get("scaling") is not None:
        factor = KeyReader(_section(r.data, "scaling", r.where), r.where + ".scaling").number("factor")
    return Rotation(dims, r.number("base"), factor)


def _softmax(m: KeyReader, rot_required: bool) -> SoftmaxAttention:
    heads = m.integer("heads")
    kv_heads = m.integer("kv_heads", default=heads)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: 'heads' {heads} is no multiple of 'kv_heads' {kv_heads}")
    dim = m.integer("dim")
    mask = KeyReader(_section(m.data, "mask", m.where), m.where + ".mask").integer("size")
    rot = _rotation(m, rot_required)
    if rot is not None and rot.dims > dim:
        raise ConfigError(f"{m.where}.rot: 'dims' {rot.dims} exceeds 'dim' {dim}")
    return SoftmaxAttention(heads, kv_heads, dim, m.integer("vdim", default=dim), m.number("scale"), mask, rot)


def _retention(m: KeyReader) -> RetentionHalf:
    heads, dim = m.integer("heads"), m.integer("dim")
    decay = m.data.get("decay")
    if not isinstance(decay, list) or len(decay) != heads or any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay):
        raise ConfigError(f"{m.where}: key 'decay' must list one number for each of the {heads} heads")
    rot = _rotation(m, False)
    if rot is not None and rot.dims > dim:
        raise ConfigError(f"{m.where}.rot: 'dims' {rot.dims} exceeds 'dim' {dim}")
    return RetentionHalf(heads, dim, m.integer("vdim", default=dim), tuple(float(x) for x in decay), rot)


@dataclass(frozen=True)
class LozezenConfig:
    vocab: int
    width: int
    layers: Tuple[LozezenLayer, ...]
    norm_eps: float
    embedding_scale: float
    max_positions: int = 1 << 17            # the design sets no limit: this bounds the rotation tables and a request's block table
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Lozezen"

    @staticmethod
    def from_dict(data: Dict[str, Any], where: str = "config.json") -> "LozezenConfig":
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
            if kind == "attention":
                mixer: Any = _softmax(m, rot_required=True)
            elif kind == "rglru":
                mixer = RecurrentUnit(m.integer("width"), m.integer("blocks"), m.integer("conv"))
                if mixer.width % mixer.blocks:
                    raise ConfigError(f"{at}.mixer: 'width' {mixer.width} is no multiple of 'blocks' {mixer.blocks}")
            else:
                left = _softmax(KeyReader(_section(m.data, "left", m.where), m.where + ".left"), rot_required=False)
                right = _retention(KeyReader(_section(m.data, "right", m.where), m.where + ".right"))
                mixer = ParallelMixer(left, right, m.number("left_scale", positive=False), m.number("right_scale", positive=False))
            ff = None
            if entry.get("mlp") is not None:
                f = KeyReader(_section(entry, "mlp", at), at + ".mlp")
                if f.data.get("kind", "dense") != "dense":
                    raise ConfigError(f"{at}.mlp: 'kind' = {f.data.get('kind')!r} is no feed-forward of this design; known: ['dense']")
                ff = f.integer("ff")
            out.append(LozezenLayer(kind, mixer, ff))
        norm = KeyReader(_section(data, "norm", where), where + ": norm")
        emb = data.get("embedding")
        scale = KeyReader(emb, where + ": embedding").number("scale", default=1.0) if isinstance(emb, dict) else 1.0
        return LozezenConfig(vocab=r.integer("vocab"), width=r.integer("width"), layers=tuple(out), norm_eps=norm.number("eps"),
                             embedding_scale=scale, max_positions=r.integer("max_positions", default=1 << 17),
                             eos_token_ids=r.token_ids("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""

        def rot(x: Optional[Rotation]):
            if x is None:
                return None
            d: Dict[str, Any] = {"dims": x.dims, "base": x.base}
            if x.factor != 1.0:
                d["scaling"] = {"factor": x.factor}
            return d

        def softmax(a: SoftmaxAttention):
            d = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale, "mask": {"size": a.mask}}
            if a.rot is not None:
                d["rot"] = rot(a.rot)
            return d

        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "attention":
                md = softmax(m)
            elif layer.type == "rglru":
                md = {"width": m.width, "blocks": m.blocks, "conv": m.conv}
            else:
                right = {"heads": m.right.heads, "dim": m.right.dim, "vdim": m.right.vdim, "decay": list(m.right.decay)}
                if m.right.rot is not None:
                    right["rot"] = rot(m.right.rot)
                md = {"left": softmax(m.left), "right": right, "left_scale": m.left_scale, "right_scale": m.right_scale}
            layers.append({"type": layer.type, "mixer": md, "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "max_positions": self.max_positions}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
