"""Typed configuration of the Miberax decoder: a list of layers, each a pair of mixers side by side
(rotary attention under a chunked mask, and a gated delta rule behind short convolutions) whose
normalised outputs are averaged, and a feed-forward that is dense with a polynomial activation, a
mixture of clamped experts behind a grouped router, or absent. Pre-norm layers with RMS norms in
groups, a 32-bit residual stream, a head tied to the embedding.

``config.json`` keys: ``vocab``, ``width``, ``norm.eps``, ``norm.groups`` and ``layers``: a list of
``{"type": "parallel", "mixer": {"left": {...}, "right": {...}}, "mlp": {...} | null}``.
``mixer.left``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size`` (absent: every earlier
position is seen), ``rot.{dims, base, scaling.factor}`` (absent: no rotation).
``mixer.right``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``.
``mlp``: ``{"kind": "dense", "ff"}`` or ``{"kind": "moe", "expert": {ff, limit},
"router": {experts, top, identity, scale, groups: {count, keep}}, "shared": {ff, limit} | absent}``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from .errors import UnsupportedModelError
from .makodra import _need, _positive

LAYER_TYPES = ("parallel",)
MLP_KINDS = ("dense", "moe")


def _grouping(m: Mapping[str, Any], where: str) -> tuple[int, int]:
    heads = _positive(_need(m, "heads", where), where + ".heads")
    kv = _positive(m.get("kv_heads") or heads, where + ".kv_heads")
    if heads % kv:
        raise UnsupportedModelError(f"{where}: {heads} heads do not group onto {kv} kv_heads")
    return heads, kv


@dataclass(frozen=True)
class MiberaxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0             # mask.size (0: every earlier position is seen)
    rot_dims: int = 0          # 0: no rotation
    rot_base: float = 10000.0
    rot_factor: float = 1.0    # linear scaling: every frequency is divided by it

    @staticmethod
    def parse(m: Mapping[str, Any], where: str) -> "MiberaxAttention":
        heads, kv = _grouping(m, where)
        dim = _positive(_need(m, "dim", where), where + ".dim")
        mask = dict(m.get("mask") or {})
        unknown = set(mask) - {"size"}
        if unknown:
            raise UnsupportedModelError(f"{where}.mask has keys that are not implemented: {sorted(unknown)}")
        fields: dict[str, Any] = {}
        rot = m.get("rot")
        if rot:
            dims = _positive(_need(rot, "dims", where + ".rot"), where + ".rot.dims")
            if dims % 2 or dims > dim:
                raise UnsupportedModelError(f"{where}.rot.dims={dims} must be even and at most dim={dim}")
            scaling = dict(rot.get("scaling") or {})
            unknown = set(scaling) - {"factor"}
            if unknown:
                raise UnsupportedModelError(f"{where}.rot.scaling has keys that are not implemented: {sorted(unknown)}")
            factor = float(scaling.get("factor", 1.0))
            if not factor > 0:
                raise UnsupportedModelError(f"{where}.rot.scaling.factor={factor} must be positive")
            fields = dict(rot_dims=dims, rot_base=float(_need(rot, "base", where + ".rot")), rot_factor=factor)
        return MiberaxAttention(
            heads=heads, kv_heads=kv, dim=dim, vdim=_positive(m.get("vdim") or dim, where + ".vdim"),
            scale=float(_need(m, "scale", where)),
            chunk=_positive(mask["size"], where + ".mask.size") if mask.get("size") is not None else 0, **fields)


@dataclass(frozen=True)
class MiberaxDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @staticmethod
    def parse(m: Mapping[str, Any], where: str) -> "MiberaxDelta":
        heads, kv = _grouping(m, where)
        dim = _positive(_need(m, "dim", where), where + ".dim")
        conv = _positive(_need(m, "conv", where), where + ".conv")
        if conv > 16:
            raise UnsupportedModelError(f"{where}.conv={conv}: the convolution kernel takes up to 16 taps")
        return MiberaxDelta(heads=heads, kv_heads=kv, dim=dim, vdim=_positive(m.get("vdim") or dim, where + ".vdim"), conv=conv)


@dataclass(frozen=True)
class MiberaxMLP:
    kind: str
    ff: int = 0                 # dense: the hidden size; moe: an expert's
    limit: float = 0.0          # moe: the experts' clamp
    experts: int = 0
    top: int = 0
    identity: int = 0
    scale: float = 1.0
    groups: int = 1
    groups_kept: int = 1
    shared_ff: int = 0          # 0: no shared expert
    shared_limit: float = 0.0

    @staticmethod
    def parse(raw: Mapping[str, Any], where: str) -> "MiberaxMLP":
        kind = raw.get("kind", "dense")
        if kind not in MLP_KINDS:
            raise UnsupportedModelError(f"{where}.kind={kind!r}; known: {MLP_KINDS}")
        if kind == "dense":
            return MiberaxMLP(kind=kind, ff=_positive(_need(raw, "ff", where), where + ".ff"))
        expert, router = _need(raw, "expert", where), _need(raw, "router", where)
        experts = _positive(_need(router, "experts", where + ".router"), where + ".router.experts")
        identity = int(router.get("identity") or 0)
        top = _positive(_need(router, "top", where + ".router"), where + ".router.top")
        groups = dict(router.get("groups") or {})
        count, keep = int(groups.get("count") or 1), int(groups.get("keep") or groups.get("count") or 1)
        total = experts + identity
        if identity < 0 or top > total or count < 1 or total % count or not 1 <= keep <= count or keep * (total // count) < top:
            raise UnsupportedModelError(f"{where}.router: {top} of {experts}+{identity} outputs in {count} groups "
                                        f"of which {keep} are kept cannot be chosen")
        shared = raw.get("shared")
        return MiberaxMLP(
            kind=kind, ff=_positive(_need(expert, "ff", where + ".expert"), where + ".expert.ff"),
            limit=float(_need(expert, "limit", where + ".expert")), experts=experts, top=top, identity=identity,
            scale=float(router.get("scale", 1.0)), groups=count, groups_kept=keep,
            shared_ff=_positive(_need(shared, "ff", where + ".shared"), where + ".shared.ff") if shared else 0,
            shared_limit=float(_need(shared, "limit", where + ".shared")) if shared else 0.0)


@dataclass(frozen=True)
class MiberaxLayer:
    type: str
    left: MiberaxAttention
    right: MiberaxDelta
    mlp: Optional[MiberaxMLP]

    @staticmethod
    def parse(raw: Mapping[str, Any], index: int) -> "MiberaxLayer":
        where = f"layers[{index}]"
        kind = _need(raw, "type", where)
        if kind not in LAYER_TYPES:
            raise UnsupportedModelError(f"{where}.type={kind!r}; known: {LAYER_TYPES}")
        m = _need(raw, "mixer", where)
        mlp = raw.get("mlp")
        return MiberaxLayer(type=kind, left=MiberaxAttention.parse(_need(m, "left", where + ".mixer"), where + ".mixer.left"),
                            right=MiberaxDelta.parse(_need(m, "right", where + ".mixer"), where + ".mixer.right"),
                            mlp=MiberaxMLP.parse(mlp, where + ".mlp") if mlp is not None else None)


@dataclass(frozen=True)
class MiberaxConfig:
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    layers: tuple[MiberaxLayer, ...]

    architecture = "Miberax"

    # the names under which the engine's tools ask any configuration for its common sizes
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "MiberaxConfig":
        layers = _need(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise UnsupportedModelError("layers must be a list with at least one layer")
        norm = _need(raw, "norm", "")
        width = _positive(_need(raw, "width", ""), "width")
        groups = _positive(norm.get("groups") or 1, "norm.groups")
        if width % groups:
            raise UnsupportedModelError(f"width={width} does not split into norm.groups={groups} equal parts")
        return cls(vocab=_positive(_need(raw, "vocab", ""), "vocab"), width=width,
                   norm_eps=float(_need(norm, "eps", "norm")), norm_groups=groups,
                   layers=tuple(MiberaxLayer.parse(l, i) for i, l in enumerate(layers)))
