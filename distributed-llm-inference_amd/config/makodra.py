"""Typed configuration of the Makodra decoder: a list of layers, each with one mixer (attention
with changed scores, a generalized delta rule, or decayed sums with token shift) and an optional
gated feed-forward, norms on the sublayers' outputs, sinusoidal positions added to the embedding,
a tied head with a soft cap on the logits.

``config.json`` keys: ``vocab``, ``width``, ``norm.eps``, ``logit_softcap``, and ``layers``: a list of
``{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}``. Mixer keys by type:
``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size``, ``v_mix``;
``general_delta`` and ``wkv``: ``heads``, ``dim`` (and optionally ``rank``, the rank of the decay's
low-rank projection, which a checkpoint's tensors give by themselves).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from .errors import MissingConfigKeyError, UnsupportedModelError

MIXER_TYPES = ("attention", "general_delta", "wkv")


def _need(d: Mapping[str, Any], key: str, where: str) -> Any:
    if key not in d or d[key] is None:
        raise MissingConfigKeyError(f"{where}.{key}" if where else key)
    return d[key]


def _positive(value: Any, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise UnsupportedModelError(f"{name}={value!r} must be a positive integer")
    return value


@dataclass(frozen=True)
class MakodraLayer:
    type: str
    heads: int
    dim: int
    kv_heads: int = 0          # attention
    vdim: int = 0              # attention
    scale: float = 0.0         # attention
    chunk: int = 0             # attention: mask.size (0: every earlier position is seen)
    v_mix: bool = False        # attention
    rank: Optional[int] = None  # general_delta, wkv
    ff: int = 0                # 0: no feed-forward

    @staticmethod
    def parse(raw: Mapping[str, Any], index: int) -> "MakodraLayer":
        where = f"layers[{index}]"
        kind = _need(raw, "type", where)
        if kind not in MIXER_TYPES:
            raise UnsupportedModelError(f"{where}.type={kind!r}; known: {MIXER_TYPES}")
        m = _need(raw, "mixer", where)
        heads = _positive(_need(m, "heads", where + ".mixer"), where + ".mixer.heads")
        dim = _positive(_need(m, "dim", where + ".mixer"), where + ".mixer.dim")
        fields: dict[str, Any] = {}
        if kind == "attention":
            kv = _positive(m.get("kv_heads") or heads, where + ".mixer.kv_heads")
            if heads % kv:
                raise UnsupportedModelError(f"{where}: {heads} heads do not group onto {kv} kv_heads")
            mask = dict(m.get("mask") or {})
            if str(mask.pop("kind", "chunk")).lower() not in ("chunk", "chunked"):
                raise UnsupportedModelError(f"{where}.mixer.mask.kind={m['mask']['kind']!r}; known: 'chunk'")
            unknown = set(mask) - {"size"}
            if unknown:
                raise UnsupportedModelError(f"{where}.mixer.mask has keys that are not implemented: {sorted(unknown)}")
            fields = dict(kv_heads=kv, vdim=_positive(m.get("vdim") or dim, where + ".mixer.vdim"),
                          scale=float(_need(m, "scale", where + ".mixer")),
                          chunk=_positive(mask["size"], where + ".mixer.mask.size") if mask.get("size") is not None else 0,
                          v_mix=bool(m.get("v_mix", False)))
        elif m.get("rank") is not None:
            fields = dict(rank=_positive(m["rank"], where + ".mixer.rank"))
        mlp = raw.get("mlp")
        ff = 0
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise UnsupportedModelError(f"{where}.mlp.kind={mlp.get('kind')!r}; known: 'dense'")
            ff = _positive(_need(mlp, "ff", where + ".mlp"), where + ".mlp.ff")
        return MakodraLayer(type=kind, heads=heads, dim=dim, ff=ff, **fields)


@dataclass(frozen=True)
class MakodraConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: float
    layers: tuple[MakodraLayer, ...]

    architecture = "Makodra"

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
    def from_dict(cls, raw: Mapping[str, Any]) -> "MakodraConfig":
        layers = _need(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise UnsupportedModelError("layers must be a list with at least one layer")
        norm = _need(raw, "norm", "")
        cap = raw.get("logit_softcap")
        return cls(vocab=_positive(_need(raw, "vocab", ""), "vocab"), width=_positive(_need(raw, "width", ""), "width"),
                   norm_eps=float(_need(norm, "eps", "norm")), logit_softcap=float(cap) if cap else 0.0,
                   layers=tuple(MakodraLayer.parse(l, i) for i, l in enumerate(layers)))
