"""A plain, slow Makodra in float64 on the CPU: one function per mechanism, whole sequences only,
no cache, no batching. It shares nothing with the engine: it reads ``config.json`` as a dictionary
and the tensors by their checkpoint names.

Notation: ``h [n, width]`` is a sublayer's input, positions count from 0, ``rms(x) = x / sqrt(mean(x^2) + eps)``
over the last axis.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np
import torch

F = torch.float64


# ------------------------------------------------------------------------------ small pieces

def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sinusoid(positions: torch.Tensor, width: int, base: float = 10000.0) -> torch.Tensor:
    """``[n, width]``: column ``2i`` is ``sin(p base^(-2i/width))``, column ``2i+1`` the cosine."""
    i = torch.arange((width + 1) // 2, dtype=F)
    angle = positions.to(F)[:, None] * torch.pow(torch.tensor(base, dtype=F), -2.0 * i / width)[None, :]
    pe = torch.zeros(positions.shape[0], 2 * i.shape[0], dtype=F)
    pe[:, 0::2], pe[:, 1::2] = torch.sin(angle), torch.cos(angle)
    return pe[:, :width]


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(x / cap) if cap > 0 else x


def gated_mlp(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    g = h @ gate.T
    return ((g * torch.sigmoid(g)) * (h @ up.T)) @ down.T


def lowrank(h: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w0: torch.Tensor) -> torch.Tensor:
    return torch.tanh(h @ w1.T) @ w2.T + w0


# ------------------------------------------------------------------------------ attention

def visible(n: int, chunk: int = 0, window: int = 0, first: int = 0) -> torch.Tensor:
    """``[n, n]`` booleans: query ``i`` (at position ``first + i``) sees key ``j``."""
    p = torch.arange(first, first + n)
    ok = p[None, :] <= p[:, None]
    if chunk > 0:
        ok = ok & (p[None, :] // chunk == p[:, None] // chunk)
    if window > 0:
        ok = ok & (p[None, :] > p[:, None] - window)
    return ok


def sink_softmax(scores: torch.Tensor, ok: torch.Tensor, sink: bool) -> torch.Tensor:
    """Weights ``exp(s_j) / (sink + sum_visible exp(s_j))``; a row that sees nothing is all zeros."""
    e = torch.where(ok, torch.exp(scores), torch.zeros_like(scores))
    total = e.sum(-1, keepdim=True) + (1.0 if sink else 0.0)
    return torch.where(total > 0, e / total, torch.zeros_like(e))


def scored_attention_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, *, chunk: int = 0,
                          window: int = 0, sink: bool = False, r1=None, r2=None) -> torch.Tensor:
    """``q [n, H, D]``, ``k [n, G, D]``, ``v [n, G, V]`` of one sequence from position 0 -> ``[n, H, V]``."""
    n, H, _ = q.shape
    G = k.shape[1]
    p = torch.arange(n)
    dist = (p[:, None] - p[None, :]).clamp(min=0).to(F)
    ok = visible(n, chunk, window)
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if r1 is not None:
            s = s - r1[h] * torch.log1p(r2[h] * dist)
        out[:, h] = sink_softmax(s, ok, sink) @ v[:, g]
    return out


def attention_mixer(h: torch.Tensor, W: dict, p: str, m: dict, eps: float, shared: dict) -> torch.Tensor:
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    G, V = m.get("kv_heads") or H, m.get("vdim") or D
    q = rms((h @ W[p + "q"].T).view(n, H, D), eps)
    k = rms((h @ W[p + "k"].T).view(n, G, D), eps)
    v = (h @ W[p + "v"].T).view(n, G, V)
    if m.get("v_mix"):
        if "first" in shared:
            lam = W[p + "vmix"]
            v = (1 - lam) * v + lam * shared["first"]
        else:
            shared["first"] = v
    chunk = (m.get("mask") or {}).get("size") or 0
    o = scored_attention_core(q, k, v, m["scale"], chunk=chunk, sink=True, r1=W[p + "r1"], r2=W[p + "r2"])
    return (o.reshape(n, H * V) * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


# ------------------------------------------------------------------------------ recurrences

def delta_rule(r, k, v, w, a, state=None):
    """``r, k, v, w, a [n, H, D]`` -> ``o [n, H, D]`` and the last state ``[H, D(key), D(value)]``."""
    n, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=F) if state is None else state.clone()
    o = torch.zeros(n, H, D, dtype=F)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    for t in range(n):
        uS = torch.einsum("hk,hkv->hv", u[t], S)
        S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, r[t])
    return o, S


def bonus_rule(r, k, v, w, bonus, state=None):
    n, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=F) if state is None else state.clone()
    o = torch.zeros(n, H, D, dtype=F)
    for t in range(n):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S + bonus[:, :, None] * kv, r[t])
        S = w[t][:, :, None] * S + kv
    return o, S


def general_delta_mixer(h: torch.Tensor, W: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, D = h.shape[0], m["heads"], m["dim"]
    r, k, v = ((h @ W[p + s].T).view(n, H, D) for s in ("r", "k", "v"))
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lowrank(h, W[p + "w1"], W[p + "w2"], W[p + "w0"]))).view(n, H, D)
    a = torch.sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(n, H, D)
    o, _ = delta_rule(r, k, v, w, a)
    o = rms(o, eps).reshape(n, H * D) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def shifted(h: torch.Tensor, before=None) -> torch.Tensor:
    first = torch.zeros(1, h.shape[1], dtype=F) if before is None else before.reshape(1, -1)
    return torch.cat([first, h[:-1]], 0)


def wkv_mixer(h: torch.Tensor, W: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    n, H, D = h.shape[0], m["heads"], m["dim"]
    prev = shifted(h)
    mix = lambda s: h + (prev - h) * W[p + "mu." + s]
    r, k, v = ((mix(s) @ W[p + s].T).view(n, H, D) for s in ("r", "k", "v"))
    g = mix("g") @ W[p + "g"].T
    w = torch.exp(-torch.exp(lowrank(mix("w"), W[p + "w1"], W[p + "w2"], W[p + "w0"]))).view(n, H, D)
    o, _ = bonus_rule(r, k, v, w, W[p + "u"])
    o = rms(o, eps).reshape(n, H * D) * W[p + "norm"] * (g * torch.sigmoid(g))
    return o @ W[p + "o"].T


# ------------------------------------------------------------------------------ the model

def forward_logits(W: dict, cfg: dict, tokens, layers_out=None, operand_noise: float = 0.0) -> torch.Tensor:
    """Logits ``[n, vocab]`` of one sequence from position 0. ``operand_noise``: relative noise on
    what every sublayer reads (the size of a rounding of the products' operands), for probing how
    far rounding can move a row; 0 for the model itself."""
    n, width, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens))] + sinusoid(torch.arange(n), width)
    g = torch.Generator().manual_seed(1)
    read = (lambda t: t * (1 + operand_noise * torch.randn(t.shape, generator=g, dtype=F))) if operand_noise else (lambda t: t)
    shared: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "attention":
            y = attention_mixer(read(x), W, p, m, eps, shared)
        elif layer["type"] == "general_delta":
            y = general_delta_mixer(read(x), W, p, m, eps)
        else:
            y = wkv_mixer(read(x), W, p, m, eps)
        x = x + rms(y, eps) * W[f"l{i}.norm1"]
        if layer.get("mlp"):
            q = f"l{i}.mlp."
            x = x + rms(gated_mlp(read(x), W[q + "gate"], W[q + "up"], W[q + "down"]), eps) * W[f"l{i}.norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return softcap((rms(x, eps) * W["final.norm"]) @ W["embed"].T, cfg.get("logit_softcap") or 0.0)


def greedy_generate(W: dict, cfg: dict, prompt, n_new: int) -> list[int]:
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(forward_logits(W, cfg, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


# ------------------------------------------------------------------------------ weights of a test model

def tensor_shapes(cfg: dict, rank: int = 8) -> dict[str, tuple]:
    """Name -> shape of every tensor of a model of this configuration."""
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        out[f"l{i}.norm1"] = (w,)
        H, D = m["heads"], m["dim"]
        if layer["type"] == "attention":
            G, V = m.get("kv_heads") or H, m.get("vdim") or D
            out.update({p + "q": (H * D, w), p + "k": (G * D, w), p + "v": (G * V, w), p + "g": (H * V, w),
                        p + "o": (w, H * V), p + "r1": (H,), p + "r2": (H,)})
            if m.get("v_mix"):
                out[p + "vmix"] = ()
        else:
            c, rk = H * D, m.get("rank") or rank
            out.update({p + s: (c, w) for s in ("r", "k", "v", "g")})
            out.update({p + "w1": (rk, w), p + "w2": (c, rk), p + "w0": (c,), p + "norm": (c,), p + "o": (w, c)})
            if layer["type"] == "general_delta":
                out.update({p + "a": (c, w), p + "a.b": (c,)})
            else:
                out.update({p + "mu." + s: (w,) for s in "rkvgw"})
                out[p + "u"] = (H, D)
        if layer.get("mlp"):
            q = f"l{i}.mlp."
            out[f"l{i}.norm2"] = (w,)
            out.update({q + "gate": (layer["mlp"]["ff"], w), q + "up": (layer["mlp"]["ff"], w), q + "down": (w, layer["mlp"]["ff"])})
    return out


def random_weights(cfg: dict, seed: int, rank: int = 8) -> dict[str, torch.Tensor]:
    """Random tensors whose values are exactly representable in bfloat16 (float64 here), drawn so
    that every mechanism matters: matrices of unit-size outputs, norms near one, decays and rates
    spread out, distance penalties and the value mix well away from zero."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        leaf = name.split(".")[-1]
        if name.endswith("mix.norm") or leaf in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "r1":
            t = 0.3 + 0.5 * torch.rand(shape, generator=g)
        elif leaf == "r2":
            t = 0.2 + 1.5 * torch.rand(shape, generator=g)
        elif leaf == "vmix":
            t = torch.tensor(0.35) + 0.2 * torch.rand((), generator=g)
        elif leaf in ("w0", "b"):
            t = torch.randn(shape, generator=g)
        elif name.split(".")[-2:-1] == ["mu"]:
            t = torch.rand(shape, generator=g)
        elif leaf == "u":
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = 0.4 * torch.randn(shape, generator=g)   # logits of a few units: a soft cap of that size bends them
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1]) * (2.0 if leaf in ("q", "k", "w2") else 1.0)
        out[name] = t.to(torch.bfloat16).to(F)
    return out


def jittered(W: dict, seed: int = 0, size: float = 2.0 ** -8) -> dict:
    """Every matrix with relative noise of the size of bfloat16's rounding: how far the logits of
    a position move under it says how far rounding may move them (a row whose sign hangs on a
    dot product near zero, the first token of a recurrence for instance, moves a lot)."""
    g = torch.Generator().manual_seed(seed)
    return {n: t * (1 + size * torch.randn(t.shape, generator=g, dtype=F)) if t.dim() == 2 else t for n, t in W.items()}


def write_folder(folder: Path, cfg: dict, W: dict) -> Path:
    """``config.json`` and ``model.safetensors`` (bfloat16) of ``W``, written byte by byte here."""
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    header, blobs, at = {}, [], 0
    for name in sorted(W):
        bits = (W[name].to(torch.float32).contiguous().view(torch.int32).numpy().astype(np.uint32) >> 16).astype("<u2")
        raw = bits.tobytes()
        header[name] = {"dtype": "BF16", "shape": list(W[name].shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    head = json.dumps(header).encode()
    head += b" " * (-len(head) % 8)
    with open(folder / "model.safetensors", "wb") as f:
        f.write(len(head).to_bytes(8, "little") + head + b"".join(blobs))
    return folder
