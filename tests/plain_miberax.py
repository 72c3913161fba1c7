"""A plain, slow Miberax in float64 on the CPU: one function per mechanism, whole sequences only,
no cache, no batching. It shares nothing with the engine: it reads ``config.json`` as a dictionary
and the tensors by their checkpoint names.

Notation: ``h [n, width]`` is a sublayer's input, positions count from 0,
``rms(x) = x / sqrt(mean(x^2) + eps)`` over the last axis.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


# ------------------------------------------------------------------------------ norms

def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Each of ``groups`` equal consecutive parts of a row by its own root mean square, then ``w``."""
    n, width = x.shape
    return rms(x.reshape(n, groups, width // groups), eps).reshape(n, width) * w


# ------------------------------------------------------------------------------ left: attention

def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, factor: float) -> torch.Tensor:
    """``x [n, heads, dim]``: the first ``dims`` components of every head are rotated, component
    ``2i`` with ``2i + 1`` by the angle ``p base^(-2i/dims) / factor``; the rest pass."""
    i = torch.arange(dims // 2, dtype=F)
    freq = torch.pow(torch.tensor(base, dtype=F), -2.0 * i / dims) / factor
    angle = positions.to(F)[:, None] * freq[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def chunked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, chunk: int) -> torch.Tensor:
    """``q [n, H, D]``, ``k [n, G, D]``, ``v [n, G, V]`` of one sequence from position 0 -> ``[n, H, V]``;
    query ``i`` sees ``j <= i`` of its own chunk (``chunk`` 0: all of them)."""
    n, H, _ = q.shape
    G = k.shape[1]
    p = torch.arange(n)
    ok = p[None, :] <= p[:, None]
    if chunk > 0:
        ok = ok & (p[None, :] // chunk == p[:, None] // chunk)
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = torch.where(ok, s, torch.full_like(s, -math.inf))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def left_mixer(h: torch.Tensor, t: dict, pre: str, m: dict) -> torch.Tensor:
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(n, H, D)
    k = (h @ t[pre + "k"].T).reshape(n, G, D)
    v = (h @ t[pre + "v"].T).reshape(n, G, V)
    rot = m.get("rot")
    if rot:
        pos = torch.arange(n)
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate_interleaved(q, pos, rot["dims"], rot["base"], factor)
        k = rotate_interleaved(k, pos, rot["dims"], rot["base"], factor)
    chunk = int((m.get("mask") or {}).get("size", 0) or 0)
    o = chunked_attention(q, k, v, m["scale"], chunk)
    return o.reshape(n, H * V) @ t[pre + "o"].T


# ------------------------------------------------------------------------------ right: gated delta rule

def short_conv_silu(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x [n, channels]``, ``w [channels, taps]``: ``y[t] = sum_j w[:, taps-1-j] x[t-j]`` with zeros
    before the start, then silu."""
    n, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for j in range(taps):
        y[j:] += x[:n - j] * w[:, taps - 1 - j]
    return y * torch.sigmoid(y)


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def gated_delta_rule(q, k, v, beta, g):
    """``q, k [n, H, D]`` (already per value head), ``v [n, H, V]``, ``beta, g [n, H]`` -> ``[n, H, V]``.
    Per head: ``S <- g S``; ``u = beta (v - S^T k)``; ``S <- S + k u^T``; ``o = S^T q``."""
    n, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F)
    out = torch.zeros(n, H, V, dtype=F)
    for t in range(n):
        S = S * g[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + torch.einsum("hd,hv->hdv", k[t], u)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def right_mixer(h: torch.Tensor, t: dict, pre: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ t[pre + "q"].T, t[pre + "q.conv"]).reshape(n, G, D)
    k = short_conv_silu(h @ t[pre + "k"].T, t[pre + "k.conv"]).reshape(n, G, D)
    v = short_conv_silu(h @ t[pre + "v"].T, t[pre + "v.conv"]).reshape(n, H, V)
    q = unit(q) * D ** -0.5
    k = unit(k)
    rep = H // G
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ t[pre + "b"].T)
    g = torch.exp(-torch.exp(t[pre + "A_log"]) * torch.nn.functional.softplus(h @ t[pre + "a"].T + t[pre + "dt_bias"]))
    o = gated_delta_rule(q, k, v, beta, g)
    gate = (h @ t[pre + "g"].T).reshape(n, H, V)
    o = rms(o, eps) * t[pre + "norm"] * (gate * torch.sigmoid(gate))
    return o.reshape(n, H * V) @ t[pre + "o"].T


def parallel_mixer(h: torch.Tensor, t: dict, pre: str, m: dict, eps: float) -> torch.Tensor:
    left = rms(left_mixer(h, t, pre + "left.", m["left"]), eps) * t[pre + "left.out"]
    right = rms(right_mixer(h, t, pre + "right.", m["right"], eps), eps) * t[pre + "right.out"]
    return 0.5 * (left + right)


# ------------------------------------------------------------------------------ feed-forward

def poly_norm_mlp(h: torch.Tensor, t: dict, pre: str, eps: float) -> torch.Tensor:
    z = h @ t[pre + "up"].T
    a, b, c, e = t[pre + "act"]
    act = a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e
    return act @ t[pre + "down"].T


def clamped_expert(h: torch.Tensor, t: dict, pre: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ t[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ t[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[pre + "down"].T


def route(h: torch.Tensor, t: dict, pre: str, r: dict):
    """Chosen experts ``[n, top]`` and their weights ``[n, top]``; ids at or above ``experts`` are
    identity experts."""
    total = r["experts"] + int(r.get("identity", 0) or 0)
    s = torch.softmax(h @ t[pre + "router"].T, dim=-1)
    choice = s + t[pre + "correction"] if (pre + "correction") in t else s.clone()
    groups = r.get("groups") or {}
    count, keep = int(groups.get("count", 1) or 1), int(groups.get("keep", 1) or 1)
    if count > 1:
        per = total // count
        best = choice.reshape(-1, count, per).max(-1).values
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
        choice = torch.where(kept.repeat_interleave(per, dim=1), choice, torch.full_like(choice, -math.inf))
    chosen = choice.topk(r["top"], dim=-1).indices
    w = s.gather(1, chosen)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))
    return chosen, w


def moe(h: torch.Tensor, t: dict, pre: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    chosen, w = route(h, t, pre, r)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, we in zip(chosen[i].tolist(), w[i]):
            if e >= r["experts"]:
                out[i] += we * h[i]
            else:
                out[i] += we * clamped_expert(h[i:i + 1], t, f"{pre}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        gate = torch.sigmoid(h @ t[pre + "shared.sg"].T)
        out = out + gate * clamped_expert(h, t, pre + "shared.", mlp["shared"]["limit"])
    return out


# ------------------------------------------------------------------------------ the model

def forward(cfg: dict, tensors: dict, tokens, return_layers: bool = False):
    """Logits ``[n, vocab]`` of one sequence from position 0 (and the residual stream after every layer)."""
    t = {k: v.to(F) for k, v in tensors.items()}
    eps, groups = cfg["norm"]["eps"], int(cfg["norm"].get("groups", 1) or 1)
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        x = x + parallel_mixer(group_norm(x, t[p + "norm1"], groups, eps), t, p + "mix.", layer["mixer"], eps)
        mlp = layer.get("mlp")
        if mlp:
            h = group_norm(x, t[p + "norm2"], groups, eps)
            x = x + (poly_norm_mlp(h, t, p + "mlp.", eps) if mlp["kind"] == "dense" else moe(h, t, p + "mlp.", mlp))
        streams.append(x)
    logits = group_norm(x, t["final.norm"], groups, eps) @ t["embed"].T
    return (logits, torch.stack(streams)) if return_layers else logits


forward_logits = forward


def greedy_generate(cfg: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(forward(cfg, tensors, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


# ------------------------------------------------------------------------------ weights of a test model

def tensor_shapes(cfg: dict) -> dict[str, tuple]:
    """Name -> shape of every tensor of a model of this configuration."""
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        out[f"l{i}.norm1"] = (w,)
        a, d = layer["mixer"]["left"], layer["mixer"]["right"]
        p = f"l{i}.mix.left."
        out.update({p + "q": (a["heads"] * a["dim"], w), p + "k": (a["kv_heads"] * a["dim"], w),
                    p + "v": (a["kv_heads"] * a["vdim"], w), p + "o": (w, a["heads"] * a["vdim"]), p + "out": (w,)})
        p = f"l{i}.mix.right."
        qk, hv, taps = d["kv_heads"] * d["dim"], d["heads"] * d["vdim"], d["conv"]
        out.update({p + "q": (qk, w), p + "k": (qk, w), p + "v": (hv, w), p + "q.conv": (qk, taps), p + "k.conv": (qk, taps),
                    p + "v.conv": (hv, taps), p + "b": (d["heads"], w), p + "a": (d["heads"], w), p + "A_log": (d["heads"],),
                    p + "dt_bias": (d["heads"],), p + "norm": (d["vdim"],), p + "g": (hv, w), p + "o": (w, hv), p + "out": (w,)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        out[f"l{i}.norm2"] = (w,)
        p = f"l{i}.mlp."
        if mlp["kind"] == "dense":
            out.update({p + "up": (mlp["ff"], w), p + "down": (w, mlp["ff"]), p + "act": (4,)})
            continue
        r, f = mlp["router"], mlp["expert"]["ff"]
        total = r["experts"] + int(r.get("identity", 0) or 0)
        out.update({p + "router": (total, w), p + "correction": (total,)})
        for e in range(r["experts"]):
            out.update({f"{p}e{e}.gate": (f, w), f"{p}e{e}.up": (f, w), f"{p}e{e}.down": (w, f)})
        if mlp.get("shared"):
            s = mlp["shared"]["ff"]
            out.update({p + "shared.gate": (s, w), p + "shared.up": (s, w), p + "shared.down": (w, s), p + "shared.sg": (1, w)})
    return out


def random_weights(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """Random tensors whose values are exactly representable in bfloat16 (float64 here), drawn so that
    every mechanism matters: projections of unit-size outputs (so that the experts' clamps bite), norm
    weights near one, a router that prefers some experts clearly, corrections that change its choice
    and make some choice scores negative, decays spread out."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm", "out"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif leaf == "A_log":
            t = torch.rand(shape, generator=g) * 2.0 - 1.5
        elif leaf == "dt_bias":
            t = torch.randn(shape, generator=g)
        elif leaf == "act":
            t = torch.tensor([1.0, 0.5, -0.3, 0.1]) + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.15 * torch.randn(shape, generator=g) - 0.05
        elif leaf == "router":
            t = 3.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        elif name == "embed":
            t = 0.5 * torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1]) * (2.0 if leaf in ("q", "k") else 1.0)
        out[name] = t.to(torch.bfloat16).to(F)
    return out


def jittered(tensors: dict, seed: int = 0, size: float = 2.0 ** -8) -> dict:
    """Every matrix with relative noise of the size of bfloat16's rounding: how far the logits of a
    position move under it says how far rounding may move them."""
    g = torch.Generator().manual_seed(seed)
    return {n: t * (1 + size * torch.randn(t.shape, generator=g, dtype=F)) if t.dim() == 2 and not n.endswith("router") else t
            for n, t in tensors.items()}


def write_folder(folder, cfg: dict, tensors: dict):
    """``config.json`` and ``model.safetensors`` (bfloat16) of ``tensors``, written byte by byte here."""
    import json

    import numpy as np

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    header, blobs, at = {}, [], 0
    for name in sorted(tensors):
        bits = (tensors[name].to(torch.float32).contiguous().view(torch.int32).numpy().astype(np.uint32) >> 16).astype("<u2")
        raw = bits.tobytes()
        header[name] = {"dtype": "BF16", "shape": list(tensors[name].shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    head = json.dumps(header).encode()
    head += b" " * (-len(head) % 8)
    with open(folder / "model.safetensors", "wb") as f:
        f.write(len(head).to_bytes(8, "little") + head + b"".join(blobs))
    return folder
