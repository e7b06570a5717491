"""Whole-sequence Felosun forward, written out mechanism by mechanism with plain tensor operations.

No cache, no batching: every call recomputes one whole sequence, one (query, head) at a time where a mask is involved.
CPU tensors in the dtype of the weights passed in (float64 in the tests).  Shares nothing with the package: names of
checkpoint tensors and config.json keys are read here on their own.

Notation: n tokens, width W.  A layer is x <- x + norm1(mixer(x)), then x <- x + norm2(ff(x)): the norms act on what the
sublayers give out, the sublayers read x itself.
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension (eps under the root)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def logistic(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def pair_rates(rot: dict, dtype) -> torch.Tensor:
    """Rate of pair i: base^(-2i/dims), divided by the linear scaling factor if there is one."""
    dims = rot["dims"]
    stretch = float((rot.get("scaling") or {}).get("factor", 1.0))
    return torch.tensor([rot["base"] ** (-2.0 * i / dims) / stretch for i in range(dims // 2)], dtype=dtype)


def turn(x: torch.Tensor, rot: dict | None, layout: str, first_position: int = 0) -> torch.Tensor:
    """x [n, heads, d].  The first rot.dims dims of every head are turned by position * rate; `layout` says which dims make a
    pair: "neighbours" (2i, 2i + 1) or "halves" (i, i + dims/2).  The other dims pass."""
    if rot is None:
        return x
    n, dims = x.shape[0], rot["dims"]
    angle = (torch.arange(n, dtype=x.dtype) + first_position)[:, None, None] * pair_rates(rot, x.dtype)
    c, s = angle.cos(), angle.sin()
    out = x.clone()
    if layout == "neighbours":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def visible(i: int, j: int, mask: dict | None) -> bool:
    """Whether query position i sees key position j: causal, and behind a window the first keep_first positions stay."""
    if j > i:
        return False
    if mask is None:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def attention(x: torch.Tensor, w: dict, m: dict, eps: float, kind: str, weights_out: list | None = None) -> torch.Tensor:
    """Both attention mixers.  kind "attention": biases, neighbouring pairs, a sink in the denominator (and, as a rule, a window
    with kept first positions).  kind "attention_2": no biases, half-split pairs, a sigmoid gate per head (and, as a rule,
    linear scaling, a tanh cap on the scores, the whole context).  In both, q and k are made unit-RMS per head after the
    rotation, and the constants a layer's entry gives (mask, softcap, rot.scaling) are what it has."""
    n = x.shape[0]
    heads, groups, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    first = kind == "attention"
    q, k, v = x @ w["q"].T, x @ w["k"].T, x @ w["v"].T
    if first:
        q, k, v = q + w["q.b"], k + w["k.b"], v + w["v.b"]
    q, k, v = q.view(n, heads, d), k.view(n, groups, d), v.view(n, groups, e)
    layout = "neighbours" if first else "halves"
    q, k = unit_rms(turn(q, m.get("rot"), layout), eps), unit_rms(turn(k, m.get("rot"), layout), eps)
    mask, cap = m.get("mask"), m.get("softcap")      # written for one kind each; a layer that is given the other's has it
    out = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        for i in range(n):
            seen = [j for j in range(i + 1) if visible(i, j, mask)]
            scores = (k[seen, g] @ q[i, h]) * m["scale"]
            if cap is not None:
                scores = cap * torch.tanh(scores / cap)
            top = scores.max()
            if first:
                top = torch.maximum(top, w["sink"][h])
            weights = torch.exp(scores - top)
            total = weights.sum()
            if first:
                total = total + torch.exp(w["sink"][h] - top)      # the sink: no key, no value, counted once
            weights = weights / total
            if weights_out is not None:
                weights_out.append((h, i, seen, weights))
            out[i, h] = weights @ v[seen, g]
    if not first:
        out = out * logistic(x @ w["g"].T)[:, :, None]
    return out.reshape(n, heads * e) @ w["o"].T


def expert(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    """g = min(W_gate x, limit); u = clamp(W_up x, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(x @ gate.T, max=limit)
    u = torch.clamp(x @ up.T, min=-limit, max=limit)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ down.T


def choose(logits: torch.Tensor, top: int, margins: list | None = None):
    """(indices [n, top], scores [n, top]): the `top` largest sigmoid scores of every row, the scores as they are."""
    s = logistic(logits)
    values, indices = torch.topk(s, top, dim=-1)
    if margins is not None and top < s.shape[-1]:
        rest = torch.topk(s, top + 1, dim=-1).values
        margins.extend((rest[:, top - 1] - rest[:, top]).tolist())
    return indices, values


def routed_ff(x: torch.Tensor, w: dict, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """sum over the chosen experts of expert(score * x), and the shared expert of x itself."""
    router, sizes = mlp["router"], mlp["expert"]
    indices, scores = choose(x @ w["router"].T, router["top"], margins)
    out = torch.zeros_like(x)
    for i in range(x.shape[0]):
        for e, s in zip(indices[i].tolist(), scores[i]):
            out[i] += expert(s * x[i], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], sizes["limit"])
    shared = mlp.get("shared")
    if shared is not None:
        out = out + expert(x, w["shared.gate"], w["shared.up"], w["shared.down"], shared["limit"])
    return out


def under(weights: dict, prefix: str) -> dict:
    return {name[len(prefix):]: t for name, t in weights.items() if name.startswith(prefix)}


def forward(weights: dict, raw: dict, ids, streams: list | None = None, margins: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence from position 0; streams: gets the stream after every layer."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    eps = raw["norm"]["eps"]
    x = weights["embed"][ids] * raw["embedding"]["scale"] + weights["pos"][: len(ids)]
    for index, layer in enumerate(raw["layers"]):
        w = under(weights, f"l{layer.get('weights_of', index)}.")
        y = attention(x, under(w, "mix."), layer["mixer"], eps, layer["type"])
        x = x + unit_rms(y, eps) * w["norm1"]
        if layer.get("mlp") is not None:
            y = routed_ff(x, under(w, "mlp."), layer["mlp"], margins)
            x = x + unit_rms(y, eps) * w["norm2"]
        if streams is not None:
            streams.append(x.clone())
    x = unit_rms(x, eps) * weights["final.norm"]
    return (x @ weights["head"].T) * raw.get("logit_scale", 1.0)


def read_safetensors(path, dtype=torch.float64) -> dict:
    """name -> tensor from a safetensors file (8-byte length, a JSON header, the data); bfloat16 and float32 data widened to
    `dtype`, int32 tables left as they are."""
    data = Path(path).read_bytes()
    (size,) = struct.unpack("<Q", data[:8])
    header = json.loads(data[8:8 + size])
    out = {}
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "I32": torch.int32}
    for name, entry in header.items():
        if name == "__metadata__":
            continue
        lo, hi = entry["data_offsets"]
        t = torch.frombuffer(bytearray(data[8 + size + lo:8 + size + hi]), dtype=kinds[entry["dtype"]]).reshape(entry["shape"])
        out[name] = t if entry["dtype"] == "I32" else t.to(dtype)
    return out


def load_model_dir(folder, dtype=torch.float64):
    folder = Path(folder)
    raw = json.loads((folder / "config.json").read_text())
    return read_safetensors(folder / "model.safetensors", dtype), raw
