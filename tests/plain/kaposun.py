"""Whole-sequence Kaposun forward, written out mechanism by mechanism with plain tensor operations.

No cache, no state carried between calls, no batching: every call recomputes one whole sequence, with token loops
where the definition is a recurrence.  CPU tensors in the dtype of the weights passed in (float64 in the tests).
Shares nothing with the package: names of checkpoint tensors and config.json keys are read here on their own.

Notation: n tokens, width W.  A layer is x <- x + m * (mixer(h) + feed_forward(h)) with h = the one norm of x.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension (eps under the root)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def swish(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def logistic(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def soft_plus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def gelu_exact(x: torch.Tensor) -> torch.Tensor:
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def causal_taps(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """x [n, channels], taps [channels, t]: y[i, c] = bias[c] + sum_j taps[c, j] x[i - (t - 1 - j), c], zeros before the start."""
    n, t = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x) if bias is None else bias.expand(n, -1).clone()
    for i in range(n):
        for j in range(t):
            source = i - (t - 1 - j)
            if source >= 0:
                y[i] += taps[:, j] * x[source]
    return y


def turn_front(x: torch.Tensor, base: float, dims: int, stretch: float) -> torch.Tensor:
    """x [n, heads, d]: dim i < dims/2 of every head paired with i + dims/2 and turned by position * base^(-2i/dims) / stretch."""
    n, half = x.shape[0], dims // 2
    rate = torch.tensor([base ** (-2.0 * i / dims) / stretch for i in range(half)], dtype=x.dtype)
    angle = torch.arange(n, dtype=x.dtype)[:, None, None] * rate
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat((u * angle.cos() - v * angle.sin(), v * angle.cos() + u * angle.sin(), x[..., dims:]), -1)


def sees(i: int, j: int, window: int | None, kept: int) -> bool:
    return j <= i and (window is None or i - j < window or j < kept)


def softmax_attention(x, w, *, heads, groups, d, e, eps, scale, rot=None, window=None, kept=0, gated=False):
    """Grouped-query attention whose q and k pass an RMS norm over the whole projection (all heads at once).
    rot: (base, dims, stretch) or None; window, kept: i sees j <= i with i - j < window or j < kept; gated: the
    heads' outputs times sigmoid(W_g x) before the output matrix."""
    n = x.shape[0]
    q = unit_rms(x @ w["q"].T, eps) * w["q.norm"]
    k = unit_rms(x @ w["k"].T, eps) * w["k.norm"]
    q, k, v = q.view(n, heads, d), k.view(n, groups, d), (x @ w["v"].T).view(n, groups, e)
    if rot is not None:
        q, k = turn_front(q, *rot), turn_front(k, *rot)
    out = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        for i in range(n):
            seen = [j for j in range(i + 1) if sees(i, j, window, kept)]
            scores = (k[seen, g] @ q[i, h]) * scale
            out[i, h] = torch.softmax(scores, 0) @ v[seen, g]
    out = out.reshape(n, heads * e)
    if gated:
        out = out * logistic(x @ w["g"].T)
    return out @ w["o"].T


def state_space(x, w, *, heads, groups, state, e, taps, parts, eps):
    """Selective state space layer: per head a matrix S [state, e], S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x."""
    n, inner = x.shape[0], heads * e
    z, xbc, dt = torch.split(x @ w["in"].T, [inner, inner + 2 * groups * state, heads], -1)
    xbc = swish(causal_taps(xbc, w["conv"], w["conv.b"]))
    u, b, c = torch.split(xbc, [inner, groups * state, groups * state], -1)
    u, b, c = u.view(n, heads, e), b.view(n, groups, state), c.view(n, groups, state)
    dt = soft_plus(dt + w["dt_bias"])
    y = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        s = torch.zeros(state, e, dtype=x.dtype)
        for i in range(n):
            s = torch.exp(-torch.exp(w["A_log"][h]) * dt[i, h]) * s + dt[i, h] * torch.outer(b[i, g], u[i, h])
            y[i, h] = s.T @ c[i, g] + w["D"][h] * u[i, h]
    y = y.reshape(n, inner) * swish(z)
    y = unit_rms(y.view(n, parts, inner // parts), eps).reshape(n, inner) * w["norm"]
    return y @ w["o"].T


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def delta_rule_channel_decay(x, w, *, heads, groups, d, e, eps):
    """Gated delta rule with a decay per head and key channel: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    n = x.shape[0]
    q = unit(swish(causal_taps(x @ w["q"].T, w["q.conv"])).view(n, groups, d)) * d ** -0.5
    k = unit(swish(causal_taps(x @ w["k"].T, w["k.conv"])).view(n, groups, d))
    v = swish(causal_taps(x @ w["v"].T, w["v.conv"])).view(n, heads, e)
    beta = logistic(x @ w["b"].T)
    decay_in = soft_plus((x @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(n, heads, d)
    g = torch.exp(-torch.exp(w["A_log"])[None, :, None] * decay_in)
    gate = logistic((x @ w["g1"].T) @ w["g2"].T).view(n, heads, e)
    o = torch.zeros(n, heads, e, dtype=x.dtype)
    for h in range(heads):
        j = h // (heads // groups)
        s = torch.zeros(d, e, dtype=x.dtype)
        for i in range(n):
            s = g[i, h][:, None] * s
            u = beta[i, h] * (v[i, h] - s.T @ k[i, j])
            s = s + torch.outer(k[i, j], u)
            o[i, h] = s.T @ q[i, j]
    o = unit_rms(o, eps) * w["norm"] * gate
    return o.reshape(n, heads * e) @ w["o"].T


def under(tensors: dict, prefix: str) -> dict:
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


def mixer_output(kind: str, sizes: dict, h: torch.Tensor, w: dict, eps: float) -> torch.Tensor:
    if kind == "mamba2":
        return state_space(h, w, heads=sizes["heads"], groups=sizes["groups"], state=sizes["state"], e=sizes["vdim"], taps=sizes["conv"],
                           parts=sizes["norm_groups"], eps=eps)
    if kind == "attention":
        return _attention(sizes, h, w, eps, gated=False)
    if kind == "parallel":
        left = _attention(sizes["left"], h, under(w, "left."), eps, gated=True)
        r = sizes["right"]
        right = delta_rule_channel_decay(h, under(w, "right."), heads=r["heads"], groups=r["kv_heads"], d=r["dim"], e=r["vdim"], eps=eps)
        return sizes["left_scale"] * left + sizes["right_scale"] * right
    raise ValueError(kind)


def _attention(sizes: dict, h, w, eps, gated):
    rot = mask = None
    if sizes.get("rot") is not None:
        rot = (sizes["rot"]["base"], sizes["rot"]["dims"], (sizes["rot"].get("scaling") or {}).get("factor", 1.0))
    window, kept = None, 0
    if sizes.get("mask") is not None:
        window, kept = sizes["mask"]["size"], sizes["mask"].get("keep_first", 0)
    return softmax_attention(h, w, heads=sizes["heads"], groups=sizes["kv_heads"], d=sizes["dim"], e=sizes["vdim"], eps=eps,
                             scale=sizes["scale"], rot=rot, window=window, kept=kept, gated=gated)


def layer_order(config: dict) -> list:
    count, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return list(range(count))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], count))


def forward(config: dict, tensors: dict, tokens, streams: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence; streams (a list) receives the stream after every layer run."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = tensors["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for index in layer_order(config):
        layer, w = config["layers"][index], under(tensors, f"l{index}.")
        h = unit_rms(x, eps) * w["norm1"]
        y = mixer_output(layer["type"], layer["mixer"], h, under(w, "mix."), eps)
        if layer.get("mlp") is not None:
            y = y + gelu_exact(h @ w["mlp.up"].T) @ w["mlp.down"].T
        x = x + m * y
        if streams is not None:
            streams.append(x.clone())
    return (unit_rms(x, eps) * tensors["final.norm"]) @ tensors["embed"].T


def load_folder(folder, dtype=torch.float64) -> tuple:
    """(config dict, tensors by name) of a model folder, floating tensors widened to `dtype`."""
    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {name: t.to(dtype) if t.is_floating_point() else t for name, t in load_file(str(folder / "model.safetensors")).items()}
    return config, tensors
