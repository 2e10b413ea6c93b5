"""A plain, slow Somesun decoder on the CPU: the yardstick of the engine's tests for that design.

Whole sequences, token by token where the design is recurrent, no cache, no batching, one function per mechanism.
Nothing here is imported from the framework.  Weights are a ``dict`` from the checkpoint's tensor names to CPU
tensors of the working dtype (float64 by default); the configuration is the plain ``dict`` of config.json.

The design in this file's notation (x: a token's residual row, h: a sublayer's input):

* layer:      x += N1b(mixer(N1(x)));  x += N2b(ff(N2(x)))  with N(v) = v / sqrt(mean(v^2) + eps) * w
* mixer:      a_l * attention(h) + a_r * delta(h), both reading the same h
* attention:  q = Wq h, k = Wk h, values are the raw k; q and k are normed over the whole projection, then the first
              ``rot.dims`` columns of every head are rotated in neighbouring pairs (2i, 2i + 1) by p * base^(-2i/dims);
              position p sees j <= p with j // size == p // size; the softmax denominator also holds exp(sink_head)
* delta:      q, k, v through a causal depthwise convolution and SiLU; q, k to unit length (q also / sqrt(dim));
              beta = sigmoid(Wb h); g = exp(-exp(A_log) * softplus(Wa2 Wa1 h + dt_bias)) per head and key channel;
              S = g * S; u = beta * (v - S^T k); S += k u^T; o = S^T q; o normed per head over vdim, times
              sigmoid(Wg2 Wg1 h); then Wo
* ff:         s = sigmoid(Wr h); the ``top`` largest s_e are kept; out = sum_e expert_e(s_e * h),
              expert(z) = Wd (silu(Wg z) * (Wu z))
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

W = Dict[str, torch.Tensor]


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, heads, dim]: columns (2i, 2i + 1), i < dims / 2, turned by positions * base^(-2i/dims)."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=x.dtype)
    freq = torch.tensor(float(base), dtype=x.dtype) ** (-2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]            # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def chunked_sink_attention(h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    """The left mixer on a whole sequence h [T, width] (positions 0 .. T-1)."""
    t = h.shape[0]
    nh, nkv, dim = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[pre + "q"].T
    k = h @ w[pre + "k"].T
    v = k.view(t, nkv, dim)                                        # the values: k as projected
    q = rms_norm(q, w[pre + "q.norm"], eps).view(t, nh, dim)
    k = rms_norm(k, w[pre + "k.norm"], eps).view(t, nkv, dim)
    pos = torch.arange(t)
    q = rotate_pairs(q, pos, m["rot"]["base"], m["rot"]["dims"])
    k = rotate_pairs(k, pos, m["rot"]["base"], m["rot"]["dims"])
    size = m["mask"]["size"]
    out = torch.zeros(t, nh, v.shape[-1], dtype=h.dtype)
    for head in range(nh):
        kv = head // (nh // nkv)
        for i in range(t):
            lo = (i // size) * size
            sc = (k[lo:i + 1, kv] @ q[i, head]) * m["scale"]
            sink = w[pre + "sink"][head]
            mx = torch.maximum(sc.max(), sink)
            e = torch.exp(sc - mx)
            den = e.sum() + torch.exp(sink - mx)
            out[i, head] = (e / den) @ v[lo:i + 1, kv]
    return out.reshape(t, -1) @ w[pre + "o"].T


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K] (last column: the current token); zeros before the start."""
    t, c = x.shape
    kk = taps.shape[1]
    padded = torch.cat([torch.zeros(kk - 1, c, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(kk):
        y = y + padded[j:j + t] * taps[:, j][None, :]
    return silu(y)


def gated_delta(h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    """The right mixer on a whole sequence, one token after the other."""
    t = h.shape[0]
    nh, nkv, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ w[pre + "q"].T, w[pre + "q.conv"]).view(t, nkv, dim)
    k = causal_conv_silu(h @ w[pre + "k"].T, w[pre + "k.conv"]).view(t, nkv, dim)
    v = causal_conv_silu(h @ w[pre + "v"].T, w[pre + "v.conv"]).view(t, nh, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)                                         # [T, nh]
    dt = torch.nn.functional.softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"])
    g = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * dt.view(t, nh, dim))  # [T, nh, dim]
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(t, nh, vdim)
    o = torch.zeros(t, nh, vdim, dtype=h.dtype)
    for head in range(nh):
        kv = head // (nh // nkv)
        s = torch.zeros(dim, vdim, dtype=h.dtype)
        for i in range(t):
            s = g[i, head][:, None] * s
            u = beta[i, head] * (v[i, head] - s.T @ k[i, kv])
            s = s + torch.outer(k[i, kv], u)
            o[i, head] = s.T @ q[i, kv]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[pre + "norm"] * gate
    return o.reshape(t, -1) @ w[pre + "o"].T


def parallel_mixer(h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    return m["left_scale"] * chunked_sink_attention(h, w, pre + "left.", m["left"], eps) + \
        m["right_scale"] * gated_delta(h, w, pre + "right.", m["right"], eps)


def routed_experts(h: torch.Tensor, w: W, pre: str, m: dict) -> torch.Tensor:
    scores = torch.sigmoid(h @ w[pre + "router"].T)                                   # [T, experts]
    top = m["router"]["top"]
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        best = torch.topk(scores[t], top).indices.tolist()
        for e in best:
            z = scores[t, e] * h[t]
            p = f"{pre}e{e}."
            out[t] = out[t] + w[p + "down"] @ (silu(w[p + "gate"] @ z) * (w[p + "up"] @ z))
    return out


def forward(tokens: List[int], w: W, cfg: dict, residuals: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``residuals`` collects the residual rows after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "parallel":
            raise ValueError(f"layer {i}: unknown type {layer['type']}")
        p = f"l{i}."
        a = parallel_mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        x = x + rms_norm(a, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            f = routed_experts(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"])
            x = x + rms_norm(f, w[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy(prompt: List[int], n: int, w: W, cfg: dict) -> List[int]:
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward(seq, w, cfg)[-1].argmax()))
    return seq[len(prompt):]
