"""A plain, slow Morulix decoder on the CPU: the yardstick of the engine's tests for that design.

Whole sequences, token by token where the design is recurrent, no cache, no batching, one function per mechanism.
Nothing here is imported from the framework.  Weights are a ``dict`` from the checkpoint's tensor names to CPU
tensors of the working dtype (float64 by default); the configuration is the plain ``dict`` of config.json.

The design in this file's notation (x: a token's residual row, e: its embedding row, h: a layer's input):

* layer:      h = N(x) with N(v) = v / sqrt(mean(v^2) + eps) * (1 + w);  x += mixer(h) + ff(h)
* loop:       layers start .. stop - 1 run ``times`` times over; pass t begins with x = W_in [x; e] + step[t]
* attention:  q, k, v projections; the first ``rot.dims`` columns of every q and k head are rotated in pairs
              (i, i + dims/2) by p * f_i, f_i = base^(-2i/dims) rescaled band by band; position p sees the last
              ``mask.size`` keys, its own included; plain softmax
* latent:     c = Nplain(W_dkv h); per head k = W_uk c, v = W_uv c; position p sees every j <= p; the softmax
              denominator also holds exp(sink_head); head outputs times sigmoid(W_g h)_head; then W_o
* mamba2:     [z | x | B | C | dt] = W_in h; x, B, C through a causal depthwise convolution with bias and SiLU;
              dt = softplus(dt + dt_bias); per head S = exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x;
              y * silu(z), normed in ``norm_groups`` parts, times the weight, then W_o
* ff:         W_down (silu(W_gate h) * (W_up h))
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

W = Dict[str, torch.Tensor]


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * (1.0 + w)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def band_scaled_frequencies(base: float, dims: int, scaling: Optional[dict], dtype=torch.float64) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` (factor, low, high, original) the long wavelengths are
    slowed by ``factor``, the short ones kept, and those between blended."""
    i = torch.arange(dims // 2, dtype=dtype)
    f = torch.tensor(float(base), dtype=dtype) ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for j in range(f.numel()):
        wavelength = 2.0 * math.pi / float(f[j])
        if wavelength < orig / high:
            continue
        if wavelength > orig / low:
            out[j] = f[j] / factor
        else:
            s = (orig / wavelength - low) / (high - low)
            out[j] = (1.0 - s) * f[j] / factor + s * f[j]
    return out


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """x [T, heads, dim]: column i < dims/2 is paired with column i + dims/2 (dims = 2 len(freq)) and the pair is
    turned by positions * freq_i; the columns from dims on pass."""
    half = freq.numel()
    ang = positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    out[..., :half] = u * c - v * s
    out[..., half:2 * half] = v * c + u * s
    return out


def windowed_attention(h: torch.Tensor, w: W, pre: str, m: dict) -> torch.Tensor:
    """The 'attention' mixer on a whole sequence h [T, width] (positions 0 .. T-1)."""
    t = h.shape[0]
    nh, nkv, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(t, nh, dim)
    k = (h @ w[pre + "k"].T).view(t, nkv, dim)
    v = (h @ w[pre + "v"].T).view(t, nkv, vdim)
    rot = m.get("rot")
    if rot and rot["dims"]:
        f = band_scaled_frequencies(rot["base"], rot["dims"], rot.get("scaling"), h.dtype)
        pos = torch.arange(t)
        q, k = rotate_halves(q, pos, f), rotate_halves(k, pos, f)
    size = m["mask"]["size"] if m.get("mask") else None
    out = torch.zeros(t, nh, vdim, dtype=h.dtype)
    for head in range(nh):
        kv = head // (nh // nkv)
        for i in range(t):
            lo = max(0, i - size + 1) if size else 0
            sc = (k[lo:i + 1, kv] @ q[i, head]) * m["scale"]
            out[i, head] = torch.softmax(sc, dim=0) @ v[lo:i + 1, kv]
    return out.reshape(t, -1) @ w[pre + "o"].T


def latent_attention(h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    """The 'latent_attention' mixer on a whole sequence: keys and values of every head are made from one small
    normed vector per token."""
    t = h.shape[0]
    nh, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(t, nh, dim)
    c = rms(h @ w[pre + "dkv"].T, eps) * w[pre + "dkv.norm"]
    k = (c @ w[pre + "uk"].T).view(t, nh, dim)
    v = (c @ w[pre + "uv"].T).view(t, nh, vdim)
    gate = torch.sigmoid(h @ w[pre + "g"].T)                                  # [T, nh]
    out = torch.zeros(t, nh, vdim, dtype=h.dtype)
    for head in range(nh):
        sink = w[pre + "sink"][head]
        for i in range(t):
            sc = (k[:i + 1, head] @ q[i, head]) * m["scale"]
            mx = torch.maximum(sc.max(), sink)
            e = torch.exp(sc - mx)
            out[i, head] = (e / (e.sum() + torch.exp(sink - mx))) @ v[:i + 1, head]
    out = out * gate[:, :, None]
    return out.reshape(t, -1) @ w[pre + "o"].T


def causal_conv_bias_silu(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K] (last column: the current token's), zeros before the start."""
    t, c = x.shape
    kk = taps.shape[1]
    padded = torch.cat([torch.zeros(kk - 1, c, dtype=x.dtype), x], dim=0)
    y = bias[None, :].expand(t, c).clone()
    for j in range(kk):
        y = y + padded[j:j + t] * taps[:, j][None, :]
    return silu(y)


def mamba2(h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    """The 'mamba2' mixer on a whole sequence, one token after the other."""
    t = h.shape[0]
    nh, vdim, n, g = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * vdim
    proj = h @ w[pre + "in"].T
    z = proj[:, :inner]
    xbc = causal_conv_bias_silu(proj[:, inner: 2 * inner + 2 * g * n], w[pre + "conv"], w[pre + "conv.b"])
    x = xbc[:, :inner].view(t, nh, vdim)
    b = xbc[:, inner: inner + g * n].view(t, g, n)
    c = xbc[:, inner + g * n:].view(t, g, n)
    dt = torch.nn.functional.softplus(proj[:, 2 * inner + 2 * g * n:] + w[pre + "dt_bias"])        # [T, nh]
    a = torch.exp(-torch.exp(w[pre + "A_log"])[None, :] * dt)
    y = torch.zeros(t, nh, vdim, dtype=h.dtype)
    for head in range(nh):
        grp = head // (nh // g)
        s = torch.zeros(n, vdim, dtype=h.dtype)
        for i in range(t):
            s = a[i, head] * s + dt[i, head] * torch.outer(b[i, grp], x[i, head])
            y[i, head] = s.T @ c[i, grp] + w[pre + "D"][head] * x[i, head]
    y = y.reshape(t, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.view(t, parts, inner // parts), eps).reshape(t, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


def dense_ff(h: torch.Tensor, w: W, pre: str) -> torch.Tensor:
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def mixer(kind: str, h: torch.Tensor, w: W, pre: str, m: dict, eps: float) -> torch.Tensor:
    if kind == "attention":
        return windowed_attention(h, w, pre, m)
    if kind == "latent_attention":
        return latent_attention(h, w, pre, m, eps)
    if kind == "mamba2":
        return mamba2(h, w, pre, m, eps)
    raise ValueError(f"unknown mixer {kind}")


def run_order(cfg: dict) -> List[tuple]:
    """(layer, pass number or None) in the order the layers run; a pass number marks the first layer of a pass."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    lo, hi, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(lo)]
    for t in range(times):
        order += [(i, t if i == lo else None) for i in range(lo, hi)]
    return order + [(i, None) for i in range(hi, n)]


def forward(tokens: List[int], w: W, cfg: dict, residuals: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``residuals`` collects the residual rows after every layer run."""
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    x = x0
    for i, turn in run_order(cfg):
        if turn is not None:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][turn]
        layer = cfg["layers"][i]
        p = f"l{i}."
        h = norm_around_zero(x, w[p + "norm1"], eps)
        d = mixer(layer["type"], h, w, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {layer['mlp']['kind']}")
            d = d + dense_ff(h, w, p + "mlp.")
        x = x + d
        if residuals is not None:
            residuals.append(x.clone())
    return norm_around_zero(x, w["final.norm"], eps) @ w["head"].T


def greedy(prompt: List[int], n: int, w: W, cfg: dict) -> List[int]:
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(forward(seq, w, cfg)[-1].argmax()))
    return seq[len(prompt):]
