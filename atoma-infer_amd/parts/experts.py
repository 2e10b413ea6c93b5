"""Feed-forward layers of many small experts, of which every token uses a few.

``RoutedExperts``: router logits ``z = W_r x`` in float32, scores ``s = sigmoid(z)``; the ``top`` experts with the
largest scores are chosen (the lower index wins a tie) and weighed by those scores as they are, without
renormalising.  The weight multiplies the expert's *input*: ``out = sum_e expert_e(s_e x)`` with
``expert(z) = W_down (silu(W_gate z) * (W_up z))``, no biases.

The chosen (token, choice) pairs are ordered by expert on the device (no count or index passes the host, so a step
may be recorded into a graph), and two grouped products walk them tile by tile; the second writes choice c of
every token into plane c, and the norm behind the layer adds the planes in order.

Tensors: ``router`` [experts, width]; ``e<i>.gate``, ``e<i>.up`` [ff, width], ``e<i>.down`` [width, ff].
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightSpec, register_feed_forward
from .linear import linear


class RoutedExperts(FeedForward):
    def __init__(self, width: int, intermediate: int, experts: int, top: int):
        if not 0 < top <= experts or experts > 1024:
            raise ValueError(f"{top} of {experts} experts: top must be at least 1 and at most the number of experts "
                             f"(up to 1,024)")
        self.width, self.inter, self.experts, self.top = int(width), int(intermediate), int(experts), int(top)
        self.w_router = self.w_gate_up = self.w_down = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {"router": WeightSpec((self.experts, self.width), std=0.5)}
        for e in range(self.experts):
            specs[f"e{e}.gate"] = WeightSpec((self.inter, self.width))
            specs[f"e{e}.up"] = WeightSpec((self.inter, self.width))
            specs[f"e{e}.down"] = WeightSpec((self.width, self.inter))
        return specs

    def load(self, get, device, act_dtype) -> None:
        self.w_router = get("router").to(device).contiguous()
        # [experts, 2 ff, width]: an expert's gate rows, then its up rows
        self.w_gate_up = torch.stack([torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], dim=0)
                                      for e in range(self.experts)]).to(device).contiguous()
        self.w_down = torch.stack([get(f"e{e}.down") for e in range(self.experts)]).to(device).contiguous()

    def device_bytes(self) -> int:
        """The router and the chosen share of the experts (what a step of one token reads)."""
        per_expert = (self.w_gate_up.numel() + self.w_down.numel()) // self.experts * self.w_down.element_size()
        return self.w_router.numel() * self.w_router.element_size() + self.top * per_expert

    def forward(self, x, ctx):
        t = x.shape[0]
        ids, scores = ops.route_topk(linear(x, self.w_router, torch.float32), self.top)
        perm, offsets, tiles = ops.route_group(ids.view(-1), self.experts)
        slots = t * self.top
        gu = torch.empty((slots, 2 * self.inter), dtype=x.dtype, device=x.device)
        ops.expert_gemm(x, self.w_gate_up, gu, perm, offsets, tiles, self.top, gather=True, scale=scores.view(-1))
        h = ops.swiglu(gu)
        out = torch.empty((self.top, t, self.width), dtype=torch.float32, device=x.device)
        ops.expert_gemm(h, self.w_down, out, perm, offsets, tiles, self.top, gather=False, planes=True)
        return out


register_feed_forward("routed_experts", RoutedExperts)
