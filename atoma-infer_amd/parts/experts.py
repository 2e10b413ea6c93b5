"""Feed-forward layers of many small experts, of which every token uses a few.

``RoutedExperts``: router logits ``z = W_r x`` in float32, scores ``s = sigmoid(z)``; the ``top`` experts with the
largest scores are chosen (the lower index wins a tie) and weighed by those scores as they are, without
renormalising.  The weight multiplies the expert's *input*: ``out = sum_e expert_e(s_e x)`` with
``expert(z) = W_down (silu(W_gate z) * (W_up z))``, no biases.

The chosen (token, choice) pairs are ordered by expert on the device (no count or index passes the host, so a step
may be recorded into a graph), and two grouped products walk them tile by tile; the second writes choice c of
every token into plane c, and the norm behind the layer adds the planes in order.  In bfloat16 the products run on
the matrix cores (float32 sums): the scaled inputs are gathered in the experts' order first, and the first product
applies silu(gate) * up in its epilogue (an expert's gate and up rows are interleaved in blocks of 16 at load time
for that).  The 32-bit path, and sizes that the matrix-core kernel does not take (a width that is no multiple of 64,
an expert width that is no multiple of 16), run true float32 multiply-adds.

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
        self.mfma = False       # set at load time: the products run on the matrix cores

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
        gates, ups = [get(f"e{e}.gate") for e in range(self.experts)], [get(f"e{e}.up") for e in range(self.experts)]
        self.w_down = torch.stack([get(f"e{e}.down") for e in range(self.experts)]).to(device).contiguous()
        self.mfma = (act_dtype is torch.bfloat16 and self.w_down.dtype is torch.bfloat16
                     and all(t.dtype is torch.bfloat16 for t in gates + ups) and self.inter % 16 == 0
                     and ops.expert_gemm_mfma_ok(2 * self.inter, self.width)
                     and ops.expert_gemm_mfma_ok(self.width, self.inter))
        if self.mfma:
            # [experts, 2 ff, width]: blocks of 16 gate rows, each followed by the 16 up rows of the same outputs
            gu = [torch.stack([g.view(-1, 16, self.width), u.view(-1, 16, self.width)], dim=1).reshape(-1, self.width)
                  for g, u in zip(gates, ups)]
        else:
            gu = [torch.cat([g, u], dim=0) for g, u in zip(gates, ups)]     # gate rows, then up rows
        self.w_gate_up = torch.stack(gu).to(device).contiguous()

    def device_bytes(self) -> int:
        """The router and the chosen share of the experts (what a step of one token reads)."""
        per_expert = (self.w_gate_up.numel() + self.w_down.numel()) // self.experts * self.w_down.element_size()
        return self.w_router.numel() * self.w_router.element_size() + self.top * per_expert

    def forward(self, x, ctx):
        t = x.shape[0]
        ids, scores = ops.route_topk(linear(x, self.w_router, torch.float32), self.top)
        slots = t * self.top
        if self.mfma and x.dtype is torch.bfloat16:
            # tiles of 128 places where an expert has about a hundred or more (prompts): a weight fragment then
            # serves twice as many rows
            tile_m = 128 if slots >= 96 * self.experts else 64
            perm, offsets, tiles = ops.route_group(ids.view(-1), self.experts, tile_m)
            xs = ops.gather_scale(x, scores.view(-1), perm, self.top)
            h = torch.empty((slots, self.inter), dtype=torch.bfloat16, device=x.device)
            ops.expert_gemm_mfma(xs, self.w_gate_up, h, perm, offsets, tiles, self.top, swiglu=True, tile_m=tile_m)
            out = torch.empty((self.top, t, self.width), dtype=torch.float32, device=x.device)
            ops.expert_gemm_mfma(h, self.w_down, out, perm, offsets, tiles, self.top, planes=True, tile_m=tile_m)
            return out
        perm, offsets, tiles = ops.route_group(ids.view(-1), self.experts)
        gu = torch.empty((slots, 2 * self.inter), dtype=x.dtype, device=x.device)
        ops.expert_gemm(x, self.w_gate_up, gu, perm, offsets, tiles, self.top, gather=True, scale=scores.view(-1))
        h = ops.swiglu(gu)
        out = torch.empty((self.top, t, self.width), dtype=torch.float32, device=x.device)
        ops.expert_gemm(h, self.w_down, out, perm, offsets, tiles, self.top, gather=False, planes=True)
        return out


register_feed_forward("routed_experts", RoutedExperts)
