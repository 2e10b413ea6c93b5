"""The entry of a pass over layers that run several times in a row with the same weights.

Before the first layer of every pass the stream is mapped anew from itself and from the embedding's rows,

    x <- W_in [x; x0] + step[t],

with x0 the rows as the embedding left them and t the number of the pass.  The map is a block of its own in the run
order (it mixes nothing between tokens and keeps no cache), run once per pass; which pass it is in, the model tells
it (``takes_turn``).  The product may run in the activation dtype; its sums, the bias and the new stream are float32.

Tensors: ``in`` [width, 2 width] (the stream's columns first), ``step`` [times, width].
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Begun, Block, Mixer, WeightedSum, WeightSpec, register_block, register_mixer
from .linear import Normed, linear


class NoMixer(Mixer):
    """Mixes nothing and keeps nothing: the mixer of blocks that only map the stream."""

    def graph_safe(self) -> bool:
        return True

    def forward(self, x, ctx, cache):
        return None


class LoopEntry(Block):
    #: the model hands ``forward`` the rows of the embedding (``embedded=``) and the number of this call among the
    #: calls of this block (``turn=``)
    reads_embedding = True
    takes_turn = True

    def __init__(self, width: int, times: int, names=("in", "step")):
        self.width, self.times, self.names = int(width), int(times), tuple(names)
        self.mixer = NoMixer()
        self.w_in: Optional[torch.Tensor] = None
        self.steps: Optional[torch.Tensor] = None
        self.act_dtype = torch.float32

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        # (drawn so that a pass keeps the stream's size: two halves of about 1/sqrt(2 width) each)
        return {self.names[0]: WeightSpec((self.width, 2 * self.width), std=0.7 / self.width ** 0.5),
                self.names[1]: WeightSpec((self.times, self.width), std=0.05)}

    def load(self, get, device, act_dtype) -> None:
        self.w_in = get(self.names[0]).to(device).contiguous()
        self.steps = get(self.names[1]).to(device=device, dtype=torch.float32).contiguous()
        self.act_dtype = act_dtype

    def device_bytes(self) -> int:
        return self.w_in.numel() * self.w_in.element_size()

    def forward(self, resid, delta, ctx, cache, embedded=None, turn=0):
        if embedded is None or not 0 <= turn < self.times:
            raise RuntimeError("a loop entry needs the embedding's rows and a pass number below its number of passes")
        if isinstance(delta, (Begun, Normed)):
            pass                        # the block before has added its outputs to the stream already
        elif delta is not None:         # what the block before left pending joins the stream first
            terms = delta.terms if isinstance(delta, WeightedSum) else [(delta, 1.0)]
            ops.add_normed(resid, terms, None, 0.0)
        pair = ops.pack_pair(resid, embedded, self.act_dtype if self.w_in.dtype is torch.bfloat16 else torch.float32)
        y = linear(pair, self.w_in, torch.float32)
        ops.set_rows(resid, y, self.steps[turn])
        return None


register_mixer("none", NoMixer)
register_block("loop_entry", LoopEntry)
