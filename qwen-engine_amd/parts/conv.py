"""A short causal convolution over time on each channel, added to its input, in front of a mixer:
out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), zeros before the request's start.  It reads the 32-bit
stream and writes the activation type.  A request's last ``taps - 1`` inputs are its state, kept in a
state slot in 32-bit, so that a portion cut anywhere continues where the last one ended."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.plan import StateNeed
from ..kernels import ops
from .base import Runtime, TensorInfo
from .registry import register_part


class ShortConv:
    graph_safe = True        # one launch (two with the state's update) whose grid follows the rows alone

    def __init__(self, spec, hidden_size: int):
        self.taps = int(spec.taps)
        self.hidden = int(hidden_size)
        if self.taps < 1:
            raise ValueError(f"a convolution of {self.taps} taps")
        self.weight: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        return {"": TensorInfo((hidden, int(spec.taps)), "normal", "vector")}

    @staticmethod
    def state_need(spec, hidden: int) -> Optional[StateNeed]:
        return StateNeed(shape=(int(spec.taps) - 1, hidden), dtype="float32") if int(spec.taps) > 1 else None

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.weight = rt.place_vector(tensors[""])

    def forward(self, x: torch.Tensor, ctx, state: Optional[torch.Tensor]) -> torch.Tensor:
        """x: the 32-bit stream [T, H]; state [slots, taps - 1, H], read and brought up to date."""
        # (a step in which every request brings one token: convolution and the state's shift in one launch)
        single = all(s.q_len == 1 for s in ctx.seqs) and len(ctx.seqs) == x.shape[0]
        return ops.short_conv(x, self.weight, state, ctx.tok_seq, ctx.rt.dtype, single_rows=single)


register_part("short_conv", ShortConv)
