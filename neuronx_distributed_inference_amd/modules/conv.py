"""Short causal convolutions over time with carried state.

A depthwise FIR filter of a few taps per channel, applied along the
sequence: ``y_t = sum_j w[:, j] * x_{t-(taps-1)+j}`` plus an optional
per-channel bias (the last column of
``w`` multiplies the current token, inputs before the sequence start are
zero). The last ``taps-1`` inputs of every sequence are engine state: they
live in a :class:`RecurrentStateManager` tensor (slots, taps-1, C) so a
prompt can be fed in portions and decoding continues where prefill stopped.
Used both as a residual "input mixing" filter in front of a token mixer and
as the q/k/v pre-filter of linear-recurrence layers.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.ops import seqmix


class CausalShortConv(nn.Module):
    def __init__(self, channels: int, taps: int, activation: str = "none",
                 residual: bool = False, bias: bool = False):
        super().__init__()
        assert taps >= 1 and activation in ("none", "silu")
        self.channels = channels
        self.taps = taps
        self.activation = activation
        self.residual = residual
        # filter taps stay fp32 (a few KB; exact widening of the checkpoint)
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(channels, dtype=torch.float32),
                                 requires_grad=False) if bias else None

    def state_shape(self):
        return (max(self.taps - 1, 0), self.channels)

    def forward(self, x: torch.Tensor, tail: torch.Tensor, step: seqmix.StepLayout,
                out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """x (B,S,C). Reads the carried tail, then advances it by this
        step's inputs (two launches: every token of the step must have read
        the old tail before it is overwritten)."""
        y = seqmix.short_conv(x, self.weight, tail, step, self.activation,
                              self.residual, out_dtype, bias=self.bias)
        if self.taps > 1:
            seqmix.short_conv_commit(x, tail, step)
        return y
