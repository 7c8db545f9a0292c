"""A short causal convolution over time on every channel, added to its input: ``h_t + sum_j w[:, j] * h_(t - taps + 1 + j)``.

The taps reach back over a request's earlier steps, so its last ``taps - 1`` inputs are a per-request state (zeros
before the sequence starts).  The input is the 32-bit residual stream; the result is rounded once to the compute
type for the projections that read it.
"""
from __future__ import annotations

from .base import VECTOR, ParamSpec, Part, StateSpec


class ShortConvolution(Part):
    def __init__(self, width: int, taps: int, tensor: str = "weight"):
        if taps < 1:
            raise ValueError(f"a convolution needs at least one tap, got {taps}")
        self.width, self.taps, self.tensor = width, int(taps), tensor
        self.weight = None      # float32 [width, taps]

    def param_specs(self):
        return {self.tensor: ParamSpec((self.width, self.taps), VECTOR, "normal")}

    def assign(self, name, tensor):
        assert name == self.tensor
        self.weight = tensor

    def state_spec(self):
        """What a request carries from step to step: its last ``taps - 1`` inputs (None for a single tap)."""
        return StateSpec((self.taps - 1, self.width), "float32") if self.taps > 1 else None

    def forward(self, x, ctx, state):
        """``x [T, W]`` float32 -> ``x + conv(x)`` in the compute type; ``state [slots, taps - 1, W]`` is read, then
        brought up to date with this step's inputs."""
        out = ctx.empty(x.shape)
        single = ctx.n_tokens == ctx.n_rows         # one token a row: a row's state is one workgroup's, which moves it on itself
        ctx.ops.short_conv(x, self.weight, state, ctx.state_slots, ctx.token_row, ctx.positions, ctx.row_start, out,
                           keep=single and state is not None)
        if state is not None and not single:
            ctx.ops.short_conv_keep(x, state, ctx.state_slots, ctx.row_start, ctx.row_len, ctx.row_ctx)
        return out
