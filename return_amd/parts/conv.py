"""A causal convolution over time in front of a sublayer: what the sublayer reads, x, becomes
x + conv(x) with conv(x)_t = sum_j w[:, j] * x_(t - taps + 1 + j) on each channel, zeros before the
sequence's start. The last taps-1 inputs belong to a request's state; the block that owns the part
keeps them (state_shape) and hands them in.
"""
from __future__ import annotations

from .registry import register_part


def filter_init(shape, generator):
    """Taps of a short filter for the random-weights mode: N(0, 0.3) on every tap."""
    import torch
    return 0.3 * torch.randn(*shape, generator=generator, dtype=torch.float32, device=generator.device)


class ResidualCausalConv:
    @staticmethod
    def tensor_shapes(params):
        return {"weight": (params["size"], params["taps"])}

    @staticmethod
    def random_init(params, role):
        return filter_init

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.size = int(params["size"])
        self.taps = int(params["taps"])
        self.weight = rt.vector32(tensors["weight"])

    def state_shape(self):
        return (self.taps - 1, self.size)

    def forward(self, x, step, tail):
        out = self.rt.empty(x.shape[0], self.size)
        self.rt.ops.causal_conv(x, self.weight, tail, step, out, add_input=True)
        return out


register_part("input_conv", "residual_causal_conv", ResidualCausalConv)
