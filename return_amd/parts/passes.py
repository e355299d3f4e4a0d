"""What a looped stack does to the residual stream when a pass begins.

"concat_linear": h <- W [h ; h0] + b[t], with h0 the embedding's output, W stored [H, 2H] (the
stream's columns first) and b [passes, H] one vector per pass t. What the part before left pending
goes into the stream first. The product takes the stream and h0 rounded to the compute dtype and
gives a 32-bit result, which is the new stream; the vector is added in 32-bit.
"""
from __future__ import annotations

import torch

from .registry import register_part
from .runtime import unscaled


class ConcatLinearPassInput:
    @staticmethod
    def tensor_shapes(params):
        H = params["hidden_size"]
        return {"weight": (H, 2 * H), "step": (params["passes"], H)}

    @staticmethod
    def random_init(params, role):
        if role == "step":
            return lambda shape, gen: 0.1 * torch.randn(*shape, generator=gen, dtype=torch.float32,
                                                        device=gen.device)
        H = params["hidden_size"]
        # near [I | 0] + noise, so that a looped stream keeps its size
        def draw(shape, gen):
            w = torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device) * (0.5 / (2 * H) ** 0.5)
            w[:, :H] += 0.7 * torch.eye(H, device=gen.device)
            return w
        return draw

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = int(params["hidden_size"])
        self.passes = int(params["passes"])
        self.weight = rt.product(rt.matrix(tensors["weight"]), out_dtype=torch.float32)
        self.step = rt.vector32(tensors["step"])

    def forward(self, h, pending, h0, number):
        if not 0 <= number < self.passes:
            raise ValueError(f"pass {number} of a stack with {self.passes} passes")
        ops = self.rt.ops
        delta, factor = unscaled(pending)
        rows = self.rt.empty(h.shape[0], 2 * self.hidden)
        ops.stream_pair_rows(h, delta, factor, h0, rows)
        h = ops.linear(rows, self.weight, out_dtype=torch.float32)
        ops.add_bias(h, self.step[number])
        return h, None


register_part("pass_input", "concat_linear", ConcatLinearPassInput)
