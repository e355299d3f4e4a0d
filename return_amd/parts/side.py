"""Per-layer token input: every layer adds to the stream something of the token itself, read from a
second, narrow embedding table of which the layer owns `dim` columns starting at `offset`:

    e = table[token][offset : offset + dim]
    g = gelu_tanh(W_gate h) * e
    y = W_proj g
    h <- h + y / sqrt(mean(y^2) + eps) * w

with gelu_tanh(x) = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))). The addition of the part
before (pending) is made in the same kernel, in 32-bit.
"""
from __future__ import annotations

from .registry import register_part


class GatedTokenSide:
    @staticmethod
    def tensor_shapes(params):
        H, S = params["hidden_size"], params["dim"]
        return {"table": (params["vocab_size"], params["table_width"]), "gate": (S, H), "proj": (H, S),
                "norm": (H,)}

    @staticmethod
    def random_init(params, role):
        return {"table": "embedding", "norm": "norm"}.get(role, "matrix")

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = int(params["hidden_size"])
        self.dim = int(params["dim"])
        self.offset = int(params["offset"])
        self.eps = float(params["eps"])
        if self.offset + self.dim > int(params["table_width"]):
            raise ValueError(f"token input: columns {self.offset}..{self.offset + self.dim} lie beyond the table's "
                             f"{params['table_width']}")
        self.table = rt.matrix(tensors["table"])
        self.gate = rt.matrix(tensors["gate"])
        self.proj = rt.matrix(tensors["proj"])
        self.weight = rt.vector32(tensors["norm"])

    def forward(self, h, pending, step):
        self.rt.ops.token_side(h, pending, step.token_ids, self.table, self.offset, self.gate, self.proj,
                               self.weight, self.eps)


register_part("token_input", "gated_token_side", GatedTokenSide)
