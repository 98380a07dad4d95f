"""A per-layer token input: the layer's slice of a second embedding table (one row a token, `dim`
columns a layer), gated by the stream, projected to the stream's width, RMS-normed and added:
e = table[token, offset : offset + dim]; g = gelu_tanh(Wg x) * e; y = Wp g;
x += y / sqrt(mean(y^2) + eps) * w.  The table is one tensor that all layers read."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Part, RmsScaling, register_part
from .linear import Linear


class _PlainRms:
    """The norm's weights and eps in the form `ResidualStream.add_normed` takes."""

    def __init__(self, weight, eps):
        self._s = RmsScaling(weight, eps)

    def as_scaling(self):
        return self._s


class TokenSideInput(Part):
    category = "token_input"
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.dim = int(a["dim"])
        self.offset = int(a["offset"])               # first column of this layer's slice
        self.table_name = str(a["table"])
        self.table_shape = (int(a["vocab_size"]), int(a["table_width"]))
        self.eps = float(a["eps"])
        self.names = {"gate": "gate", "proj": "proj", "norm": "norm", **(a.get("names") or {})}
        if self.dim <= 0 or self.offset < 0 or self.offset + self.dim > self.table_shape[1]:
            raise ValueError("token input: the layer's slice lies outside the table")
        self.gate = self.proj = self.norm = self.table = None

    def expected_params(self):
        p, n = self.prefix, self.names
        return {self.table_name: ParamSpec(self.table_shape),
                p + n["gate"]: ParamSpec((self.dim, self.hidden)),
                p + n["proj"]: ParamSpec((self.hidden, self.dim)),
                p + n["norm"]: ParamSpec((self.hidden,), init="one_plus_normal")}

    def load_params(self, get):
        p, n = self.prefix, self.names
        self.table = self.rt.shared_matrix(self.table_name, lambda: get(self.table_name))
        self.gate = Linear(self.rt, get(p + n["gate"]))
        self.proj = Linear(self.rt, get(p + n["proj"]))
        self.norm = _PlainRms(self.rt.vector(get(p + n["norm"])), self.eps)

    def forward(self, stream, ctx, next_norm=None):
        x = stream.tensor()
        t = x.shape[0]
        if self.rt.dtype is torch.float32:
            xa = x
        else:
            xa = ctx.ws.buffer("token_input.x", x.shape, self.rt.dtype)
            ops.cast(x, xa)
        a = ctx.ws.buffer("token_input.gate", (t, self.dim), torch.float32)
        self.gate(xa, a, ws=ctx.ws)
        g = ctx.ws.buffer("token_input.g", (t, self.dim), self.rt.dtype)
        ops.gelu_gate_rows(a, ctx.ids, self.table, self.offset, g, ctx.id_src, ctx.feedback)
        y = ctx.ws.buffer("token_input.y", x.shape, torch.float32)
        self.proj(g, y, ws=ctx.ws)
        stream.add_normed(self.norm, y, next_norm)


register_part("token_input", "gated_table_slice", TokenSideInput)
