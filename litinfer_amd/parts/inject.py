"""Additions to the residual stream BETWEEN layers, named by entries of the execution order.

`LoopEntry`: where a run of layers is passed several times with the same weights, the stream takes, right
before the first layer of pass t, the embedding output again (not before the first pass) and the t-th row
of a table [passes, width].  The embedding output is gathered again from the table rather than kept."""
from __future__ import annotations

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Part, register_part


class LoopEntry(Part):
    category = "injection"
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.times = int(spec.args["times"])
        self.hidden = int(spec.args["hidden_size"])
        self.param = self.prefix + str(spec.args.get("param", "step"))
        self.add_embedding = bool(spec.args.get("add_embedding", True))
        self.steps = None

    def expected_params(self):
        return {self.param: ParamSpec((self.times, self.hidden))}

    def load_params(self, get):
        self.steps = self.rt.vector(get(self.param))

    def forward(self, stream, ctx, index: int, embedding) -> None:
        if not 0 <= index < self.times:
            raise IndexError(f"loop entry: pass {index} of {self.times}")
        x = stream.tensor()
        table = embedding.table if (self.add_embedding and index > 0) else None
        ops.embedding_add(x, ctx.ids, table, self.steps[index], ctx.id_src, ctx.feedback)


register_part("injection", "loop_entry", LoopEntry)
