"""Parts that change the residual stream between layers (category ``stream``): the run order names one with
``LayerCall.before`` and the model applies it right before that call.

``add_row``: one row of a learned table [rows, hidden] is added to every token's stream, h += table[row] (float32).  A
model whose layers run several times in a row adds the pass's own row before each pass.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightInfo, register_part


class AddRow(Part):
    category = "stream"
    graph_safe = True

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.row = int(spec.params["row"])
        self.rows = int(spec.params["rows"])
        if not 0 <= self.row < self.rows:
            raise ValueError(f"add_row: row {self.row} outside a table of {self.rows}")
        self.table = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        return {spec.weights["table"]: WeightInfo((int(spec.params["rows"]), hidden_size))}

    def load_weights(self, get):
        # (the stream is float32: so is what is added to it)
        self.table = self._to_device(get(self.spec.weights["table"]), torch.float32)

    def forward(self, h, ctx) -> None:
        ops.add_row(h, self.table, self.row)


register_part("stream", "add_row", AddRow)
