"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * (w + weight_offset)``.

``groups`` (default 1): the row is split into that many equal consecutive parts and each is divided by its own root
mean square; the weight spans the whole row.

``weight_offset`` (default 0) serves checkpoints that store the weight around zero: with 1.0 the stored tensor is
the deviation from one.  The offset is added once, in float32, when the weight is loaded.
``scale`` (default 1) multiplies the result: a norm behind a sublayer whose output enters the residual stream
times a constant carries the constant here (the weight is multiplied once, when it is loaded).

The reference multiplies ``x * scale * w`` with eps inside the square root,
added to the mean (/root/reference/kernels/src/ggml/ops_llama.rs:201-216).
The sum of squares and the scale are computed in float32 in every dtype.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Norm, WeightInfo, register_part


class RMSNorm(Norm):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.eps = float(spec.params["eps"])
        self.weight_offset = float(spec.params.get("weight_offset", 0.0))
        self.scale = float(spec.params.get("scale", 1.0))
        self.groups = int(spec.params.get("groups", 1) or 1)
        if self.groups < 1 or hidden_size % self.groups != 0:
            raise ValueError(f"rmsnorm: groups ({self.groups}) must divide the row ({hidden_size})")
        self.weight = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        # (a weight stored around zero is drawn like any other tensor, one stored around one as ones)
        init = "normal" if float(spec.params.get("weight_offset", 0.0)) != 0.0 else "ones"
        return {spec.weights["weight"]: WeightInfo((hidden_size,), init)}

    def load_weights(self, get):
        # Norm weights are tiny and multiply in float32: keep them in float32.
        self.weight = self._to_device(get(self.spec.weights["weight"]), torch.float32)
        if self.weight_offset != 0.0:
            self.weight = (self.weight.double() + self.weight_offset).to(torch.float32)
        if self.scale != 1.0:
            self.weight = (self.weight.double() * self.scale).to(torch.float32)

    def forward(self, h, rows=None, out_dtype=None):
        """``out_dtype``: another type than the compute dtype (float32 rows for a part that goes on in float32)."""
        if self.groups > 1:
            return ops.rmsnorm(h, self.weight, self.eps, out_dtype or self.dtype, rows, groups=self.groups)
        return ops.rmsnorm(h, self.weight, self.eps, out_dtype or self.dtype, rows)

    def deferred(self, m):
        """(weight, eps) when the two products around this norm can carry it for ``m`` rows (the one
        before prepares, the one after applies the scale), else None."""
        if self.groups == 1 and ops.split_norm_ok(m, self.hidden_size, self.dtype):
            return self.weight, self.eps
        return None


register_part("norm", "rmsnorm", RMSNorm)
