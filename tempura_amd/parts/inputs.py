"""What sublayers read of a layer's normed rows (category ``input``).

``residual_conv``: each sublayer reads n + conv(n), a causal convolution over time on every channel with a weight of
its own ([hidden, taps], no bias; conv(n)_t = sum_j w[:, j] n_(t - taps + 1 + j), zeros before a request's start).
The sublayers convolve the SAME rows, so a request carries the last ``taps - 1`` normed rows once, whatever the number
of sublayers: ``state_floats()`` float32 values of its state row, from ``state_off`` on.  Sums are float32; the results
come in the compute dtype, one tensor per sublayer (tensor role ``taps``: a list of names, one per sublayer; role
``unused``, optional: names of weights a checkpoint may hold for sublayers the layer does not have, which are ignored).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightInfo, register_part


class ResidualConv(Part):
    category = "input"
    graph_safe = True

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.taps = int(spec.params["taps"])
        self.names = list(spec.weights["taps"])
        if self.taps < 1 or not self.names:
            raise ValueError("residual_conv: at least one tap and one sublayer")
        self.state_off = 0
        self.weight = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        shape = (hidden_size, int(spec.params["taps"]))
        out = {name: WeightInfo(shape) for name in spec.weights["taps"]}
        out.update({name: WeightInfo(shape, "skip", optional=True) for name in spec.weights.get("unused", [])})
        return out

    def state_floats(self) -> int:
        return (self.taps - 1) * self.hidden_size

    def load_weights(self, get):
        # [sublayers, taps, hidden]: tap-major, so that neighbouring lanes read neighbouring channels
        self.weight = torch.stack([self._to_device(get(name), torch.float32).t() for name in self.names]).contiguous()

    def forward(self, n, ctx, cache):
        """float32 rows [tokens, hidden] -> a list of compute-dtype rows, one per sublayer."""
        return ops.residual_conv(n, self.weight, cache.state, self.state_off, ctx.cu_seqlens, ctx.token_req, ctx.state_slots,
                                 ctx.num_requests, self.dtype)


register_part("input", "residual_conv", ResidualConv)
