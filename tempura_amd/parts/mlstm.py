"""An mLSTM mixer: a linear recurrence over a matrix memory per head with exponential input gates, kept in range by a
running maximum of the log gates.

With H = ``num_heads`` heads of D = ``head_dim`` key channels and Dv = ``value_dim`` values: q = W_q x * ``q_scale``,
k = W_k x [H, D], v = W_v x [H, Dv]; per head a log input gate i = cap tanh((W_i x + b_i) / cap) and a log forget gate
f = logsigmoid(cap tanh((W_f x + b_f) / cap)) with cap = ``gate_cap``.  Per head, with S [D, Dv], n [D] and m all zero at
a request's start:

    m' = max(f + m, i)      S' = e^(f + m - m') S + e^(i - m') k v^T      n' = e^(f + m - m') n + e^(i - m') k
    o = S'^T q / (max(|n' . q|, e^(-m')) + ``denominator_eps``)

Each head's o is divided by its root mean square (``norm_eps``), the concatenated heads are multiplied by a weight
[H Dv] and by sigmoid(W_g x), then projected back.  Everything between the projections is float32 whatever the compute
dtype.

The columns of its input product are [q | k | v | gate | i | f].  Per request it keeps one float32 row: per head the
memory column by column with n as one more column ([H, Dv + 1, D]), then a copy of m for every column ([H, Dv + 1]).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BranchMixer, WeightInfo, register_part

#: what is added to the read-out's denominator: the kernels have it built in
DENOMINATOR_EPS = 1e-6


class MLSTMMixer(BranchMixer):
    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p["value_dim"])
        self.gate_cap = float(p["gate_cap"])
        self.norm_eps = float(p["norm_eps"])
        self.q_scale = float(p.get("q_scale", self.head_dim ** -0.5))
        if float(p.get("denominator_eps", DENOMINATOR_EPS)) != DENOMINATOR_EPS:
            raise ValueError(f"mlstm: the kernels add {DENOMINATOR_EPS} to the denominator, nothing else")
        if self.gate_cap <= 0:
            raise ValueError("mlstm: gate_cap must be positive")
        self.qk_dim = self.num_heads * self.head_dim
        self.inner = self.num_heads * self.value_dim

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        H, D, Dv = int(p["num_heads"]), int(p["head_dim"]), int(p["value_dim"])
        return {
            w["q"]: WeightInfo((H * D, hidden_size)), w["k"]: WeightInfo((H * D, hidden_size)), w["v"]: WeightInfo((H * Dv, hidden_size)),
            w["gate"]: WeightInfo((H * Dv, hidden_size)), w["o"]: WeightInfo((hidden_size, H * Dv)),
            w["norm"]: WeightInfo((H * Dv,), "ones"),
            w["i"]: WeightInfo((H, hidden_size)), w["i_bias"]: WeightInfo((H,)),
            w["f"]: WeightInfo((H, hidden_size)), w["f_bias"]: WeightInfo((H,)),
        }

    def state_floats(self) -> int:
        return self.num_heads * (self.value_dim + 1) * (self.head_dim + 1)

    def load_branch(self, get):
        w = self.spec.weights
        f32 = lambda name: self._to_device(get(w[name]), torch.float32)
        self.i_bias, self.f_bias, self.norm_w = f32("i_bias"), f32("f_bias"), f32("norm")
        rows = [get(w[name]) for name in ("q", "k", "v", "gate", "i", "f")]
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(get(w["o"]))

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        ops.mlstm_scan(proj, col0, self.i_bias, self.f_bias, self.gate_cap, self.q_scale, cache.state, self.state_off, ctx.cu_seqlens,
                       ctx.state_slots, ctx.num_requests, self.num_heads, self.head_dim, self.value_dim, self.norm_w, self.norm_eps,
                       scale, out, out_col0)


register_part("mixer", "mlstm", MLSTMMixer)
