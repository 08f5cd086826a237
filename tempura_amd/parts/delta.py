"""A gated delta-rule mixer: a linear recurrence over a matrix state per head that, at every token, decays the
state, corrects what the state predicts for the token's key towards the token's value, and reads the state out with
the token's query.

With H = ``num_heads``, G = ``num_kv_heads`` key heads (head h uses key head h // (H / G)), D = ``head_dim`` and
Dv = ``value_dim``: q and k [G, D] and v [H, Dv] pass a causal convolution per channel (``conv_taps`` taps, no
bias) and SiLU; q and k become unit vectors per head (x / sqrt(sum x^2 + ``unit_eps``)), q times ``q_scale``;
beta = sigmoid(W_b x) per head; the decay per head and key channel is exp(-exp(a_log[h]) * softplus(W_a2 (W_a1 x) +
dt_bias)).  Per head, with S [D, Dv] starting at zero:

    S <- decay * S      u = beta (v - S^T k)      S <- S + k u^T      o = S^T q

o is divided by its root mean square over Dv per head (``norm_eps``), times a weight [Dv] shared by the heads, times
sigmoid(W_g2 (W_g1 x)), then projected back.  Everything between the projections is float32 whatever the compute
dtype; the two low-rank second products run in float32 on the first products' float32 sums.

The columns of its input product are [q | k | v | beta | a1 | g1]; the ranks of the two low-rank projections are the
checkpoint's own.  Per request it keeps, in one float32 row, the convolution's last ``conv_taps - 1`` inputs and the
state (a head's [D, Dv] matrix column by column: [H, Dv, D]).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BranchMixer, WeightInfo, register_part


class GatedDeltaMixer(BranchMixer):
    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p["value_dim"])
        self.taps = int(p["conv_taps"])
        self.norm_eps = float(p["norm_eps"])
        self.unit_eps = float(p.get("unit_eps", 1e-6))
        self.q_scale = float(p.get("q_scale", self.head_dim ** -0.5))
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError("gated_delta: heads must be a multiple of key heads")
        if self.taps < 1:
            raise ValueError("gated_delta: conv_taps must be at least 1")
        self.qk_dim = self.num_kv_heads * self.head_dim
        self.inner = self.num_heads * self.value_dim
        self.channels = 2 * self.qk_dim + self.inner
        self.decay_dim = self.num_heads * self.head_dim
        self.conv_floats = (self.taps - 1) * self.channels

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        H, G, D, Dv, taps = p["num_heads"], p["num_kv_heads"], p["head_dim"], p["value_dim"], int(p["conv_taps"])
        # (the ranks are the checkpoint's; a configuration names them only for random weights)
        ra, rg = p.get("decay_rank"), p.get("gate_rank")
        return {
            w["q"]: WeightInfo((G * D, hidden_size)), w["k"]: WeightInfo((G * D, hidden_size)), w["v"]: WeightInfo((H * Dv, hidden_size)),
            w["q_conv"]: WeightInfo((G * D, taps)), w["k_conv"]: WeightInfo((G * D, taps)),
            w["v_conv"]: WeightInfo((H * Dv, taps)),
            w["beta"]: WeightInfo((H, hidden_size)),
            w["a_log"]: WeightInfo((H,)), w["dt_bias"]: WeightInfo((H * D,)),
            w["a1"]: WeightInfo((ra, hidden_size)), w["a2"]: WeightInfo((H * D, ra)),
            w["g1"]: WeightInfo((rg, hidden_size)), w["g2"]: WeightInfo((H * Dv, rg)),
            w["norm"]: WeightInfo((Dv,), "ones"),
            w["o"]: WeightInfo((hidden_size, H * Dv)),
        }

    def state_floats(self) -> int:
        return self.conv_floats + self.num_heads * self.head_dim * self.value_dim

    def load_branch(self, get):
        w = self.spec.weights
        f32 = lambda name: self._to_device(get(w[name]), torch.float32)
        a1, a2, g1, g2 = get(w["a1"]), f32("a2"), get(w["g1"]), f32("g2")
        if a2.shape[1] != a1.shape[0] or g2.shape[1] != g1.shape[0]:
            raise ValueError("gated_delta: the two halves of a low-rank projection disagree on its rank")
        self.a2_t, self.g2_t = a2.t().contiguous(), g2.t().contiguous()      # [rank, columns]: lanes read neighbours
        conv = torch.cat([get(w["q_conv"]), get(w["k_conv"]), get(w["v_conv"])], dim=0)
        self.conv_w = self._to_device(conv, torch.float32).t().contiguous()  # tap-major for the kernel
        self.a_log, self.dt_bias, self.norm_w = f32("a_log"), f32("dt_bias"), f32("norm")
        rows = [get(w["q"]), get(w["k"]), get(w["v"]), get(w["beta"]), a1, g1]
        self.beta_col = self.channels
        self.a1_col = self.beta_col + self.num_heads
        self.g1_col = self.a1_col + a1.shape[0]
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(get(w["o"]))

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        qkv = ops.causal_conv(proj, col0, self.channels, self.conv_w, None, cache.state, ctx.cu_seqlens, ctx.token_req,
                              ctx.state_slots, ctx.num_requests, state_off=self.state_off, act=True)
        decay = ops.lowrank_up(proj, col0 + self.a1_col, self.a2_t, "decay", self.a_log, self.dt_bias, self.head_dim)
        gate = ops.lowrank_up(proj, col0 + self.g1_col, self.g2_t, "sigmoid")
        o = ops.delta_scan(qkv, decay, proj, col0 + self.beta_col, cache.state, self.state_off + self.conv_floats, ctx.cu_seqlens,
                           ctx.state_slots, ctx.num_requests, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                           self.q_scale, self.unit_eps)
        ops.head_norm_gate(o, self.norm_w, gate, self.norm_eps, scale, self.num_heads, out, out_col0)


register_part("mixer", "gated_delta", GatedDeltaMixer)


class GeneralDeltaMixer(BranchMixer):
    """A generalized delta-rule mixer.  With H = ``num_heads`` heads of D = ``head_dim``: r, k, v = W_r x, W_k x, W_v x
    [H, D]; a decay per head and key channel w = exp(-``decay_rate`` * sigmoid(W_w2 tanh(W_w1 x) + w0)); a removal rate
    per head and key channel a = sigmoid(W_a x + a_bias).  With the unit key u = k / sqrt(sum k^2 + ``unit_eps``), per
    head and with S [D, D] starting at zero:

        S <- diag(w) S - (a u) (u^T S) + k v^T        (both terms read the old S)        o = S^T r

    o is divided by its root mean square per head (``norm_eps``), the concatenated heads times a weight [H D], times
    sigmoid(W_g x), then projected back.  Everything between the projections is float32 whatever the compute dtype.

    The columns of its input product are [r | k | v | a | gate | w1]; the rank of the decay's low-rank projection is the
    checkpoint's own.  Per request it keeps the state in one float32 row (a head's matrix column by column: [H, D, D])."""

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.norm_eps = float(p["norm_eps"])
        self.unit_eps = float(p.get("unit_eps", 1e-6))
        self.decay_rate = float(p["decay_rate"])
        self.inner = self.num_heads * self.head_dim

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        n = int(p["num_heads"]) * int(p["head_dim"])
        rank = p.get("decay_rank")
        out = {w[name]: WeightInfo((n, hidden_size)) for name in ("r", "k", "v", "gate", "a")}
        out.update({w["a_bias"]: WeightInfo((n,)), w["w1"]: WeightInfo((rank, hidden_size)), w["w2"]: WeightInfo((n, rank)),
                    w["w0"]: WeightInfo((n,)), w["norm"]: WeightInfo((n,), "ones"), w["o"]: WeightInfo((hidden_size, n))})
        return out

    def state_floats(self) -> int:
        return self.num_heads * self.head_dim * self.head_dim

    def load_branch(self, get):
        w = self.spec.weights
        f32 = lambda name: self._to_device(get(w[name]), torch.float32)
        w1, w2 = get(w["w1"]), f32("w2")
        if w2.shape[1] != w1.shape[0]:
            raise ValueError("general_delta: the two halves of the decay's projection disagree on its rank")
        self.w2_t = w2.t().contiguous()      # [rank, columns]: lanes read neighbours
        self.a_bias, self.w0, self.norm_w = f32("a_bias"), f32("w0"), f32("norm")
        rows = [get(w["r"]), get(w["k"]), get(w["v"]), get(w["a"]), get(w["gate"]), w1]
        self.gate_col = 4 * self.inner
        self.w1_col = 5 * self.inner
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(get(w["o"]))

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        decay = ops.lowrank_up(proj, col0 + self.w1_col, self.w2_t, "rate_sigmoid", bias=self.w0, rate=self.decay_rate, in_act="tanh")
        o = ops.general_delta_scan(proj, col0, decay, self.a_bias, cache.state, self.state_off, ctx.cu_seqlens, ctx.state_slots,
                                   ctx.num_requests, self.num_heads, self.head_dim, self.unit_eps)
        ops.head_norm_gate(o, self.norm_w, None, self.norm_eps, scale, self.num_heads, out, out_col0, gate_rows=proj,
                           gate_col0=col0 + self.gate_col)


register_part("mixer", "general_delta", GeneralDeltaMixer)
