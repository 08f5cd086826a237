"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases
(/root/reference/engine/src/model.rs:1203-1231,1301-1313;
``silu(x) = x / (1 + exp(-x))``, /root/reference/kernels/src/ggml/vec_llama.rs:808-810).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, WeightInfo, register_part


class SwiGLU(FeedForward):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph
    split_norm = True      # takes rows whose norm its first product finishes; prepares the next norm in its last

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.w13 = None
        self.w2 = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {
            w["gate"]: WeightInfo((i, hidden_size)),
            w["up"]: WeightInfo((i, hidden_size)),
            w["down"]: WeightInfo((hidden_size, i)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        gate, up = self._to_device(get(w["gate"])), self._to_device(get(w["up"]))
        # One matrix, one product instead of two.  In bfloat16 the rows alternate eight of gate and
        # eight of up, so that the product's epilogue applies silu(g) * u to its float32 sums.
        self.fused = self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        if self.fused:
            self.w13 = ops.tile_weight(ops.interleave_gate_up(gate, up))
        else:
            self.w13 = ops.tile_weight(torch.cat([gate, up], dim=0).contiguous())
        self.w2 = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual, next_norm=None):
        if self.fused:
            # (a few rows go to the next product k-blocked: it reads them straight from global memory)
            a = ops.linear_swiglu(x, self.w13, blocked_out=True)
        else:
            gu = ops.linear(x, self.w13, torch.float32)
            a = ops.swiglu(gu, self.dtype)
        if next_norm is None:
            ops.linear(a, self.w2, torch.float32, residual=residual)
            return None
        return ops.linear(a, self.w2, torch.float32, residual=residual, next_norm=next_norm)[1]


class GatedFFN(FeedForward):
    """``down(act(gate(x), up(x)))`` with ``act(g, u) = g' * sigmoid(slope * g') * (u' + up_offset)``, where
    g' = min(g, limit) and u' = clamp(u, -limit, limit) when ``limit`` is given.  slope 1, no limit and offset 0 is
    SwiGLU; the constants are parameters of the part.  The activation reads the float32 sums of the gate/up
    product, whatever the compute dtype."""
    graph_safe = True
    returns_output = True      # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.intermediate_size = int(p["intermediate_size"])
        self.slope = float(p.get("sigmoid_slope", 1.0))
        self.limit = float(p["limit"]) if p.get("limit") is not None else 0.0
        self.up_offset = float(p.get("up_offset", 0.0))
        if self.limit < 0:
            raise ValueError("gated feed-forward: limit must be positive when given")
        self.w13 = None
        self.w2 = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {
            w["gate"]: WeightInfo((i, hidden_size)),
            w["up"]: WeightInfo((i, hidden_size)),
            w["down"]: WeightInfo((hidden_size, i)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        gate, up = self._to_device(get(w["gate"])), self._to_device(get(w["up"]))
        # One product.  In bfloat16 the rows alternate eight of gate and eight of up, and the product's epilogue
        # applies the activation to its float32 sums; else gate columns, then up columns, and a kernel of its own.
        self.fused = self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        if self.fused:
            self.w13 = ops.tile_weight(ops.interleave_gate_up(gate, up))
        else:
            self.w13 = ops.tile_weight(torch.cat([gate, up], dim=0).contiguous())
        self.w2 = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual=None):
        if self.fused and x.shape[0] >= ops.gated_epilogue_rows:
            a = ops.linear_swiglu(x, self.w13, slope=self.slope, limit=self.limit, up_offset=self.up_offset)
        else:
            # (a few rows, or sizes the fused product does not take: the product's float32 sums, then the activation)
            gu = ops.linear(x, self.w13, torch.float32)
            a = ops.gated_act(gu, self.dtype, self.slope, self.limit, self.up_offset, interleaved=self.fused)
        return ops.linear(a, self.w2, torch.float32, residual=residual)


class DenseMLP(FeedForward):
    """``down(act(up(x)))`` without a gate; ``activation`` names the function (``gelu_tanh``, ``silu``), which reads
    the float32 sums of the up product."""
    graph_safe = True
    returns_output = True      # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "gelu_tanh"))
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"mlp: activation {self.activation!r} unknown (known: {sorted(ops.ACTIVATIONS)})")
        self.w_up = self.w_down = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {w["up"]: WeightInfo((i, hidden_size)), w["down"]: WeightInfo((hidden_size, i))}

    def load_weights(self, get):
        w = self.spec.weights
        self.w_up = ops.tile_weight(self._to_device(get(w["up"])))
        self.w_down = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual=None):
        u = ops.linear(x, self.w_up, torch.float32)
        a = ops.activation(u, self.activation, self.dtype)
        return ops.linear(a, self.w_down, torch.float32, residual=residual)


class RoutedExperts(FeedForward):
    """A mixture of ``experts`` gated feed-forwards (``down(silu(gate(x)) * up(x))``, no biases) of which every token
    uses ``top``.  Router: logits = W_router x with float32 sums (in bfloat16 the operands are the bfloat16 rows and
    the checkpoint's bfloat16 weights, whose products are exact in float32); scores s = softmax over all experts;
    the choice adds ``correction`` to s and, with ``groups`` (``count`` equal groups of neighbouring experts,
    ``keep``), only looks at the experts of the ``keep`` groups whose best choice score is largest; the weights are
    the chosen experts' s, not renormalised.  The output is the weighted sum of the chosen experts' outputs.

    Two ways through the experts.  A step of single tokens (decoding; it may be captured): ONE gate/up product
    over the stacked weights of all experts, then every expert's activations times the row's weight for it (zero
    where the expert was not chosen; ``ops.moe_spread``), then the experts' down products one after the other into
    one sum, ascending; nothing of the batch is read on the host, and at a few rows with several experts each
    nearly every expert's weights are read anyway.  A step with portions of prompts: the
    chosen (token, expert) pairs are brought into the order of the experts, the host reads how many rows each expert
    has (the one wait of the layer), every expert with rows is one pair of products over its rows, and a token's
    sum adds its experts' rows in the order of its choice.  Either way a row's result does not depend on what else
    is in the batch; the two ways differ in rounding only.  Tensor roles: ``router``,
    ``correction``, and ``gate`` / ``up`` / ``down`` as name patterns with ``{}`` for the expert's number.

    Parameters of the router beyond that: ``score`` (``"softmax"`` or ``"sigmoid"``: s = sigmoid(logit), each expert by
    itself); a spec without a ``correction`` tensor has none; ``group_best`` (default 1): a group is ranked by the sum
    of that many of its largest choice scores; ``normalize``: the weights are the chosen s over their sum (plus
    ``sum_eps``); ``scale`` multiplies the weights; a ``router_bias`` tensor [experts] is added to the logits.  (A softmax
    over the chosen logits alone is ``normalize`` with ``sum_eps`` 0.)

    ``expert`` (default ``"gated"``): ``"plain"`` experts are ``down(act(up(x)))`` without a gate, ``activation`` naming the
    function (``ops.ACTIVATIONS``; it reads the float32 sums of the up product).
    ``shared`` (``{"intermediate_size", "activation"}``, tensor roles ``shared_up``, ``shared_down``, ``shared_gate`` [1,
    hidden]): one more plain expert that every token uses, its output times sigmoid(w_gate . x), one number a token, added
    to the routed sum.  The gate row rides along in the shared up product, and the gate multiplies the activations in
    front of the down product (which is linear), not its result."""
    graph_safe = True
    returns_output = True

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.experts = int(p["experts"])
        self.top = int(p["top"])
        self.intermediate_size = int(p["intermediate_size"])
        g = p.get("groups")
        self.groups = int(g["count"]) if g else 1
        self.keep = int(g["keep"]) if g else 1
        if not 0 < self.top <= self.experts:
            raise ValueError("moe: top must lie between 1 and the number of experts")
        if self.groups > 1 and (self.experts % self.groups != 0 or not 0 < self.keep <= self.groups
                                or self.keep * (self.experts // self.groups) < self.top):
            raise ValueError("moe: groups must divide the experts and the kept groups must hold at least top experts")
        self.score = str(p.get("score", "softmax"))
        if self.score not in ops.ROUTE_SCORES:
            raise ValueError(f"moe: score {self.score!r} unknown (known: {sorted(ops.ROUTE_SCORES)})")
        self.group_best = int(p.get("group_best", 1))
        self.normalize = bool(p.get("normalize", False))
        self.sum_eps = float(p.get("sum_eps", 0.0))
        self.weight_scale = float(p.get("scale", 1.0))
        if self.group_best < 1:
            raise ValueError("moe: group_best must be at least 1")
        self.expert_kind = str(p.get("expert", "gated"))
        if self.expert_kind not in ("gated", "plain"):
            raise ValueError(f"moe: expert kind {self.expert_kind!r} unknown (known: gated, plain)")
        self.activation = str(p.get("activation", "silu"))
        if self.expert_kind == "plain" and self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"moe: activation {self.activation!r} unknown (known: {sorted(ops.ACTIVATIONS)})")
        self.shared = p.get("shared")
        if self.shared is not None and str(self.shared.get("activation", "silu")) not in ops.ACTIVATIONS:
            raise ValueError(f"moe: shared activation {self.shared.get('activation')!r} unknown")
        self.has_router_bias = "router_bias" in spec.weights
        self.plain_router = (self.score, self.group_best, self.normalize, self.weight_scale) == ("softmax", 1, False, 1.0) \
            and not self.has_router_bias
        self.w_router = self.correction = self.router_bias = None
        self.w_shared_up = self.w_shared_down = None
        self.w13, self.w2 = [], []

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        i, e = p["intermediate_size"], p["experts"]
        out = {w["router"]: WeightInfo((e, hidden_size))}
        if "correction" in w:
            out[w["correction"]] = WeightInfo((e,))
        if "router_bias" in w:
            out[w["router_bias"]] = WeightInfo((e,))
        gated = p.get("expert", "gated") == "gated"
        for n in range(e):
            if gated:
                out[w["gate"].format(n)] = WeightInfo((i, hidden_size))
            out[w["up"].format(n)] = WeightInfo((i, hidden_size))
            out[w["down"].format(n)] = WeightInfo((hidden_size, i))
        if p.get("shared") is not None:
            si = int(p["shared"]["intermediate_size"])
            out[w["shared_up"]] = WeightInfo((si, hidden_size))
            out[w["shared_down"]] = WeightInfo((hidden_size, si))
            out[w["shared_gate"]] = WeightInfo((1, hidden_size))
        return out

    def load_weights(self, get):
        from .base import pad_rows
        w = self.spec.weights
        self.w_router = ops.tile_weight(pad_rows(self._to_device(get(w["router"])), 16))
        self.correction = self._to_device(get(w["correction"]), torch.float32) if "correction" in w else None
        self.router_bias = self._to_device(get(w["router_bias"]), torch.float32) if self.has_router_bias else None
        if self.shared is not None:
            # the gate's row behind the up rows: one product gives the activations' sums and the gate's
            self.shared_size = int(self.shared["intermediate_size"])
            self.w_shared_up = ops.tile_weight(pad_rows(torch.cat([self._to_device(get(w["shared_up"])),
                                                                   self._to_device(get(w["shared_gate"])).reshape(1, -1)], dim=0), 16))
            self.w_shared_down = ops.tile_weight(self._to_device(get(w["shared_down"])))
        gated = self.expert_kind == "gated"
        self.fused = gated and self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        stack, self.w2 = [], []
        for n in range(self.experts):
            up = self._to_device(get(w["up"].format(n)))
            if gated:
                gate = self._to_device(get(w["gate"].format(n)))
                stack.append(ops.interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], dim=0))
            else:
                stack.append(up)
            self.w2.append(ops.tile_weight(self._to_device(get(w["down"].format(n)))))
        # the gate/up weights of all experts are one matrix (decoding runs them as one product); an expert's own
        # are rows of it, without a copy (tiled weights are cut at multiples of sixteen rows)
        rows = (2 if gated else 1) * self.intermediate_size
        stacked = torch.cat(stack, dim=0).contiguous()
        self.w13_all = ops.tile_weight(stacked) if rows % 16 == 0 else stacked
        self.w13 = [ops.weight_rows(self.w13_all, n * rows, (n + 1) * rows) for n in range(self.experts)]

    def _expert(self, n, rows):
        if self.expert_kind == "plain":
            return ops.activation(ops.linear(rows, self.w13[n], torch.float32), self.activation, self.dtype)
        if self.fused:
            return ops.linear_swiglu(rows, self.w13[n])
        return ops.swiglu(ops.linear(rows, self.w13[n], torch.float32), self.dtype)

    def _add_shared(self, x, y):
        """y += down_s(act(up_s x) * sigmoid(w_gate . x)): the expert every token uses."""
        u = ops.linear(x, self.w_shared_up, torch.float32)
        a = ops.activation(u, str(self.shared.get("activation", "silu")), self.dtype, 0, self.shared_size, self.shared_size)
        ops.linear(a, self.w_shared_down, torch.float32, residual=y)

    def forward(self, x, ctx, residual=None):
        if self.shared is None:
            return self._routed(x, ctx, residual)
        y = self._routed(x, ctx, residual)
        self._add_shared(x, residual if residual is not None else y)
        return y

    def _routed(self, x, ctx, residual=None):
        logits = ops.linear(x, self.w_router, torch.float32)
        if self.router_bias is not None:
            dense, ids, weights = ops.moe_route(logits, self.correction, self.experts, self.top, self.groups, self.keep, score=self.score,
                                                group_best=self.group_best, normalize=self.normalize, sum_eps=self.sum_eps,
                                                scale=self.weight_scale, bias=self.router_bias)
        elif self.plain_router and self.correction is not None:
            dense, ids, weights = ops.moe_route(logits, self.correction, self.experts, self.top, self.groups, self.keep)
        else:
            dense, ids, weights = ops.moe_route(logits, self.correction, self.experts, self.top, self.groups, self.keep, score=self.score,
                                                group_best=self.group_best, normalize=self.normalize, sum_eps=self.sum_eps,
                                                scale=self.weight_scale)
        if getattr(ctx, "max_q_len", 1) <= 1:
            if self.expert_kind == "plain":
                a = ops.activation(ops.linear(x, self.w13_all, torch.float32), self.activation, self.dtype)
            elif self.fused:
                a = ops.linear_swiglu(x, self.w13_all)
            else:
                gu = ops.linear(x, self.w13_all, torch.float32)
                a = ops.swiglu(gu.view(-1, 2 * self.intermediate_size), self.dtype).view(x.shape[0], -1)
            parts = ops.moe_spread(a, dense, self.experts)
            y = residual      # (None: the first expert's product starts a new tensor)
            for n in range(self.experts):
                y = ops.linear(parts[n], self.w2[n], torch.float32, residual=y) if y is not None else ops.linear(parts[n], self.w2[n], torch.float32)
            return y if residual is None else None
        counts, offsets, rank = ops.moe_plan(ids, self.experts)
        xg, row_of = ops.moe_gather(x, ids, rank, offsets)
        yg = torch.zeros((xg.shape[0], self.hidden_size), dtype=torch.float32, device=xg.device)
        at = 0
        for n, m in enumerate(counts.tolist()):      # (the host waits here for the router)
            if m:
                ops.linear(self._expert(n, xg[at: at + m]), self.w2[n], torch.float32, residual=yg[at: at + m])
                at += m
        y = ops.moe_scatter(yg, row_of, weights, residual)
        return y if residual is None else None


register_part("ffn", "mlp", DenseMLP)
register_part("ffn", "moe", RoutedExperts)
register_part("ffn", "swiglu", SwiGLU)
register_part("ffn", "gated", GatedFFN)
