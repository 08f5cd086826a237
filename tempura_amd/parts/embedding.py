"""Token embedding and output head.

``hidden[t] = embed[token[t]]`` with no scaling
(/root/reference/engine/src/model.rs:672-684); logits are
``norm(hidden)[rows] @ lm_head^T`` in float32, and when the checkpoint has no
output matrix the embedding matrix is used for it
(/root/reference/engine/src/weights.rs:156-166).

Two options beyond that: the embedding may add a sinusoidal position vector (``position: "sinusoid"`` with
``position_base`` b: element 2i of position p gets sin(p * b^(-2i / hidden)), element 2i + 1 the cosine), and the
head may multiply its logits by a constant (``scale``).

``bigram`` (``{"buckets", "mul_prev", "mul_cur"}``, tensor role ``bigram`` [buckets + 1, hidden]): a second row is
added to every token's, chosen by a hash of the token before it and the token itself,
(previous * mul_prev + token * mul_cur) mod buckets; a request's first token reads the last row.  The token before a
step's first one is per-request state: the embedding says so with ``state_spec()`` (one int32 per request), the model
asks for a state tensor on its behalf and hands it to ``forward``.

``scale`` multiplies the token's row (not the other rows).  ``position: "learned"`` (tensor role ``position``
[``max_positions``, hidden]) adds the row of the token's position; it combines with a bigram table.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, StateSpec, WeightInfo, register_part


class TokenEmbedding(Part):
    category = "embedding"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None
        kind = spec.params.get("position")
        if kind not in (None, "sinusoid", "learned"):
            raise ValueError(f"embedding: position {kind!r} unknown (known: sinusoid, learned)")
        self.scale = float(spec.params.get("scale", 1.0))
        self.learned = kind == "learned"
        self.pos_table = None
        if self.scale != 1.0 and kind == "sinusoid":
            raise ValueError("embedding: a scale and a sinusoidal position vector together are not supported")
        self.inv_freq = None
        if kind == "sinusoid":
            base = float(spec.params.get("position_base", 10000.0))
            i = torch.arange((hidden_size + 1) // 2, dtype=torch.float64)
            # float64 on the host; the kernel forms the angle in float64 too
            self.inv_freq = torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / hidden_size).to(device)
        self.bigram = spec.params.get("bigram")
        self.bigram_table = None
        if self.bigram is not None:
            if kind == "sinusoid":
                raise ValueError("embedding: a bigram table and a sinusoidal position vector together are not supported")
            for key in ("buckets", "mul_prev", "mul_cur"):
                if int(self.bigram[key]) < (1 if key == "buckets" else 0):
                    raise ValueError(f"embedding: bigram {key} must be {'positive' if key == 'buckets' else 'non-negative'}")

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        out = {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size))}
        if spec.params.get("bigram") is not None:
            out[spec.weights["bigram"]] = WeightInfo((int(spec.params["bigram"]["buckets"]) + 1, hidden_size))
        if spec.params.get("position") == "learned":
            rows = spec.params.get("max_positions")      # (None: the tensor's own)
            out[spec.weights["position"]] = WeightInfo((None if rows is None else int(rows), hidden_size))
        return out

    def load_weights(self, get):
        self.weight = self._to_device(get(self.spec.weights["weight"]))
        if self.bigram is not None:
            self.bigram_table = self._to_device(get(self.spec.weights["bigram"]))
        if self.learned:
            self.pos_table = self._to_device(get(self.spec.weights["position"]))

    def state_spec(self):
        """Per-request state of the embedding: the request's last token, for the bigram row of the next step's first."""
        return StateSpec((1,), torch.int32) if self.bigram is not None else None

    def forward(self, tokens, positions=None, streams: int = 1, ctx=None, state=None):
        """int32 [tokens] -> float32 [tokens, streams * hidden]: ``streams`` copies of the residual stream."""
        if self.bigram is not None or self.learned or self.scale != 1.0:
            if streams != 1:
                raise ValueError("embedding: a bigram table, a scale or learned positions with several copies of the stream are not supported")
            b = self.bigram or {"mul_prev": 0, "mul_cur": 0, "buckets": 0}
            if self.learned and getattr(ctx, "max_context_len", 0) > self.pos_table.shape[0]:
                raise ValueError(f"embedding: position {ctx.max_context_len - 1} lies beyond the {self.pos_table.shape[0]} learned positions")
            if self.scale == 1.0 and not self.learned:
                return ops.embed_bigram(tokens, self.weight, self.bigram_table, ctx.positions, ctx.token_req, ctx.cu_seqlens,
                                        ctx.state_slots, state, ctx.num_requests, int(b["mul_prev"]), int(b["mul_cur"]), int(b["buckets"]))
            return ops.embed_bigram(tokens, self.weight, self.bigram_table, ctx.positions, ctx.token_req, ctx.cu_seqlens,
                                    ctx.state_slots, state, ctx.num_requests, int(b["mul_prev"]), int(b["mul_cur"]), int(b["buckets"]),
                                    self.scale, self.pos_table)
        if self.inv_freq is None and streams == 1:
            return ops.embed(tokens, self.weight)
        return ops.embed(tokens, self.weight, positions, self.inv_freq, streams)


class OutputHead(Part):
    category = "lm_head"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None
        self.tied = bool(spec.params.get("tied", False))
        self.scale = float(spec.params.get("scale", 1.0))

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        # Tied: the tensor is neither required nor generated, and is ignored if present.
        init = "skip" if spec.params.get("tied", False) else "normal"
        return {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size), init, optional=True)}

    def load_weights(self, get, embedding: TokenEmbedding = None):
        t = None if self.tied else get(self.spec.weights["weight"], optional=True)
        if t is None:
            if embedding is None or embedding.weight is None:
                raise ValueError("output head is tied but no embedding matrix is loaded")
            # The products read tiled weights at nearly twice the rate of row-major ones (the head of the 3B shape,
            # 128256 x 3072: 208 us row-major, 120 us tiled), and the lookup needs the rows as they are: the head
            # takes a tiled copy where the kernels have a tiled form (bfloat16 on the GPU; vocab x hidden x 2 bytes
            # more), else the same buffer.
            self.weight = ops.tile_weight(embedding.weight)
            self.tied = True
        else:
            self.weight = ops.tile_weight(self._to_device(t))

    def forward(self, x):
        """normed rows [m, hidden] -> float32 logits [m, vocab]."""
        logits = ops.linear(x, self.weight, torch.float32)
        return logits if self.scale == 1.0 else ops.scale_(logits, self.scale)


register_part("embedding", "embedding", TokenEmbedding)
register_part("lm_head", "lm_head", OutputHead)
