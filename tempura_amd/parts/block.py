"""Block arrangements.

``prenorm``: ``h += mixer(norm(h)); h += ffn(norm(h))`` — sequential, two
residual adds (/root/reference/engine/src/model.rs:952-1314; declared as
[PreNormAttention, PreNormFfn], /root/reference/engine/src/architecture.rs:56-65).
The residual stream ``h`` is float32 in every dtype.

A norm may be carried by the two products around it instead of running as a kernel of its own
(``Norm.deferred``, ``ops.Prenormed``): the part before it prepares the rows in the epilogue of its last
product, the part after it finishes them in its first.  The block arranges that for parts that declare
``split_norm``; any other part gets plain normed rows and returns nothing.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightInfo, build_part, part_class, register_part


class ArrangedBlock:
    """Base of the arrangements: builds the parts a ``LayerSpec`` names, by the categories the arrangement
    declares in ``ROLES`` (name -> ``"mixer"``, ``"ffn"`` or ``"norm"``), in that order, each as an attribute of
    its name.  A subclass writes ``forward(h, ctx, cache)`` and registers itself under ``"block"``; the model
    asks ``cache_owner()`` which part's cache and state needs a call of the layer has."""

    category = "block"
    ROLES: dict = {}
    #: roles a layer may leave out (the attribute is then None)
    OPTIONAL: frozenset = frozenset()
    #: what this arrangement hands to the block behind it (blocks of the same kind only): see ``entry_norm``
    handoff = None

    def __init__(self, layer_spec, hidden_size, dtype, device):
        self.layer_spec = layer_spec
        missing = [name for name in self.ROLES if name not in layer_spec.parts and name not in self.OPTIONAL]
        extra = [name for name in layer_spec.parts if name not in self.ROLES]
        if missing or extra:
            raise ValueError(f"block {layer_spec.block!r} arranges the parts {sorted(self.ROLES)}: "
                             f"missing {missing}, not its own {extra}")
        for name, cat in self.ROLES.items():
            ps = layer_spec.parts.get(name)
            setattr(self, name, None if ps is None else build_part(cat, ps, hidden_size, dtype, device))

    def parts(self):
        return [getattr(self, name) for name in self.ROLES if getattr(self, name) is not None]

    def cache_owner(self):
        """The part whose ``cache_spec()`` / ``state_spec()`` this layer's cache slot serves."""
        return self.mixer

    @classmethod
    def expected_weights(cls, layer_spec, hidden_size):
        out = {}
        for name, cat in cls.ROLES.items():
            ps = layer_spec.parts.get(name)
            if ps is None:
                continue
            out.update(part_class(cat, ps.kind).expected_weights(ps, hidden_size))
        return out

    def load_weights(self, get):
        for p in self.parts():
            p.load_weights(get)


class PreNormBlock(ArrangedBlock):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "ffn"}
    handoff = "split_norm"

    def entry_norm(self, m):
        """What the part before this block needs to prepare this block's first norm for ``m`` rows, or None."""
        if getattr(self.mixer, "split_norm", False) and hasattr(self.mixer_norm, "deferred"):
            return self.mixer_norm.deferred(m)
        return None

    def forward(self, h, ctx, cache, x=None, next_norm=None):
        """``x``: rows handed over by the block before (its last product prepared ``mixer_norm``);
        ``next_norm``: the ``entry_norm`` of the block after.  Returns the rows handed to that block, or None."""
        if x is None:
            x = self.mixer_norm.forward(h)
        x2 = None
        if getattr(self.mixer, "split_norm", False):
            mid = None
            if getattr(self.ffn, "split_norm", False) and hasattr(self.ffn_norm, "deferred"):
                mid = self.ffn_norm.deferred(h.shape[0])
            x2 = self.mixer.forward(x, ctx, cache, h, next_norm=mid)
        else:
            self.mixer.forward(x, ctx, cache, h)
        if x2 is None:
            x2 = self.ffn_norm.forward(h)
        if next_norm is not None and getattr(self.ffn, "split_norm", False):
            return self.ffn.forward(x2, ctx, h, next_norm=next_norm)
        self.ffn.forward(x2, ctx, h)
        return None


register_part("block", "prenorm", PreNormBlock)


class HyperConnection(Part):
    """How a sublayer is wired to ``streams`` copies of the residual stream: its input is
    sum_a in[a] x_a, and its output y updates every copy at once, x_b <- sum_a mix[a, b] x_a + out[b] * y
    (``mix`` is indexed [from, to]).  Three small tensors, kept in float32."""

    category = "connection"
    graph_safe = True      # three tensors read by kernels: nothing of the batch is seen on the host

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.streams = int(spec.params["streams"])
        self.in_coef = self.out_coef = self.mix = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        s, w = int(spec.params["streams"]), spec.weights
        return {w["in"]: WeightInfo((s,), "fraction"), w["out"]: WeightInfo((s,), "ones"), w["mix"]: WeightInfo((s, s), "identity")}

    def load_weights(self, get):
        w = self.spec.weights
        self.in_coef = self._to_device(get(w["in"]), torch.float32)
        self.out_coef = self._to_device(get(w["out"]), torch.float32)
        self.mix = self._to_device(get(w["mix"]), torch.float32)


register_part("connection", "hyper_connection", HyperConnection)


class StreamOpening:
    """What the kernel that closes one sublayer needs to open the next: the input coefficients of its connection
    (None: the plain sum) and the weight and eps of its norm."""
    __slots__ = ("in_coef", "weight", "eps")

    def __init__(self, in_coef, weight, eps):
        self.in_coef, self.weight, self.eps = in_coef, weight, eps


class HyperBlock(ArrangedBlock):
    """Pre-norm sublayers around several copies of the residual stream.  ``h`` is float32 [tokens, streams * hidden].
    For the mixer and then the feed-forward (which a layer may leave out): u = sum_a in[a] x_a, y = sublayer(norm(u)),
    then every copy is updated from the old ones (see ``HyperConnection``).  A sublayer without a connection part
    has the plain residual sum (one copy, x <- x + y).

    One kernel closes a sublayer and opens the next (update of the copies, the next input combination and its
    norm), also across layers: ``entry_norm`` says what the block before needs for that."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_link": "connection",
             "ffn_norm": "norm", "ffn": "ffn", "ffn_link": "connection"}
    OPTIONAL = frozenset({"mixer_link", "ffn_norm", "ffn", "ffn_link"})
    handoff = "streams"

    def __init__(self, layer_spec, hidden_size, dtype, device):
        super().__init__(layer_spec, hidden_size, dtype, device)
        if (self.ffn is None) != (self.ffn_norm is None):
            raise ValueError("block 'hyper': a feed-forward and its norm come together")
        links = [l for l in (self.mixer_link, self.ffn_link) if l is not None]
        self.streams = links[0].streams if links else 1
        if any(l.streams != self.streams for l in links) or (self.streams > 1 and (self.mixer_link is None or (self.ffn is not None and self.ffn_link is None))):
            raise ValueError("block 'hyper': every sublayer of a layer is wired to the same number of copies")
        self.hidden_size = hidden_size
        self.dtype = dtype

    @staticmethod
    def _opening(norm, link):
        if hasattr(norm, "weight") and hasattr(norm, "eps") and type(norm).__name__ == "RMSNorm" and getattr(norm, "groups", 1) == 1:
            return StreamOpening(None if link is None else link.in_coef, norm.weight, norm.eps)
        return None

    def entry_norm(self, m):
        """What the block before needs to prepare this block's first sublayer input (None: this block does it)."""
        return self._opening(self.mixer_norm, self.mixer_link)

    def _open(self, h, norm, link):
        """The normed input of a sublayer from the copies as they stand."""
        op = self._opening(norm, link)
        if op is not None:
            return ops.stream_step(h, self.streams, in_coef=op.in_coef, norm_weight=op.weight, eps=op.eps, out_dtype=self.dtype)
        u = ops.stream_step(h, self.streams, in_coef=None if link is None else link.in_coef, out_dtype=torch.float32)
        return norm.forward(u)

    def _close(self, h, y, link, opening):
        """Update the copies with a sublayer's output; with ``opening`` also return the next sublayer's input."""
        mix = None if link is None else link.mix
        out = None if link is None else link.out_coef
        if opening is None:
            ops.stream_step(h, self.streams, y, mix, out)
            return None
        return ops.stream_step(h, self.streams, y, mix, out, opening.in_coef, opening.weight, opening.eps, self.dtype)

    def _run(self, part, x, ctx, cache, n, device):
        """A sublayer's output as a tensor of its own, float32 [tokens, hidden]."""
        args = (x, ctx, cache) if cache is not None else (x, ctx)
        if getattr(part, "returns_output", False):
            return part.forward(*args, None)
        y = torch.zeros((n, self.hidden_size), dtype=torch.float32, device=device)
        part.forward(*args, y)
        return y

    def forward(self, h, ctx, cache, x=None, next_norm=None):
        n = h.shape[0]
        if x is None:
            x = self._open(h, self.mixer_norm, self.mixer_link)
        y = self._run(self.mixer, x, ctx, cache, n, h.device)
        after = next_norm if isinstance(next_norm, StreamOpening) else None
        if self.ffn is None:
            return self._close(h, y, self.mixer_link, after)
        mid = self._opening(self.ffn_norm, self.ffn_link)
        x2 = self._close(h, y, self.mixer_link, mid)
        if x2 is None:
            x2 = self._open(h, self.ffn_norm, self.ffn_link)
        y2 = self._run(self.ffn, x2, ctx, None, n, h.device)
        return self._close(h, y2, self.ffn_link, after)


register_part("block", "hyper", HyperBlock)


class SandwichBlock(ArrangedBlock):
    """A norm before and a norm behind each sublayer: ``h += post(mixer(pre(h)))``, then, when the layer has a
    feed-forward, ``h += post(ffn(pre(h)))``.  A constant that multiplies what enters the stream is the ``scale`` of
    the norm behind the sublayer.  The norms behind the sublayers are RMS norms; one kernel norms a sublayer's
    output, adds it into the stream and norms the stream for the next sublayer, also across layers (``entry_norm``
    says what the block before needs for that)."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm",
             "ffn_norm": "norm", "ffn": "ffn", "ffn_post_norm": "norm"}
    OPTIONAL = frozenset({"ffn_norm", "ffn", "ffn_post_norm"})
    handoff = "sandwich"

    def __init__(self, layer_spec, hidden_size, dtype, device):
        super().__init__(layer_spec, hidden_size, dtype, device)
        if len({self.ffn is None, self.ffn_norm is None, self.ffn_post_norm is None}) != 1:
            raise ValueError("block 'sandwich': a feed-forward and its two norms come together")
        for post in (self.mixer_post_norm, self.ffn_post_norm):
            if post is not None and (type(post).__name__ != "RMSNorm" or getattr(post, "groups", 1) != 1):
                raise ValueError("block 'sandwich': the norm behind a sublayer must be an RMS norm")
        self.hidden_size = hidden_size
        self.dtype = dtype

    @staticmethod
    def _rms(norm):
        """(weight, eps) of an RMS norm that the closing kernel can apply, else None."""
        if type(norm).__name__ == "RMSNorm" and getattr(norm, "groups", 1) == 1:
            return norm.weight, norm.eps
        return None

    def entry_norm(self, m):
        return self._rms(self.mixer_norm)

    def _run(self, part, x, ctx, cache, n, device):
        """A sublayer's output as a tensor of its own, float32 [tokens, hidden]."""
        args = (x, ctx, cache) if cache is not None else (x, ctx)
        if getattr(part, "returns_output", False):
            return part.forward(*args, None)
        y = torch.zeros((n, self.hidden_size), dtype=torch.float32, device=device)
        part.forward(*args, y)
        return y

    def _close(self, h, y, post, opening):
        """Norm ``y``, add it into the stream; with ``opening`` (weight, eps) also return the stream normed for the
        next sublayer."""
        if opening is None:
            ops.norm_add(h, y, post.weight, post.eps)
            return None
        return ops.norm_add(h, y, post.weight, post.eps, opening[0], opening[1], self.dtype)

    def forward(self, h, ctx, cache, x=None, next_norm=None):
        n = h.shape[0]
        if x is None:
            x = self.mixer_norm.forward(h)
        y = self._run(self.mixer, x, ctx, cache, n, h.device)
        after = next_norm if isinstance(next_norm, tuple) else None
        if self.ffn is None:
            return self._close(h, y, self.mixer_post_norm, after)
        x2 = self._close(h, y, self.mixer_post_norm, self._rms(self.ffn_norm))
        if x2 is None:
            x2 = self.ffn_norm.forward(h)
        y2 = self._run(self.ffn, x2, ctx, None, n, h.device)
        return self._close(h, y2, self.ffn_post_norm, after)


register_part("block", "sandwich", SandwichBlock)


class SharedNormBlock(ArrangedBlock):
    """ONE norm whose output both sublayers read, their outputs entering the stream together:
    n = norm(h); h += mixer(in_0(n)) + ffn(in_1(n)).  ``inputs`` (optional, category ``input``) says what each sublayer
    reads of n (``residual_conv``: n plus a short convolution of n over time, one weight per sublayer); without it both
    read n itself.  A layer may have no feed-forward.

    The layer's state row holds the input part's carried rows first and the mixer's state behind them, so the mixer is
    one that takes an offset into its row (a ``BranchMixer``) or keeps no state."""
    ROLES = {"norm": "norm", "inputs": "input", "mixer": "mixer", "ffn": "ffn"}
    OPTIONAL = frozenset({"inputs", "ffn"})

    def __init__(self, layer_spec, hidden_size, dtype, device):
        super().__init__(layer_spec, hidden_size, dtype, device)
        self.dtype = dtype
        self.front = self.inputs.state_floats() if self.inputs is not None else 0
        if self.front:
            if self.mixer.state_spec() is not None and not hasattr(self.mixer, "state_floats"):
                raise ValueError(f"block 'shared_norm': mixer {self.mixer.spec.kind!r} cannot share a state row (no state offset)")
            if hasattr(self.mixer, "state_floats"):
                self.mixer.state_off = self.front
        if self.inputs is not None and len(self.inputs.names) != (1 if self.ffn is None else 2):
            raise ValueError("block 'shared_norm': the input part needs one weight per sublayer")

    def cache_owner(self):
        return self

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        from .base import StateSpec
        if not self.front:
            return self.mixer.state_spec()
        behind = self.mixer.state_floats() if hasattr(self.mixer, "state_floats") else 0
        return StateSpec((self.front + behind,), torch.float32)

    def forward(self, h, ctx, cache) -> None:
        if self.inputs is not None:
            xs = self.inputs.forward(self.norm.forward(h, out_dtype=torch.float32), ctx, cache)
        else:
            xs = [self.norm.forward(h)] * 2
        self.mixer.forward(xs[0], ctx, cache, h)
        if self.ffn is not None:
            self.ffn.forward(xs[1], ctx, h)


register_part("block", "shared_norm", SharedNormBlock)
