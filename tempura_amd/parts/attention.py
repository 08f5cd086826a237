"""Grouped-query attention over the paged cache.

Per token: q, k, v projections (no bias), position encoding on q and k, k and v
stored into the cache pages, causal (optionally windowed) softmax attention
over the request's cached keys with ``kv_head = head // (heads / kv_heads)``,
output projection added into the residual stream
(/root/reference/engine/src/model.rs:1007-1152,
/root/reference/kernels/src/attention.rs:28-87).
A window of ``w`` lets query position p see keys p-w+1 .. p
(/root/reference/kernels/src/attention.rs:55-59).

Options beyond that, each a parameter of the part:
* ``bias``: the q and k projections have biases (tensors ``q_bias``, ``k_bias``);
* ``values: "keys"``: there is no value projection, a head's values are its keys as projected;
* ``distance_bias``: a learned bias per head and distance is added to the scaled score (the scale does not
  multiply it).  Kind ``"log_buckets"``: the tensor has B rows of one value per head, and distance n reads row
  n while n < B // 2, else row min(B - 1, B // 2 + floor(ln(n / (B // 2)) / ln(max_distance / (B // 2)) * (B - B // 2))).
  B is the tensor's own first dimension.
The first two need a position encoding that does not rotate (``"none"``).
* ``qk_norm`` (``{"eps"}``, tensors ``q_norm``, ``k_norm`` of [head_dim]): every head of q and of k is divided by its
  root mean square and multiplied by the weight (one weight for all q heads, one for all k heads), before any rotation;
* ``value_dim``: the values of a head have another size than its keys;
* ``sink`` (tensor ``sink`` [heads]): the softmax's denominator holds one more term exp(sink[head]) that has no key
  and no value;
* ``keep_first``: under a ``window`` a query also sees the request's first ``keep_first`` keys (their pages stay held).
The last four run without projection biases, own values, and a rows-in-float32 projection (no split norm).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ..kernels import ops
from .base import BranchMixer, CacheSpec, Mixer, WeightInfo, build_part, part_class, register_part


def log_bucket(n: int, buckets: int, max_distance: int) -> int:
    """The row of a ``log_buckets`` table that distance ``n`` >= 0 reads: exact below half the table, then
    logarithmic up to ``max_distance``, then the last row."""
    half = buckets // 2
    if n < half:
        return n
    if half == 0 or max_distance <= half:
        return buckets - 1
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(max_distance / half) * (buckets - half))))


def distance_table(rows: torch.Tensor, max_distance: int, window) -> torch.Tensor:
    """float32 [heads, L] from a ``log_buckets`` tensor [B, heads]: entry n is the bias of distance n; every
    distance from L - 1 on has the value of entry L - 1 (the last row, or never occurs under the window)."""
    buckets = rows.shape[0]
    length = 1
    while log_bucket(length - 1, buckets, max_distance) < buckets - 1 and (window is None or length < window):
        length += 1
    index = torch.tensor([log_bucket(n, buckets, max_distance) for n in range(length)], dtype=torch.long)
    return rows.to(torch.float32)[index].t().contiguous()


class PagedAttention(Mixer):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph
    #: the value cache is transposed, eight consecutive tokens of one element being one 16-byte piece: a portion that
    #: starts at a multiple of eight positions (and of eight rows of the batch) has its values stored piece by piece
    preferred_portion_align = 8
    split_norm = True      # takes rows whose norm its first product finishes; prepares the next norm in its last
    returns_output = True  # with ``residual`` None the output comes back instead of being added

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError("attention: heads must be a multiple of kv heads")
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.q_dim = self.num_heads * self.head_dim
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.position = build_part("position", p["position"], hidden_size, dtype, device)
        self.has_bias = bool(p.get("bias", False))
        values = p.get("values", "own")
        if values not in ("own", "keys"):
            raise ValueError(f"attention: values {values!r} unknown (known: own, keys)")
        self.values_are_keys = values == "keys"
        self.distance_bias = p.get("distance_bias")
        if self.distance_bias is not None and self.distance_bias.get("kind") != "log_buckets":
            raise ValueError(f"attention: distance bias {self.distance_bias.get('kind')!r} unknown (known: log_buckets)")
        if (self.has_bias or self.values_are_keys) and self.position.rotary() is not None:
            raise ValueError("attention: projection biases and values that are the keys need a position encoding that does not rotate")
        if self.has_bias and not self.values_are_keys:
            raise ValueError("attention: projection biases are supported together with values that are the keys")
        #: q and k come straight from the projection (biases added, keys stored as keys and as values): no rotation kernel
        self.plain_qk = self.values_are_keys
        self.qk_norm = p.get("qk_norm")
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.has_sink = bool(p.get("sink", False))
        self.keep_first = int(p.get("keep_first") or 0)
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise ValueError("attention: keep_first needs a window and must not be negative")
        #: the options that take the projection's float32 rows through kernels of their own
        self.extended = self.qk_norm is not None or self.value_dim != self.head_dim or self.has_sink or self.keep_first > 0
        if self.extended and (self.plain_qk or self.has_bias or self.distance_bias is not None):
            raise ValueError("attention: qk_norm, value_dim, sink and keep_first do not combine with biases, values that are the keys "
                             "or a distance bias")
        self.v_dim = self.num_kv_heads * self.value_dim
        # values wider than keys, of a size the matrix-core attention kernels take: q and the cached keys get zeros
        # behind their own elements up to the values' size (no score changes), so that those kernels serve
        self.key_dim = self.head_dim
        if (dtype == torch.bfloat16 and self.head_dim < self.value_dim <= 128 and self.value_dim % 32 == 0 and self.head_dim % 2 == 0
                and ops.fast_attention_takes(self.has_sink, self.keep_first)):
            self.key_dim = self.value_dim
        self.split_norm = not self.plain_qk and not self.extended      # (these projections take finished rows only)
        self.q_norm_w = self.k_norm_w = self.sink_w = None
        self.wqkv = None
        self.wo = None
        self.q_bias = self.k_bias = self.dist_table = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        q_dim = p["num_heads"] * p["head_dim"]
        kv_dim = p["num_kv_heads"] * p["head_dim"]
        out = {
            w["q"]: WeightInfo((q_dim, hidden_size)),
            w["k"]: WeightInfo((kv_dim, hidden_size)),
            w["o"]: WeightInfo((hidden_size, q_dim)),
        }
        vd = int(p.get("value_dim") or p["head_dim"])
        if p.get("values", "own") != "keys":
            out[w["v"]] = WeightInfo((p["num_kv_heads"] * vd, hidden_size))
        out[w["o"]] = WeightInfo((hidden_size, p["num_heads"] * vd))
        if p.get("qk_norm") is not None:
            out[w["q_norm"]] = WeightInfo((p["head_dim"],), "ones")
            out[w["k_norm"]] = WeightInfo((p["head_dim"],), "ones")
        if p.get("sink", False):
            out[w["sink"]] = WeightInfo((p["num_heads"],))
        if p.get("bias", False):
            out[w["q_bias"]] = WeightInfo((q_dim,))
            out[w["k_bias"]] = WeightInfo((kv_dim,))
        if p.get("distance_bias") is not None:
            # (the number of rows is the tensor's own; a configuration may name it for random weights)
            out[w["distance_bias"]] = WeightInfo((p["distance_bias"].get("buckets"), p["num_heads"]))
        # a position encoding may have tensors of its own (a rotary one has none)
        out.update(part_class("position", p["position"].kind).expected_weights(p["position"], hidden_size))
        return out

    def _paired(self, t: torch.Tensor) -> torch.Tensor:
        """The rows of a q or k projection with every head's rotary elements in paired order: rows
        (2 d, 2 d + 1) of a head are rows (d, d + rotary_dim / 2) of the checkpoint's split-half order, so
        that the two elements that rotate together are neighbours (the rotation kernels expect that, and a
        product's epilogue can rotate what it holds).  q and k are permuted alike, which leaves every score
        as it was; the cache then holds keys in this order."""
        rot = self.position.rotary()
        if rot is None or rot[1] == 0:
            return t
        rd, half, d = rot[1], rot[1] // 2, self.head_dim
        order = torch.arange(d)
        order[0:rd:2] = torch.arange(half)
        order[1:rd:2] = torch.arange(half) + half
        heads = t.shape[0] // d
        return t.view(heads, d, -1)[:, order.to(t.device), :].reshape(t.shape)

    def load_weights(self, get):
        w = self.spec.weights
        if self.has_bias:
            self.q_bias = self._to_device(get(w["q_bias"]), torch.float32)
            self.k_bias = self._to_device(get(w["k_bias"]), torch.float32)
        if self.distance_bias is not None:
            self.dist_table = self._to_device(distance_table(get(w["distance_bias"]), int(self.distance_bias["max_distance"]),
                                                             self.window), torch.float32)
        # One [q_dim + 2 kv_dim, hidden] matrix: one product instead of three.
        parts = [self._paired(get(w["q"])), self._paired(get(w["k"]))]
        if not self.values_are_keys:
            parts.append(get(w["v"]))
        # (stored tiled where the sizes allow: the products then read whole cache lines)
        self.wqkv = ops.tile_weight(torch.cat([self._to_device(t) for t in parts], dim=0).contiguous())
        self.wo = ops.tile_weight(self._to_device(get(w["o"])))
        if self.qk_norm is not None:
            self.q_norm_w = self._to_device(get(w["q_norm"]), torch.float32)
            self.k_norm_w = self._to_device(get(w["k_norm"]), torch.float32)
        if self.has_sink:
            self.sink_w = self._to_device(get(w["sink"]), torch.float32)
        self.position.load_weights(get)

    def cache_spec(self):
        kind = "window" if self.window is not None else "full"
        if self.keep_first:
            return SizedValueCacheSpec("window_keep_first", self.num_kv_heads, self.key_dim, self.window, self.value_dim, self.keep_first)
        if self.value_dim != self.key_dim:
            return SizedValueCacheSpec(kind, self.num_kv_heads, self.key_dim, self.window, self.value_dim)
        return CacheSpec(kind, self.num_kv_heads, self.key_dim, self.window)

    def forward(self, x, ctx, cache, residual, next_norm=None):
        rot = self.position.rotary()
        q = None
        if self.plain_qk:
            q = self._project_plain(x, ctx, cache)
        elif rot is not None and cache.writes and not self.extended:
            rows = x.x if isinstance(x, ops.Prenormed) else x
            if ops.linear_rope_ok(x.shape[0], self.wqkv.shape[0], x.shape[1], self.head_dim, rot[1], cache.k.shape[2],
                                  rows.dtype, cache.k.dtype, isinstance(x, ops.Prenormed)):
                # a few rows (decoding) or a long step: the projection rotates and stores its rows itself
                table = self.position.table(ctx, always=True) if hasattr(self.position, "table") else None
                q = ops.linear_rope_kv(x, self.wqkv, ctx.positions, ctx.slot_mapping[cache.group], rot[0], rot[1], rot[2],
                                       self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v, table)
        if q is None:
            q = self._project_and_rotate(x, ctx, cache, rot)
        if self.extended:
            a = ops.paged_attention(
                q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
                ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len,
                ctx.num_single, sink=self.sink_w, keep_first=self.keep_first)
        elif self.dist_table is not None:
            a = ops.paged_attention(
                q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
                ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len,
                ctx.num_single, dist_bias=self.dist_table)
        else:
            a = ops.paged_attention(
                q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
                ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len,
                ctx.num_single)
        if residual is None:
            return ops.linear(a, self.wo, torch.float32)
        if next_norm is None:
            ops.linear(a, self.wo, torch.float32, residual=residual)
            return None
        return ops.linear(a, self.wo, torch.float32, residual=residual, next_norm=next_norm)[1]

    def _project_plain(self, x, ctx, cache):
        """q ([n, heads, head_dim]) of a projection without rotation: biases added, k stored as keys and, when the
        values are the keys, as values too (the value cache is transposed, so it is a second store, not a view)."""
        if isinstance(x, ops.Prenormed):
            raise ValueError("attention: rows with an unfinished norm need a rotary projection")
        if cache.writes:
            rows = ops.linear(x, self.wqkv, torch.float32)
            return ops.qk_store(rows, self.q_bias, self.k_bias, ctx.slot_mapping[cache.group], self.num_heads,
                                self.num_kv_heads, self.head_dim, cache.k, cache.v, self.dtype)
        rows = ops.linear(x, ops.weight_rows(self.wqkv, 0, self.q_dim), torch.float32)
        return ops.qk_store(rows, self.q_bias, None, None, self.num_heads, self.num_kv_heads, self.head_dim, None, None, self.dtype)

    def _project_extended(self, x, ctx, cache, rot):
        """q of a projection with a norm per head and/or values of their own size: the float32 rows are normed in
        place, then rotated (if the position part rotates) and stored by the cache-write kernel."""
        if rot is None and type(self.position).__name__ != "NoPosition":
            raise ValueError("attention: qk_norm, value_dim, sink and keep_first need a rotary position part or none")
        writes = cache.writes
        w = self.wqkv if writes else ops.weight_rows(self.wqkv, 0, self.q_dim)
        qkv = ops.linear(x, w, torch.float32)
        if self.qk_norm is not None:
            ops.head_rmsnorm(qkv, 0, self.num_heads, self.q_norm_w, self.q_dim, self.num_kv_heads if writes else 0, self.k_norm_w,
                             self.head_dim, float(self.qk_norm["eps"]))
        inv_freq, rotary_dim, factor, table = None, 0, 1.0, None
        if rot is not None:
            inv_freq, rotary_dim, factor = rot
            table = self.position.table(ctx) if hasattr(self.position, "table") else None
        return ops.rope_kv_write(qkv, ctx.positions, ctx.slot_mapping[cache.group] if writes else None, inv_freq, rotary_dim, factor,
                                 self.num_heads, self.num_kv_heads, self.head_dim, cache.k if writes else None,
                                 cache.v if writes else None, self.dtype, table, value_dim=self.value_dim, pad_dim=self.key_dim)

    def _project_and_rotate(self, x, ctx, cache, rot):
        """q (rotated, [n, heads, head_dim]) of the projection; k and v go to the cache."""
        # (with a rotary position the next kernel may add the projection's partial sums itself)
        if self.extended:
            return self._project_extended(x, ctx, cache, rot)
        if cache.writes:
            qkv = ops.linear(x, self.wqkv, torch.float32, partial_ok=rot is not None)
        else:
            # A call that reads another call's cache needs queries only.
            qkv = ops.linear(x, ops.weight_rows(self.wqkv, 0, self.q_dim), torch.float32, partial_ok=rot is not None)
        if rot is None:
            q = qkv[:, : self.q_dim]
            k = qkv[:, self.q_dim: self.q_dim + self.kv_dim] if cache.writes else None
            q2, k2 = self.position.apply(q, k, ctx.positions)
            if cache.writes:
                qkv = torch.cat([q2, k2, qkv[:, self.q_dim + self.kv_dim:]], dim=1).contiguous()
            else:
                qkv = q2.contiguous()
            inv_freq, rotary_dim, factor, table = None, 0, 1.0, None
        else:
            inv_freq, rotary_dim, factor = rot
            table = self.position.table(ctx) if hasattr(self.position, "table") else None
        q = ops.rope_kv_write(
            qkv, ctx.positions, ctx.slot_mapping[cache.group] if cache.writes else None,
            inv_freq, rotary_dim, factor, self.num_heads, self.num_kv_heads, self.head_dim,
            cache.k if cache.writes else None, cache.v if cache.writes else None, self.dtype, table)
        return q


register_part("mixer", "attention", PagedAttention)


@dataclass(frozen=True)
class SizedValueCacheSpec(CacheSpec):
    """Keys of ``head_dim`` and values of ``value_dim``: keys [kv_heads, page_size, head_dim] as ever, values
    transposed [kv_heads, value_dim, page_size]."""
    value_dim: int = 0
    #: with kind ``"window_keep_first"``: the request's first keys that stay visible (and held) under the window
    keep_first: int = 0

    def planes(self, page_size: int):
        return {"k": (self.num_kv_heads, page_size, self.head_dim), "v": (self.num_kv_heads, self.value_dim, page_size)}


class ConvAttention(BranchMixer):
    """Grouped-query softmax attention over the paged cache whose q, k and v pass a short causal convolution per
    channel right behind their projections (``conv_taps`` taps, no bias, no activation, zeros before a request's
    start; before any rotation), whose values may have another size than its keys (``value_dim``), and whose
    concatenated heads are multiplied by sigmoid(W_g x) before the output projection (``gate``).  The position
    encoding, the scale and an optional window are parameters as for ``attention``.

    The columns of its input product are [q | k | v | gate]; a request's state is the convolution's last
    ``conv_taps - 1`` inputs [conv_taps - 1, q | k | v], float32."""
    preferred_portion_align = 8      # (the value cache is transposed: see ``PagedAttention``)

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError("conv_attention: heads must be a multiple of kv heads")
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.taps = int(p["conv_taps"])
        if self.taps < 1:
            raise ValueError("conv_attention: conv_taps must be at least 1")
        self.gate = bool(p.get("gate", False))
        self.position = build_part("position", p["position"], hidden_size, dtype, device)
        self.q_dim = self.num_heads * self.head_dim
        self.k_dim = self.num_kv_heads * self.head_dim
        self.v_dim = self.num_kv_heads * self.value_dim
        self.channels = self.q_dim + self.k_dim + self.v_dim
        self.inner = self.num_heads * self.value_dim
        # values wider than keys, of a size the matrix-core attention kernels take: q and the cached keys get zeros
        # behind their own elements up to the values' size (no score changes; the key pages are that much wider),
        # so that those kernels serve; every other pair of sizes runs the general kernel
        self.key_dim = self.head_dim
        if dtype == torch.bfloat16 and self.head_dim < self.value_dim <= 128 and self.value_dim % 32 == 0 and self.head_dim % 2 == 0:
            self.key_dim = self.value_dim
        self.conv_w = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        vd = int(p.get("value_dim") or p["head_dim"])
        q_dim, k_dim, v_dim = p["num_heads"] * p["head_dim"], p["num_kv_heads"] * p["head_dim"], p["num_kv_heads"] * vd
        taps = int(p["conv_taps"])
        out = {
            w["q"]: WeightInfo((q_dim, hidden_size)), w["k"]: WeightInfo((k_dim, hidden_size)), w["v"]: WeightInfo((v_dim, hidden_size)),
            w["q_conv"]: WeightInfo((q_dim, taps)), w["k_conv"]: WeightInfo((k_dim, taps)),
            w["v_conv"]: WeightInfo((v_dim, taps)),
            w["o"]: WeightInfo((hidden_size, p["num_heads"] * vd)),
        }
        if p.get("gate", False):
            out[w["gate"]] = WeightInfo((p["num_heads"] * vd, hidden_size))
        out.update(part_class("position", p["position"].kind).expected_weights(p["position"], hidden_size))
        return out

    def state_floats(self) -> int:
        return (self.taps - 1) * self.channels

    def cache_spec(self):
        kind = "window" if self.window is not None else "full"
        if self.value_dim == self.key_dim:
            return CacheSpec(kind, self.num_kv_heads, self.key_dim, self.window)
        return SizedValueCacheSpec(kind, self.num_kv_heads, self.key_dim, self.window, self.value_dim)

    def _paired(self, t: torch.Tensor) -> torch.Tensor:
        """Rows of a q or k tensor (projection or convolution) with every head's rotary elements in paired order
        (see ``PagedAttention._paired``: the rotation kernels take neighbours as pairs)."""
        rot = self.position.rotary()
        if rot is None or rot[1] == 0:
            return t
        rd, half, d = rot[1], rot[1] // 2, self.head_dim
        order = torch.arange(d)
        order[0:rd:2] = torch.arange(half)
        order[1:rd:2] = torch.arange(half) + half
        return t.view(t.shape[0] // d, d, -1)[:, order.to(t.device), :].reshape(t.shape)

    def load_branch(self, get):
        w = self.spec.weights
        rows = [self._paired(get(w["q"])), self._paired(get(w["k"])), get(w["v"])]
        if self.gate:
            rows.append(get(w["gate"]))
        conv = torch.cat([self._paired(get(w["q_conv"])), self._paired(get(w["k_conv"])), get(w["v_conv"])], dim=0)
        self.conv_w = self._to_device(conv, torch.float32).t().contiguous()      # tap-major for the kernel
        self.position.load_weights(get)
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(get(w["o"]))

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        if not cache.writes:
            raise ValueError("conv_attention: a call that reads another call's cache is not supported")
        qkv = ops.causal_conv(proj, col0, self.channels, self.conv_w, None, cache.state, ctx.cu_seqlens, ctx.token_req,
                              ctx.state_slots, ctx.num_requests, state_off=self.state_off, act=False)
        rot = self.position.rotary()
        inv_freq, rotary_dim, factor, table = None, 0, 1.0, None
        if rot is not None:
            inv_freq, rotary_dim, factor = rot
            table = self.position.table(ctx) if hasattr(self.position, "table") else None
        q = ops.rope_kv_write(qkv, ctx.positions, ctx.slot_mapping[cache.group], inv_freq, rotary_dim, factor, self.num_heads,
                              self.num_kv_heads, self.head_dim, cache.k, cache.v, self.dtype, table, value_dim=self.value_dim,
                              pad_dim=self.key_dim)
        a = ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
                                ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len, ctx.num_single)
        ops.sigmoid_gate(a, proj if self.gate else None, col0 + self.channels, scale, out, out_col0)


register_part("mixer", "conv_attention", ConvAttention)


class LatentAttention(BranchMixer):
    """Softmax attention whose keys and values are expanded from one compressed vector per token.  With H =
    ``num_heads``, per head D = ``head_dim`` unrotated and R = ``rotary_dim`` rotated query/key elements, values of
    ``value_dim`` and a latent of L = ``latent_dim``: q = W_q x, per head [D unrotated | R rotated]; W_down x has L + R
    rows: the first L, RMS-normed (``norm_eps``) with a weight, are the latent c, the last R (not normed) are ONE rotated
    key part shared by all heads.  Head h's unrotated key is W_uk[h] c, its value W_uv[h] c; the score is
    (q_plain . k_plain + q_rot . k_rot) * ``scale``.  The position part rotates neighbouring pairs (2i, 2i + 1) of the R
    rotated elements of q and of the shared key part.  ``window``, ``gate`` (sigmoid(W_g x) on the concatenated heads) as
    for ``conv_attention``.

    The cache holds expanded keys and values per head: keys [rotated | unrotated] of R + D, values of ``value_dim``.
    Every model of this kind here runs under a sliding window, which bounds what a request holds, and a decode step
    then needs no products with the expansion weights for the keys it reads.  At load the rows of W_q are brought into
    the cache's order per head, [rotated | unrotated]; q and k are ordered alike, so no score changes.

    The columns of its input product are [q | down | gate]; it keeps no per-request state."""
    preferred_portion_align = 8      # (the value cache is transposed: see ``PagedAttention``)

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.rotary_dim = int(p["rotary_dim"])
        self.value_dim = int(p["value_dim"])
        self.latent_dim = int(p["latent_dim"])
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.norm_eps = float(p["norm_eps"])
        self.gate = bool(p.get("gate", False))
        self.position = build_part("position", p["position"], hidden_size, dtype, device)
        rot = self.position.rotary()
        if (rot[1] if rot is not None else 0) != self.rotary_dim:
            raise ValueError("latent_attention: the position part must rotate exactly the rotated elements")
        self.key_dim = self.head_dim + self.rotary_dim
        self.q_dim = self.num_heads * self.key_dim
        self.down_dim = self.latent_dim + self.rotary_dim
        self.inner = self.num_heads * self.value_dim

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        H, D, R, Dv, L = (int(p[k]) for k in ("num_heads", "head_dim", "rotary_dim", "value_dim", "latent_dim"))
        out = {w["q"]: WeightInfo((H * (D + R), hidden_size)), w["down"]: WeightInfo((L + R, hidden_size)),
               w["latent_norm"]: WeightInfo((L,), "ones"), w["up_k"]: WeightInfo((H * D, L)), w["up_v"]: WeightInfo((H * Dv, L)),
               w["o"]: WeightInfo((hidden_size, H * Dv))}
        if p.get("gate", False):
            out[w["gate"]] = WeightInfo((H * Dv, hidden_size))
        out.update(part_class("position", p["position"].kind).expected_weights(p["position"], hidden_size))
        return out

    def cache_spec(self):
        kind = "window" if self.window is not None else "full"
        if self.value_dim == self.key_dim:
            return CacheSpec(kind, self.num_heads, self.key_dim, self.window)
        return SizedValueCacheSpec(kind, self.num_heads, self.key_dim, self.window, self.value_dim)

    def load_branch(self, get):
        from .base import pad_rows
        w = self.spec.weights
        H, D, R = self.num_heads, self.head_dim, self.rotary_dim
        q = get(w["q"])
        q = torch.cat([q.view(H, D + R, -1)[:, D:], q.view(H, D + R, -1)[:, :D]], dim=1).reshape(q.shape)      # per head [rotated | unrotated]
        rows = [q, get(w["down"])]
        if self.gate:
            rows.append(get(w["gate"]))
        self.latent_norm_w = self._to_device(get(w["latent_norm"]), torch.float32)
        self.w_up = ops.tile_weight(pad_rows(torch.cat([self._to_device(get(w["up_k"])), self._to_device(get(w["up_v"]))], dim=0), 16))
        self.position.load_weights(get)
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(get(w["o"]))

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        if not cache.writes:
            raise ValueError("latent_attention: a call that reads another call's cache is not supported")
        H = self.num_heads
        c = ops.rmsnorm_cols(proj, col0 + self.q_dim, self.latent_dim, self.latent_norm_w, self.norm_eps, self.dtype)
        up = ops.linear(c, self.w_up, torch.float32)
        rows = ops.latent_rows(proj, col0, col0 + self.q_dim + self.latent_dim, up, H, self.head_dim, self.rotary_dim, self.value_dim)
        inv_freq, rotary_dim, factor = self.position.rotary()
        table = self.position.table(ctx) if hasattr(self.position, "table") else None
        q = ops.rope_kv_write(rows, ctx.positions, ctx.slot_mapping[cache.group], inv_freq, rotary_dim, factor, H, H, self.key_dim,
                              cache.k, cache.v, self.dtype, table, value_dim=self.value_dim)
        a = ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
                                ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len, ctx.num_single)
        ops.sigmoid_gate(a, proj if self.gate else None, col0 + self.q_dim + self.down_dim, scale, out, out_col0)


register_part("mixer", "latent_attention", LatentAttention)


class LatentCacheAttention(BranchMixer):
    """Softmax attention without positions whose cache holds ONE compressed vector a token, the latent c, from which
    every head's keys and values are linear maps.  With H = ``num_heads``, per head D = ``head_dim`` query/key elements
    and Dv = ``value_dim`` values, a latent of L = ``latent_dim`` and a query latent of ``query_rank``:

        c_q = rmsnorm(W_dq x) * w_dq      q_h = W_uq[h] c_q                       (queries through a latent of their own)
        c   = rmsnorm(W_dkv x) * w_dkv    k_h = W_uk[h] c    v_h = W_uv[h] c      score = (q_h . k_h) * ``scale``

    causal (or under a ``window``), optionally with a ``sink`` per head in the softmax's denominator, then W_o on the
    concatenated heads.  ``own_latent`` False: the layer has no W_dkv; its call of the run order names the cache slot of
    the layer whose latents it reads (with its own W_uk, W_uv and everything else).

    The maps are folded into the two ends: q_h . (W_uk[h] c) = (W_uk[h]^T q_h) . c and W_o[:, h] W_uv[h] (sum_j p_j c_j), so
    the attention itself is one shared key/value head of L elements whose values are its keys, read straight from the
    cache: a step expands nothing of what it reads, however long the context.  The folded weights W_uk[h]^T W_uq[h]
    [H L, query_rank] and W_o[:, h] W_uv[h] [hidden, H L] are formed once at load (in float64, then rounded to the
    compute dtype); per token they cost H L (query_rank + hidden) multiply-adds against H (D query_rank + Dv hidden) plus
    H L (D + Dv) for the maps one after the other, which is the price of a cache and a decode step that stay small.

    The columns of its input product are [dq | dkv]; it keeps no per-request state.  A page holds the latents as keys
    [1, page_size, L] and once more transposed as values [1, L, page_size], the layout every attention kernel reads."""
    preferred_portion_align = 8      # (the value cache is transposed: see ``PagedAttention``)

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.head_dim = int(p["head_dim"])
        self.value_dim = int(p["value_dim"])
        self.latent_dim = int(p["latent_dim"])
        #: the query latent's size: the configuration's, or (None) the checkpoint's own, known once the tensors are loaded
        self.query_rank = int(p["query_rank"]) if p.get("query_rank") is not None else None
        self.scale = float(p["scale"])
        self.norm_eps = float(p["norm_eps"])
        self.window = p.get("window")
        self.has_sink = bool(p.get("sink", False))
        self.own_latent = bool(p.get("own_latent", True))
        self.inner = self.num_heads * self.latent_dim
        self.sink_w = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        H, D, Dv, L = (int(p[k]) for k in ("num_heads", "head_dim", "value_dim", "latent_dim"))
        Q = int(p["query_rank"]) if p.get("query_rank") is not None else None      # (None: the checkpoint says it)
        out = {w["dq"]: WeightInfo((Q, hidden_size)), w["dq_norm"]: WeightInfo((Q,), "ones"), w["uq"]: WeightInfo((H * D, Q)),
               w["uk"]: WeightInfo((H * D, L)), w["uv"]: WeightInfo((H * Dv, L)), w["o"]: WeightInfo((hidden_size, H * Dv))}
        if p.get("own_latent", True):
            out[w["dkv"]] = WeightInfo((L, hidden_size))
            out[w["dkv_norm"]] = WeightInfo((L,), "ones")
        if p.get("sink", False):
            out[w["sink"]] = WeightInfo((H,))
        return out

    def cache_spec(self):
        return CacheSpec("window" if self.window is not None else "full", 1, self.latent_dim, self.window)

    def load_branch(self, get):
        w = self.spec.weights
        H, D, Dv, L = self.num_heads, self.head_dim, self.value_dim, self.latent_dim
        f64 = lambda name: get(w[name]).to(torch.float64)
        dq = get(w["dq"])
        if self.query_rank is None:
            self.query_rank = int(dq.shape[0])
        if get(w["uq"]).shape[1] != self.query_rank or dq.shape[0] != self.query_rank:
            raise ValueError("latent_cache_attention: the two halves of the query projection disagree on its latent's size")
        uq, uk, uv, o = f64("uq").view(H, D, -1), f64("uk").view(H, D, L), f64("uv").view(H, Dv, L), f64("o").view(-1, H, Dv)
        # queries into the latent's space: rows h L .. (h + 1) L are W_uk[h]^T W_uq[h]
        q_fold = torch.einsum("hdl,hdq->hlq", uk, uq).reshape(H * L, -1)
        self.w_q = ops.tile_weight(self._to_device(q_fold))
        # and the heads' sums over the latents back out: columns h L .. (h + 1) L are W_o[:, h] W_uv[h]
        o_fold = torch.einsum("whv,hvl->whl", o, uv).reshape(-1, H * L)
        self.dq_norm_w = self._to_device(get(w["dq_norm"]), torch.float32)
        rows = [dq]
        if self.own_latent:
            rows.append(get(w["dkv"]))
            self.dkv_norm_w = self._to_device(get(w["dkv_norm"]), torch.float32)
        if self.has_sink:
            self.sink_w = self._to_device(get(w["sink"]), torch.float32)
        return torch.cat([self._to_device(t) for t in rows], dim=0).contiguous(), self._to_device(o_fold)

    def run(self, proj, col0, ctx, cache, out, out_col0, scale):
        if cache.writes != self.own_latent:
            raise ValueError("latent_cache_attention: a layer with a latent of its own writes its cache slot, one without reads another's")
        n = proj.shape[0]
        if cache.writes:
            c = ops.rmsnorm_cols(proj, col0 + self.query_rank, self.latent_dim, self.dkv_norm_w, self.norm_eps, cache.k.dtype)
            ops.vector_store(c, ctx.slot_mapping[cache.group], cache.k, cache.v)
        cq = ops.rmsnorm_cols(proj, col0, self.query_rank, self.dq_norm_w, self.norm_eps, self.dtype)
        q = ops.linear(cq, self.w_q, self.dtype).view(n, self.num_heads, self.latent_dim)
        a = ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens, ctx.token_req,
                                self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len, ctx.num_single, sink=self.sink_w)
        ops.sigmoid_gate(a, None, 0, scale, out, out_col0)


register_part("mixer", "latent_cache_attention", LatentCacheAttention)
