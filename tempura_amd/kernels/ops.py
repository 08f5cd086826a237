"""The operations the parts are written against, bound to the gfx950 kernel library.

Every function checks shapes, dtypes, contiguity and device on the host before a
kernel is launched (a kernel never sees an operand it was not written for), then
calls the library's C entry point on the current stream.  There is no CPU path:
without the compiled library or without a GPU the first call raises.

Tests may install another backend with ``set_backend`` (an object with the same
functions) to exercise the engine's bookkeeping on the host; nothing in the
product does.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_F32, _BF16 = 0, 1
_backend = None


def set_backend(backend) -> None:
    """Install an object providing this module's functions (tests only); None restores the library."""
    global _backend
    _backend = backend


class KernelError(RuntimeError):
    pass


class _Library:
    """The compiled kernel library, loaded on first use."""

    _lib = None

    @classmethod
    def get(cls):
        if cls._lib is None:
            if not torch.cuda.is_available():
                raise KernelError("tempura_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
            from ..csrc.build import ensure_built
            path = ensure_built()
            try:
                lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelError(f"cannot load the kernel library {path}: {e}") from e
            lib.tp_last_error.restype = ctypes.c_char_p
            cls._lib = lib
            cls.path = path
        return cls._lib


def library():
    return _Library.get()


class KernelTimer:
    """Times every call into the kernel library made while it is active (``with KernelTimer() as t:``), with a pair
    of events on the current stream around each call: eager steps only (events cannot be recorded into a graph
    that is replayed), and the pairs serialise nothing, so a call's time includes what its kernels wait for.
    ``label`` (settable at any time) is stored with every call; ``table()`` waits for the device and returns
    rows (entry point, label, calls, total microseconds), largest first."""

    def __init__(self):
        self.label = ""
        self._events = []

    def __enter__(self):
        global _timer
        self._before, _timer = _timer, self
        return self

    def __exit__(self, *exc):
        global _timer
        _timer = self._before
        return False

    def table(self, by_label: bool = False):
        torch.cuda.synchronize()
        total = {}
        for name, label, e0, e1 in self._events:
            key = (name, label if by_label else "")
            calls, us = total.get(key, (0, 0.0))
            total[key] = (calls + 1, us + 1e3 * e0.elapsed_time(e1))
        return sorted(((k[0], k[1], c, us) for k, (c, us) in total.items()), key=lambda r: -r[3])


_timer: Optional[KernelTimer] = None


def _call(name: str, *args, tag: Optional[tuple] = None) -> None:
    """``tag``: what distinguishes this call in a ``KernelTimer``'s table (a product's sizes)."""
    lib = _Library.get()
    t = _timer
    if t is not None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(f"{name}: {lib.tp_last_error().decode()}")
    if t is not None:
        e1.record()
        t._events.append((name if tag is None else name + " " + "x".join(map(str, tag)), t.label, e0, e1))


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _F32
    if t.dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"unsupported dtype {t.dtype}")


def _dtcode(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"unsupported dtype {dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream():
    """The current stream's handle (of the current device).  Asked for at every launch: the direct call is
    some 8 us cheaper than ``torch.cuda.current_stream()``, a quarter of an eager launch's host time."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev_ok(*ts) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "operand is not on the GPU")
            _need(t.is_contiguous(), "operand is not contiguous")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    _need(t.dtype == torch.int32 and t.numel() >= n and t.dim() >= 1, f"{what}: need int32 with {n} elements")


# ---------------------------------------------------------------------------------
def embed(tokens: torch.Tensor, table: torch.Tensor, positions: Optional[torch.Tensor] = None,
          inv_freq: Optional[torch.Tensor] = None, streams: int = 1) -> torch.Tensor:
    """int32 [n] , [vocab, hidden] -> float32 [n, hidden]; with ``streams`` > 1, [n, streams * hidden] holding that
    many copies of each row.  With ``inv_freq`` (float64 [ceil(hidden / 2)]) and ``positions`` (int32 [n]) a
    sinusoidal position vector is added: element 2i gets sin(p * inv_freq[i]), element 2i + 1 the cosine."""
    if _backend is not None:
        if inv_freq is None and streams == 1:
            return _backend.embed(tokens, table)
        return _backend.embed(tokens, table, positions, inv_freq, streams)
    _dev_ok(tokens, table, positions, inv_freq)
    n = tokens.numel()
    _i32(tokens, n, "embed tokens")
    _need(table.dim() == 2, "embed: table must be [vocab, hidden]")
    hidden = table.shape[1]
    if inv_freq is None and streams == 1:
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
        _call("tp_embed", _ptr(tokens), _ptr(table), _dt(table), _ptr(out), n, hidden, _stream())
        return out
    _need(streams >= 1, "embed: streams must be positive")
    if inv_freq is not None:
        _need(positions is not None, "embed: positions missing")
        _i32(positions, n, "embed positions") if n else None
        _need(inv_freq.dtype == torch.float64 and inv_freq.numel() == (hidden + 1) // 2, "embed: inv_freq must be float64 [ceil(hidden / 2)]")
    out = torch.empty((n, streams * hidden), dtype=torch.float32, device=table.device)
    _call("tp_embed_pos", _ptr(tokens), _ptr(positions), _ptr(table), _dt(table), _ptr(inv_freq), _ptr(out), n, hidden,
          int(streams), _stream())
    return out


def stream_step(h: torch.Tensor, streams: int, y: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                out_coef: Optional[torch.Tensor] = None, in_coef: Optional[torch.Tensor] = None,
                norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0, out_dtype: Optional[torch.dtype] = None,
                rows: Optional[torch.Tensor] = None, write_back: bool = True) -> Optional[torch.Tensor]:
    """One step of ``streams`` copies of the residual stream, h float32 [n, streams * width], per row:
    with ``y`` (float32 [n, width], a sublayer's output) every stream b becomes sum_a mix[a, b] h[a] + out_coef[b] * y
    (``mix`` float32 [streams, streams], None: identity; ``out_coef`` [streams], None: ones), written back into
    ``h`` when ``write_back``; then, with ``out_dtype``, the result is u = sum_a in_coef[a] h[a] (None: the plain
    sum), normed with ``norm_weight`` (float32 [width]; u / sqrt(mean(u^2) + eps) * weight) when that is given,
    as ``out_dtype`` [n or len(rows), width].  ``rows`` (int32) picks the rows."""
    if _backend is not None:
        return _backend.stream_step(h, streams, y, mix, out_coef, in_coef, norm_weight, eps, out_dtype, rows, write_back)
    _dev_ok(h, y, mix, out_coef, in_coef, norm_weight, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2 and streams >= 1 and h.shape[1] % streams == 0,
          "stream_step: h must be float32 [n, streams * width]")
    n, width = h.shape[0], h.shape[1] // streams
    if y is not None:
        _need(y.dtype == torch.float32 and tuple(y.shape) == (n, width), "stream_step: y must be float32 [n, width]")
    for t, size, what in ((mix, streams * streams, "mix"), (out_coef, streams, "out_coef"), (in_coef, streams, "in_coef"),
                          (norm_weight, width, "norm_weight")):
        if t is not None:
            _need(t.dtype == torch.float32 and t.numel() == size, f"stream_step: {what} must be float32 with {size} elements")
    n_out = n
    if rows is not None:
        n_out = rows.numel()
        _i32(rows, n_out, "stream_step rows") if n_out else None
        _need(not (write_back and y is not None) or out_dtype is None, "stream_step: a step over chosen rows cannot write all streams back")
    out = None
    if out_dtype is not None:
        out = torch.empty((n_out, width), dtype=out_dtype, device=h.device)
        if n_out == 0:
            return out          # (a step in which no row is wanted)
    else:
        _need(y is not None and write_back, "stream_step: nothing to do")
    _call("tp_hc_step", _ptr(h), _ptr(y), _ptr(mix), _ptr(out_coef), _ptr(in_coef), _ptr(norm_weight), ctypes.c_float(eps),
          _ptr(out), _dtcode(out_dtype) if out_dtype is not None else _F32, _ptr(rows), n_out, int(streams), width,
          int(bool(write_back) and y is not None), _stream())
    return out


def scale_(x: torch.Tensor, scale: float) -> torch.Tensor:
    """x *= scale in place (float32)."""
    if _backend is not None:
        return _backend.scale_(x, scale)
    _dev_ok(x)
    _need(x.dtype == torch.float32, "scale_: needs float32")
    _call("tp_scale_f32", _ptr(x), ctypes.c_size_t(x.numel()), ctypes.c_float(scale), _stream())
    return x


def gated_act(gu: torch.Tensor, out_dtype: torch.dtype, slope: float = 1.0, limit: float = 0.0, up_offset: float = 0.0,
              interleaved: bool = False) -> torch.Tensor:
    """[m, 2i] (gate columns then up columns; ``interleaved``: eight gate and eight up columns in turn, the layout of
    ``interleave_gate_up``) -> out_dtype [m, i]: g = min(gate, limit), u = clamp(up, -limit, limit)
    (limit <= 0: none), g * sigmoid(slope * g) * (u + up_offset)."""
    if _backend is not None:
        return _backend.gated_act(gu, out_dtype, slope, limit, up_offset, interleaved)
    _dev_ok(gu)
    _need(gu.dim() == 2 and gu.shape[1] % 2 == 0, "gated_act: input must be [m, 2i]")
    m, i2 = gu.shape
    out = torch.empty((m, i2 // 2), dtype=out_dtype, device=gu.device)
    _call("tp_gated_act", _ptr(gu), _dt(gu), _ptr(out), _dtcode(out_dtype), m, i2 // 2, ctypes.c_float(slope),
          ctypes.c_float(limit), ctypes.c_float(up_offset), int(bool(interleaved)), _stream())
    return out


def qk_store(rows: torch.Tensor, q_bias: Optional[torch.Tensor], k_bias: Optional[torch.Tensor], slots: Optional[torch.Tensor],
             num_heads: int, num_kv_heads: int, head_dim: int, k_cache: Optional[torch.Tensor],
             v_cache: Optional[torch.Tensor], q_dtype: torch.dtype) -> torch.Tensor:
    """float32 rows [n, (heads + kv_heads) * head_dim] of a projection (no rotation): biases (float32, per column)
    are added, q is returned as q_dtype [n, heads, head_dim], k goes to the cache rows ``slots`` of ``k_cache`` and,
    when ``v_cache`` is given (values that are the keys), into the transposed value cache too.  ``slots`` None: the
    rows hold q only."""
    if _backend is not None:
        return _backend.qk_store(rows, q_bias, k_bias, slots, num_heads, num_kv_heads, head_dim, k_cache, v_cache, q_dtype)
    _dev_ok(rows, q_bias, k_bias, slots, k_cache, v_cache)
    _need(rows.dtype == torch.float32 and rows.dim() == 2, "qk_store: rows must be float32 [n, width]")
    n = rows.shape[0]
    width = (num_heads + (num_kv_heads if slots is not None else 0)) * head_dim
    _need(rows.shape[1] == width, f"qk_store: row width {rows.shape[1]} != {width}")
    for b, size in ((q_bias, num_heads * head_dim), (k_bias, num_kv_heads * head_dim)):
        if b is not None:
            _need(b.dtype == torch.float32 and b.numel() == size, "qk_store: bias must be float32, one value per column")
    page_size, cache_dt = 1, _F32
    if slots is not None:
        _i32(slots, n, "slots") if n else None
        _need(k_cache is not None and k_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim,
              "qk_store: k cache must be [pages, kv_heads, page_size, head_dim]")
        page_size, cache_dt = k_cache.shape[2], _dt(k_cache)
        if v_cache is not None:
            _need(tuple(v_cache.shape) == (k_cache.shape[0], num_kv_heads, head_dim, page_size) and v_cache.dtype == k_cache.dtype,
                  "qk_store: v cache must be [pages, kv_heads, head_dim, page_size] of the key cache's type")
    q = torch.empty((n, num_heads, head_dim), dtype=q_dtype, device=rows.device)
    _call("tp_qk_store", _ptr(rows), rows.shape[1], _ptr(q_bias), _ptr(k_bias), _ptr(slots), n, num_heads, num_kv_heads, head_dim,
          _ptr(q), _dtcode(q_dtype), _ptr(k_cache if slots is not None else None), _ptr(v_cache if slots is not None else None),
          cache_dt, page_size, _stream())
    return q


def causal_conv(proj: torch.Tensor, col0: int, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                cu_seqlens: torch.Tensor, token_req: torch.Tensor, state_slots: torch.Tensor, num_requests: int,
                state_off: int = 0, act: bool = True) -> torch.Tensor:
    """Causal convolution per channel over each request's run of tokens, then SiLU (``act`` False: the sums
    themselves).  ``proj`` float32 [n, width] holds the inputs at columns col0 .. col0 + channels; ``weight``
    [taps, channels] (tap-major; the last tap is the current token's), ``bias`` [channels] or None; ``state`` float32
    [slots, row] whose rows hold, from element ``state_off`` on, the carried inputs [taps - 1, channels] (oldest
    first) of the request in that slot: they are read for the first tokens of a run and replaced by the run's last
    inputs.  Returns float32 [n, channels]."""
    if _backend is not None:
        if state_off == 0 and act and bias is not None:
            return _backend.causal_conv(proj, col0, channels, weight, bias, state, cu_seqlens, token_req, state_slots, num_requests)
        return _backend.causal_conv(proj, col0, channels, weight, bias, state, cu_seqlens, token_req, state_slots, num_requests,
                                    state_off, act)
    _dev_ok(proj, weight, bias, state, cu_seqlens, token_req, state_slots)
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and 0 <= col0 and col0 + channels <= proj.shape[1], "causal_conv: bad rows")
    _need(weight.dtype == torch.float32 and weight.dim() == 2 and weight.shape[1] == channels, "causal_conv: weight must be float32 [taps, channels]")
    taps = weight.shape[0]
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == channels), "causal_conv: bias must be float32 [channels]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state_off >= 0 and state.shape[1] >= state_off + (taps - 1) * channels,
          "causal_conv: state rows too short")
    n = proj.shape[0]
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    _i32(token_req, n, "token_req") if n else None
    out = torch.empty((n, channels), dtype=torch.float32, device=proj.device)
    _call("tp_causal_conv", _ptr(proj), proj.shape[1], int(col0), _ptr(weight), _ptr(bias), _ptr(state),
          ctypes.c_size_t(state.shape[1]), ctypes.c_size_t(state_off), _ptr(cu_seqlens), _ptr(token_req), _ptr(state_slots), _ptr(out),
          n, int(num_requests), channels, taps, int(bool(act)), _stream())
    return out


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_col0: int, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
             state: torch.Tensor, state_off: int, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, num_requests: int,
             num_heads: int, head_dim: int, state_size: int, groups: int, max_run: Optional[int] = None) -> torch.Tensor:
    """The selective recurrence per head over each request's run: with dt = softplus(proj[:, dt_col0 + h] + dt_bias[h])
    and a = exp(-exp(a_log[h]) * dt):  S <- a S + dt B x^T,  y = S^T C + d_skip[h] x.  ``xbc`` float32 [n, channels]
    holds x [heads * head_dim] | B [groups * state] | C [groups * state]; the state [heads, state, head_dim] of a
    request lives at ``state[slot, state_off:]`` (float32), is read at the start of the run and left as the run
    leaves it.  ``max_run``: the longest run of the batch (None: the number of rows); long runs are cut into
    pieces that run side by side, which changes rounding only.  Returns y float32 [n, heads * head_dim]."""
    if _backend is not None:
        return _backend.ssm_scan(xbc, proj, dt_col0, dt_bias, a_log, d_skip, state, state_off, cu_seqlens, state_slots,
                                 num_requests, num_heads, head_dim, state_size, groups)
    _dev_ok(xbc, proj, dt_bias, a_log, d_skip, state, cu_seqlens, state_slots)
    inner = num_heads * head_dim
    channels = inner + 2 * groups * state_size
    _need(xbc.dtype == torch.float32 and xbc.dim() == 2 and xbc.shape[1] == channels, f"ssm_scan: xbc must be float32 [n, {channels}]")
    n = xbc.shape[0]
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[0] == n and 0 <= dt_col0 and dt_col0 + num_heads <= proj.shape[1],
          "ssm_scan: bad projection rows")
    for t in (dt_bias, a_log, d_skip):
        _need(t.dtype == torch.float32 and t.numel() == num_heads, "ssm_scan: per-head constants must be float32 [heads]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= state_off + num_heads * state_size * head_dim,
          "ssm_scan: state rows too short")
    _need(num_heads % groups == 0 and state_size <= 2048, "ssm_scan: heads must be a multiple of groups, state size at most 2048")
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    y = torch.empty((n, inner), dtype=torch.float32, device=xbc.device)
    max_run = n if max_run is None else min(int(max_run), n)
    lib = _Library.get()
    lib.tp_ssm_scan_scratch.restype = ctypes.c_size_t
    need = lib.tp_ssm_scan_scratch(int(num_requests), max_run, num_heads, head_dim, state_size, None)
    scratch = torch.empty((need,), dtype=torch.float32, device=xbc.device) if need else None
    _call("tp_ssm_scan", _ptr(xbc), _ptr(proj), proj.shape[1], int(dt_col0), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state),
          ctypes.c_size_t(state.shape[1]), ctypes.c_size_t(state_off), _ptr(cu_seqlens), _ptr(state_slots), _ptr(y),
          int(num_requests), num_heads, head_dim, state_size, groups, max_run, _ptr(scratch), ctypes.c_size_t(need), _stream())
    return y


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_col0: int, weight: torch.Tensor, eps: float, groups: int,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """v = y * silu(proj[:, z_col0 + j]), normed in ``groups`` equal parts (each by its own root mean square, eps
    inside the root), times ``weight``; float32 in, ``out_dtype`` [n, inner] out."""
    if _backend is not None:
        return _backend.gated_group_norm(y, proj, z_col0, weight, eps, groups, out_dtype)
    _dev_ok(y, proj, weight)
    _need(y.dtype == torch.float32 and y.dim() == 2, "gated_group_norm: y must be float32 [n, inner]")
    n, inner = y.shape
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[0] == n and 0 <= z_col0 and z_col0 + inner <= proj.shape[1],
          "gated_group_norm: bad projection rows")
    _need(weight.dtype == torch.float32 and weight.numel() == inner and groups > 0 and inner % groups == 0, "gated_group_norm: bad weight or groups")
    out = torch.empty((n, inner), dtype=out_dtype, device=y.device)
    _call("tp_gated_group_norm", _ptr(y), _ptr(proj), proj.shape[1], int(z_col0), _ptr(weight), ctypes.c_float(eps), _ptr(out),
          _dtcode(out_dtype), n, inner, int(groups), _stream())
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None, groups: int = 1) -> torch.Tensor:
    """float32 [n, hidden] -> out_dtype [n or len(rows), hidden].  ``groups`` > 1: the row is split into that many
    equal consecutive parts and each is divided by its own root mean square."""
    if _backend is not None:
        if groups != 1:
            return _backend.rmsnorm(h, weight, eps, out_dtype, rows, groups)
        return _backend.rmsnorm(h, weight, eps, out_dtype, rows)
    _dev_ok(h, weight, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2, "rmsnorm: input must be float32 [n, hidden]")
    _need(weight.dtype == torch.float32 and weight.numel() == h.shape[1], "rmsnorm: weight must be float32 [hidden]")
    n_out = h.shape[0]
    if rows is not None:
        n_out = rows.numel()
        _i32(rows, n_out, "rmsnorm rows") if n_out else None
    out = torch.empty((n_out, h.shape[1]), dtype=out_dtype, device=h.device)
    if groups != 1:
        _need(groups > 0 and h.shape[1] % groups == 0, "rmsnorm: groups must divide the row")
        _call("tp_group_rmsnorm", _ptr(h), ctypes.c_size_t(h.shape[1]), 0, _ptr(weight), _ptr(rows), _ptr(out), _dtcode(out_dtype),
              n_out, h.shape[1], int(groups), ctypes.c_float(eps), _stream())
        return out
    _call("tp_rmsnorm", _ptr(h), _ptr(weight), _ptr(rows), _ptr(out), _dtcode(out_dtype), n_out, h.shape[1],
          ctypes.c_float(eps), _stream())
    return out


#: bfloat16 products may use the matrix-core kernels (tests switch this off to grade the general kernel)
allow_mfma = True


#: a gate with constants of its own runs in the product's epilogue from this many rows on (the products of fewer
#: rows stream the weights once and have the plain gated SiLU only)
gated_epilogue_rows = 17


def gated_layout_ok(n_rows: int, k: int) -> bool:
    """Whether ``linear_swiglu`` takes a weight of 2 * n_rows rows and k columns."""
    return n_rows % 8 == 0 and k % 32 == 0


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[i, k], [i, k] -> [2i, k] with eight gate rows and eight up rows in turn, the layout
    ``linear_swiglu`` reads."""
    i, k = gate.shape
    return torch.stack([gate.reshape(i // 8, 8, k), up.reshape(i // 8, 8, k)], dim=1).reshape(2 * i, k).contiguous()


class Prenormed:
    """Rows whose root-mean-square norm is finished by the product that consumes them: ``x`` is
    bfloat16(h * norm weight) [m, k]; ``ss`` [ceil(k / 16), 16] float32 holds, per block of 16 columns
    and row, the sum of squares of h; the consumer multiplies its float32 result rows by
    rsqrt(sum(ss) / k + eps).  Made by ``linear(..., residual=h, next_norm=(weight, eps))``."""
    __slots__ = ("x", "ss", "eps", "blocked")

    def __init__(self, x, ss, eps, blocked=None):
        self.x, self.ss, self.eps = x, ss, float(eps)
        #: None: ``x`` is row-major [m, k]; (m, k): ``x`` is stored k-blocked, [k / 8, m, 8] (see ``KBlocked``)
        self.blocked = blocked

    @property
    def shape(self):
        return self.x.shape if self.blocked is None else self.blocked

    def rows(self):
        """``x`` as a row-major [m, k] tensor (a copy when it is stored k-blocked)."""
        if self.blocked is None:
            return self.x
        m, k = self.blocked
        return self.x.permute(1, 0, 2).reshape(m, k)


class KBlocked:
    """bfloat16 activations of at most 16 rows stored k-blocked, ``data`` [k / 8, m, 8]: eight consecutive
    columns of all rows side by side.  A product of a few rows that reads its activations straight from
    global memory then fetches neighbouring bytes instead of short pieces of several rows.  Made by
    ``linear_swiglu(..., blocked_out=True)``, taken by ``linear``."""
    __slots__ = ("data", "rows", "width")

    def __init__(self, data, rows, width):
        self.data, self.rows, self.width = data, rows, width

    @property
    def shape(self):
        return (self.rows, self.width)

    def row_major(self) -> torch.Tensor:
        return self.data.permute(1, 0, 2).reshape(self.rows, self.width).contiguous()


class TiledWeight:
    """A bfloat16 weight [n, k] (n % 16 == 0, k % 64 == 0) stored tiled, ``data`` [n / 16, k / 32, 64, 8]: the block
    of rows 16 i.. and columns 32 j.. as 1,024 contiguous bytes in the matrix cores' operand order, lane l = (column
    group l / 16, row l % 16) holding eight consecutive columns.  The products read it with whole-cache-line loads
    where the row-major form makes a wave fetch 64-byte pieces of sixteen rows.  Made by ``tile_weight``; taken by
    ``linear``, ``linear_swiglu`` and ``linear_rope_kv``."""
    __slots__ = ("data", "n", "k")

    def __init__(self, data, n, k):
        self.data, self.n, self.k = data, n, k

    @property
    def shape(self):
        return (self.n, self.k)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def dim(self) -> int:
        return 2

    def rows(self, lo: int, hi: int) -> "TiledWeight":
        """Rows lo..hi (multiples of 16) as a weight of their own; no copy."""
        _need(lo % 16 == 0 and hi % 16 == 0 and 0 <= lo < hi <= self.n, f"tiled weight: rows {lo}..{hi} of {self.n}")
        return TiledWeight(self.data[lo // 16: hi // 16], hi - lo, self.k)

    def row_major(self) -> torch.Tensor:
        """The plain [n, k] tensor (a copy)."""
        return self.data.view(self.n // 16, self.k // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(self.n, self.k).contiguous()


#: weights that fit are stored tiled (False, or TEMPURA_TILE_WEIGHTS=0 in the environment: every weight stays row-major)
tile_weights = os.environ.get("TEMPURA_TILE_WEIGHTS", "1") != "0"


def tile_weight(w: torch.Tensor):
    """A weight [n, k] for the products: ``TiledWeight`` when it is bfloat16 on the GPU with n % 16 == 0 and
    k % 64 == 0 and the matrix-core kernels are in use, else ``w`` itself.  No value changes."""
    if not (tile_weights and _backend is None and allow_mfma and isinstance(w, torch.Tensor) and w.is_cuda
            and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 16 == 0 and w.shape[1] % 64 == 0):
        return w
    n, k = w.shape
    data = w.view(n // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(n // 16, k // 32, 64, 8)
    return TiledWeight(data, n, k)


def weight_rows(w, lo: int, hi: int):
    """Rows lo..hi of a weight, tiled or not, without a copy."""
    return w.rows(lo, hi) if isinstance(w, TiledWeight) else w[lo:hi]


def _w_args(w):
    """(tensor whose memory the kernel reads, layout bit) of a weight."""
    if isinstance(w, TiledWeight):
        return w.data, 4
    return w, 0


class Partials:
    """The float32 partial sums [splits, m, n] of a product whose K was split over blocks, not yet added:
    the kernel that consumes the rows adds them (in ascending order), which saves the reduction kernel.
    Made by ``linear(..., partial_ok=True)``, taken by ``rope_kv_write``."""
    __slots__ = ("data",)

    def __init__(self, data):
        self.data = data

    @property
    def shape(self):
        return tuple(self.data.shape[1:])


def split_norm_ok(m: int, width: int, dtype: torch.dtype) -> bool:
    """Whether the product before a norm over ``width`` columns of ``m`` rows can carry it (``linear`` with
    ``next_norm``): up to 16 rows the two products around the norm share it; with more rows the kernel that
    adds the product's partial sums into the residual stream also norms the rows, where the product splits K
    (``linear`` says whether it did)."""
    if _backend is not None:
        return _backend.split_norm_ok(m, width, dtype)
    return allow_mfma and dtype == torch.bfloat16 and 0 < m and width % 32 == 0


def _pre_args(x):
    """(the tensor a product reads, the arguments of its row scale, its rows and columns, layout bit 1 when the
    tensor is k-blocked) of plain rows or of ``Prenormed`` rows."""
    if isinstance(x, Prenormed):
        _dev_ok(x.x, x.ss)
        m, k = x.shape
        _need(x.x.dtype == torch.bfloat16 and x.ss.dtype == torch.float32 and x.x.numel() == m * k and
              tuple(x.ss.shape) == ((k + 15) // 16, 16), "linear: malformed handed-over rows")
        return x.x, (_ptr(x.ss), x.ss.shape[0], ctypes.c_float(x.eps)), (m, k), (1 if x.blocked is not None else 0)
    return x, (_ptr(None), 0, ctypes.c_float(0.0)), (tuple(x.shape) if x.dim() == 2 else None), 0


def linear_swiglu(x, w: torch.Tensor, blocked_out: bool = False, slope: float = 1.0, limit: float = 0.0, up_offset: float = 0.0):
    """bfloat16 x [m, k] (or ``Prenormed``), interleaved gate/up weight [2i, k] -> bfloat16 [m, i] =
    silu(x g^T) * (x u^T), the gate applied to the float32 accumulators (no rounding in between).
    With ``blocked_out`` the result comes as ``KBlocked`` when there are at most 16 rows and i % 32 == 0 (else as a tensor).
    ``slope``, ``limit``, ``up_offset``: the general gate of ``gated_act`` (g' * sigmoid(slope g') * (u' + up_offset)
    with both branches limited when limit > 0) in the same epilogue; the defaults are SwiGLU.  The products of at
    most 16 rows have the default gate only (``gated_epilogue_rows``)."""
    if _backend is not None:
        if (slope, limit, up_offset) != (1.0, 0.0, 0.0):
            return _backend.linear_swiglu(x, w, blocked_out, slope, limit, up_offset)
        return _backend.linear_swiglu(x, w, blocked_out) if blocked_out else _backend.linear_swiglu(x, w)
    x, pre, mk, xl = _pre_args(x)
    wd, wl = _w_args(w)
    _dev_ok(x, wd)
    _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear_swiglu: shapes {mk} x {tuple(w.shape)}")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "linear_swiglu: operands must be bfloat16")
    m, k = mk
    n = w.shape[0]
    _need(n % 16 == 0 and k % 32 == 0, "linear_swiglu: needs 2i % 16 == 0 and k % 32 == 0")
    # (the product that takes such rows is an MFMA kernel over K in steps of 32)
    blocked_out = blocked_out and allow_mfma and 0 < m <= 16 and (n // 2) % 32 == 0
    if blocked_out:
        out = KBlocked(torch.empty((n // 16, m, 8), dtype=torch.bfloat16, device=x.device), m, n // 2)
    else:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    scratch, nscratch = _splitk_scratch(x, m, n)
    _call("tp_linear_fused", _ptr(x), _ptr(wd), _BF16, _ptr(out.data if blocked_out else out), _BF16, 2, m, n, k, 1,
          _ptr(scratch), ctypes.c_size_t(nscratch), *pre, _ptr(None), _ptr(None), _ptr(None), (2 if blocked_out else 0) | wl | xl,
          0, _ptr(None), ctypes.c_float(slope), ctypes.c_float(limit), ctypes.c_float(up_offset), _stream(), tag=(m, n, k))
    return out


def _splitk_scratch(x: torch.Tensor, m: int, n: int):
    """Room for the partial sums of a bfloat16 product whose K is split over blocks: products of 17..128
    rows (64-row blocks up to 64 rows, 128-row blocks above), and larger ones with too few result tiles (256 x 128)
    to give every CU work."""
    if x.dtype != torch.bfloat16 or m <= 16:
        return None, 0
    if m <= 128:
        splits = min(16, max(1, -(-512 // (-(-n // 128) * -(-m // 64)))))
    else:
        tiles = -(-m // 256) * -(-n // 128)
        if tiles >= 128:
            return None, 0
        splits = min(16, 2 * -(-256 // tiles))      # (room for the library to choose: it prices the candidates)
    count = splits * m * n
    return torch.empty((count,), dtype=torch.float32, device=x.device), count


def linear(x, w: torch.Tensor, out_dtype: torch.dtype, residual: Optional[torch.Tensor] = None, next_norm=None,
           partial_ok: bool = False):
    """x [m, k] (or ``Prenormed`` / ``KBlocked``) @ w[n, k]^T -> out_dtype [m, n]; with ``residual`` (float32
    [m, n]) the product is added into it in place and it is returned.
    With ``next_norm`` = (float32 weight [n], eps) (needs ``residual``) the result is the pair (residual, rows
    for the part behind that norm): ``Prenormed`` rows up to 16 rows of bfloat16, the normed rows themselves
    from 17 rows on when the product's K was split (one kernel adds the partial sums into the residual and norms
    it), or None when the norm has to run on its own.
    With ``partial_ok`` (float32 output, no residual) the result may be ``Partials``."""
    if _backend is not None:
        if next_norm is not None:
            return _backend.linear(x, w, out_dtype, residual, next_norm)
        return _backend.linear(x, w, out_dtype, residual)
    layout = 0
    wd, wl = _w_args(w)
    if isinstance(x, KBlocked):
        _need(allow_mfma and x.data.dtype == torch.bfloat16 and tuple(x.data.shape) == (x.width // 8, x.rows, 8)
              and x.width % 32 == 0, "linear: malformed k-blocked rows")
        kb, layout = x, 1
        x, pre = x.data, (_ptr(None), 0, ctypes.c_float(0.0))
        m, k = kb.rows, kb.width
        _dev_ok(x, wd, residual)
        _need(w.dim() == 2 and w.shape[1] == k and w.dtype == torch.bfloat16, f"linear: shapes {(m, k)} x {tuple(w.shape)}")
    else:
        x, pre, mk, layout = _pre_args(x)
        _dev_ok(x, wd, residual)
        _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear: shapes {mk} x {tuple(w.shape)}")
        _need(x.dtype == w.dtype, f"linear: operand dtypes differ ({x.dtype}, {w.dtype})")
        m, k = mk
    n = w.shape[0]
    if residual is not None:
        _need(residual.dtype == torch.float32 and tuple(residual.shape) == (m, n), "linear: residual must be float32 [m, n]")
        out, acc = residual, 1
    else:
        out, acc = torch.empty((m, n), dtype=out_dtype, device=x.device), 0
    post, handed = (_ptr(None), _ptr(None), _ptr(None)), None
    if next_norm is not None and split_norm_ok(m, n, x.dtype) and k % 32 == 0 and m <= 16:
        weight, eps = next_norm
        _dev_ok(weight)
        _need(residual is not None, "linear: next_norm needs a residual")
        _need(weight.dtype == torch.float32 and weight.numel() == n, "linear: norm weight must be float32 [n]")
        # (the rows go on k-blocked where the consumer can read them so: a product of a few rows then takes its
        # activations straight from memory as operands instead of staging them through LDS)
        hand_blocked = handoff_blocked and n % 32 == 0
        handed = Prenormed(torch.empty((n // 8, m, 8) if hand_blocked else (m, n), dtype=torch.bfloat16, device=x.device),
                           torch.empty(((n + 15) // 16, 16), dtype=torch.float32, device=x.device), eps,
                           (m, n) if hand_blocked else None)
        post = (_ptr(weight), _ptr(handed.x), _ptr(handed.ss))
        if hand_blocked:
            layout |= 8
    scratch, nscratch = _splitk_scratch(x, m, n) if allow_mfma else (None, 0)
    # from 17 rows on: the partial sums of a split K may stay unadded for the kernel that consumes the rows
    layout |= wl
    defer = scratch is not None and 16 < m and (layout & 3) == 0 and \
        ((next_norm is not None and residual is not None and split_norm_ok(m, n, x.dtype) and n % 4 == 0 and n <= 16384) or
         (partial_ok and residual is None and out_dtype == torch.float32))
    splits = ctypes.c_int(1)
    _call("tp_linear_fused", _ptr(x), _ptr(wd), _dt(x), _ptr(out), _dt(out), acc, m, n, k, int(allow_mfma), _ptr(scratch),
          ctypes.c_size_t(nscratch), *pre, *post, layout, int(defer), ctypes.byref(splits), ctypes.c_float(1.0),
          ctypes.c_float(0.0), ctypes.c_float(0.0), _stream(), tag=(m, n, k))
    if defer and splits.value > 1:
        if next_norm is None:
            return Partials(scratch[: splits.value * m * n].view(splits.value, m, n))
        weight, eps = next_norm
        _dev_ok(weight)
        _need(weight.dtype == torch.float32 and weight.numel() == n, "linear: norm weight must be float32 [n]")
        normed = torch.empty((m, n), dtype=x.dtype, device=x.device)
        _call("tp_splitk_add_rmsnorm", _ptr(scratch), splits.value, _ptr(residual), _ptr(weight), ctypes.c_float(eps),
              _ptr(normed), _dt(normed), m, n, _stream())
        return out, normed
    return out if next_norm is None else (out, handed)


#: rows handed from one product to the next with a norm between them travel k-blocked (up to 16 rows)
handoff_blocked = True
#: long steps may rotate and store in the projection's epilogue too (False: only the few rows of decoding)
rope_in_long_products = True


def linear_rope_ok(m: int, n: int, k: int, head_dim: int, rotary_dim: int, page_size: int, x_dtype: torch.dtype,
                   cache_dtype: torch.dtype, prenormed: bool = False) -> bool:
    """Whether ``linear_rope_kv`` takes a projection of m rows onto n columns: a few rows (decoding), or a long
    step with enough result tiles (128 x 128) to give half the CUs work without splitting K, heads of a multiple of 64."""
    if not (_backend is None and allow_mfma and x_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16):
        return False
    if 0 < m <= 16:
        return k % 32 == 0 and head_dim % 16 == 0
    tiles = -(-m // 128) * -(-n // 128)      # (of 128 x 128, the smallest blocks of the pipelined products)
    return (rope_in_long_products and m > 128 and tiles >= 128 and k % 64 == 0 and 255 * k * 2 + 128 < 2 ** 31 and head_dim % 64 == 0
            and rotary_dim % 8 == 0 and page_size % 8 == 0 and not prenormed)


def linear_rope_kv(x, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, inv_freq: Optional[torch.Tensor],
                   rotary_dim: int, factor: float, num_heads: int, num_kv_heads: int, head_dim: int,
                   k_cache: torch.Tensor, v_cache: torch.Tensor, cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The q/k/v projection of bfloat16 rows (at most 16, also ``Prenormed``; or a long step, see
    ``linear_rope_ok``) with the rotation and the cache write in its epilogue: the same result as ``linear``
    to float32 followed by ``rope_kv_write`` (w's q and k heads in paired order), without the kernel and the
    rows in between.  Returns q as bfloat16 [m, heads, head_dim]."""
    x, pre, mk, xl = _pre_args(x)
    wd, wl = _w_args(w)
    _dev_ok(x, wd, positions, slots, inv_freq, k_cache, v_cache)
    _need(mk is not None and w.dim() == 2 and mk[1] == w.shape[1], f"linear_rope_kv: shapes {mk} x {tuple(w.shape)}")
    m, k = mk
    n = w.shape[0]
    _need(linear_rope_ok(m, n, k, head_dim, rotary_dim, k_cache.shape[2] if k_cache.dim() == 4 else 0, x.dtype, k_cache.dtype,
                         pre[1] != 0) and w.dtype == torch.bfloat16,
          "linear_rope_kv: sizes or dtypes that the fused projection does not take (see linear_rope_ok)")
    _need(m <= 16 or cos_sin is not None, "linear_rope_kv: a long step needs the table of cosines and sines")
    _need(n == (num_heads + 2 * num_kv_heads) * head_dim, f"linear_rope_kv: {n} weight rows for {num_heads} + 2 x {num_kv_heads} heads of {head_dim}")
    _i32(positions, m, "positions")
    _i32(slots, m, "slots")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim
          and tuple(v_cache.shape) == (k_cache.shape[0], k_cache.shape[1], k_cache.shape[3], k_cache.shape[2])
          and v_cache.dtype == torch.bfloat16,
          "linear_rope_kv: caches must be k [pages, kv_heads, page_size, head_dim], v [pages, kv_heads, head_dim, page_size]")
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
              "linear_rope_kv: inv_freq must be float64 [rotary_dim / 2]")
    if cos_sin is not None:
        _dev_ok(cos_sin)
        _need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and tuple(cos_sin.shape) == (m, rotary_dim // 2, 2),
              "linear_rope_kv: table must be float32 [m, rotary_dim / 2, 2]")
    q = torch.empty((m, num_heads, head_dim), dtype=torch.bfloat16, device=x.device)
    _call("tp_linear_rope", _ptr(x), _ptr(wd), int(wl != 0) | (2 if xl else 0), m, n, k, *pre, _ptr(positions), _ptr(slots), _ptr(inv_freq), rotary_dim,
          ctypes.c_float(factor), num_heads, num_kv_heads, head_dim, _ptr(q), _ptr(k_cache), _ptr(v_cache),
          k_cache.shape[2], _ptr(cos_sin), _stream(), tag=(m, n, k))
    return q


def rope_kv_write(qkv, positions: torch.Tensor, slots: Optional[torch.Tensor],
                  inv_freq: Optional[torch.Tensor], rotary_dim: int, factor: float, num_heads: int,
                  num_kv_heads: int, head_dim: int, k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor], q_dtype: torch.dtype,
                  cos_sin: Optional[torch.Tensor] = None, value_dim: Optional[int] = None,
                  pad_dim: Optional[int] = None) -> torch.Tensor:
    """Rotate q and k of float32 rows [n, (heads + 2 kv_heads) * head_dim] (or the ``Partials`` of the
    projection that makes them), store k and v into the cache rows ``slots`` and return q as q_dtype
    [n, heads, head_dim].  With ``slots`` None the rows hold q only and nothing is stored.
    ``value_dim``: the size of a value head when it is not head_dim (the rows are then
    [n, (heads + kv_heads) * head_dim + kv_heads * value_dim], the value cache [pages, kv_heads, value_dim, page_size]).
    ``pad_dim`` (>= head_dim): q comes back as [n, heads, pad_dim] and the key cache has heads of pad_dim, zeros
    behind each head's own elements (scores are unchanged; attention kernels that want keys as wide as values then serve).
    The q and k heads are in PAIRED order: elements (2 d, 2 d + 1) of a head rotate together by the angle
    of pair d (they are elements (d, d + rotary_dim / 2) of the split-half order).
    ``cos_sin``: this step's table from ``rope_table`` (the same values, computed once for all layers)."""
    vd = head_dim if value_dim is None else int(value_dim)
    od = head_dim if pad_dim is None else int(pad_dim)
    if _backend is not None:
        if vd != head_dim or od != head_dim:
            return _backend.rope_kv_write(qkv, positions, slots, inv_freq, rotary_dim, factor, num_heads,
                                          num_kv_heads, head_dim, k_cache, v_cache, q_dtype, value_dim=vd, pad_dim=od)
        return _backend.rope_kv_write(qkv, positions, slots, inv_freq, rotary_dim, factor, num_heads,
                                      num_kv_heads, head_dim, k_cache, v_cache, q_dtype)
    splits = 1
    if isinstance(qkv, Partials):
        splits, qkv = qkv.data.shape[0], qkv.data.view(-1, qkv.data.shape[2])[: qkv.data.shape[1]]
        _need(qkv.is_contiguous() or splits == 1, "rope_kv_write: malformed partial sums")
    _dev_ok(positions, slots, inv_freq, k_cache, v_cache)
    _need(qkv.is_cuda, "operand is not on the GPU")
    _need(qkv.dtype == torch.float32 and qkv.dim() == 2, "rope_kv_write: rows must be float32 [n, width]")
    n = qkv.shape[0]
    width = (num_heads + (num_kv_heads if slots is not None else 0)) * head_dim + (num_kv_heads * vd if slots is not None else 0)
    _need(qkv.shape[1] == width, f"rope_kv_write: row width {qkv.shape[1]} != {width}")
    _i32(positions, n, "positions") if n else None
    page_size, cache_dt = 1, _F32
    if slots is not None:
        _i32(slots, n, "slots") if n else None
        _need(k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4
              and tuple(v_cache.shape) == (k_cache.shape[0], k_cache.shape[1], vd, k_cache.shape[2]),
              "rope_kv_write: caches must be k [pages, kv_heads, page_size, head_dim], v [pages, kv_heads, value_dim, page_size]")
        _need(k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == od, "rope_kv_write: cache layout mismatch")
        _need(k_cache.dtype == v_cache.dtype, "rope_kv_write: cache dtypes differ")
        page_size, cache_dt = k_cache.shape[2], _dt(k_cache)
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
              "rope_kv_write: inv_freq must be float64 [rotary_dim / 2]")
    if cos_sin is not None:
        _need(cos_sin.is_cuda and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and tuple(cos_sin.shape) == (n, rotary_dim // 2, 2), "rope_kv_write: table must be float32 [n, rotary_dim / 2, 2]")
    _need(od >= head_dim and od % 2 == 0, "rope_kv_write: pad_dim must be even and at least head_dim")
    q = torch.empty((n, num_heads, od), dtype=q_dtype, device=qkv.device)
    _call("tp_rope_kv_write", _ptr(qkv), qkv.shape[1], _ptr(positions), _ptr(slots), _ptr(inv_freq), rotary_dim,
          ctypes.c_float(factor), n, num_heads, num_kv_heads, head_dim, _ptr(q), _dtcode(q_dtype),
          _ptr(k_cache), _ptr(v_cache), cache_dt, page_size, splits, _ptr(cos_sin), vd, od, _stream())
    return q


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, rotary_dim: int, factor: float) -> torch.Tensor:
    """float32 [n, rotary_dim / 2, 2]: cosine and sine (times factor) of every token's angles, as
    ``rope_kv_write`` would compute them itself."""
    if _backend is not None:
        return None
    _dev_ok(positions, inv_freq)
    n = positions.numel()
    _i32(positions, n, "positions") if n else None
    _need(rotary_dim > 0 and inv_freq.dtype == torch.float64 and inv_freq.numel() == rotary_dim // 2,
          "rope_table: inv_freq must be float64 [rotary_dim / 2]")
    table = torch.empty((n, rotary_dim // 2, 2), dtype=torch.float32, device=positions.device)
    _call("tp_rope_table", _ptr(positions), _ptr(inv_freq), rotary_dim, ctypes.c_float(factor), n, _ptr(table), _stream())
    return table


#: bfloat16 attention may use the matrix-core kernels
allow_fast_attention = True
#: the split decode kernel aims at this many blocks (of four waves) in flight
decode_target_blocks = 256


def decode_rows_padded(rows: int) -> int:
    """The number of rows a decode step of `rows` requests is sized for: the next power of two up to 128, beyond
    that the next multiple of 128.  A captured step has that many rows and an eager one chooses its kernels and
    splits as if it had, so the two give the same bits."""
    if rows > 128:
        return (rows + 127) // 128 * 128
    padded = 1
    while padded < rows:
        padded *= 2
    return padded
#: and at least this many splits while a split has at most 64 blocks
decode_min_splits = 8
#: measurements: this many splits whatever the batch (0: chosen by the rules below)
decode_force_splits = 0
#: portions of prompts with fewer query blocks than this have their keys split over blocks (1: never)
portion_target_blocks = 1024
#: in parts of at least this many keys
portion_min_keys = 1024
#: and only while the partial results stay below this many bytes
portion_scratch_limit = 256 << 20


def fast_attention_takes(has_sink: bool, keep_first: int) -> bool:
    """Whether the matrix-core attention kernels take a softmax with a sink and kept first keys (else the general
    kernel runs, and no splits or partial results are prepared for them): both (kept first keys by the kernels that
    load keys and values per wave, whose portions are never split over blocks)."""
    return True


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    cu_seqlens: torch.Tensor, context_lens: torch.Tensor, token_req: torch.Tensor,
                    scale: float, window: int, max_q_len: int, max_context_len: int,
                    num_single: Optional[int] = None, dist_bias: Optional[torch.Tensor] = None,
                    sink: Optional[torch.Tensor] = None, keep_first: int = 0) -> torch.Tensor:
    """q [n, heads, head_dim] over k [pages, kv_heads, page_size, head_dim] and transposed
    v [pages, kv_heads, value_dim, page_size] -> [n, heads * value_dim] (value_dim is the value cache's own; the
    matrix-core kernels take value_dim == head_dim, other sizes run the general kernel).
    ``dist_bias`` (float32 [heads, L]): added to the scaled score of a query at position p and a key at j as
    dist_bias[head, min(p - j, L - 1)].
    ``sink`` (float32 [heads]): the softmax's denominator holds one more term, exp(sink[head]), without key or value.
    ``keep_first``: under a window, the request's first ``keep_first`` keys stay visible as well."""
    if _backend is not None:
        if sink is not None or keep_first:
            return _backend.paged_attention(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens,
                                            token_req, scale, window, max_q_len, max_context_len, dist_bias=dist_bias,
                                            sink=sink, keep_first=keep_first)
        if dist_bias is not None:
            return _backend.paged_attention(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens,
                                            token_req, scale, window, max_q_len, max_context_len, dist_bias=dist_bias)
        return _backend.paged_attention(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens,
                                        token_req, scale, window, max_q_len, max_context_len)
    # num_single: requests that bring exactly one token (None: all of them iff max_q_len == 1, else unknown
    # and every request is treated as a portion).
    _dev_ok(q, k_cache, v_cache, block_tables, cu_seqlens, context_lens, token_req)
    _need(q.dim() == 3 and k_cache.dim() == 4 and v_cache.dim() == 4, "paged_attention: bad operand ranks")
    n, heads, d = q.shape
    pages, kvh, page_size, d2 = k_cache.shape
    vd = v_cache.shape[2]
    _need(tuple(v_cache.shape) == (pages, kvh, vd, page_size), "paged_attention: v cache must be [pages, kv_heads, value_dim, page_size]")
    _need(d == d2, "paged_attention: head_dim of q and cache differ")
    _need(q.dtype == k_cache.dtype == v_cache.dtype, "paged_attention: q and cache dtypes differ")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32, "paged_attention: block_tables must be int32 [r, width]")
    r, width = block_tables.shape
    _i32(cu_seqlens, r + 1, "cu_seqlens")
    _i32(context_lens, r, "context_lens")
    _i32(token_req, n, "token_req") if n else None
    _need(pages * kvh * page_size < 2 ** 31, "paged_attention: cache pool too large for 32-bit row indices")
    _need(max_context_len <= width * page_size, "paged_attention: block table narrower than the longest context")
    out = torch.empty((n, heads * vd), dtype=q.dtype, device=q.device)
    if num_single is None:
        num_single = r if max_q_len == 1 else 0
    _need(0 <= num_single <= r, "paged_attention: num_single out of range")
    if dist_bias is not None:
        _dev_ok(dist_bias)
        _need(dist_bias.dtype == torch.float32 and dist_bias.dim() == 2 and dist_bias.shape[0] == heads and dist_bias.shape[1] > 0,
              "paged_attention: dist_bias must be float32 [heads, L]")
    if sink is not None:
        _dev_ok(sink)
        _need(sink.dtype == torch.float32 and sink.numel() == heads, "paged_attention: sink must be float32 [heads]")
    _need(keep_first >= 0, "paged_attention: keep_first must be >= 0")
    if not window:
        keep_first = 0
    fast = allow_fast_attention and q.dtype == torch.bfloat16 and d % 32 == 0 and d <= 128 and page_size % 8 == 0 and vd == d
    fast = fast and fast_attention_takes(sink is not None, keep_first) and not (keep_first and dist_bias is not None)
    splits, scratch = 1, None
    if fast and num_single > 0:
        # enough blocks to fill 256 CUs, but at least 128 keys per block
        blocks_per_split = decode_rows_padded(num_single) * kvh * ((heads // kvh + 15) // 16)
        # (two blocks fit a CU, 512 the chip.  From 65 to 256 blocks per split, as many splits as fill it once: measured
        # alone at 2,100 keys, 16 requests 35.8 -> 33.5 us, 20 requests 47.2 -> 38.5, 32 requests 54.3 -> 52.7, and more
        # for contexts that differ; through the engine 16 requests of the 8B shape 4.33 -> 4.25 ms a step, 32 requests
        # 5.27 -> 5.20; 12 requests in five splits against three 4.11 / 4.27, 20 in three against two 4.77 / 4.92, 24 in
        # two against three 4.97 / 5.21.)
        if blocks_per_split <= 64:
            want = -(-decode_target_blocks // blocks_per_split)
        elif blocks_per_split <= decode_target_blocks:
            want = max(1, 2 * decode_target_blocks // blocks_per_split)
        else:
            # (more blocks than half the chip's places: no split.  Through the engine, requests of 2,048+ keys of the 8B
            # shape, one split against two: 36 requests 6.06 / 5.97 ms a step, 40: 6.14 / 6.04, 48: 6.27 / 6.49,
            # 56: 6.42 / 6.68, 64: 6.62 / 6.89; three splits at 36 and 40 requests, which the kernel timed alone
            # prefers, 6.07 and 6.13)
            want = 1
        if blocks_per_split <= 64:
            want = max(want, decode_min_splits)     # (batch 8 of the 8B shape: eight splits 3.87 ms a step, four 3.94)
        if decode_force_splits > 0:
            want = decode_force_splits
        # (at least 128 keys a split, by the longest context rounded up to a power of two from 256: a step captured
        # for a bound on the context and an eager step at the actual length then cut alike and give the same bits)
        bound = 256
        while bound < max_context_len:
            bound *= 2
        splits = max(1, min(64, want, bound // 128))
        if splits > 1:
            scratch = torch.empty((r * heads * splits * (d + 2),), dtype=torch.float32, device=q.device)
    parts, part_scratch = 1, None
    # (the kernel with a distance bias does not split a portion's keys)
    if fast and dist_bias is None and not keep_first and num_single < r and d in (32, 64, 128) and page_size & (page_size - 1) == 0 and page_size >= max(8, 512 // d):
        # Few query blocks under a long context (a portion of a prompt behind a long cached prefix): the keys of
        # every portion are split over blocks until the chip is full (T = 512 behind 7,680 keys: 219 -> 137 us).
        q_blocks = -(-(n - num_single) // 32) + (r - num_single)
        blocks = q_blocks * kvh * ((heads // kvh + 3) // 4)
        # (a query block is split into at most as many parts as it has portion_min_keys keys: the short blocks
        # of a prompt from an empty cache stay whole)
        parts = max(1, min(16, portion_target_blocks // blocks, max_context_len // portion_min_keys, 65535 // r))
        if parts > 1 and n * heads * parts * (d + 4) * 4 > portion_scratch_limit:
            parts = 1
        if parts > 1:
            part_scratch = torch.empty((n * heads * parts * (d + 4),), dtype=torch.float32, device=q.device)
    _call("tp_paged_attention", _ptr(q), _dt(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables), width,
          _ptr(cu_seqlens), _ptr(context_lens), _ptr(token_req), _ptr(out), n, r, heads, kvh, d, page_size,
          ctypes.c_float(scale), int(window), int(max_q_len), int(max_context_len), int(fast),
          int(num_single), int(splits), _ptr(scratch), int(parts), max(1, portion_min_keys // 32), _ptr(part_scratch),
          _ptr(dist_bias), 0 if dist_bias is None else dist_bias.shape[1], int(vd), int(keep_first), _ptr(sink), _stream())
    return out


def swiglu(gu: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[m, 2i] (gate columns then up columns) -> out_dtype [m, i]."""
    if _backend is not None:
        return _backend.swiglu(gu, out_dtype)
    _dev_ok(gu)
    _need(gu.dim() == 2 and gu.shape[1] % 2 == 0, "swiglu: input must be [m, 2i]")
    m, i2 = gu.shape
    out = torch.empty((m, i2 // 2), dtype=out_dtype, device=gu.device)
    _call("tp_swiglu", _ptr(gu), _dt(gu), _ptr(out), _dtcode(out_dtype), m, i2 // 2, _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """float32 [m, vocab] -> int32 [m]; the last maximum wins on exact ties."""
    if _backend is not None:
        return _backend.argmax(logits)
    _dev_ok(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits must be float32 [m, vocab]")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    part = torch.empty((logits.shape[0] * 128,), dtype=torch.float32, device=logits.device)
    _call("tp_argmax", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _ptr(part), _stream())
    return out


class HostCopy:
    """A small device tensor on its way to the host: the copy into pinned memory is queued when the object is
    made, ``result()`` waits for that copy alone (not for work queued behind it) and returns a list.  The pinned
    buffers are taken in turn from a ring, so at most ``RING`` copies may be outstanding."""
    RING = 8
    _ring: list = []
    _next = 0

    def __init__(self, t: torch.Tensor):
        cls = HostCopy
        n = t.numel()
        if not cls._ring:
            cls._ring = [None] * cls.RING
        slot = cls._ring[cls._next]
        if slot is None or slot[0].numel() < n or slot[0].dtype != t.dtype:
            slot = (torch.empty(max(n, 256), dtype=t.dtype, pin_memory=True), torch.cuda.Event())
            cls._ring[cls._next] = slot
        cls._next = (cls._next + 1) % cls.RING
        self._buf, self._event, self._n = slot[0], slot[1], n
        self._buf[:n].copy_(t.reshape(-1), non_blocking=True)
        self._event.record()

    def result(self) -> list:
        self._event.synchronize()
        return self._buf[: self._n].tolist()


class _Staging:
    """Small per-call option arrays on their way to the device through pinned memory: the copy is queued behind
    the work in flight instead of making the host wait for it (a pageable copy would).  Buffers are taken in
    turn from a ring and reused once their copy has run."""
    RING = 8
    _ring: list = []
    _next = 0

    @classmethod
    def send(cls, arrays, device) -> list:
        """``arrays``: numpy arrays of 4-byte elements, each [rows..]; returns device tensors of the same shapes
        and dtypes (views of one packed transfer)."""
        import numpy as np
        total = sum(a.size for a in arrays)
        if not cls._ring:
            cls._ring = [None] * cls.RING
        slot = cls._ring[cls._next]
        if slot is None or slot[0].numel() < total:
            slot = (torch.empty(max(total, 1024), dtype=torch.int32, pin_memory=True), torch.cuda.Event())
            cls._ring[cls._next] = slot
        cls._next = (cls._next + 1) % cls.RING
        host, event = slot
        event.synchronize()                       # the copy that last used this buffer has run
        flat = host.numpy()
        views, off = [], 0
        for a in arrays:
            flat[off: off + a.size] = np.ascontiguousarray(a).reshape(-1).view(np.int32)
            off += a.size
        dev = host[:total].to(device, non_blocking=True)
        event.record()
        off = 0
        for a in arrays:
            t = dev[off: off + a.size]
            views.append((t.view(torch.float32) if a.dtype == np.float32 else t).view(a.shape))
            off += a.size
        return views


def apply_penalties(logits: torch.Tensor, rows, tokens, counts, in_window, presence, frequency, repeat) -> None:
    """In place on float32 [m, vocab]: for entry i, logits[rows[i], tokens[i]] gets the presence/frequency
    penalty when counts[i] > 0 and the repetition penalty when in_window[i]; penalties are per row."""
    if _backend is not None:
        return _backend.apply_penalties(logits, rows, tokens, counts, in_window, presence, frequency, repeat)
    import numpy as np
    _dev_ok(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "apply_penalties: logits must be float32 [m, vocab]")
    m, vocab = logits.shape
    n = len(rows)
    _need(len(tokens) == n and len(counts) == n and len(in_window) == n, "apply_penalties: entry lists differ in length")
    _need(len(presence) == m and len(frequency) == m and len(repeat) == m, "apply_penalties: one penalty per row")
    _need(all(0 <= r < m for r in rows), "apply_penalties: row out of range")
    dev = logits.device
    ints, fl = _Staging.send([np.asarray([rows, tokens, counts, in_window], dtype=np.int32),
                              np.asarray([presence, frequency, repeat], dtype=np.float32)], dev)
    _call("tp_apply_penalties", _ptr(logits), vocab, _ptr(ints[0]), _ptr(ints[1]), _ptr(ints[2]), _ptr(ints[3]),
          _ptr(fl[0]), _ptr(fl[1]), _ptr(fl[2]), n, _stream())


_SAMPLE_LIMITS: Optional[tuple] = None


def _sample_limits() -> tuple:
    """(pieces of a row, candidates per piece, largest top_k settled from candidates, most elements of a piece,
    bins of a counting pass) as the sampling kernels were compiled; ``sample`` sizes their scratch by these."""
    global _SAMPLE_LIMITS
    if _SAMPLE_LIMITS is None:
        buf = (ctypes.c_int * 5)()
        lib = _Library.get()
        if lib.tp_sample_limits(buf) != 0:
            raise KernelError(f"tp_sample_limits: {lib.tp_last_error().decode()}")
        _SAMPLE_LIMITS = tuple(int(v) for v in buf)
    return _SAMPLE_LIMITS


def sample(logits: torch.Tensor, work: torch.Tensor, temperature, top_k, top_p, min_p, rnd, typical_p=None,
           info: Optional[torch.Tensor] = None, settled: Optional[list] = None) -> torch.Tensor:
    """float32 [m, vocab] and per-row options (host arrays) -> int32 [m] chosen tokens.
    ``work`` is float32 scratch of at least [m, vocab].  temperature 0 rows return the argmax.
    ``typical_p`` None leaves that filter off (1.0) in every row.
    ``info``: float32 [m, 4] that receives, per row, what log-probabilities of the filtered distribution need
    (maximum, ln of the normaliser, smallest surviving value) and the chosen token's log-probability in column 3;
    ``work`` then holds the filtered, scaled logits for ``top_logprobs``.
    ``settled``: a list that receives, per row, 1 when the row was settled from the candidates of its pieces (a
    small top_k, or top_p alone on a row whose kept prefix is short) and 0 when the one block per row did it; for tests."""
    if typical_p is None:
        typical_p = [1.0] * len(temperature)
    if _backend is not None:
        if settled is not None:
            settled[:] = [0] * len(temperature)
        return _backend.sample(logits, work, temperature, top_k, top_p, min_p, rnd, typical_p, info)
    import numpy as np
    _dev_ok(logits, work)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample: logits must be float32 [m, vocab]")
    m, vocab = logits.shape
    _need(work.dtype == torch.float32 and work.numel() >= m * vocab, "sample: work buffer too small")
    for a in (temperature, top_k, top_p, min_p, rnd, typical_p):
        _need(len(a) == m, "sample: one option per row")
    dev = logits.device
    fl, tk = _Staging.send([np.asarray([temperature, top_p, min_p, rnd, typical_p], dtype=np.float32),
                            np.asarray(top_k, dtype=np.int32)], dev)
    out = torch.empty((m,), dtype=torch.int32, device=dev)
    # (the scratch buffers are laid out by the library's own sizes, asked of it once: pieces of a row, candidates a
    # piece may hand over, the largest top_k settled from candidates, the most elements of a piece, bins of a pass)
    pieces, ccap, kmax, per_max, bins = _sample_limits()
    part_max = torch.empty((m * pieces,), dtype=torch.float32, device=dev)    # (maxima of the pieces of each row)
    # rows that are only scaled (and cut by min_p) before the draw get the masses of their pieces from a kernel
    # of many blocks; worth it when there is such a row
    plain_rows = any(t > 0 and not (0 < k < vocab) and not (0.0 < p < 1.0) and not (ty < 1.0)
                     for t, k, p, ty in zip(temperature, top_k, top_p, typical_p))
    # rows cut by top_p alone are settled from the candidates of their pieces against the mass of the whole row
    piece_ok = -(-vocab // pieces) <= per_max and info is None
    topp_rows = piece_ok and vocab > kmax and any(
        t > 0 and not (0 < k < vocab) and 0.0 < p < 1.0 and not (ty < 1.0)
        for t, k, p, ty in zip(temperature, top_k, top_p, typical_p))
    part_mass = torch.empty((m * pieces,), dtype=torch.int64, device=dev) if (plain_rows or topp_rows) and info is None else None
    # rows cut by top_k have the first pass of their selection counted by the kernel of many blocks that scales the row
    # ... unless top_k is small: such a row is settled from the few candidates that each piece of it hands over
    small = lambda k, ty: 0 < k <= kmax and not (ty < 1.0) and piece_ok
    topk_rows = [(k, ty) for t, k, ty in zip(temperature, top_k, typical_p) if t > 0 and 0 < k < vocab]
    part_cnt = None
    if any(not small(k, ty) for k, ty in topk_rows):
        part_cnt = torch.empty((m * pieces * bins,), dtype=torch.int32, device=dev)
    cand_val = cand_idx = cand_cnt = cand_thr = done = None
    if topp_rows or any(small(k, ty) for k, ty in topk_rows):
        cand_val = torch.empty((m * pieces * ccap,), dtype=torch.float32, device=dev)
        cand_idx = torch.empty((m * pieces * ccap,), dtype=torch.int32, device=dev)
        cand_cnt = torch.empty((m * pieces,), dtype=torch.int32, device=dev)
        cand_thr = torch.empty((m * pieces,), dtype=torch.int32, device=dev)
        done = torch.empty((m,), dtype=torch.int32, device=dev)
    if info is not None:
        _dev_ok(info)
        _need(info.dtype == torch.float32 and info.is_contiguous() and tuple(info.shape) == (m, 4), "sample: info must be float32 [m, 4]")
    _call("tp_sample", _ptr(logits), _ptr(work), m, vocab, _ptr(fl[0]), _ptr(tk), _ptr(fl[1]), _ptr(fl[2]),
          _ptr(fl[4]), _ptr(fl[3]), _ptr(out), _ptr(info), _ptr(part_max), _ptr(part_mass), _ptr(part_cnt),
          _ptr(cand_val), _ptr(cand_idx), _ptr(cand_cnt), _ptr(cand_thr), _ptr(done), _stream())
    if settled is not None:
        settled[:] = [0] * m if done is None else done.tolist()
    return out


def top_logprobs(work: torch.Tensor, info: torch.Tensor, vocab: int, n: int):
    """After ``sample(..., info=info)``: the ``n`` most probable tokens of each row's filtered distribution,
    most probable first (ties by index), as (int32 [m, n] ids, float32 [m, n] log-probabilities); id -1 where a
    row has fewer survivors."""
    if _backend is not None:
        return _backend.top_logprobs(work, info, vocab, n)
    _dev_ok(work, info)
    m = info.shape[0]
    _need(info.dtype == torch.float32 and info.is_contiguous() and tuple(info.shape) == (m, 4), "top_logprobs: info must be float32 [m, 4]")
    _need(work.dtype == torch.float32 and work.is_contiguous() and work.numel() >= m * vocab, "top_logprobs: work buffer too small")
    _need(0 <= n <= vocab, "top_logprobs: n out of range")
    ids = torch.empty((m, n), dtype=torch.int32, device=info.device)
    lps = torch.empty((m, n), dtype=torch.float32, device=info.device)
    _call("tp_top_logprobs", _ptr(work), _ptr(info), m, vocab, n, _ptr(ids), _ptr(lps), _stream())
    return ids, lps


def take_rows(t: torch.Tensor, rows=None) -> torch.Tensor:
    """A new tensor holding rows ``rows`` (a list of indices; None: all of them, a plain copy) of a float32 or
    int32 tensor [n] or [n, width], by the library's own copy kernel."""
    if _backend is not None:
        return _backend.take_rows(t, rows)
    import numpy as np
    _dev_ok(t)
    _need(t.dtype in (torch.float32, torch.int32) and t.dim() in (1, 2), "take_rows: needs float32 or int32 [n] or [n, width]")
    n_in = t.shape[0]
    width = 1 if t.dim() == 1 else t.shape[1]
    if rows is None:
        n, idx = n_in, None
    else:
        n = len(rows)
        _need(all(0 <= int(r) < n_in for r in rows), "take_rows: row out of range")
        idx = _Staging.send([np.asarray(rows, dtype=np.int32)], t.device)[0] if n else None
    out = torch.empty((n,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
    if n and width:
        _call("tp_copy_rows4", _ptr(t), _ptr(idx), _ptr(out), n, width, _stream())
    return out


def zero_rows(t: torch.Tensor, rows) -> None:
    """t[rows] = 0 in place for a float32 or int32 tensor [n, ...] (rows: a list of indices)."""
    if _backend is not None:
        return _backend.zero_rows(t, rows)
    import numpy as np
    _dev_ok(t)
    _need(t.dtype in (torch.float32, torch.int32) and t.dim() >= 1, "zero_rows: needs a float32 or int32 tensor")
    n_in = t.shape[0]
    width = t[0].numel() if n_in else 0
    _need(all(0 <= int(r) < n_in for r in rows), "zero_rows: row out of range")
    if len(rows) and width:
        idx = _Staging.send([np.asarray(rows, dtype=np.int32)], t.device)[0]
        _call("tp_zero_rows4", _ptr(t), _ptr(idx), len(rows), width, _stream())


def fill_normal(out: torch.Tensor, seed: int, mean: float, std: float) -> torch.Tensor:
    """Fill a device tensor with mean + std * N(0, 1); element i depends only on (seed, i) and has the bits
    that ``weights.random_init.fill_normal_host`` gives it on the host."""
    if _backend is not None:
        return _backend.fill_normal(out, seed, mean, std)
    _dev_ok(out)
    _call("tp_fill_normal", _ptr(out), _dt(out), ctypes.c_size_t(out.numel()), ctypes.c_ulonglong(seed & (2 ** 64 - 1)),
          ctypes.c_double(mean), ctypes.c_double(std), _stream())
    return out


# ---------------------------------------------------------------------------------
# Operations of layers with a hashed bigram embedding, norms behind the sublayers, a gated delta-rule mixer and
# routed experts.

def embed_bigram(tokens: torch.Tensor, table: torch.Tensor, bigram: Optional[torch.Tensor], positions: torch.Tensor,
                 token_req: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, prev_state: torch.Tensor,
                 num_requests: int, mul_prev: int, mul_cur: int, buckets: int, scale: float = 1.0,
                 pos_table: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [n, hidden] = table[token] * scale + bigram[row], row = (previous * mul_prev + token * mul_cur) mod buckets,
    and row ``buckets`` for a token at position 0.  The previous token of a run's first token is what
    ``prev_state`` (int32 [slots, 1]) holds for the request's slot; each run's last token is left there.
    ``pos_table`` ([positions, hidden], of the tables' type): its row of the token's position is added as well.
    ``bigram`` None: no second row (and nothing is read from or left in ``prev_state``, which may be None too)."""
    if _backend is not None:
        if scale != 1.0 or pos_table is not None:
            return _backend.embed_bigram(tokens, table, bigram, positions, token_req, cu_seqlens, state_slots, prev_state,
                                         num_requests, mul_prev, mul_cur, buckets, scale, pos_table)
        return _backend.embed_bigram(tokens, table, bigram, positions, token_req, cu_seqlens, state_slots, prev_state,
                                     num_requests, mul_prev, mul_cur, buckets)
    _dev_ok(tokens, table, bigram, positions, token_req, cu_seqlens, state_slots, prev_state, pos_table)
    n = tokens.numel()
    _need(pos_table is None or (pos_table.dim() == 2 and pos_table.shape[1] == table.shape[1] and pos_table.dtype == table.dtype),
          "embed_bigram: the position table must be [positions, hidden] of the tables' type")
    _need(table.dim() == 2, "embed_bigram: tables must be [rows, hidden] of one type")
    if bigram is not None:
        _need(bigram.dim() == 2 and bigram.shape[1] == table.shape[1] and bigram.dtype == table.dtype,
              "embed_bigram: tables must be [rows, hidden] of one type")
        _need(bigram.shape[0] == buckets + 1, f"embed_bigram: the bigram table needs {buckets + 1} rows, has {bigram.shape[0]}")
        _need(prev_state is not None and prev_state.dtype == torch.int32, "embed_bigram: the state must be int32")
    _i32(tokens, n, "embed tokens") if n else None
    _i32(positions, n, "embed positions") if n else None
    _i32(token_req, n, "token_req") if n else None
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    hidden = table.shape[1]
    out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    _call("tp_embed_bigram", _ptr(tokens), _ptr(positions), _ptr(token_req), _ptr(cu_seqlens), _ptr(state_slots), _ptr(prev_state),
          _ptr(table), _ptr(bigram), _dt(table), _ptr(out), n, int(num_requests), hidden, ctypes.c_longlong(mul_prev),
          ctypes.c_longlong(mul_cur), ctypes.c_longlong(buckets), ctypes.c_float(scale), _ptr(pos_table), _stream())
    return out


def sigmoid_gate(a: torch.Tensor, proj: Optional[torch.Tensor], gate_col0: int, scale: float, out: torch.Tensor, out_col0: int) -> None:
    """out[:, out_col0 + c] = a[:, c] * sigmoid(proj[:, gate_col0 + c]) * scale (``proj`` float32 rows; None: no
    gate); ``a`` and ``out`` are of one type, ``out`` [n, wider]."""
    if _backend is not None:
        return _backend.sigmoid_gate(a, proj, gate_col0, scale, out, out_col0)
    _dev_ok(a, proj, out)
    _need(a.dim() == 2 and out.dim() == 2 and a.dtype == out.dtype and a.shape[0] == out.shape[0], "sigmoid_gate: bad operands")
    n, width = a.shape
    _need(0 <= out_col0 and out_col0 + width <= out.shape[1], "sigmoid_gate: output rows too short")
    if proj is not None:
        _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[0] == n and 0 <= gate_col0 and gate_col0 + width <= proj.shape[1],
              "sigmoid_gate: bad gate rows")
    _call("tp_sigmoid_gate", _ptr(a), _dt(a), _ptr(proj), 0 if proj is None else proj.shape[1], int(gate_col0), ctypes.c_float(scale),
          _ptr(out), out.shape[1], int(out_col0), n, width, _stream())


def norm_add(h: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, next_weight: Optional[torch.Tensor] = None,
             next_eps: float = 0.0, out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """h += y / sqrt(mean(y^2) + eps) * weight, per row, in place (float32 [n, width]).  With ``next_weight`` the
    rows of the new h normed with it (and ``next_eps``) come back as ``out_dtype``."""
    if _backend is not None:
        return _backend.norm_add(h, y, weight, eps, next_weight, next_eps, out_dtype)
    _dev_ok(h, y, weight, next_weight)
    _need(h.dtype == torch.float32 and h.dim() == 2 and y.dtype == torch.float32 and tuple(y.shape) == tuple(h.shape),
          "norm_add: h and y must be float32 [n, width]")
    n, width = h.shape
    _need(weight.dtype == torch.float32 and weight.numel() == width, "norm_add: weight must be float32 [width]")
    x = None
    if next_weight is not None:
        _need(next_weight.dtype == torch.float32 and next_weight.numel() == width and out_dtype is not None, "norm_add: bad next norm")
        x = torch.empty((n, width), dtype=out_dtype, device=h.device)
    _call("tp_norm_add", _ptr(h), _ptr(y), _ptr(weight), ctypes.c_float(eps), _ptr(next_weight), ctypes.c_float(next_eps), _ptr(x),
          _dtcode(out_dtype) if x is not None else _F32, n, width, _stream())
    return x


ACTIVATIONS = {"gelu_tanh": 0, "silu": 1, "gelu_erf": 2}


def activation(u: torch.Tensor, kind: str, out_dtype: torch.dtype, col0: int = 0, width: Optional[int] = None,
               gate_col: Optional[int] = None) -> torch.Tensor:
    """Element by element: ``gelu_tanh`` (0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))), ``gelu_erf``
    (0.5 z (1 + erf(z / sqrt(2)))) or ``silu``, formed in float32, as ``out_dtype``.
    With ``width`` (``u`` float32 rows [n, wider]): the columns col0 .. col0 + width of every row, and with ``gate_col``
    each row's results times the sigmoid of that column of the row."""
    _need(kind in ACTIVATIONS, f"activation: {kind!r} unknown (known: {sorted(ACTIVATIONS)})")
    if _backend is not None:
        if width is not None:
            return _backend.activation(u, kind, out_dtype, col0, width, gate_col)
        return _backend.activation(u, kind, out_dtype)
    _dev_ok(u)
    if width is not None:
        _need(u.dtype == torch.float32 and u.dim() == 2 and 0 <= col0 and col0 + width <= u.shape[1] and width > 0,
              "activation: rows must be float32 [n, wider]")
        _need(gate_col is None or 0 <= gate_col < u.shape[1], "activation: gate column outside the rows")
        out = torch.empty((u.shape[0], width), dtype=out_dtype, device=u.device)
        _call("tp_activation_rows", _ptr(u), ctypes.c_size_t(u.shape[1]), int(col0), int(width), -1 if gate_col is None else int(gate_col),
              _ptr(out), _dtcode(out_dtype), u.shape[0], ACTIVATIONS[kind], _stream())
        return out
    out = torch.empty(u.shape, dtype=out_dtype, device=u.device)
    _call("tp_activation", _ptr(u), _dt(u), _ptr(out), _dtcode(out_dtype), ctypes.c_size_t(u.numel()), ACTIVATIONS[kind], _stream())
    return out


ROUTE_SCORES = {"softmax": 0, "sigmoid": 1}


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], experts: int, top: int, groups: int, keep: int,
              score: str = "softmax", group_best: int = 1, normalize: bool = False, sum_eps: float = 0.0, scale: float = 1.0,
              bias: Optional[torch.Tensor] = None):
    """Router of a mixture of experts over float32 logits [n, >= experts]: s = softmax over the experts (``score``
    ``"sigmoid"``: the sigmoid of each logit by itself); an expert's choice score is s + correction (None: s); with
    ``groups`` > 1 only the experts of the ``keep`` groups (of neighbours) whose ``group_best`` largest choice scores
    add up highest can be chosen; the ``top`` best allowed experts are chosen and weigh s, with ``normalize`` divided by
    the chosen experts' sum (+ ``sum_eps``), times ``scale``.  Returns (dense float32 [n, experts] with a chosen expert's
    weight and 0 elsewhere, ids int32 [n, top], weights [n, top]).  ``bias`` (float32 [experts]) is added to the logits
    first.  (A softmax over the chosen logits alone is ``normalize`` without ``sum_eps``: the chosen experts' shares of
    the full softmax over their sum.)"""
    _need(score in ROUTE_SCORES, f"moe_route: score {score!r} unknown")
    if _backend is not None:
        if bias is not None:
            return _backend.moe_route(logits, correction, experts, top, groups, keep, score, group_best, normalize, sum_eps, scale, bias)
        if (score, group_best, normalize, scale) == ("softmax", 1, False, 1.0) and correction is not None:
            return _backend.moe_route(logits, correction, experts, top, groups, keep)
        return _backend.moe_route(logits, correction, experts, top, groups, keep, score, group_best, normalize, sum_eps, scale)
    _dev_ok(logits, correction, bias)
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == experts), "moe_route: bias must be float32 [experts]")
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[1] >= experts, "moe_route: logits must be float32 [n, experts]")
    _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == experts), "moe_route: correction must be float32 [experts]")
    _need(group_best >= 1, "moe_route: group_best must be at least 1")
    n = logits.shape[0]
    dense = torch.empty((n, experts), dtype=torch.float32, device=logits.device)
    ids = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=logits.device)
    _call("tp_moe_route", _ptr(logits), logits.shape[1], _ptr(correction), int(experts), int(top), int(groups), int(keep), _ptr(dense),
          _ptr(ids), _ptr(weights), n, ROUTE_SCORES[score], int(group_best), int(bool(normalize)), ctypes.c_float(sum_eps),
          ctypes.c_float(scale), _ptr(bias), _stream())
    return dense, ids, weights


LOWRANK_MODES = {"plain": 0, "sigmoid": 1, "decay": 2, "rate_sigmoid": 3}


def lowrank_up(x: torch.Tensor, col0: int, weight_t: torch.Tensor, mode: str = "plain", a_log: Optional[torch.Tensor] = None,
               bias: Optional[torch.Tensor] = None, per_head: int = 0, rate: float = 0.0, in_act: Optional[str] = None) -> torch.Tensor:
    """The second product of a low-rank projection: float32 [n, N] = f(g(x[:, col0: col0 + r]) @ weight_t), ``x`` float32
    rows (the first product's sums), ``weight_t`` float32 [r, N].  f: ``plain``; ``sigmoid``; ``decay``:
    exp(-exp(a_log[c // per_head]) * softplus(sum + bias[c])); ``rate_sigmoid``: exp(-rate * sigmoid(sum + bias[c])).
    g: the identity, or tanh with ``in_act`` ``"tanh"``."""
    _need(in_act in (None, "tanh"), f"lowrank_up: input function {in_act!r} unknown")
    if _backend is not None:
        if mode == "rate_sigmoid" or in_act is not None:
            return _backend.lowrank_up(x, col0, weight_t, mode, a_log, bias, per_head, rate, in_act)
        return _backend.lowrank_up(x, col0, weight_t, mode, a_log, bias, per_head)
    _dev_ok(x, weight_t, a_log, bias)
    _need(mode in LOWRANK_MODES, f"lowrank_up: mode {mode!r} unknown")
    _need(x.dtype == torch.float32 and x.dim() == 2 and weight_t.dtype == torch.float32 and weight_t.dim() == 2, "lowrank_up: float32 operands")
    r, n_out = weight_t.shape
    _need(0 <= col0 and col0 + r <= x.shape[1], "lowrank_up: rows too short")
    if mode == "decay":
        _need(a_log is not None and bias is not None and per_head > 0 and n_out % per_head == 0 and a_log.dtype == torch.float32
              and bias.dtype == torch.float32 and a_log.numel() == n_out // per_head and bias.numel() == n_out, "lowrank_up: bad decay constants")
    if mode == "rate_sigmoid":
        _need(bias is not None and bias.dtype == torch.float32 and bias.numel() == n_out, "lowrank_up: bad decay biases")
    out = torch.empty((x.shape[0], n_out), dtype=torch.float32, device=x.device)
    _call("tp_lowrank_up", _ptr(x), x.shape[1], int(col0), r, _ptr(weight_t), _ptr(out), x.shape[0], n_out, LOWRANK_MODES[mode],
          _ptr(a_log), _ptr(bias), int(per_head), 1 if in_act == "tanh" else 0, ctypes.c_float(rate), _stream())
    return out


def delta_scan(qkv: torch.Tensor, decay: torch.Tensor, proj: torch.Tensor, beta_col0: int, state: torch.Tensor, state_off: int,
               cu_seqlens: torch.Tensor, state_slots: torch.Tensor, num_requests: int, heads: int, kv_heads: int, dim: int,
               vdim: int, q_scale: float, unit_eps: float) -> torch.Tensor:
    """The gated delta rule per head over each request's run.  ``qkv`` float32 [n, q | k | v] with q and k
    [kv_heads * dim] and v [heads * vdim]; q and k are made unit vectors per head (x / sqrt(sum x^2 + unit_eps), q times
    ``q_scale``); beta = sigmoid(proj[:, beta_col0 + h]); ``decay`` float32 [n, heads * dim].  Per head, with S
    [dim, vdim] (kept at ``state[slot, state_off:]`` column by column, [heads, vdim, dim]):  S <- decay * S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
    Returns o float32 [n, heads * vdim]; the state is left as the run leaves it.  (q and k of ``qkv`` are left as
    unit vectors: the rows are a temporary of the caller's.)"""
    if _backend is not None:
        return _backend.delta_scan(qkv, decay, proj, beta_col0, state, state_off, cu_seqlens, state_slots, num_requests, heads,
                                   kv_heads, dim, vdim, q_scale, unit_eps)
    _dev_ok(qkv, decay, proj, state, cu_seqlens, state_slots)
    n = qkv.shape[0]
    _need(qkv.dtype == torch.float32 and qkv.dim() == 2 and qkv.shape[1] == 2 * kv_heads * dim + heads * vdim, "delta_scan: bad q | k | v rows")
    _need(decay.dtype == torch.float32 and tuple(decay.shape) == (n, heads * dim), "delta_scan: decay must be float32 [n, heads * dim]")
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[0] == n and 0 <= beta_col0 and beta_col0 + heads <= proj.shape[1],
          "delta_scan: bad projection rows")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state_off >= 0 and state.shape[1] >= state_off + heads * dim * vdim,
          "delta_scan: state rows too short")
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    y = torch.empty((n, heads * vdim), dtype=torch.float32, device=qkv.device)
    kq = torch.empty((n, kv_heads), dtype=torch.float32, device=qkv.device)      # k . q per token and key head
    _call("tp_delta_scan", _ptr(qkv), qkv.shape[1], _ptr(decay), _ptr(proj), proj.shape[1], int(beta_col0), _ptr(state),
          ctypes.c_size_t(state.shape[1]), ctypes.c_size_t(state_off), _ptr(cu_seqlens), _ptr(state_slots), _ptr(y), _ptr(kq), n,
          int(num_requests), int(heads), int(kv_heads), int(dim), int(vdim), ctypes.c_float(q_scale), ctypes.c_float(unit_eps), _stream())
    return y


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: Optional[torch.Tensor], eps: float, scale: float, heads: int,
                   out: torch.Tensor, out_col0: int, gate_rows: Optional[torch.Tensor] = None, gate_col0: int = 0) -> None:
    """out[:, out_col0 + h * vdim + d] = o[:, h, d] / sqrt(mean_d o^2 + eps) * weight[d] * gate[:, h * vdim + d] * scale:
    ``o`` float32 [n, heads * vdim]; ``weight`` float32 [vdim] shared by the heads, or [heads * vdim], every head its own;
    ``gate`` float32 like ``o`` or None.  ``gate_rows`` (float32 rows [n, wider], instead of ``gate``): the gate is the
    sigmoid of their columns gate_col0 .. gate_col0 + heads * vdim."""
    if _backend is not None:
        if gate_rows is not None:
            return _backend.head_norm_gate(o, weight, gate, eps, scale, heads, out, out_col0, gate_rows, gate_col0)
        return _backend.head_norm_gate(o, weight, gate, eps, scale, heads, out, out_col0)
    _dev_ok(o, weight, gate, out, gate_rows)
    _need(o.dtype == torch.float32 and o.dim() == 2 and o.shape[1] % heads == 0, "head_norm_gate: o must be float32 [n, heads * vdim]")
    n, vdim = o.shape[0], o.shape[1] // heads
    _need(weight.dtype == torch.float32 and weight.numel() in (vdim, heads * vdim), "head_norm_gate: weight must be float32 [vdim] or [heads * vdim]")
    # (one head: a weight of [vdim] is both)
    per_head = int(weight.numel() == heads * vdim and heads > 1)
    _need(gate is None or gate_rows is None, "head_norm_gate: one gate")
    _need(gate is None or (gate.dtype == torch.float32 and tuple(gate.shape) == tuple(o.shape)), "head_norm_gate: gate must match o")
    _need(out.dim() == 2 and out.shape[0] == n and 0 <= out_col0 and out_col0 + o.shape[1] <= out.shape[1], "head_norm_gate: output rows too short")
    gate_ptr, gate_stride, raw = _ptr(gate), o.shape[1], 0
    if gate_rows is not None:
        _need(gate_rows.dtype == torch.float32 and gate_rows.dim() == 2 and gate_rows.shape[0] == n and 0 <= gate_col0
              and gate_col0 + o.shape[1] <= gate_rows.shape[1], "head_norm_gate: bad gate rows")
        gate_ptr, gate_stride, raw = ctypes.c_void_p(gate_rows.data_ptr() + 4 * int(gate_col0)), gate_rows.shape[1], 1
    _call("tp_head_norm_gate", _ptr(o), _ptr(weight), gate_ptr, ctypes.c_float(eps), ctypes.c_float(scale), _ptr(out), _dt(out),
          out.shape[1], int(out_col0), n, int(heads), vdim, per_head, ctypes.c_size_t(gate_stride), raw, _stream())


def moe_plan(ids: torch.Tensor, experts: int):
    """Where every chosen (token, expert) pair goes when the pairs are brought into the order of the experts:
    ``ids`` int32 [n, top] -> (counts int32 [experts], offsets int32 [experts + 1], rank int32 [n, top]); pair (t, k)
    goes to row offsets[ids[t, k]] + rank[t, k], the pairs of one expert keeping the order of the tokens."""
    if _backend is not None:
        return _backend.moe_plan(ids, experts)
    _dev_ok(ids)
    _need(ids.dtype == torch.int32 and ids.dim() == 2, "moe_plan: ids must be int32 [n, top]")
    counts = torch.empty((experts,), dtype=torch.int32, device=ids.device)
    offsets = torch.empty((experts + 1,), dtype=torch.int32, device=ids.device)
    rank = torch.empty(ids.shape, dtype=torch.int32, device=ids.device)
    _call("tp_moe_plan", _ptr(ids), ids.shape[0], ids.shape[1], int(experts), _ptr(counts), _ptr(offsets), _ptr(rank), _stream())
    return counts, offsets, rank


def moe_gather(x: torch.Tensor, ids: torch.Tensor, rank: torch.Tensor, offsets: torch.Tensor):
    """(rows [n * top, width] of ``x`` [n, width] in the order of the experts, row_of int32 [n, top]: the row of pair (t, k))."""
    if _backend is not None:
        return _backend.moe_gather(x, ids, rank, offsets)
    _dev_ok(x, ids, rank, offsets)
    n, top = ids.shape
    _need(x.dim() == 2 and x.shape[0] == n and (x.shape[1] * x.element_size()) % 4 == 0, "moe_gather: rows must be a multiple of four bytes")
    _need(rank.dtype == torch.int32 and tuple(rank.shape) == (n, top) and offsets.dtype == torch.int32, "moe_gather: bad plan")
    xg = torch.empty((n * top, x.shape[1]), dtype=x.dtype, device=x.device)
    row_of = torch.empty((n, top), dtype=torch.int32, device=x.device)
    _call("tp_moe_gather", _ptr(x), _ptr(ids), _ptr(rank), _ptr(offsets), _ptr(xg), _ptr(row_of), n, top, x.shape[1] * x.element_size(), _stream())
    return xg, row_of


def moe_scatter(yg: torch.Tensor, row_of: torch.Tensor, weights: torch.Tensor, y: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[t] (+)= sum_k weights[t, k] * yg[row_of[t, k]] (k ascending); ``y`` None: a new tensor."""
    if _backend is not None:
        return _backend.moe_scatter(yg, row_of, weights, y)
    _dev_ok(yg, row_of, weights, y)
    n, top = row_of.shape
    _need(yg.dtype == torch.float32 and yg.dim() == 2 and yg.shape[0] == n * top and weights.dtype == torch.float32
          and tuple(weights.shape) == (n, top) and row_of.dtype == torch.int32, "moe_scatter: bad operands")
    acc = y is not None
    if not acc:
        y = torch.empty((n, yg.shape[1]), dtype=torch.float32, device=yg.device)
    _need(y.dtype == torch.float32 and tuple(y.shape) == (n, yg.shape[1]), "moe_scatter: y must be float32 [n, width]")
    _call("tp_moe_scatter", _ptr(yg), _ptr(row_of), _ptr(weights), _ptr(y), n, top, yg.shape[1], int(acc), _stream())
    return y


def moe_spread(a: torch.Tensor, dense: torch.Tensor, experts: int) -> torch.Tensor:
    """``a`` [n, experts * ff] (all experts' activations of every row) -> [experts, n, ff]: each expert's activations
    as rows of its own, times the row's weight for the expert (``dense`` float32 [n, experts], zero where the expert
    was not chosen); the product is formed in float32 and rounded once."""
    if _backend is not None:
        return _backend.moe_spread(a, dense, experts)
    _dev_ok(a, dense)
    _need(a.dim() == 2 and a.shape[1] % experts == 0 and dense.dtype == torch.float32 and tuple(dense.shape) == (a.shape[0], experts),
          "moe_spread: bad operands")
    n, ff = a.shape[0], a.shape[1] // experts
    out = torch.empty((experts, n, ff), dtype=a.dtype, device=a.device)
    _call("tp_moe_spread", _ptr(a), _dt(a), _ptr(dense), _ptr(out), n, int(experts), ff, _stream())
    return out


# ---------------------------------------------------------------------------------
# Operations of layers with one norm for both sublayers, inputs convolved over time, a generalized delta rule, an
# attention over keys and values expanded from a latent, and a vector added to the stream between layers.

def rmsnorm_cols(x: torch.Tensor, col0: int, width: int, weight: torch.Tensor, eps: float, out_dtype: torch.dtype, groups: int = 1) -> torch.Tensor:
    """The RMS norm (in ``groups`` equal parts) of columns col0 .. col0 + width of float32 rows [n, wider], times
    ``weight`` [width] -> out_dtype [n, width]."""
    if _backend is not None:
        return _backend.rmsnorm_cols(x, col0, width, weight, eps, out_dtype, groups)
    _dev_ok(x, weight)
    _need(x.dtype == torch.float32 and x.dim() == 2 and 0 <= col0 and col0 + width <= x.shape[1], "rmsnorm_cols: bad rows")
    _need(weight.dtype == torch.float32 and weight.numel() == width and groups > 0 and width % groups == 0, "rmsnorm_cols: bad weight or groups")
    out = torch.empty((x.shape[0], width), dtype=out_dtype, device=x.device)
    _call("tp_group_rmsnorm", _ptr(x), ctypes.c_size_t(x.shape[1]), int(col0), _ptr(weight), _ptr(None), _ptr(out), _dtcode(out_dtype),
          x.shape[0], int(width), int(groups), ctypes.c_float(eps), _stream())
    return out


def residual_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, state_off: int, cu_seqlens: torch.Tensor,
                  token_req: torch.Tensor, state_slots: torch.Tensor, num_requests: int, out_dtype: torch.dtype):
    """What sublayers read of rows ``x`` (float32 [n, width]): for each of the ``weight`` [subs, taps, width] (tap-major,
    the last tap the current token's) x + conv(x) over each request's run of tokens, as ``out_dtype``; a list of
    ``subs`` tensors [n, width].  ``state`` float32 [slots, row]: from element ``state_off`` on a request's carried
    rows [taps - 1, width] (oldest first), read for the first tokens of a run and replaced by the run's last rows."""
    if _backend is not None:
        return _backend.residual_conv(x, weight, state, state_off, cu_seqlens, token_req, state_slots, num_requests, out_dtype)
    _dev_ok(x, weight, state, cu_seqlens, token_req, state_slots)
    _need(x.dtype == torch.float32 and x.dim() == 2, "residual_conv: rows must be float32 [n, width]")
    n, width = x.shape
    _need(weight.dtype == torch.float32 and weight.dim() == 3 and weight.shape[2] == width, "residual_conv: weight must be float32 [subs, taps, width]")
    subs, taps = weight.shape[0], weight.shape[1]
    # (one tap carries nothing: a layer whose parts keep no state then has no state tensor)
    _need((state is None and taps == 1) or (state is not None and state.dtype == torch.float32 and state.dim() == 2 and state_off >= 0
                                            and state.shape[1] >= state_off + (taps - 1) * width), "residual_conv: state rows too short")
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    _i32(token_req, n, "token_req") if n else None
    out = torch.empty((subs, n, width), dtype=out_dtype, device=x.device)
    _call("tp_residual_conv", _ptr(x), _ptr(weight), _ptr(state), ctypes.c_size_t(0 if state is None else state.shape[1]), ctypes.c_size_t(state_off),
          _ptr(cu_seqlens), _ptr(token_req), _ptr(state_slots), _ptr(out), _dtcode(out_dtype), n, int(num_requests), width, taps, subs,
          _stream())
    return [out[i] for i in range(subs)]


def add_row(h: torch.Tensor, table: torch.Tensor, row: int) -> None:
    """h[t] += table[row] for every row t, in place (float32)."""
    if _backend is not None:
        return _backend.add_row(h, table, row)
    _dev_ok(h, table)
    _need(h.dtype == torch.float32 and h.dim() == 2 and table.dtype == torch.float32 and table.dim() == 2 and table.shape[1] == h.shape[1]
          and 0 <= row < table.shape[0], "add_row: h float32 [n, width], table float32 [rows, width]")
    _call("tp_add_row", _ptr(h), ctypes.c_void_p(table.data_ptr() + 4 * int(row) * table.shape[1]), h.shape[0], h.shape[1], _stream())


def general_delta_scan(proj: torch.Tensor, col0: int, decay: torch.Tensor, a_bias: torch.Tensor, state: torch.Tensor, state_off: int,
                       cu_seqlens: torch.Tensor, state_slots: torch.Tensor, num_requests: int, heads: int, dim: int,
                       unit_eps: float) -> torch.Tensor:
    """The generalized delta rule per head over each request's run.  ``proj`` float32 rows hold, from column ``col0``
    on, r | k | v | a_raw, each [heads * dim]; a = sigmoid(a_raw + a_bias); ``decay`` float32 [n, heads * dim].  With the
    unit key u = k / sqrt(sum k^2 + unit_eps) and S [dim, dim] per head (kept at ``state[slot, state_off:]`` column by
    column):  S <- diag(decay) S - (a u) (u^T S) + k v^T (both terms read the old S);  o = S^T r.
    Returns o float32 [n, heads * dim]; the state is left as the run leaves it."""
    if _backend is not None:
        return _backend.general_delta_scan(proj, col0, decay, a_bias, state, state_off, cu_seqlens, state_slots, num_requests, heads, dim, unit_eps)
    _dev_ok(proj, decay, a_bias, state, cu_seqlens, state_slots)
    n, hd = proj.shape[0], heads * dim
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and 0 <= col0 and col0 + 4 * hd <= proj.shape[1], "general_delta_scan: bad r | k | v | a rows")
    _need(decay.dtype == torch.float32 and tuple(decay.shape) == (n, hd), "general_delta_scan: decay must be float32 [n, heads * dim]")
    _need(a_bias.dtype == torch.float32 and a_bias.numel() == hd, "general_delta_scan: a_bias must be float32 [heads * dim]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state_off >= 0 and state.shape[1] >= state_off + hd * dim,
          "general_delta_scan: state rows too short")
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    y = torch.empty((n, hd), dtype=torch.float32, device=proj.device)
    scratch = torch.empty((max(1, n * 2 * hd + n * heads * 2),), dtype=torch.float32, device=proj.device)
    _call("tp_gdelta_scan", _ptr(proj), proj.shape[1], int(col0), _ptr(decay), _ptr(a_bias), _ptr(state), ctypes.c_size_t(state.shape[1]),
          ctypes.c_size_t(state_off), _ptr(cu_seqlens), _ptr(state_slots), _ptr(y), _ptr(scratch), n, int(num_requests), int(heads),
          int(dim), ctypes.c_float(unit_eps), _stream())
    return y


def latent_rows(proj: torch.Tensor, q_col0: int, rot_col0: int, up: torch.Tensor, heads: int, dim: int, rot: int, vdim: int) -> torch.Tensor:
    """The rows q | k | v that ``rope_kv_write`` takes, for an attention whose keys and values are expanded from a
    latent: q [heads, rot + dim] is columns q_col0 .. of ``proj`` (float32 rows) as they stand; head h's key is the
    shared part proj[:, rot_col0 : rot_col0 + rot] followed by up[:, h * dim : (h + 1) * dim]; its value
    up[:, heads * dim + h * vdim : ...].  ``up`` float32 [n, >= heads * (dim + vdim)].  Returns float32
    [n, 2 * heads * (rot + dim) + heads * vdim]."""
    if _backend is not None:
        return _backend.latent_rows(proj, q_col0, rot_col0, up, heads, dim, rot, vdim)
    _dev_ok(proj, up)
    n = proj.shape[0]
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and up.dtype == torch.float32 and up.dim() == 2 and up.shape[0] == n,
          "latent_rows: float32 rows")
    _need(0 <= q_col0 and q_col0 + heads * (rot + dim) <= proj.shape[1] and 0 <= rot_col0 and rot_col0 + rot <= proj.shape[1]
          and up.shape[1] >= heads * (dim + vdim), "latent_rows: rows too short")
    out = torch.empty((n, 2 * heads * (rot + dim) + heads * vdim), dtype=torch.float32, device=proj.device)
    _call("tp_latent_rows", _ptr(proj), ctypes.c_size_t(proj.shape[1]), int(q_col0), int(rot_col0), _ptr(up), ctypes.c_size_t(up.shape[1]),
          _ptr(out), n, int(heads), int(dim), int(rot), int(vdim), _stream())
    return out


def head_rmsnorm(rows: torch.Tensor, col_a: int, heads_a: int, weight_a: Optional[torch.Tensor], col_b: int, heads_b: int,
                 weight_b: Optional[torch.Tensor], dim: int, eps: float) -> None:
    """In place on float32 rows [n, wider]: each of the ``heads_a`` heads of ``dim`` columns from col_a on becomes
    x / sqrt(mean(x^2) + eps) * weight_a (float32 [dim], one for all heads), and likewise the ``heads_b`` heads from col_b
    on with weight_b (the queries and the keys of an attention in one launch)."""
    if _backend is not None:
        return _backend.head_rmsnorm(rows, col_a, heads_a, weight_a, col_b, heads_b, weight_b, dim, eps)
    _dev_ok(rows, weight_a, weight_b)
    _need(rows.dtype == torch.float32 and rows.dim() == 2, "head_rmsnorm: rows must be float32 [n, width]")
    for col, heads, w in ((col_a, heads_a, weight_a), (col_b, heads_b, weight_b)):
        _need(heads >= 0 and col >= 0 and col + heads * dim <= rows.shape[1], "head_rmsnorm: heads outside the rows")
        _need(heads == 0 or (w is not None and w.dtype == torch.float32 and w.numel() == dim), "head_rmsnorm: weight must be float32 [dim]")
    _call("tp_head_rmsnorm", _ptr(rows), ctypes.c_size_t(rows.shape[1]), int(col_a), int(heads_a), _ptr(weight_a), int(col_b), int(heads_b),
          _ptr(weight_b), int(dim), ctypes.c_float(eps), rows.shape[0], _stream())


def vector_store(c: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """One vector a token, ``c`` [n, dim], into cache place ``slots`` of keys [pages, 1, page_size, dim] and of transposed
    values [pages, 1, dim, page_size] (an attention whose keys are its values reads both)."""
    if _backend is not None:
        return _backend.vector_store(c, slots, k_cache, v_cache)
    _dev_ok(c, slots, k_cache, v_cache)
    _need(c.dim() == 2 and k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == 1, "vector_store: bad operand ranks")
    n, dim = c.shape
    pages, _, page_size, d2 = k_cache.shape
    _need(d2 == dim and tuple(v_cache.shape) == (pages, 1, dim, page_size), "vector_store: caches must be k [pages, 1, page_size, dim], v [pages, 1, dim, page_size]")
    _need(c.dtype == k_cache.dtype == v_cache.dtype, "vector_store: vector and cache types differ")
    _i32(slots, n, "slots") if n else None
    _call("tp_vector_store", _ptr(c), _dt(c), _ptr(slots), _ptr(k_cache), _ptr(v_cache), n, dim, page_size, _stream())


def mlstm_scan(proj: torch.Tensor, col0: int, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float, q_scale: float,
               state: torch.Tensor, state_off: int, cu_seqlens: torch.Tensor, state_slots: torch.Tensor, num_requests: int,
               heads: int, dim: int, vdim: int, norm_weight: torch.Tensor, eps: float, scale: float, out: torch.Tensor,
               out_col0: int) -> None:
    """The matrix-memory recurrence of an mLSTM mixer over each request's run of tokens, and its read-out as the rows
    of the output product.  ``proj`` float32 [n, wider] holds from col0 on [q | k | v | gate | i | f] (heads * dim,
    heads * dim, heads * vdim, heads * vdim, heads, heads columns).  With i = cap tanh((x_i + i_bias) / cap) and
    f = logsigmoid(cap tanh((x_f + f_bias) / cap)) per head: m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T;
    n' likewise with k alone; o = S'^T (q * q_scale) / (max(|n' . q|, e^(-m')) + 1e-6).  Then per head o over its root
    mean square (``eps``), times ``norm_weight`` [heads * vdim], times sigmoid(gate), times ``scale``, into columns
    out_col0 .. of ``out``.  A request's state (float32 row of ``state`` from state_off on, heads * (vdim + 1) * (dim + 1)
    numbers: per head the memory column by column with n as the last column, then a copy of m per column) is read and
    left updated."""
    if _backend is not None:
        return _backend.mlstm_scan(proj, col0, i_bias, f_bias, cap, q_scale, state, state_off, cu_seqlens, state_slots, num_requests,
                                   heads, dim, vdim, norm_weight, eps, scale, out, out_col0)
    _dev_ok(proj, i_bias, f_bias, state, cu_seqlens, state_slots, norm_weight, out)
    _need(proj.dtype == torch.float32 and proj.dim() == 2, "mlstm_scan: rows must be float32 [n, width]")
    n = proj.shape[0]
    width = 2 * heads * dim + 2 * heads * vdim + 2 * heads
    _need(0 <= col0 and col0 + width <= proj.shape[1], "mlstm_scan: rows too short")
    for b in (i_bias, f_bias):
        _need(b.dtype == torch.float32 and b.numel() == heads, "mlstm_scan: gate biases must be float32 [heads]")
    _need(norm_weight.dtype == torch.float32 and norm_weight.numel() == heads * vdim, "mlstm_scan: norm weight must be float32 [heads * vdim]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= state_off + heads * (vdim + 1) * (dim + 1),
          "mlstm_scan: state rows too short")
    _i32(cu_seqlens, num_requests + 1, "cu_seqlens")
    _i32(state_slots, num_requests, "state_slots")
    _need(out.dim() == 2 and out.shape[0] == n and 0 <= out_col0 and out_col0 + heads * vdim <= out.shape[1], "mlstm_scan: output rows too short")
    scratch = torch.empty((max(2, n * heads * (vdim + 4)),), dtype=torch.float32, device=proj.device)
    _call("tp_mlstm_scan", _ptr(proj), proj.shape[1], int(col0), _ptr(i_bias), _ptr(f_bias), ctypes.c_float(cap), ctypes.c_float(q_scale),
          _ptr(state), ctypes.c_size_t(state.shape[1]), ctypes.c_size_t(state_off), _ptr(cu_seqlens), _ptr(state_slots), _ptr(scratch),
          _ptr(norm_weight), ctypes.c_float(eps), ctypes.c_float(scale), _ptr(out), _dt(out), out.shape[1], int(out_col0), n,
          int(num_requests), int(heads), int(dim), int(vdim), _stream())
