"""The Zemarax design written out plainly in float64, one function per mechanism, token by token where the design
is recurrent.  It shares no code with the product: tensors come as a dict name -> tensor, the configuration as the
dict that config.json holds.  Slow on purpose.

Notation: x is the residual stream [T, W]; u is a sublayer's input (the normed stream); a layer is
x += post1(mixer(pre1(x))), then x += post2(ff(pre2(x))) when it has a feed-forward.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    """x over the root of (mean of squares + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# ---- embedding --------------------------------------------------------------------------------------------
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the hashed pair table for every token; a sequence's first token reads the row behind the buckets."""
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((int(a) * mul_prev + int(b) * mul_cur) % buckets)
    return rows


def embed(tokens, W, cfg):
    e = cfg["embedding"]
    bg = e["bigram"]
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] * float(e["scale"])
    x = x + W["bigram"][torch.tensor(bigram_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"]))]
    return x + W["pos"][:T]


# ---- softmax with a sink and a mask -------------------------------------------------------------------------
def visible(T, window=None, keep_first=0):
    """Boolean [T, T]: query i sees key j when j <= i and (no window, or i - j < window, or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def sink_softmax(scores, mask, sink):
    """scores [H, T, T], mask [T, T], sink [H]: softmax over the visible keys and one more term exp(sink) that
    has no value (it only enlarges the denominator)."""
    H, T, _ = scores.shape
    s = scores.masked_fill(~mask[None], -math.inf)
    full = torch.cat([s, sink.reshape(H, 1, 1).expand(H, T, 1)], dim=-1)
    return torch.softmax(full, dim=-1)[..., :T]


# ---- mixer: attention -----------------------------------------------------------------------------------------
def attention(u, W, p, c, eps):
    T = u.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (u @ W[p + ".q"].T).reshape(T, H, D)
    k = (u @ W[p + ".k"].T).reshape(T, G, D)
    v = (u @ W[p + ".v"].T).reshape(T, G, Dv)
    q = unit_rms(q, eps) * W[p + ".q.norm"]
    k = unit_rms(k, eps) * W[p + ".k.norm"]
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * float(c["scale"])
    mask = c.get("mask")
    ok = visible(T, None if mask is None else int(mask["size"]), 0 if mask is None else int(mask.get("keep_first", 0)))
    prob = sink_softmax(scores, ok, W[p + ".sink"])
    o = torch.einsum("hij,jhd->ihd", prob, v).reshape(T, H * Dv)
    return o @ W[p + ".o"].T


# ---- mixer: mlstm ---------------------------------------------------------------------------------------------
def mlstm_chain(q, k, v, i_log, f_log):
    """q, k [T, H, D]; v [T, H, Dv]; i_log, f_log [T, H].  Matrix memory S [D, Dv], normaliser n [D] and a running
    maximum m per head, all from zero: m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T; n' likewise with
    k; read-out S'^T q over (max(|n' . q|, e^(-m')) + 1e-6)."""
    T, H, D = q.shape
    Dv = v.shape[2]
    S = torch.zeros(H, D, Dv, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    m = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(f_log[t] + m, i_log[t])
        keep = torch.exp(f_log[t] + m - m_new)
        put = torch.exp(i_log[t] - m_new)
        S = keep[:, None, None] * S + put[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + put[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    return out


def mlstm(u, W, p, c, eps):
    T = u.shape[0]
    H, D, Dv, cap = c["heads"], c["dim"], c["vdim"], float(c["gate_cap"])
    q = (u @ W[p + ".q"].T).reshape(T, H, D) * D ** -0.5
    k = (u @ W[p + ".k"].T).reshape(T, H, D)
    v = (u @ W[p + ".v"].T).reshape(T, H, Dv)
    i_log = cap * torch.tanh((u @ W[p + ".i"].T + W[p + ".i.b"]) / cap)
    f_log = torch.nn.functional.logsigmoid(cap * torch.tanh((u @ W[p + ".f"].T + W[p + ".f.b"]) / cap))
    o = unit_rms(mlstm_chain(q, k, v, i_log, f_log), eps).reshape(T, H * Dv) * W[p + ".norm"]
    o = o * torch.sigmoid(u @ W[p + ".g"].T)
    return o @ W[p + ".o"].T


# ---- mixer: latent_attention ------------------------------------------------------------------------------------
def latent_of(u, W, p, eps):
    """The compressed vector a token leaves behind: the normed down projection."""
    return unit_rms(u @ W[p + ".dkv"].T, eps) * W[p + ".dkv.norm"]


def latent_attention(u, W, p, c, eps, latent):
    """``latent`` [T, R]: this layer's own, or the one of the layer it borrows from."""
    T = u.shape[0]
    H, D, Dv = c["heads"], c["dim"], c["vdim"]
    cq = unit_rms(u @ W[p + ".dq"].T, eps) * W[p + ".dq.norm"]
    q = (cq @ W[p + ".uq"].T).reshape(T, H, D)
    k = (latent @ W[p + ".uk"].T).reshape(T, H, D)
    v = (latent @ W[p + ".uv"].T).reshape(T, H, Dv)
    scores = torch.einsum("ihd,jhd->hij", q, k) * float(c["scale"])
    prob = sink_softmax(scores, visible(T), W[p + ".sink"])
    o = torch.einsum("hij,jhd->ihd", prob, v).reshape(T, H * Dv)
    return o @ W[p + ".o"].T


# ---- feed-forwards --------------------------------------------------------------------------------------------------
def dense_ff(u, W, p):
    return (silu(u @ W[p + ".gate"].T) * (u @ W[p + ".up"].T)) @ W[p + ".down"].T


def plain_expert(u, W, p):
    return gelu_erf(u @ W[p + ".up"].T) @ W[p + ".down"].T


def route(u, W, p, top):
    """(ids [T, top], weights [T, top]): the ``top`` largest logits (the lower index wins a tie) and a softmax over
    those logits alone."""
    z = u @ W[p + ".router"].T + W[p + ".router.b"]
    T, E = z.shape
    ids = torch.zeros(T, top, dtype=torch.long)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))
        ids[t] = torch.tensor(order[:top])
    chosen = torch.gather(z, 1, ids)
    return ids, torch.softmax(chosen, dim=-1)


def moe_ff(u, W, p, c):
    T = u.shape[0]
    top = int(c["router"]["top"])
    ids, weights = route(u, W, p, top)
    y = torch.zeros(T, W[p + ".e0.down"].shape[0], dtype=F64)
    for t in range(T):
        for j in range(top):
            y[t] += weights[t, j] * plain_expert(u[t: t + 1], W, f"{p}.e{int(ids[t, j])}")[0]
    if c.get("shared") is not None:
        y = y + torch.sigmoid(u @ W[p + ".shared.sg"].T) * plain_expert(u, W, p + ".shared")
    return y


# ---- the model ----------------------------------------------------------------------------------------------
def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after every layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, W, cfg)
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        p, c = f"l{i}", layer["mixer"]
        u = norm_around_zero(x, W[p + ".norm1"], eps)
        if layer["type"] == "attention":
            y = attention(u, W, p + ".mix", c, eps)
        elif layer["type"] == "mlstm":
            y = mlstm(u, W, p + ".mix", c, eps)
        elif layer["type"] == "latent_attention":
            src = c.get("kv_from")
            if src is None:
                latents[i] = latent_of(u, W, p + ".mix", eps)
                src = i
            y = latent_attention(u, W, p + ".mix", c, eps, latents[src])
        else:
            raise ValueError(layer["type"])
        x = x + norm_around_zero(y, W[p + ".norm1b"], eps)
        if layer.get("mlp") is not None:
            u = norm_around_zero(x, W[p + ".norm2"], eps)
            y = dense_ff(u, W, p + ".mlp") if layer["mlp"]["kind"] == "dense" else moe_ff(u, W, p + ".mlp", layer["mlp"])
            x = x + norm_around_zero(y, W[p + ".norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = norm_around_zero(x, W["final.norm"], eps)
    return (x @ W["head"].T) * float(cfg.get("logit_scale", 1.0))


def greedy(config, weights, prompt, n_new):
    """The tokens that greedy decoding appends to ``prompt`` (the whole sequence is run anew for every token)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(config, weights, toks)[-1])))
    return toks[len(prompt):]


def logit_error(got, ref):
    """Largest difference between two sets of logits after taking each row's mean off, relative to the reference's
    spread."""
    g, r = got.to(F64).cpu(), ref.to(F64)
    d = (g - g.mean(-1, keepdim=True)) - (r - r.mean(-1, keepdim=True))
    return float(d.abs().max() / r.std())
