"""The Golavik design written out plainly in float64, one function per mechanism, token by token where the design
is recurrent.  It shares no code with the product: tensors come as a dict name -> tensor, the configuration as the
dict that config.json holds.  Slow on purpose.

Notation: x is the residual stream [T, W]; n = norm(x) is what a layer's two sublayers both start from; each
sublayer reads n + conv(n) with a convolution of its own over time.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def group_norm(x, w, eps, groups):
    """x [T, W] split into ``groups`` equal consecutive parts, each divided by its own root mean square."""
    T, W = x.shape
    p = x.reshape(T, groups, W // groups)
    p = p / torch.sqrt((p * p).mean(dim=-1, keepdim=True) + eps)
    return p.reshape(T, W) * w


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def time_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j: j + T] * w[:, j]
    return y


# ---- mixer: channel_delta ------------------------------------------------------------------------------
def gated_delta_chain(q, k, v, beta, g):
    """q, k, g [T, H, D]; v [T, H, Dv]; beta [T, H].  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=F64)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def channel_delta(h, W, p, c, eps):
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(time_conv(h @ W[p + ".q"].T, W[p + ".q.conv"])).reshape(T, G, D)
    k = silu(time_conv(h @ W[p + ".k"].T, W[p + ".k.conv"])).reshape(T, G, D)
    v = silu(time_conv(h @ W[p + ".v"].T, W[p + ".v.conv"])).reshape(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(h @ W[p + ".b"].T)
    step = torch.nn.functional.softplus((h @ W[p + ".a1"].T) @ W[p + ".a2"].T + W[p + ".dt_bias"]).reshape(T, H, D)
    g = torch.exp(-torch.exp(W[p + ".A_log"])[None, :, None] * step)
    o = gated_delta_chain(q, k, v, beta, g)
    o = rms(o, eps) * W[p + ".norm"]
    o = o.reshape(T, H * Dv) * torch.sigmoid((h @ W[p + ".g1"].T) @ W[p + ".g2"].T)
    return o @ W[p + ".o"].T


# ---- mixer: general_delta ------------------------------------------------------------------------------
def general_delta_chain(r, k, v, w, a):
    """All [T, H, D].  With the unit key u: S <- diag(w) S - (a u) (u^T S) + k v^T (both read the old S); o = S^T r."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=F64)
    out = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        seen = torch.einsum("hd,hdv->hv", u, S)
        S = w[t][:, :, None] * S - (a[t] * u)[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, r[t])
    return out


def general_delta(h, W, p, c, eps):
    T = h.shape[0]
    H, D = c["heads"], c["dim"]
    r = (h @ W[p + ".r"].T).reshape(T, H, D)
    k = (h @ W[p + ".k"].T).reshape(T, H, D)
    v = (h @ W[p + ".v"].T).reshape(T, H, D)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W[p + ".w1"].T) @ W[p + ".w2"].T + W[p + ".w0"])).reshape(T, H, D)
    a = torch.sigmoid(h @ W[p + ".a"].T + W[p + ".a.b"]).reshape(T, H, D)
    o = rms(general_delta_chain(r, k, v, w, a), eps).reshape(T, H * D) * W[p + ".norm"]
    o = o * torch.sigmoid(h @ W[p + ".g"].T)
    return o @ W[p + ".o"].T


# ---- mixer: latent_attention ---------------------------------------------------------------------------
def yarn_frequencies(dims, base, scaling):
    """(frequencies [dims / 2], magnitude of cos and sin)."""
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def corr(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(corr(float(scaling["fast"]))), 0)
    hi = min(math.ceil(corr(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, mag):
    """x [T, ..., dims]: element 2i rotates with element 2i + 1 by the angle position * freqs[i]."""
    ang = positions.to(F64)[:, None] * freqs[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [freqs.shape[0]]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, v = x[..., 0::2], x[..., 1::2]
    return torch.stack([u * c - v * s, v * c + u * s], dim=-1).reshape(x.shape)


def latent_attention(h, W, p, c, eps, positions):
    T = h.shape[0]
    H, D, R, Dv, L = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    q = (h @ W[p + ".q"].T).reshape(T, H, D + R)
    down = h @ W[p + ".dkv"].T
    lat = rms(down[:, :L], eps) * W[p + ".dkv.norm"]
    f, mag = yarn_frequencies(R, float(c["rot"]["base"]), c["rot"].get("scaling"))
    k_rot = rotate_pairs(down[:, L:], positions, f, mag)                  # [T, R], one for all heads
    q_rot = rotate_pairs(q[..., D:], positions, f, mag)
    k_plain = (lat @ W[p + ".uk"].T).reshape(T, H, D)
    v = (lat @ W[p + ".uv"].T).reshape(T, H, Dv)
    window = c.get("mask", {}).get("size") if c.get("mask") else None
    i = torch.arange(T)
    hidden = i[None, :] > i[:, None]
    if window:
        hidden = hidden | (i[:, None] - i[None, :] >= window)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :D] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * float(c["scale"])
        out[:, hd] = torch.softmax(s.masked_fill(hidden, float("-inf")), dim=-1) @ v[:, hd]
    a = out.reshape(T, H * Dv) * torch.sigmoid(h @ W[p + ".g"].T)
    return a @ W[p + ".o"].T


# ---- feed-forward ----------------------------------------------------------------------------------------
def route(h, W, p, r):
    """(chosen experts [T, top], their weights [T, top]): sigmoid scores, a group's score is the sum of its two
    largest, only the best groups' experts can be chosen; weights are the chosen scores over their sum, times a
    constant."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ W[p + ".router"].T)
    choice = s.clone()
    groups = r.get("groups")
    if groups is not None:
        per = E // groups["count"]
        best = torch.topk(s.reshape(-1, groups["count"], per), min(2, per), dim=-1).values.sum(-1)
        keep = torch.topk(best, groups["keep"], dim=-1).indices
        allowed = torch.zeros(h.shape[0], groups["count"], dtype=torch.bool)
        allowed.scatter_(1, keep, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    idx = torch.topk(choice, top, dim=-1).indices
    wts = torch.gather(s, 1, idx)
    return idx, wts / (wts.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))


def moe(h, W, p, mlp):
    idx, wts = route(h, W, p, mlp["router"])
    out = torch.zeros(h.shape[0], W[p + ".e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wts[t]):
            q = f"{p}.e{e}"
            out[t] += w * ((silu(h[t] @ W[q + ".gate"].T) * (h[t] @ W[q + ".up"].T)) @ W[q + ".down"].T)
    return out


# ---- the model -------------------------------------------------------------------------------------------
def run_order(config):
    """[(layer index, pass number or None, first of its pass)] in the order the layers run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None, False) for i in range(a)]
    for t in range(times):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def layer(x, W, i, L, config, positions):
    eps, groups = float(config["norm"]["eps"]), int(config["norm"].get("groups", 1))
    p = f"l{i}"
    n = group_norm(x, W[p + ".norm1"], eps, groups)
    hm = n + time_conv(n, W[p + ".canon1"])
    kind, c = L["type"], L["mixer"]
    if kind == "channel_delta":
        y = channel_delta(hm, W, p + ".mix", c, eps)
    elif kind == "general_delta":
        y = general_delta(hm, W, p + ".mix", c, eps)
    elif kind == "latent_attention":
        y = latent_attention(hm, W, p + ".mix", c, eps, positions)
    else:
        raise ValueError(kind)
    if L.get("mlp") is not None:
        hf = n + time_conv(n, W[p + ".canon2"])
        y = y + moe(hf, W, p + ".mlp", L["mlp"])
    return x + y


def forward(config, weights, tokens, layer_outputs=None):
    """Logits [T, vocab] of one whole sequence; ``layer_outputs`` (a list) receives the residual stream after
    every layer run."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    x = W["embed"][torch.tensor(list(tokens))]
    positions = torch.arange(len(tokens))
    for i, t, first in run_order(config):
        if first:
            x = x + W["loop.step"][t]
        x = layer(x, W, i, config["layers"][i], config, positions)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    eps, groups = float(config["norm"]["eps"]), int(config["norm"].get("groups", 1))
    return group_norm(x, W["final.norm"], eps, groups) @ W["embed"].T


def greedy(config, weights, prompt, n_new):
    """The tokens that greedy decoding appends to ``prompt`` (the whole sequence is run anew for every token)."""
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(config, weights, toks)[-1])))
    return toks[len(prompt):]


def logit_error(got, ref):
    """Largest difference between two sets of logits after taking each row's mean off, relative to the reference's
    spread."""
    g, r = got.to(F64), ref.to(F64)
    d = (g - g.mean(-1, keepdim=True)) - (r - r.mean(-1, keepdim=True))
    return float(d.abs().max() / r.std())
