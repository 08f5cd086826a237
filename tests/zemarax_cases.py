"""Small Zemarax configurations and random weights of the tests' own making (stored as bfloat16 values, so that the
float32 and the bfloat16 engine and the plain implementation all read the same numbers)."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import torch


def _attention(heads, kv, dim, vdim, scale, window=None, keep=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
        if keep is not None:
            m["mask"]["keep_first"] = keep
    return "attention", m


def _mlstm(heads, dim, vdim, cap):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _latent(heads, dim, vdim, rank, q_rank, scale, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "latent_attention", m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def _layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def _case(vocab, width, layers, eps, emb_scale, logit_scale, bigram, max_positions=256):
    return {"architecture": "Zemarax", "vocab": vocab, "width": width, "max_positions": max_positions, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "embedding": {"scale": emb_scale, "bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))},
            "layers": layers}


#: name -> config.json content
CASES: Dict[str, dict] = {
    # the three mixers and both feed-forwards; grouped key heads, values narrower than keys, a window shorter than the
    # prompts that keeps three first tokens; two borrowers of one layer's latents; an attention without a window; a layer
    # without a feed-forward; experts with and without the shared one
    "mix": _case(90, 48, [_layer(_mlstm(3, 10, 6, 8.0), _moe(16, 6, 2, shared=12)),
                          _layer(_latent(3, 8, 6, 20, 12, 0.4), _dense(40)),
                          _layer(_attention(4, 2, 12, 10, 0.3, window=9, keep=3), None),
                          _layer(_latent(2, 10, 14, 20, 9, 0.25, kv_from=1), _moe(24, 5, 3)),
                          _layer(_attention(2, 1, 8, 8, 0.35), _dense(24)),
                          _layer(_latent(4, 6, 4, 20, 16, 0.5, kv_from=1), None)], 1e-5, 2.5, 0.5, (61, 7, 13)),
    # values that a model may happen to make 1 or equal: one head, one key head, one expert a token, a shared expert only
    # worth its gate, scales of 1, a window of exactly one page that keeps nothing, a window that keeps more than it
    # spans, sizes that fill no power of two, attention first and the recurrence last
    "one": _case(40, 32, [_layer(_attention(1, 1, 20, 28, 0.2, window=16, keep=0), _moe(8, 4, 1, shared=8)),
                          _layer(_attention(3, 3, 6, 6, 0.4, window=5, keep=11), _dense(16)),
                          _layer(_latent(1, 7, 5, 11, 6, 0.3), _moe(16, 3, 3)),
                          _layer(_mlstm(1, 7, 5, 3.0), None)], 1e-6, 1.0, 1.0, (17, 3, 5)),
    # sizes the matrix-core kernels take: keys and values of 64, a latent of 96, a recurrence of 128 x 64 and one of
    # 32 x 128; sixteen experts; two layers with latents of their own (of different sizes) and a borrower of the second
    "wide": _case(96, 128, [_layer(_latent(4, 32, 32, 96, 64, 0.18), _moe(64, 16, 3, shared=32)),
                            _layer(_mlstm(2, 128, 64, 12.0), _dense(256)),
                            _layer(_attention(4, 2, 64, 64, 0.125, window=40, keep=8), _moe(32, 8, 2)),
                            _layer(_latent(2, 64, 32, 64, 32, 0.125), _dense(128)),
                            _layer(_mlstm(4, 32, 128, 6.0), None),
                            _layer(_latent(4, 16, 48, 64, 48, 0.25, kv_from=3), _dense(128))], 1e-5, 1.75, 1.5, (127, 29, 11), 512),
}


def config_json(name: str, every_expert: bool = False) -> dict:
    """The case as config.json would hold it.  ``every_expert``: each token uses all experts, so that no choice is
    there for a rounding to flip (for runs in bfloat16; the logits still weigh the experts)."""
    cfg = json.loads(json.dumps(CASES[name]))
    for layer in cfg["layers"]:
        if every_expert and layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return cfg


def make_weights(name: str, seed: int = 0, sharp: float = 1.0, cfg: dict = None) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by checkpoint name, drawn so that every mechanism matters to the logits.  ``sharp`` multiplies
    the queries of both attentions: with large values a query's softmax rests on one or two keys somewhere among those
    it sees, far ones as often as near ones (and the sink's share shrinks to nothing)."""
    cfg = cfg if cfg is not None else CASES[name]
    g = torch.Generator().manual_seed(seed)
    W: Dict[str, torch.Tensor] = {}

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g, dtype=torch.float64) * std + mean

    width = cfg["width"]
    W["embed"] = normal(cfg["vocab"], width, std=0.6)
    W["bigram"] = normal(cfg["embedding"]["bigram"]["buckets"] + 1, width, std=0.8)
    W["pos"] = normal(cfg["max_positions"], width, std=0.8)
    W["final.norm"] = normal(width, std=0.2)
    W["head"] = normal(cfg["vocab"], width, std=width ** -0.5)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if layer["mlp"] is not None else ()):
            W[f"{p}.{nm}"] = normal(width, std=0.2)
        kind, m = layer["type"], layer["mixer"]
        q = f"{p}.mix"
        if kind == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[q + ".q"] = normal(H * D, width, std=width ** -0.5)
            W[q + ".k"] = normal(G * D, width, std=width ** -0.5)
            W[q + ".v"] = normal(G * Dv, width, std=width ** -0.5)
            W[q + ".q.norm"] = normal(D, std=0.3, mean=sharp * 1.6)
            W[q + ".k.norm"] = normal(D, std=0.3, mean=1.6)
            W[q + ".sink"] = normal(H, std=1.0, mean=1.0)
            W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        elif kind == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            for nm, rows in (("q", H * D), ("k", H * D), ("v", H * Dv), ("g", H * Dv)):
                W[f"{q}.{nm}"] = normal(rows, width, std=1.3 * width ** -0.5)
            # gates that move: inputs spread over several units around zero, forgetting from nearly none to a lot
            W[q + ".i"] = normal(H, width, std=2.5 * width ** -0.5)
            W[q + ".i.b"] = normal(H, std=1.0)
            W[q + ".f"] = normal(H, width, std=2.5 * width ** -0.5)
            W[q + ".f.b"] = normal(H, std=1.0, mean=2.0)
            W[q + ".norm"] = normal(H * Dv, std=0.2, mean=1.0)
            W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        else:
            H, D, Dv, L, Q = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            W[q + ".dq"] = normal(Q, width, std=width ** -0.5)
            W[q + ".dq.norm"] = normal(Q, std=0.2, mean=1.0)
            W[q + ".uq"] = normal(H * D, Q, std=sharp * 1.5 * Q ** -0.5)
            if m.get("kv_from") is None:
                W[q + ".dkv"] = normal(L, width, std=width ** -0.5)
                W[q + ".dkv.norm"] = normal(L, std=0.2, mean=1.0)
            W[q + ".uk"] = normal(H * D, L, std=1.5 * L ** -0.5)
            W[q + ".uv"] = normal(H * Dv, L, std=L ** -0.5)
            W[q + ".sink"] = normal(H, std=1.0, mean=1.0)
            W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            W[f"{p}.mlp.gate"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.up"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.down"] = normal(width, ff, std=ff ** -0.5)
            continue
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        W[f"{p}.mlp.router"] = normal(E, width, std=2.0 * width ** -0.5)
        W[f"{p}.mlp.router.b"] = normal(E, std=1.0)
        for e in range(E):
            W[f"{p}.mlp.e{e}.up"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.e{e}.down"] = normal(width, ff, std=ff ** -0.5)
        if mlp.get("shared") is not None:
            sf = mlp["shared"]["ff"]
            W[f"{p}.mlp.shared.up"] = normal(sf, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.shared.down"] = normal(width, sf, std=sf ** -0.5)
            W[f"{p}.mlp.shared.sg"] = normal(1, width, std=2.0 * width ** -0.5)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def write_model(name: str, folder: str, seed: int = 0, weights=None, config=None) -> str:
    from tempura_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config if config is not None else config_json(name), f)
    W = weights if weights is not None else make_weights(name, seed)
    write_safetensors(os.path.join(folder, "model.safetensors"), W.items(), metadata={"format": "pt"})
    return folder


def tokens(name: str, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(4321 + seed)
    return torch.randint(0, CASES[name]["vocab"], (n,), generator=g).tolist()


#: request lengths per case: one token, a few, around pages' and windows' edges, long
LENGTHS = {"mix": {"m0": 1, "m1": 6, "m2": 23, "m3": 49, "m4": 33, "m5": 16},
           "one": {"o0": 2, "o1": 31, "o2": 17, "o3": 1, "o4": 40},
           "wide": {"w0": 5, "w1": 70, "w2": 33, "w3": 129, "w4": 48}}


def requests(name: str) -> Dict[str, List[int]]:
    return {rid: tokens(name, n, i) for i, (rid, n) in enumerate(LENGTHS[name].items())}
