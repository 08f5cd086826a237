"""Small Golavik configurations and random weights of the tests' own making (stored as bfloat16 values, so that the
float32 and the bfloat16 engine and the plain implementation all read the same numbers)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List

import torch


def _channel(heads, kv, dim, vdim, conv, ra, rg):
    return "channel_delta", {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "_ranks": (ra, rg)}


def _general(heads, dim, rw):
    return "general_delta", {"heads": heads, "dim": dim, "_ranks": (rw,)}


def _latent(heads, dim, rot, vdim, rank, window, base=10000.0, scaling=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "rot": {"dims": rot, "base": base},
         "scale": scale if scale is not None else (dim + rot) ** -0.5}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        m["mask"] = {"size": window}
    return "latent_attention", m


def _moe(ff, experts, top, scale, groups=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def _layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def _case(vocab, width, layers, taps, groups, eps, loop=None):
    d = {"architecture": "Golavik", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "canon": {"taps": taps},
         "layers": layers}
    if loop:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


#: name -> config.json content ("_ranks": ranks of a mixer's low-rank projections, sizes only the tensors say)
CASES: Dict[str, dict] = {
    # the three mixers, the middle two run three times; grouped key heads; a window shorter than the prompts, rotation
    # with scaling; a layer without a feed-forward; experts in three groups of which two are kept
    "trio": _case(90, 48, [_layer(_channel(4, 2, 12, 10, 2, 5, 7), _moe(16, 6, 2, 1.7, (3, 2))),
                           _layer(_general(3, 10, 4), _moe(24, 6, 3, 0.6, (2, 1))),
                           _layer(_latent(3, 8, 4, 6, 20, 9, base=5000.0, scaling=(4.0, 64, 8.0, 1.0), scale=0.4), None),
                           _layer(_channel(2, 2, 20, 18, 4, 9, 3), _moe(16, 6, 2, 1.7, (3, 2)))], 3, 3, 1e-5, loop=(1, 3, 3)),
    # no loop, one norm group, one tap (nothing carried), no expert groups, one expert a token, weights times 1, one head,
    # a window of one page, a key size that fills no power of two, groups of one expert
    "solo": _case(40, 32, [_layer(_general(1, 20, 2), _moe(16, 4, 1, 1.0)),
                           _layer(_latent(2, 6, 2, 12, 7, 16, base=100.0), _moe(8, 5, 2, 1.0, (5, 3))),
                           _layer(_channel(1, 1, 7, 5, 1, 3, 2), None)], 1, 1, 1e-6),
    # sizes the matrix-core kernels take, the whole model run twice: keys of 64 + 32 under values as wide, a general
    # delta rule of 64, a channel delta rule with keys of 128; eight experts in four groups; four taps
    "wide": _case(96, 128, [_layer(_latent(4, 64, 32, 96, 64, 40, base=500000.0, scaling=(6.0, 128, 16.0, 2.0), scale=0.11),
                                   _moe(64, 8, 3, 2.0, (4, 2))),
                            _layer(_general(2, 64, 16), _moe(32, 8, 2, 1.5, (2, 1))),
                            _layer(_channel(4, 2, 128, 64, 3, 16, 8), _moe(64, 8, 3, 2.0, (4, 2)))], 4, 2, 1e-5, loop=(0, 3, 2)),
}


def config_json(name: str, every_expert: bool = False) -> dict:
    """The case as config.json would hold it (without the tests' private keys).  ``every_expert``: each token uses
    all experts, without groups, so that no choice is there for a rounding to flip (for runs in bfloat16; the scores
    still weigh the experts)."""
    cfg = json.loads(json.dumps(CASES[name]))
    for layer in cfg["layers"]:
        layer["mixer"].pop("_ranks", None)
        if every_expert and layer["mlp"] is not None:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
            layer["mlp"]["router"].pop("groups", None)
    return cfg


def make_weights(name: str, seed: int = 0, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by checkpoint name, drawn so that every mechanism matters to the logits.  ``sharp`` multiplies
    the attention's query projections: with large values a query's softmax rests on one or two keys somewhere in its
    window, far ones as often as near ones."""
    cfg = CASES[name]
    g = torch.Generator().manual_seed(seed)
    W: Dict[str, torch.Tensor] = {}

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g, dtype=torch.float64) * std + mean

    width, taps = cfg["width"], cfg["canon"]["taps"]
    W["embed"] = normal(cfg["vocab"], width)
    W["final.norm"] = normal(width, std=0.2, mean=1.0)
    if "loop" in cfg:
        W["loop.step"] = normal(cfg["loop"]["times"], width, std=0.8)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        W[f"{p}.norm1"] = normal(width, std=0.2, mean=1.0)
        W[f"{p}.canon1"] = normal(width, taps, std=0.5)
        kind, m = layer["type"], layer["mixer"]
        q = f"{p}.mix"
        if kind == "channel_delta":
            H, G, D, Dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            ra, rg = m["_ranks"]
            for nm, ch in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                W[f"{q}.{nm}"] = normal(ch, width, std=width ** -0.5)
                W[f"{q}.{nm}.conv"] = normal(ch, K, std=0.5)
            W[q + ".b"] = normal(H, width, std=width ** -0.5)
            W[q + ".A_log"] = torch.log(torch.rand(H, generator=g, dtype=torch.float64) * 1.5 + 0.05)
            W[q + ".dt_bias"] = normal(H * D, std=0.8, mean=-1.5)
            W[q + ".a1"] = normal(ra, width, std=width ** -0.5)
            W[q + ".a2"] = normal(H * D, ra, std=ra ** -0.5)
            W[q + ".g1"] = normal(rg, width, std=width ** -0.5)
            W[q + ".g2"] = normal(H * Dv, rg, std=rg ** -0.5)
            W[q + ".norm"] = normal(Dv, std=0.2, mean=1.0)
            W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        elif kind == "general_delta":
            H, D = m["heads"], m["dim"]
            (rw,) = m["_ranks"]
            for nm in ("r", "k", "v", "g", "a"):
                W[f"{q}.{nm}"] = normal(H * D, width, std=width ** -0.5)
            W[q + ".a.b"] = normal(H * D, std=0.7, mean=0.3)
            W[q + ".w1"] = normal(rw, width, std=width ** -0.5)
            W[q + ".w2"] = normal(H * D, rw, std=2.0 * rw ** -0.5)
            W[q + ".w0"] = normal(H * D, std=1.5, mean=-1.0)
            W[q + ".norm"] = normal(H * D, std=0.2, mean=1.0)
            W[q + ".o"] = normal(width, H * D, std=(H * D) ** -0.5)
        else:
            H, D, R, Dv, L = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[q + ".q"] = normal(H * (D + R), width, std=sharp * 1.5 * width ** -0.5)
            W[q + ".dkv"] = normal(L + R, width, std=1.5 * width ** -0.5)
            W[q + ".dkv.norm"] = normal(L, std=0.2, mean=1.0)
            W[q + ".uk"] = normal(H * D, L, std=1.5 * L ** -0.5)
            W[q + ".uv"] = normal(H * Dv, L, std=L ** -0.5)
            W[q + ".g"] = normal(H * Dv, width, std=width ** -0.5)
            W[q + ".o"] = normal(width, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        W[f"{p}.canon2"] = normal(width, taps, std=0.5)
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        W[f"{p}.mlp.router"] = normal(E, width, std=2.0 * width ** -0.5)
        for e in range(E):
            W[f"{p}.mlp.e{e}.gate"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.e{e}.up"] = normal(ff, width, std=1.5 * width ** -0.5)
            W[f"{p}.mlp.e{e}.down"] = normal(width, ff, std=ff ** -0.5)
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
    g = torch.Generator().manual_seed(8765 + seed)
    return torch.randint(0, CASES[name]["vocab"], (n,), generator=g).tolist()


#: request lengths per case: one token, a few, around pages' and windows' edges, long
LENGTHS = {"trio": {"t0": 1, "t1": 6, "t2": 23, "t3": 49, "t4": 33, "t5": 16},
           "solo": {"s0": 2, "s1": 31, "s2": 17, "s3": 1, "s4": 40},
           "wide": {"w0": 5, "w1": 70, "w2": 33, "w3": 129, "w4": 48}}


def requests(name: str) -> Dict[str, List[int]]:
    return {rid: tokens(name, n, i) for i, (rid, n) in enumerate(LENGTHS[name].items())}
