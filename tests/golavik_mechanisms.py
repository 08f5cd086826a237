"""Each mechanism of the Golavik design alone: the framework's part, taken out of a loaded model and run on random
rows through the step's own context, cache and state, against the plain function of tests/plain_golavik.py for it.
Used by the host tests (over the stand-in operations) and by the GPU tests (over the kernels)."""
from __future__ import annotations

import torch

import golavik_cases as cases
import plain_golavik as plain


def _err(got, ref):
    got, ref = got.double().cpu(), ref.double()
    return float((got - ref).abs().max() / ref.abs().max())


def check(folder: str, name: str, device: str, tol: float, seed: int = 0, cuts=(0, 21, 23, 37)) -> None:
    """Asserts, for every layer of case ``name``: the norm, the convolved inputs, the mixer and the feed-forward alone,
    as a prompt cut at ``cuts`` (so that carried rows, states and cached keys cross the steps' borders)."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    cfg, W = cases.config_json(name), cases.make_weights(name)
    W64 = {k: v.double() for k, v in W.items()}
    model = load_model(folder, "float32", device)
    runner = ModelRunner(model, 16, 8, max_requests=2)
    g = torch.Generator().manual_seed(seed)
    n = cuts[-1]
    toks = cases.tokens(name, n, 3)
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"])
    x = torch.randn(n, cfg["width"], generator=g)
    first_call = {c.layer: i for i, c in reversed(list(enumerate(model.order)))}
    runner.add_request("r")
    outs = {}
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        tok_dev, ctx = runner._pack_step([StepEntry("r", toks[lo:hi], [])])
        runner._clear_state([s for s, q, c in zip(ctx.state_slot_list, ctx.q_lens, ctx.ctx_lens) if c == q])
        rows = x[lo:hi].to(device)
        for i, block in enumerate(model.layers):
            cache = runner.layer_caches[first_call[i]]
            outs.setdefault((i, "norm"), []).append(block.norm.forward(rows, out_dtype=torch.float32).cpu())
            ins = block.inputs.forward(rows, ctx, cache)
            outs.setdefault((i, "in0"), []).append(ins[0].cpu())
            if len(ins) > 1:
                outs.setdefault((i, "in1"), []).append(ins[1].cpu())
            outs.setdefault((i, "mixer"), []).append(block.mixer.forward(rows, ctx, cache).cpu())
            if block.ffn is not None:
                outs.setdefault((i, "ffn"), []).append(block.ffn.forward(rows, ctx).cpu())
        runner.cache.commit_many(["r"], ctx.q_lens)
    xd, pos = x.double(), torch.arange(n)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        assert _err(torch.cat(outs[(i, "norm")]), plain.group_norm(xd, W64[p + ".norm1"], eps, groups)) < tol, f"layer {i}: norm"
        assert _err(torch.cat(outs[(i, "in0")]), xd + plain.time_conv(xd, W64[p + ".canon1"])) < tol, f"layer {i}: mixer input"
        kind, c = layer["type"], layer["mixer"]
        if kind == "channel_delta":
            ref = plain.channel_delta(xd, W64, p + ".mix", c, eps)
        elif kind == "general_delta":
            ref = plain.general_delta(xd, W64, p + ".mix", c, eps)
        else:
            ref = plain.latent_attention(xd, W64, p + ".mix", c, eps, pos)
        assert _err(torch.cat(outs[(i, "mixer")]), ref) < tol, f"layer {i}: {kind}"
        if layer["mlp"] is not None:
            assert _err(torch.cat(outs[(i, "in1")]), xd + plain.time_conv(xd, W64[p + ".canon2"])) < tol, f"layer {i}: feed-forward input"
            assert _err(torch.cat(outs[(i, "ffn")]), plain.moe(xd, W64, p + ".mlp", layer["mlp"])) < tol, f"layer {i}: feed-forward"
