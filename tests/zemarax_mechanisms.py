"""Each mechanism of the Zemarax design alone: the framework's part, taken out of a loaded model and run on random
rows through the step's own context, cache and state, against the plain function of tests/plain_zemarax.py for it.
Used by the host tests (over the stand-in operations) and by the GPU tests (over the kernels)."""
from __future__ import annotations

import torch

import plain_zemarax as plain
import zemarax_cases as cases


def _err(got, ref):
    got, ref = got.double().cpu(), ref.double()
    return float((got - ref).abs().max() / ref.abs().max())


def check(folder: str, name: str, device: str, tol: float, seed: int = 0, cuts=(0, 21, 23, 37, 38), dtype: str = "float32", cfg=None,
          W=None) -> None:
    """Asserts, for every layer of case ``name``: the mixer and the feed-forward alone, as a prompt cut at ``cuts`` (so
    that states and cached keys cross the steps' borders, the last step being one token), and the embedding."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    cfg = cfg if cfg is not None else cases.config_json(name)
    W = W if W is not None else cases.make_weights(name)
    W64 = {k: v.double() for k, v in W.items()}
    model = load_model(folder, dtype, device)
    runner = ModelRunner(model, 16, 8, max_requests=2)
    g = torch.Generator().manual_seed(seed)
    n = cuts[-1]
    toks = cases.tokens(name, n, 3)
    eps = float(cfg["norm"]["eps"])
    x = torch.randn(n, cfg["width"], generator=g)
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    runner.add_request("r")
    outs = {}
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        tok_dev, ctx = runner._pack_step([StepEntry("r", toks[lo:hi], [])])
        runner._clear_state([s for s, q, c in zip(ctx.state_slot_list, ctx.q_lens, ctx.ctx_lens) if c == q])
        rows = x[lo:hi].to(device=device, dtype=model.dtype)
        outs.setdefault("embed", []).append(model.embedding.forward(tok_dev, ctx.positions, 1, ctx=ctx,
                                                                    state=runner.pools.state[model.EMBEDDING_STATE]).cpu())
        for i, block in enumerate(model.layers):
            cache = runner.layer_caches[i]
            outs.setdefault((i, "mixer"), []).append(block.mixer.forward(rows, ctx, cache, None).cpu())
            if block.ffn is not None:
                outs.setdefault((i, "ffn"), []).append(block.ffn.forward(rows, ctx).cpu())
        runner.cache.commit_many(["r"], ctx.q_lens)
    xd = x.double()
    assert _err(torch.cat(outs["embed"]), plain.embed(toks, W64, cfg)) < min(tol, 1e-5), "embedding"
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        kind, c = layer["type"], layer["mixer"]
        if kind == "attention":
            ref = plain.attention(xd, W64, p + ".mix", c, eps)
        elif kind == "mlstm":
            ref = plain.mlstm(xd, W64, p + ".mix", c, eps)
        else:
            src = c.get("kv_from")
            if src is None:
                latents[i] = plain.latent_of(xd, W64, p + ".mix", eps)
                src = i
            ref = plain.latent_attention(xd, W64, p + ".mix", c, eps, latents[src])
        assert _err(torch.cat(outs[(i, "mixer")]), ref) < tol, f"layer {i}: {kind}"
        if layer["mlp"] is not None:
            ref = plain.dense_ff(xd, W64, p + ".mlp") if layer["mlp"]["kind"] == "dense" else plain.moe_ff(xd, W64, p + ".mlp", layer["mlp"])
            assert _err(torch.cat(outs[(i, "ffn")]), ref) < tol, f"layer {i}: feed-forward"
