"""The Zemarax design through the engine's own model, cache and state manager, step function and scheduler on the
host: the kernel operations are replaced by their plain PyTorch stand-ins (tests/emu_ops.py), the expected values
come from the plain implementation in tests/plain_zemarax.py.  A difference here is a fault of the configuration,
the parts, the cache, the state slots or the batch."""
import copy
import json

import pytest
import torch

import helpers
import plain_zemarax as plain
import zemarax_cases as cases
from emu_ops import EmuOps

TOL = 2e-5      # float32 storage of activations against float64


@pytest.fixture(autouse=True)
def host_ops():
    from tempura_amd.kernels import ops
    ops.set_backend(EmuOps())
    yield
    ops.set_backend(None)


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("zemarax")
    return {name: cases.write_model(name, str(root / name)) for name in cases.CASES}


def _runner(folder, max_tokens, page_size=16, max_requests=4):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(folder, "float32", "cpu")
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests)


def _plain(name):
    return cases.config_json(name), cases.make_weights(name)


# ---- configuration ------------------------------------------------------------------------------
def test_config_reads_every_size_and_writes_it_back():
    from tempura_amd.config import ConfigError
    from tempura_amd.config.zemarax import ZemaraxConfig
    from tempura_amd.parts.inventory import expected_weights
    for name in cases.CASES:
        d = cases.config_json(name)
        cfg = ZemaraxConfig.from_dict(d)
        assert ZemaraxConfig.from_json(cfg.to_json()) == cfg
        assert cfg.width == d["width"] and cfg.vocab == d["vocab"] and cfg.logit_scale == d["logit_scale"]
        assert cfg.embedding_scale == d["embedding"]["scale"] and cfg.norm_eps == d["norm"]["eps"]
        want = {k: tuple(v.shape) for k, v in cases.make_weights(name).items()}
        got = {k: v for k, v in expected_weights(cfg.build_spec()).items() if v.init != "skip"}
        assert set(got) == set(want)
        for k, info in got.items():
            assert all(e is None or e == f for e, f in zip(info.shape, want[k])) and len(info.shape) == len(want[k]), k
    spec = ZemaraxConfig.from_dict(cases.config_json("mix")).build_spec()
    # the borrowers name the lender's cache slot; everybody else has a slot of their own
    assert [c.cache for c in spec.order] == [None, 1, None, 1, None, 1]
    for change in (lambda c: c["layers"][0].__setitem__("type", "lstm"),
                   lambda c: c["layers"][2]["mixer"].__setitem__("kv_heads", 3),
                   lambda c: c["layers"][0]["mixer"].pop("gate_cap"),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"),
                   lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 7),
                   lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 2),       # not a latent layer
                   lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 5),       # a borrower, and a later layer
                   lambda c: c["layers"][3]["mixer"].__setitem__("kv_rank", 24),      # not the lender's size
                   lambda c: c["embedding"].pop("bigram"),
                   lambda c: c.pop("layers")):
        bad = cases.config_json("mix")
        change(bad)
        with pytest.raises(ConfigError):
            ZemaraxConfig.from_dict(bad)


def test_registry_chooses_the_design_by_config_json(dirs):
    from tempura_amd.config import load_config
    from tempura_amd.config.zemarax import ZemaraxConfig
    assert isinstance(load_config(dirs["one"]), ZemaraxConfig)


def test_a_checkpoint_with_a_wrong_tensor_is_refused(dirs, tmp_path):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.weights import WeightsError
    W = cases.make_weights("mix")
    W["l0.mix.norm"] = W["l0.mix.norm"][:10].contiguous()
    del W["l0.mlp.e3.up"]
    del W["pos"]
    W["l3.mix.dkv"] = W["l1.mix.dkv"]      # a borrower has no down projection of its own
    cases.write_model("mix", str(tmp_path / "bad"), weights=W)
    with pytest.raises(WeightsError) as e:
        load_model(str(tmp_path / "bad"), "float32", "cpu")
    assert {"l0.mlp.e3.up", "pos"} <= set(e.value.missing) and "l0.mix.norm" in e.value.wrong_shape
    assert e.value.unexpected == ["l3.mix.dkv"]


def test_caches_states_and_groups_of_a_model(dirs):
    runner = _runner(dirs["mix"], 64)
    m = runner.model
    assert m.call_writes == [True, True, True, False, True, False]
    # the borrowers read the very tensors the lender writes
    k = [runner.layer_caches[i].k for i in (1, 3, 5)]
    assert k[0].data_ptr() == k[1].data_ptr() == k[2].data_ptr() and k[0].shape[1:] == (1, 16, 20)
    kinds = sorted(g.kind for g in m.cache_groups)
    assert kinds == ["full", "full", "window_keep_first"]
    # the recurrence: per head the memory with the normaliser as one more column, and a running maximum a column
    assert runner.layer_caches[0].state.shape[1] == 3 * (6 + 1) * (10 + 1)
    assert all(runner.layer_caches[i].state is None for i in (1, 2, 3, 4, 5))
    assert m.EMBEDDING_STATE in runner.pools.state      # the token before a step's first


# ---- mechanisms alone, against the plain functions ----------------------------------------------
def test_router_stand_in_is_the_plain_router():
    g = torch.Generator().manual_seed(5)
    for E, top in [(6, 2), (8, 4), (4, 1), (12, 3), (5, 5), (16, 2)]:
        h = torch.randn(40, 24, generator=g, dtype=torch.float64)
        W = {"m.router": torch.randn(E, 24, generator=g, dtype=torch.float64), "m.router.b": torch.randn(E, generator=g, dtype=torch.float64)}
        idx, wts = plain.route(h, W, "m", top)
        dense, ids, w2 = EmuOps().moe_route((h @ W["m.router"].T).float(), None, E, top, 1, 1, "softmax", 1, True, 0.0, 1.0, W["m.router.b"].float())
        assert torch.equal(ids.long(), idx), (E, top)
        assert torch.allclose(w2.double(), wts, atol=1e-6) and torch.allclose(dense.double().sum(1), torch.ones(40, dtype=torch.float64), atol=1e-5)
        assert int((dense > 0).sum()) == 40 * top


def test_the_bias_of_the_router_decides_who_is_chosen():
    """Without its bias the router of the plain implementation chooses other experts: the test's weights make the
    bias matter."""
    cfg, W = _plain("mix")
    g = torch.Generator().manual_seed(2)
    u = torch.randn(30, 48, generator=g, dtype=torch.float64)
    W64 = {k: v.double() for k, v in W.items()}
    ids, _ = plain.route(u, W64, "l0.mlp", 2)
    W64["l0.mlp.router.b"] = torch.zeros(6, dtype=torch.float64)
    ids0, _ = plain.route(u, W64, "l0.mlp", 2)
    assert not torch.equal(ids, ids0)


@pytest.mark.parametrize("name", ["mix", "one"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import zemarax_mechanisms
    zemarax_mechanisms.check(dirs[name], name, "cpu", TOL)


# ---- the model through the step function --------------------------------------------------------
@pytest.mark.parametrize("name", ["mix", "one"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_every_cutting_matches_plain(dirs, name, mode):
    cfg, W = _plain(name)
    reqs = cases.requests(name)
    lengths = cases.LENGTHS[name]
    if mode == "mixed":
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=11)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": lambda l: helpers.schedule_bulk_tail(l, tail=12),
                 "portions": lambda l: helpers.schedule_portions(l, sizes=(7, 2, 16, 3, 2, 5, 2, 9, 2, 17))}[mode](lengths)
    runner = _runner(dirs[name], max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid, toks in reqs.items():
        ref = plain.forward(cfg, W, toks)
        bad = helpers.first_difference(got[rid], ref, TOL)
        assert bad is None, f"{name}/{mode}: request {rid} first differs at position {bad}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_residual_after_every_layer_matches_plain(dirs):
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("mix")
    toks = cases.tokens("mix", 19, 7)
    want = []
    plain.forward(cfg, W, toks, want)
    runner = _runner(dirs["mix"], 64)
    seen = {}
    runner.model.observer = lambda i, h: seen.__setitem__(i, h.double().clone())
    runner.add_request("r")
    runner.step([StepEntry("r", toks, [])])
    assert len(want) == 6
    for i, ref in enumerate(want):
        assert float((seen[i + 1] - ref).abs().max() / ref.abs().max()) < TOL, f"after layer {i}"


def test_state_slots_and_pages_are_used_again(dirs):
    """Two state slots and a pool of six pages for five requests one after the other and side by side: a slot's
    or a page's last owner must leave nothing behind (a memory, a running maximum, the token before, keys, latents)."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("mix")
    runner = _runner(dirs["mix"], 96, max_requests=2)
    reqs = cases.requests("mix")
    order = ["m2", "m1", "m4", "m0", "m5"]
    slots_seen = []
    for k in range(0, len(order), 2):
        pair = order[k: k + 2]
        for rid in pair:
            runner.add_request(rid)
            slots_seen.append(runner.cache.state_slot(rid))
        done = {rid: 0 for rid in pair}
        got = {rid: [] for rid in pair}
        while any(done[r] < len(reqs[r]) for r in pair):
            batch = []
            for rid in pair:
                c = min(5, len(reqs[rid]) - done[rid])
                if c > 0:
                    batch.append(StepEntry(rid, reqs[rid][done[rid]: done[rid] + c], list(range(c))))
                    done[rid] += c
            logits = runner.step(batch)
            row = 0
            for e in batch:
                got[e.rid].append(logits[row: row + len(e.tokens)].clone())
                row += len(e.tokens)
        for rid in pair:
            runner.end_request(rid)
            ref = plain.forward(cfg, W, reqs[rid])
            assert helpers.first_difference(torch.cat(got[rid]), ref, TOL) is None, rid
    assert len(set(slots_seen)) == 2 and len(slots_seen) == 5


def _sharp(tmp_path, window, keep, name="mix"):
    """A model whose attention queries are many times larger than drawn: a query's softmax rests on one or two keys
    anywhere among those it sees, so a key that is lost, misplaced or wrongly visible changes the logits beyond any
    tolerance."""
    cfg = cases.config_json(name)
    for layer in cfg["layers"]:
        if layer["type"] == "attention" and "mask" in layer["mixer"]:
            layer["mixer"]["mask"] = {"size": window, "keep_first": keep}
    W = cases.make_weights(name, sharp=8.0)
    return cfg, W, cases.write_model(name, str(tmp_path / f"sharp{window}_{keep}"), weights=W, config=cfg)


@pytest.mark.parametrize("window,keep", [(9, 3), (16, 1), (17, 16), (33, 17), (5, 40), (20, 0)])
def test_the_edges_of_the_window_and_of_the_kept_tokens(tmp_path, window, keep):
    """Windows shorter than a page, of exactly one page, one more, and two pages and one, keeping a few first tokens,
    one, a page's worth, a page and one, more than the window spans, none: a prompt in portions that end at and beside
    page borders, then decoding across more borders.  The premise is checked first: the plain implementation with a
    window or a kept count one longer or one shorter gives other logits."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W, folder = _sharp(tmp_path, window, keep)
    toks = cases.tokens("mix", 90, 5)
    ref = plain.forward(cfg, W, toks)
    first = max(window, keep) + 1
    others = [(window - 1, keep), (window + 1, keep), (window, keep + 1)] + ([(window, keep - 1)] if keep > 0 else [])
    for w2, k2 in others:
        c2 = copy.deepcopy(cfg)
        c2["layers"][2]["mixer"]["mask"] = {"size": w2, "keep_first": k2}
        assert plain.logit_error(plain.forward(c2, W, toks)[first:], ref[first:]) > 0.05, (w2, k2)
    runner = _runner(folder, 128)
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 7, 10):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]))
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4
    # pages whose keys no query can see any more went back to the pool while the request was live; those of the
    # kept first tokens did not
    g = [i for i, s in enumerate(runner.model.cache_groups) if s.kind == "window_keep_first"]
    if g:
        held = 8 - runner.cache.free_pages()[g[0]]
        assert (keep + 15) // 16 + (window + 15) // 16 <= held <= (keep + 15) // 16 + (window + 15) // 16 + 2
        assert held < 6 or keep + window > 48


def test_a_far_latent_decides(tmp_path):
    """Sharp queries over the cached latents: the layer that borrows reads the lender's pages, hundreds of tokens
    back, in prompts cut anywhere and in decoding."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("mix")
    cfg["max_positions"] = 400
    W = cases.make_weights("mix", sharp=8.0, cfg=cfg)
    folder = cases.write_model("mix", str(tmp_path / "far"), weights=W, config=cfg)
    toks = cases.tokens("mix", 330, 17)
    ref = plain.forward(cfg, W, toks)
    runner = _runner(folder, 384)
    runner.add_request("r")
    rows, at = [], 0
    for c in (130, 2, 61, 100, 7):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]))
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4


def test_first_tokens_and_single_token_requests(dirs):
    """From the very first token on, one token a step: the bigram table's last row, states that start at zero, a
    running maximum that starts at zero and not below, a window that is not yet full."""
    from tempura_amd.engine.runner import StepEntry
    for name in ("mix", "one"):
        cfg, W = _plain(name)
        runner = _runner(dirs[name], 64)
        toks = cases.tokens(name, 6, 9)
        ref = plain.forward(cfg, W, toks)
        runner.add_request("x")
        rows = [runner.step([StepEntry("x", [t], [0])]) for t in toks]
        assert plain.logit_error(torch.cat(rows), ref) < 1e-4, name
        # the slot's next owner starts from nothing as well
        runner.end_request("x")
        runner.add_request("y")
        again = runner.step([StepEntry("y", toks[:3], [0, 1, 2])])
        assert plain.logit_error(again, ref[:3]) < 1e-4, name


def test_long_decoding_keeps_the_states(dirs):
    """A short prompt, then 150 tokens one by one: the recurrence's memory and maximum, the token before, and a window
    that passes over decoded tokens only."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("mix")
    toks = cases.tokens("mix", 155, 13)
    ref = plain.forward(cfg, W, toks)
    runner = _runner(dirs["mix"], 192)
    runner.add_request("r")
    rows = [runner.step([StepEntry("r", toks[:5], list(range(5)))])]
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[5:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4


def test_the_sink_and_the_running_maximum_matter():
    """Premises of the tests above, in the plain implementation: without the sinks the logits differ, and so they do
    with a running maximum that starts far below zero (as if it started at minus infinity)."""
    cfg, W = _plain("mix")
    toks = cases.tokens("mix", 20, 4)
    ref = plain.forward(cfg, W, toks)
    W2 = dict(W)
    for k in W:
        if k.endswith(".sink"):
            W2[k] = torch.full_like(W[k], -30.0)
    assert plain.logit_error(plain.forward(cfg, W2, toks), ref) > 0.01
    chain = plain.mlstm_chain
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(5, 2, 4, generator=g, dtype=torch.float64) for _ in range(3))
    i_log, f_log = torch.randn(5, 2, generator=g, dtype=torch.float64) - 3.0, -torch.rand(5, 2, generator=g, dtype=torch.float64)
    out = chain(q, k, v, i_log, f_log)
    # with every log input gate below zero the maximum stays at its start for a while: the floor e^(-m) is then 1
    num = torch.einsum("hdv,hd->hv", torch.exp(i_log[0])[:, None, None] * k[0][:, :, None] * v[0][:, None, :], q[0])
    den = torch.maximum((torch.exp(i_log[0])[:, None] * k[0] * q[0]).sum(-1).abs(), torch.ones(2, dtype=torch.float64)) + 1e-6
    assert torch.allclose(out[0], num / den[:, None], atol=1e-12)


# ---- generation through the engine's entry point and scheduler ----------------------------------
@pytest.mark.parametrize("name", ["mix", "one"])
def test_engine_generates_what_plain_greedy_generates(dirs, name):
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = _plain(name)
    prompts = [cases.tokens(name, n, 20 + i) for i, n in enumerate((3, 18, 9))]
    eng = Engine(dirs[name], dtype="float32", page_size=16, kv_pages=12, max_batch_size=2, max_num_batched_tokens=16,
                 prefill_chunk_size=7, device="cpu", use_graph=False)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=6))
    for p, o in zip(prompts, outs):
        assert o == plain.greedy(cfg, W, p, 6)


def test_command_line_inspects_and_writes_random_folders(dirs, tmp_path, capsys):
    """`tempura inspect` on a folder of the design, and `tempura random-model --config-json` for it."""
    from tempura_amd.cli import main
    from tempura_amd.engine.loading import load_model
    assert main(["inspect", dirs["mix"]]) == 0
    text = capsys.readouterr().out
    assert "Zemarax" in text and "6 experts of 16, 2 a token, shared expert of 12" in text and "latents of layer 1" in text
    assert "window 9 keeping the first 3" in text
    path = tmp_path / "c.json"
    path.write_text(json.dumps(cases.config_json("one")))
    assert main(["random-model", "--config-json", str(path), "--out", str(tmp_path / "rnd"), "--std", "0.3"]) == 0
    model = load_model(str(tmp_path / "rnd"), "float32", "cpu")
    assert model.layers[3].mixer.norm_w.shape == (5,) and model.layers[2].mixer.w_q.shape == (11, 6)


def test_a_size_the_configuration_leaves_out_is_the_tensors_own(tmp_path):
    """Without `q_rank` the query latent's size comes from the checkpoint, without `vdim` values are as wide as keys,
    without `max_positions` the position table has the rows it has."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("one")
    W = cases.make_weights("one")
    del cfg["layers"][2]["mixer"]["q_rank"]
    del cfg["layers"][1]["mixer"]["vdim"]
    del cfg["max_positions"]
    folder = cases.write_model("one", str(tmp_path / "lean"), weights=W, config=cfg)
    runner = _runner(folder, 64)
    assert runner.model.layers[2].mixer.query_rank == 6
    toks = cases.tokens("one", 21, 3)
    runner.add_request("r")
    got = runner.step([StepEntry("r", toks, list(range(21)))])
    assert plain.logit_error(got, plain.forward(cases.config_json("one"), W, toks)) < 1e-4
