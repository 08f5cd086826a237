"""The Golavik design through the engine's own model, cache and state manager, step function and scheduler on the
host: the kernel operations are replaced by their plain PyTorch stand-ins (tests/emu_ops.py), the expected values
come from the plain implementation in tests/plain_golavik.py.  A difference here is a fault of the configuration,
the parts, the cache, the state slots or the batch."""
import copy
import json

import pytest
import torch

import golavik_cases as cases
import helpers
import plain_golavik as plain
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
    root = tmp_path_factory.mktemp("golavik")
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
    from tempura_amd.config import ConfigError, GolavikConfig
    from tempura_amd.parts.inventory import expected_weights
    for name in cases.CASES:
        d = cases.config_json(name)
        cfg = GolavikConfig.from_dict(d)
        assert GolavikConfig.from_json(cfg.to_json()) == cfg
        assert cfg.width == d["width"] and cfg.vocab == d["vocab"] and cfg.norm_groups == d["norm"]["groups"] and cfg.canon_taps == d["canon"]["taps"]
        want = {k: tuple(v.shape) for k, v in cases.make_weights(name).items()}
        got = {k: v for k, v in expected_weights(cfg.build_spec()).items() if v.init != "skip"}
        assert set(got) == set(want)
        for k, info in got.items():
            assert all(e is None or e == f for e, f in zip(info.shape, want[k])) and len(info.shape) == len(want[k]), k
    spec = GolavikConfig.from_dict(cases.config_json("trio")).build_spec()
    assert [c.layer for c in spec.order] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [None if c.before is None else c.before.params["row"] for c in spec.order] == [None, 0, None, 1, None, 2, None, None]
    assert [c.layer for c in GolavikConfig.from_dict(cases.config_json("wide")).build_spec().order] == [0, 1, 2, 0, 1, 2]
    for change in (lambda c: c["layers"][0].__setitem__("type", "serial"),
                   lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3),
                   lambda c: c["layers"][0]["mixer"].pop("vdim"),
                   lambda c: c["layers"][1]["mlp"].__setitem__("kind", "dense"),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 4),      # more than the kept groups hold
                   lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 2),      # not the rotated part's size
                   lambda c: c["norm"].__setitem__("groups", 5),
                   lambda c: c.pop("canon"),
                   lambda c: c["loop"].__setitem__("stop", 7)):
        bad = cases.config_json("trio")
        change(bad)
        with pytest.raises(ConfigError):
            GolavikConfig.from_dict(bad)


def test_registry_chooses_the_design_by_config_json(dirs):
    from tempura_amd.config import GolavikConfig, load_config
    assert isinstance(load_config(dirs["solo"]), GolavikConfig)


def test_a_checkpoint_with_a_wrong_tensor_is_refused(dirs, tmp_path):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.weights import WeightsError
    W = cases.make_weights("trio")
    W["l1.mix.norm"] = W["l1.mix.norm"][:10].contiguous()
    del W["l1.mlp.e3.up"]
    del W["loop.step"]
    W["l2.canon2"] = W["l2.canon1"]          # a layer without a feed-forward may hold the unused weight: ignored
    W["l2.mlp.router"] = W["l1.mlp.router"]
    cases.write_model("trio", str(tmp_path / "bad"), weights=W)
    with pytest.raises(WeightsError) as e:
        load_model(str(tmp_path / "bad"), "float32", "cpu")
    assert {"l1.mlp.e3.up", "loop.step"} <= set(e.value.missing) and "l1.mix.norm" in e.value.wrong_shape
    assert e.value.unexpected == ["l2.mlp.router"]


def test_every_pass_of_the_loop_has_a_cache_and_a_state_of_its_own(dirs):
    runner = _runner(dirs["trio"], 64)
    m = runner.model
    assert len(m.order) == 8 and len({c.cache for c in m.order}) == 8 and all(m.call_writes)
    assert m.layers[m.order[1].layer] is m.layers[m.order[3].layer] is m.layers[m.order[5].layer]
    states = [runner.layer_caches[i].state for i in range(8)]
    assert len({s.data_ptr() for s in states}) == 8
    # carried rows of the input convolution in front of the mixer's own state; an attention layer carries only those
    assert states[1].shape[1] == 2 * 48 + 3 * 10 * 10 and states[2].shape[1] == 2 * 48
    assert states[0].shape[1] == 2 * 48 + (2 * 2 * 12 + 4 * 10) + 4 * 12 * 10
    keys = [runner.layer_caches[i].k for i in (2, 4, 6)]
    assert all(k is not None for k in keys) and len({k.data_ptr() for k in keys}) == 3
    # one tap, a mixer without state: no state tensor at all
    solo = _runner(dirs["solo"], 64)
    assert solo.layer_caches[1].state is None and solo.layer_caches[0].state.shape[1] == 20 * 20


# ---- mechanisms alone, against the plain functions ----------------------------------------------
def test_router_stand_in_is_the_plain_router():
    g = torch.Generator().manual_seed(5)
    for E, top, groups, scale in [(6, 2, (3, 2), 1.7), (8, 4, (4, 3), 2.5), (4, 1, None, 1.0), (12, 3, (2, 1), 0.5), (5, 5, None, 1.0),
                                  (16, 2, (16, 3), 3.0), (6, 3, (1, 1), 1.0)]:
        h = torch.randn(40, 24, generator=g, dtype=torch.float64)
        W = {"m.router": torch.randn(E, 24, generator=g, dtype=torch.float64)}
        r = {"experts": E, "top": top, "scale": scale}
        if groups:
            r["groups"] = {"count": groups[0], "keep": groups[1]}
        idx, wts = plain.route(h, W, "m", r)
        dense, ids, w2 = EmuOps().moe_route((h @ W["m.router"].T).float(), None, E, top, groups[0] if groups else 1, groups[1] if groups else 1,
                                            "sigmoid", 2, True, 1e-20, scale)
        assert torch.equal(ids.long(), idx), (E, top, groups)
        assert torch.allclose(w2.double(), wts, atol=1e-6) and torch.allclose(dense.double().sum(1), torch.full((40,), scale, dtype=torch.float64), atol=1e-5)
        assert int((dense > 0).sum()) == 40 * top


def test_a_group_is_ranked_by_its_two_best_scores_not_by_its_best():
    """Group 0 holds the single best expert, group 1 the better pair: the pair's group is kept."""
    logits = torch.tensor([[3.0, -4.0, -4.0, 1.5, 1.4, -4.0]])
    for ops_like in (EmuOps(),):
        dense, ids, w = ops_like.moe_route(logits, None, 6, 2, 2, 1, "sigmoid", 2, True, 1e-20, 1.0)
        assert sorted(ids[0].tolist()) == [3, 4]
        dense, ids, w = ops_like.moe_route(logits, None, 6, 2, 2, 1, "sigmoid", 1, True, 1e-20, 1.0)
        assert sorted(ids[0].tolist()) == [0, 1]


@pytest.mark.parametrize("name", ["trio", "solo"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import golavik_mechanisms
    golavik_mechanisms.check(dirs[name], name, "cpu", TOL)


# ---- the model through the step function --------------------------------------------------------
@pytest.mark.parametrize("name", ["trio", "solo"])
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


def test_residual_after_every_layer_run_matches_plain(dirs):
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("trio")
    toks = cases.tokens("trio", 19, 7)
    want = []
    plain.forward(cfg, W, toks, want)
    runner = _runner(dirs["trio"], 64)
    seen = {}
    runner.model.observer = lambda i, h: seen.__setitem__(i, h.double().clone())
    runner.add_request("r")
    runner.step([StepEntry("r", toks, [])])
    assert len(want) == 8
    for i, ref in enumerate(want):
        assert float((seen[i + 1] - ref).abs().max() / ref.abs().max()) < TOL, f"after layer run {i}"


def test_state_slots_and_pages_are_used_again(dirs):
    """Two state slots and a pool of six pages for five requests one after the other and side by side: a slot's
    or a page's last owner must leave nothing behind (carried rows, a recurrent state, keys)."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("trio")
    runner = _runner(dirs["trio"], 96, max_requests=2)
    reqs = cases.requests("trio")
    order = ["t2", "t1", "t4", "t0", "t5"]
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


def _sharp(tmp_path, name="trio", window=None):
    """A model whose attention queries are many times larger than drawn: a query's softmax rests on one or two keys
    anywhere in its window, so a key that is lost, misplaced or wrongly visible changes the logits beyond any
    tolerance."""
    cfg = cases.config_json(name)
    if window is not None:
        for layer in cfg["layers"]:
            if layer["type"] == "latent_attention":
                layer["mixer"]["mask"]["size"] = window
    W = cases.make_weights(name, sharp=8.0)
    return cfg, W, cases.write_model(name, str(tmp_path / f"sharp{window}"), weights=W, config=cfg)


@pytest.mark.parametrize("window", [9, 16, 17, 33])
def test_the_windows_edge_in_prompts_and_in_decoding(tmp_path, window):
    """Windows shorter than a page, of exactly one page, one more, and two pages and one: a prompt in portions that
    end at and beside page borders, then decoding across more borders.  The premise is checked first: the plain
    implementation with a window one longer or one shorter gives other logits."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W, folder = _sharp(tmp_path, window=window)
    toks = cases.tokens("trio", 90, 5)
    ref = plain.forward(cfg, W, toks)
    for other in (window - 1, window + 1):
        c2 = copy.deepcopy(cfg)
        c2["layers"][2]["mixer"]["mask"]["size"] = other
        assert plain.logit_error(plain.forward(c2, W, toks)[window:], ref[window:]) > 0.05, other
    runner = _runner(folder, 128)
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 7, 10):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]))
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4
    # pages whose keys no query can see any more went back to the pool while the request was live
    assert runner.cache.free_pages()[0] >= 8 - (window + 15) // 16 - 2


def test_first_tokens_and_single_token_requests(dirs):
    """From the very first token on, one token a step: zeros before the start of every convolution, states that start
    at zero, a window that is not yet full."""
    from tempura_amd.engine.runner import StepEntry
    for name in ("trio", "solo"):
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
    """A short prompt, then 150 tokens one by one: the recurrences' states, the carried rows and a window that passes
    over decoded tokens only."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = _plain("trio")
    toks = cases.tokens("trio", 155, 13)
    ref = plain.forward(cfg, W, toks)
    runner = _runner(dirs["trio"], 192)
    runner.add_request("r")
    rows = [runner.step([StepEntry("r", toks[:5], list(range(5)))])]
    rows += [runner.step([StepEntry("r", [t], [0])]) for t in toks[5:]]
    assert plain.logit_error(torch.cat(rows), ref) < 1e-4


def test_the_pass_vector_is_added_once_a_pass(dirs, tmp_path):
    """Without the table's rows the logits differ; with rows swapped they differ too (each pass adds its own)."""
    cfg, W = _plain("trio")
    toks = cases.tokens("trio", 12, 2)
    ref = plain.forward(cfg, W, toks)
    W2 = dict(W)
    W2["loop.step"] = W["loop.step"].flip(0).contiguous()
    assert plain.logit_error(plain.forward(cfg, W2, toks), ref) > 0.01
    from tempura_amd.engine.runner import StepEntry
    folder = cases.write_model("trio", str(tmp_path / "flipped"), weights=W2)
    for f, want in ((folder, plain.forward(cfg, W2, toks)),):
        runner = _runner(f, 64)
        runner.add_request("r")
        got = runner.step([StepEntry("r", toks, list(range(12)))])
        assert plain.logit_error(got, want) < 1e-4


# ---- generation through the engine's entry point and scheduler ----------------------------------
@pytest.mark.parametrize("name", ["trio", "solo"])
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
    """`tempura inspect` on a folder of the design, and `tempura random-model --config-json` for it (the ranks of the
    low-rank projections named in the file, since no checkpoint is there to say them)."""
    from tempura_amd.cli import main
    from tempura_amd.engine.loading import load_model
    assert main(["inspect", dirs["trio"]]) == 0
    text = capsys.readouterr().out
    assert "Golavik" in text and "6 experts of 24, 3 a token, weights times 0.6, 1 of 2 groups" in text and "layers 1 to 2, 3 times" in text
    cfg = cases.config_json("solo")
    cfg["layers"][0]["mixer"]["decay_rank"] = 2
    cfg["layers"][2]["mixer"]["decay_rank"], cfg["layers"][2]["mixer"]["gate_rank"] = 3, 2
    path = tmp_path / "c.json"
    path.write_text(json.dumps(cfg))
    assert main(["random-model", "--config-json", str(path), "--out", str(tmp_path / "rnd"), "--std", "0.3"]) == 0
    model = load_model(str(tmp_path / "rnd"), "float32", "cpu")
    assert model.layers[0].mixer.w2_t.shape == (2, 20) and model.layers[2].mixer.g2_t.shape == (2, 5)
