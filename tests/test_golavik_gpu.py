"""The Golavik design on the GPU: every new or changed kernel alone against its plain PyTorch version
(tests/emu_ops.py), and the model through the engine's own step function, cache and state manager, graphs and
scheduler against the plain implementation (tests/plain_golavik.py), in float32 and bfloat16."""
import copy
import json

import pytest
import torch

import golavik_cases as cases
import helpers
import plain_golavik as plain
from emu_ops import EmuOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# plain.logit_error of a whole model: the largest difference of any logit, in units of the logits' spread.  The
# bfloat16 bound is for a position's error by rounding alone.  A router whose two candidates lie closer than that
# rounding would choose another expert, and the recurrences carry what that changes to every position behind it: the
# bfloat16 runs therefore use every expert for every token (the scores still weigh them), the float32 runs choose.
TOL = {"float32": 1e-4, "bfloat16": 1.5e-1}
emu = EmuOps()


def _ops():
    from tempura_amd.kernels import ops
    return ops


class _Folders:
    """Model folders by case; for bfloat16 runs with every expert used by every token."""

    def __init__(self, root):
        self.root, self.made = root, {}

    def get(self, name, dtype="float32"):
        every = dtype == "bfloat16"
        if (name, every) not in self.made:
            self.made[(name, every)] = cases.write_model(name, str(self.root / f"{name}{int(every)}"), config=cases.config_json(name, every))
        return self.made[(name, every)]

    def __getitem__(self, name):
        return self.get(name)


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    return _Folders(tmp_path_factory.mktemp("golavik_gpu"))


def _close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    err = float((got - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err <= tol, f"relative error {err:.3e} > {tol:.1e}"


def _batch(runs, slots):
    """cu_seqlens, token_req, state slots of a batch of runs."""
    cu = torch.tensor([0] + list(torch.tensor(runs).cumsum(0)), dtype=torch.int32)
    token_req = torch.tensor([i for i, l in enumerate(runs) for _ in range(l)], dtype=torch.int32)
    return cu, token_req, torch.tensor(slots, dtype=torch.int32)


# ---- kernels alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("width,groups", [(48, 3), (192, 4), (37, 1), (1030, 5), (4096, 8), (64, 64)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_in_groups(width, groups, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(width)
    h, w = torch.randn(13, width, generator=g) * 3, torch.randn(width, generator=g)
    h[:, : width // groups] *= 20                      # (a part much larger than the others: each has its own scale)
    rows = torch.tensor([12, 0, 5], dtype=torch.int32)
    tol = 2e-6 if out_dtype == torch.float32 else 8e-3
    _close(ops.rmsnorm(h.to(DEV), w.to(DEV), 1e-5, out_dtype, None, groups=groups), emu.rmsnorm(h, w, 1e-5, out_dtype, None, groups), tol)
    _close(ops.rmsnorm(h.to(DEV), w.to(DEV), 1e-5, out_dtype, rows.to(DEV), groups=groups), emu.rmsnorm(h, w, 1e-5, out_dtype, rows, groups), tol)
    if width > 20:
        wide = torch.randn(13, width + 9, generator=g)
        _close(ops.rmsnorm_cols(wide.to(DEV), 4, width - 1 if groups == 1 else width, (w[:-1] if groups == 1 else w).contiguous().to(DEV), 1e-6, out_dtype, groups),
               emu.rmsnorm_cols(wide, 4, width - 1 if groups == 1 else width, w[:-1] if groups == 1 else w, 1e-6, out_dtype, groups), tol)


@pytest.mark.parametrize("width,taps,subs", [(40, 3, 2), (7, 1, 1), (130, 2, 2), (300, 5, 1), (1024, 4, 2)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rows_plus_their_convolution_with_carried_rows(width, taps, subs, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(width)
    off = 17
    w = torch.randn(subs, taps, width, generator=g)
    state = torch.randn(5, off + (taps - 1) * width + 13, generator=g)
    cu, token_req, slots = _batch([3, 1, 2, 9], [4, 0, 2, 1])
    x = torch.randn(15, width, generator=g)
    s_ref, s_dev = state.clone(), state.to(DEV)
    for _ in range(3):                                      # three steps in a row: what one leaves the next reads
        want = emu.residual_conv(x, w, s_ref, off, cu, token_req, slots, 4, out_dtype)
        got = ops.residual_conv(x.to(DEV), w.to(DEV), s_dev, off, cu.to(DEV), token_req.to(DEV), slots.to(DEV), 4, out_dtype)
        assert len(got) == subs
        for a, b in zip(got, want):
            _close(a, b, 2e-6 if out_dtype == torch.float32 else 8e-3)
        _close(s_dev, s_ref, 0)
        x = x * 0.9 + 0.1
    assert torch.equal(s_dev.cpu()[3], state[3]) and torch.equal(s_dev.cpu()[:, :off], state[:, :off])
    if taps == 1:
        got = ops.residual_conv(x.to(DEV), w.to(DEV), None, 0, cu.to(DEV), token_req.to(DEV), slots.to(DEV), 4, out_dtype)
        _close(got[0], emu.residual_conv(x, w, None, 0, cu, token_req, slots, 4, out_dtype)[0], 2e-6 if out_dtype == torch.float32 else 8e-3)


def test_a_row_added_to_the_stream():
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    h, table = torch.randn(23, 77, generator=g), torch.randn(3, 77, generator=g)
    dev = h.to(DEV)
    ops.add_row(dev, table.to(DEV), 2)
    assert torch.equal(dev.cpu(), h + table[2])


@pytest.mark.parametrize("E,top,groups,keep,best", [(6, 2, 3, 2, 2), (8, 4, 4, 3, 2), (4, 1, 1, 1, 2), (12, 3, 2, 1, 2), (5, 5, 1, 1, 1), (16, 2, 16, 3, 2),
                                                    (128, 6, 8, 4, 2), (16, 4, 2, 1, 3), (200, 8, 4, 2, 2)])
@pytest.mark.parametrize("score", ["sigmoid", "softmax"])
def test_router_with_sigmoid_scores_group_sums_and_normalised_weights(E, top, groups, keep, best, score):
    ops = _ops()
    g = torch.Generator().manual_seed(E + top)
    logits = torch.randn(77, E + 3, generator=g) * 2
    logits[5, :E] = 0.25                                       # all equal: the lower index wins every tie
    corr = torch.randn(E, generator=g) * 0.2 if score == "softmax" else None
    for normalize, scale in ((True, 2.5), (False, 1.0), (True, 1.0), (False, 0.3)):
        want = emu.moe_route(logits, corr, E, top, groups, keep, score, best, normalize, 1e-20, scale)
        got = ops.moe_route(logits.to(DEV), None if corr is None else corr.to(DEV), E, top, groups, keep, score=score, group_best=best,
                            normalize=normalize, sum_eps=1e-20, scale=scale)
        assert torch.equal(got[1].cpu(), want[1]), (normalize, scale)
        _close(got[2], want[2], 1e-5)
        _close(got[0], want[0], 1e-5)


def test_a_group_is_ranked_by_its_two_best_scores_on_the_gpu():
    ops = _ops()
    logits = torch.tensor([[3.0, -4.0, -4.0, 1.5, 1.4, -4.0]], device=DEV)
    assert sorted(ops.moe_route(logits, None, 6, 2, 2, 1, score="sigmoid", group_best=2, normalize=True, sum_eps=1e-20, scale=1.0)[1][0].tolist()) == [3, 4]
    assert sorted(ops.moe_route(logits, None, 6, 2, 2, 1, score="sigmoid", group_best=1, normalize=True, sum_eps=1e-20, scale=1.0)[1][0].tolist()) == [0, 1]


@pytest.mark.parametrize("rank,n_out", [(4, 30), (16, 384), (33, 200), (64, 4096)])
def test_low_rank_second_product_with_a_tanh_in_front_and_a_bounded_decay_behind(rank, n_out):
    ops = _ops()
    g = torch.Generator().manual_seed(rank)
    x, wt, b = torch.randn(19, rank + 11, generator=g) * 2, torch.randn(rank, n_out, generator=g), torch.randn(n_out, generator=g)
    want = emu.lowrank_up(x, 7, wt, "rate_sigmoid", None, b, 0, 0.6065, "tanh")
    got = ops.lowrank_up(x.to(DEV), 7, wt.to(DEV), "rate_sigmoid", bias=b.to(DEV), rate=0.6065, in_act="tanh")
    _close(got, want, 3e-6)
    assert float(got.min()) >= 0.545 and float(got.max()) <= 1.0
    _close(ops.lowrank_up(x.to(DEV), 7, wt.to(DEV), "sigmoid"), emu.lowrank_up(x, 7, wt, "sigmoid"), 3e-6)      # (the modes that were there)


@pytest.mark.parametrize("H,D", [(3, 10), (1, 20), (2, 64), (6, 64), (2, 128), (1, 200), (2, 48)])
def test_general_delta_rule_over_runs_with_carried_states(H, D):
    ops = _ops()
    g = torch.Generator().manual_seed(H * 1000 + D)
    runs, slots = [3, 1, 40, 9], [4, 0, 2, 1]
    cu, token_req, sl = _batch(runs, slots)
    n, hd, col0, off = sum(runs), H * D, 5, 11
    state = torch.randn(6, off + hd * D + 3, generator=g) * 0.3
    s_ref, s_dev = state.clone(), state.to(DEV)
    a_bias = torch.randn(hd, generator=g)
    for step in range(2):
        proj = torch.randn(n, col0 + 4 * hd + 6, generator=g)
        decay = torch.rand(n, hd, generator=g) * 0.45 + 0.55
        want = emu.general_delta_scan(proj, col0, decay, a_bias, s_ref, off, cu, sl, 4, H, D, 1e-6)
        got = ops.general_delta_scan(proj.to(DEV), col0, decay.to(DEV), a_bias.to(DEV), s_dev, off, cu.to(DEV), sl.to(DEV), 4, H, D, 1e-6)
        _close(got, want, 2e-5)
        _close(s_dev, s_ref, 2e-5)
    assert torch.equal(s_dev.cpu()[3], state[3]) and torch.equal(s_dev.cpu()[:, :off], state[:, :off])


def test_general_delta_rule_token_by_token_is_the_run():
    """A run cut anywhere gives the bits of the whole run: every token is one step of the same chain."""
    ops = _ops()
    g = torch.Generator().manual_seed(3)
    H, D, n = 2, 64, 50
    hd = H * D
    proj, decay = torch.randn(n, 4 * hd, generator=g).to(DEV), (torch.rand(n, hd, generator=g) * 0.4 + 0.6).to(DEV)
    a_bias = torch.randn(hd, generator=g).to(DEV)
    s1, s2 = torch.zeros(1, hd * D, device=DEV), torch.zeros(1, hd * D, device=DEV)
    one = torch.zeros(1, dtype=torch.int32, device=DEV)
    whole = ops.general_delta_scan(proj, 0, decay, a_bias, s1, 0, torch.tensor([0, n], dtype=torch.int32, device=DEV), one, 1, H, D, 1e-6)
    cu1 = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    rows = [ops.general_delta_scan(proj[t: t + 1].contiguous(), 0, decay[t: t + 1].contiguous(), a_bias, s2, 0, cu1, one, 1, H, D, 1e-6) for t in range(n)]
    assert torch.equal(torch.cat(rows), whole) and torch.equal(s1, s2)


@pytest.mark.parametrize("heads,vdim", [(4, 10), (1, 40), (3, 130), (6, 64)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_per_head_with_a_weight_per_head_and_a_gate_from_raw_rows(heads, vdim, out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(heads + vdim)
    n = 11
    o = torch.randn(n, heads * vdim, generator=g) * 5
    w, rows = torch.randn(heads * vdim, generator=g), torch.randn(n, heads * vdim + 14, generator=g) * 2
    out = torch.zeros(n, heads * vdim + 9).to(out_dtype)
    ref = out.clone()
    dev = out.to(DEV)
    ops.head_norm_gate(o.to(DEV), w.to(DEV), None, 1e-5, 0.9, heads, dev, 5, gate_rows=rows.to(DEV), gate_col0=6)
    emu.head_norm_gate(o, w, None, 1e-5, 0.9, heads, ref, 5, rows, 6)
    _close(dev, ref, 2e-6 if out_dtype == torch.float32 else 8e-3)


def test_rows_of_an_attention_expanded_from_a_latent():
    ops = _ops()
    g = torch.Generator().manual_seed(9)
    for H, D, R, Dv in ((3, 8, 4, 6), (4, 64, 32, 80), (1, 5, 2, 9)):
        proj, up = torch.randn(21, 7 + H * (D + R) + 40, generator=g), torch.randn(21, H * (D + Dv) + 5, generator=g)
        got = ops.latent_rows(proj.to(DEV), 7, 7 + H * (D + R) + 3, up.to(DEV), H, D, R, Dv)
        assert torch.equal(got.cpu(), emu.latent_rows(proj, 7, 7 + H * (D + R) + 3, up, H, D, R, Dv))


# ---- the model through the step function --------------------------------------------------------
def _runner(folder, dtype, max_tokens, page_size=16, max_requests=4, use_graph=False):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(folder, dtype, DEV)
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=max_requests, use_graph=use_graph)


_REFS = {}


def _ref(name, rid, dtype):
    key = (name, rid, dtype == "bfloat16")
    if key not in _REFS:
        _REFS[key] = plain.forward(cases.config_json(name, key[2]), cases.make_weights(name), cases.requests(name)[rid])
    return _REFS[key]


@pytest.mark.parametrize("name", ["trio", "solo", "wide"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import golavik_mechanisms
    golavik_mechanisms.check(dirs[name], name, DEV, 2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["trio", "solo", "wide"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_every_cutting_matches_plain(dirs, name, mode, dtype):
    reqs = cases.requests(name)
    lengths = cases.LENGTHS[name]
    if mode == "mixed":
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=11)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": lambda l: helpers.schedule_bulk_tail(l, tail=40),
                 "portions": lambda l: helpers.schedule_portions(l, sizes=(7, 2, 16, 3, 2, 31, 5, 2, 64, 9, 2, 17))}[mode](lengths)
    runner = _runner(dirs.get(name, dtype), dtype, max_tokens)
    got = helpers.run_schedule(runner, reqs, steps)
    for rid in reqs:
        err = plain.logit_error(got[rid], _ref(name, rid, dtype))
        assert err < TOL[dtype], f"{name}/{mode}/{dtype}: request {rid}: error {err:.3e}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_cutting_changes_rounding_only(dirs):
    """The same request whole, in portions and beside others, in float32: summation order only."""
    reqs = cases.requests("wide")
    lengths = cases.LENGTHS["wide"]
    runs = []
    for steps in (helpers.schedule_whole(lengths), helpers.schedule_portions(lengths, sizes=(2, 9, 33, 2, 16, 5)),
                  helpers.schedule_mixed(lengths, 448, seed=3)):
        runs.append(helpers.run_schedule(_runner(dirs["wide"], "float32", 448), reqs, steps))
    for rid in reqs:
        for other in runs[1:]:
            assert plain.logit_error(other[rid], runs[0][rid]) < 2e-5, rid


@pytest.mark.parametrize("window", [16, 17, 40])
def test_the_windows_edge_on_the_gpu(tmp_path, window):
    """Queries many times larger than drawn (a softmax that rests on one or two keys anywhere in the window), windows
    of one page, one page and one key, and two pages and a half: a prompt whole, then in portions that end at and beside
    page borders with decoding behind them.  The premise first: a window one longer or one shorter gives other logits."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("wide")
    cfg["layers"][0]["mixer"]["mask"]["size"] = window
    W = cases.make_weights("wide", sharp=6.0)
    folder = cases.write_model("wide", str(tmp_path / "sharp"), weights=W, config=cfg)
    toks = cases.tokens("wide", 200, 5)
    ref = plain.forward(cfg, W, toks)
    for other in (window - 1, window + 1):
        c2 = copy.deepcopy(cfg)
        c2["layers"][0]["mixer"]["mask"]["size"] = other
        assert plain.logit_error(plain.forward(c2, W, toks)[window:], ref[window:]) > 0.05, other
    runner = _runner(folder, "float32", 256 + 128)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", toks, list(range(200)))]).cpu()
    assert plain.logit_error(whole, ref) < TOL["float32"]
    runner.end_request("w")
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 31, 57, 40, 3):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]).cpu())
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]).cpu() for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < TOL["float32"]


def test_long_decoding_through_a_captured_step(dirs):
    """Two requests decoded token by token for 150 steps through the graph path: pages, carried rows and recurrent
    states all move along, and the window passes over decoded tokens."""
    from tempura_amd.engine.runner import StepEntry
    cfg, W = cases.config_json("wide"), cases.make_weights("wide")
    runner = _runner(dirs["wide"], "float32", 512, use_graph=True)
    assert runner.use_graph, "every part of the design may be captured"
    seqs = {"p": cases.tokens("wide", 170, 41), "q": cases.tokens("wide", 158, 42)}
    start = {"p": 20, "q": 8}
    got = {rid: [] for rid in seqs}
    for rid in seqs:
        runner.add_request(rid)
        got[rid].append(runner.step([StepEntry(rid, seqs[rid][: start[rid]], list(range(start[rid])))]).cpu())
    for i in range(150):
        logits = runner.step([StepEntry(rid, [seqs[rid][start[rid] + i]], [0]) for rid in seqs]).cpu()
        for k, rid in enumerate(seqs):
            got[rid].append(logits[k: k + 1].clone())
    assert runner.graph_steps >= 149
    for rid in seqs:
        assert plain.logit_error(torch.cat(got[rid]), plain.forward(cfg, W, seqs[rid])) < TOL["float32"], rid


@pytest.mark.parametrize("name", ["trio", "wide"])
@pytest.mark.parametrize("use_graph", [False, True])
def test_engine_generates_what_plain_greedy_generates(dirs, name, use_graph):
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = cases.config_json(name), cases.make_weights(name)
    prompts = [cases.tokens(name, n, 20 + i) for i, n in enumerate((3, 18, 9, 40, 1))]
    eng = Engine(dirs[name], dtype="float32", page_size=16, kv_pages=24, max_batch_size=3, max_num_batched_tokens=32,
                 prefill_chunk_size=7, device=DEV, use_graph=use_graph)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12))
    for p, o in zip(prompts, outs):
        assert o == plain.greedy(cfg, W, p, 12)
    if use_graph:
        assert eng.runner.graph_steps > 0


def test_replay_program_on_a_model_folder(dirs, tmp_path):
    """bin/trace_run on a small folder: steps on standard input, logits files out, against the plain result."""
    import os
    import subprocess
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    toks = cases.tokens("trio", 30, 5)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[11:13], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[13:], "want": [16]}, {"id": "b", "tokens": toks[:4], "want": [3]}], "end": ["a", "b"]}]
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", dirs["trio"], "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = plain.forward(cases.config_json("trio"), cases.make_weights("trio"), toks)
    vocab = ref.shape[1]
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
    assert plain.logit_error(torch.cat([a, c]), torch.stack([ref[0], ref[10], ref[29], ref[3]])) < TOL["float32"]
