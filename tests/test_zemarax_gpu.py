"""The Zemarax design on the GPU: every new or changed kernel alone against its plain PyTorch version
(tests/emu_ops.py), and the model through the engine's own step function, cache and state manager, graphs and
scheduler against the plain implementation (tests/plain_zemarax.py), in float32 and bfloat16."""
import copy
import json

import pytest
import torch

import helpers
import plain_zemarax as plain
import zemarax_cases as cases
from emu_ops import EmuOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# plain.logit_error of a whole model: the largest difference of any logit, in units of the logits' spread.  The
# bfloat16 bound is for a position's error by rounding alone.  A router whose two candidates lie closer than that
# rounding would choose another expert, and the recurrence carries what that changes to every position behind it: the
# bfloat16 runs therefore use every expert for every token (the logits still weigh them), the float32 runs choose.
TOL = {"float32": 1e-4, "bfloat16": 1.5e-1}
# Models with sharpened queries amplify float32 rounding (scores of several tens); a key that is lost or wrongly seen
# costs at least 0.05 there (each such test asserts that first), 25 times this bound.
SHARP_TOL = 2e-3
emu = EmuOps()


def _assert_logits(got, ref, dtype, what):
    """float32: every logit within TOL.  bfloat16: with these weights (norms behind every sublayer, peaked softmaxes)
    the rounding of stored activations moves single positions by up to 0.4 of the logits' spread while the typical
    position moves by 0.02 to 0.04; the host stand-in of the same arithmetic shows the same figures at the same
    positions.  So the bound is on the distribution over positions: the median, nine tenths of them, and the worst."""
    if dtype == "float32":
        err = plain.logit_error(got, ref)
        assert err < TOL[dtype], f"{what}: error {err:.3e}"
        return
    g, r = got.double().cpu(), ref.double()
    d = (g - g.mean(-1, keepdim=True)) - (r - r.mean(-1, keepdim=True))
    per = (d.abs().max(-1).values / r.std()).sort().values
    n = per.numel()
    assert float(per[n // 2]) < 0.08 and float(per[(9 * n) // 10 - (1 if n >= 10 else 0)]) < 0.2 + (0.3 if n < 10 else 0.0) and float(per[-1]) < 1.0, \
        f"{what}: median {float(per[n // 2]):.3f}, worst {float(per[-1]):.3f}"


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
    return _Folders(tmp_path_factory.mktemp("zemarax_gpu"))


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
@pytest.mark.parametrize("H,D,Dv", [(3, 10, 6), (1, 7, 5), (2, 128, 64), (4, 32, 128), (2, 256, 40), (1, 24, 200), (2, 520, 9), (5, 64, 63)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_matrix_memory_recurrence(H, D, Dv, out_dtype):
    """Runs of 1 to 40 tokens of four requests, three steps in a row (what one leaves in the state the next reads),
    with gates that span the cap, against the stand-in; slots that are not in the batch stay as they were."""
    ops = _ops()
    g = torch.Generator().manual_seed(H * 1000 + D)
    off, col0, out0 = 11, 5, 3
    width = 2 * H * D + 2 * H * Dv + 2 * H
    n_state = H * (Dv + 1) * (D + 1)
    state = torch.zeros(6, off + n_state + 7)
    state[:, :off] = 3.0
    state[:, off + n_state:] = -2.0
    cu, token_req, slots = _batch([3, 1, 40, 17], [4, 0, 2, 1])
    ib, fb = torch.randn(H, generator=g), torch.randn(H, generator=g) + 1.5
    nw = torch.randn(H * Dv, generator=g) * 0.3 + 1.0
    s_ref, s_dev = state.clone(), state.to(DEV)
    tol = 3e-5 if out_dtype == torch.float32 else 1e-2
    for step in range(3):
        proj = torch.randn(61, col0 + width + 4, generator=g)
        proj[:, col0: col0 + 2 * H * D] *= 1.5
        proj[:, col0 + width - 2 * H:] *= 4.0                      # gates: log inputs and forgets over several units
        want = torch.zeros(61, out0 + H * Dv + 2, dtype=out_dtype)
        got = torch.zeros(61, out0 + H * Dv + 2, dtype=out_dtype, device=DEV)
        emu.mlstm_scan(proj, col0, ib, fb, 6.0, D ** -0.5, s_ref, off, cu, slots, 4, H, D, Dv, nw, 1e-5, 0.8, want, out0)
        ops.mlstm_scan(proj.to(DEV), col0, ib.to(DEV), fb.to(DEV), 6.0, D ** -0.5, s_dev, off, cu.to(DEV), slots.to(DEV), 4, H, D, Dv,
                       nw.to(DEV), 1e-5, 0.8, got, out0)
        _close(got, want, tol)
        _close(s_dev[:, off: off + H * (Dv + 1) * D], s_ref[:, off: off + H * (Dv + 1) * D], 3e-5)
        assert torch.equal(got.cpu()[:, :out0], want[:, :out0]) and torch.equal(got.cpu()[:, out0 + H * Dv:], want[:, out0 + H * Dv:])
    after = s_dev.cpu()
    assert torch.equal(after[3], state[3]) and torch.equal(after[5], state[5])
    assert torch.equal(after[:, :off], state[:, :off]) and torch.equal(after[:, off + n_state:], state[:, off + n_state:])


def test_matrix_memory_token_by_token_is_the_run():
    """One request as one run of 50 tokens and as 50 steps of one token: the same outputs and the same state to float32
    rounding (the running maximum over a run comes from sums in another order; the read-out does not depend on it)."""
    ops = _ops()
    g = torch.Generator().manual_seed(4)
    H, D, Dv = 2, 48, 20
    width = 2 * H * D + 2 * H * Dv + 2 * H
    proj = torch.randn(50, width, generator=g).to(DEV)
    proj[:, -2 * H:] *= 5.0
    ib, fb, nw = torch.zeros(H, device=DEV), torch.ones(H, device=DEV), torch.ones(H * Dv, device=DEV)
    n_state = H * (Dv + 1) * (D + 1)
    s_run, s_tok = torch.zeros(2, n_state, device=DEV), torch.zeros(2, n_state, device=DEV)
    out_run, out_tok = torch.zeros(50, H * Dv, device=DEV), torch.zeros(50, H * Dv, device=DEV)
    slots = torch.tensor([1], dtype=torch.int32, device=DEV)
    ops.mlstm_scan(proj, 0, ib, fb, 9.0, 0.2, s_run, 0, torch.tensor([0, 50], dtype=torch.int32, device=DEV), slots, 1, H, D, Dv, nw, 1e-6, 1.0, out_run, 0)
    one = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    for t in range(50):
        o = torch.zeros(1, H * Dv, device=DEV)
        ops.mlstm_scan(proj[t: t + 1].contiguous(), 0, ib, fb, 9.0, 0.2, s_tok, 0, one, slots, 1, H, D, Dv, nw, 1e-6, 1.0, o, 0)
        out_tok[t] = o[0]
    _close(out_tok, out_run, 2e-5)
    # the memories agree once both are brought to one maximum: S e^m is what the two runs share
    S = [s[1, : H * (Dv + 1) * D].reshape(H, Dv + 1, D).double() * torch.exp(s[1, H * (Dv + 1) * D:].reshape(H, Dv + 1).double())[:, :, None]
         for s in (s_run, s_tok)]
    _close(S[1], S[0], 2e-5)


def _paged(ctx_lens, kvh, d, vd, ps, dtype, g, spare=3):
    """Random keys and values of requests with the given context lengths, spread over shuffled pages."""
    pages_of = [(c + ps - 1) // ps for c in ctx_lens]
    total = sum(pages_of) + spare
    order = torch.randperm(total, generator=g).tolist()
    k = torch.randn(total + 1, kvh, ps, d, generator=g).to(dtype)
    v = torch.randn(total + 1, kvh, vd, ps, generator=g).to(dtype)
    width = max(pages_of)
    bt = torch.full((len(ctx_lens), width), total, dtype=torch.int32)
    at = 0
    for r, n in enumerate(pages_of):
        bt[r, :n] = torch.tensor(order[at: at + n], dtype=torch.int32)
        at += n
    return k, v, bt


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kvh,d,vd,window,keep", [(4, 2, 12, 10, 9, 3), (1, 1, 20, 28, 16, 0), (3, 3, 6, 6, 5, 11), (4, 2, 64, 64, 40, 8),
                                                      (8, 1, 96, 96, 0, 0), (2, 1, 64, 80, 33, 17), (4, 4, 32, 32, 64, 64), (4, 2, 128, 128, 50, 0),
                                                      (16, 1, 64, 64, 0, 0), (2, 2, 32, 32, 0, 0)])
def test_attention_with_a_sink_and_kept_first_keys(dtype, heads, kvh, d, vd, window, keep):
    """Portions behind cached prefixes and single tokens in one batch; with and without the sink; large sinks too."""
    ops = _ops()
    g = torch.Generator().manual_seed(heads * 100 + d)
    q_lens, ctx_lens = [1, 37, 5, 1, 70], [150, 37, 120, 3, 200]
    k, v, bt = _paged(ctx_lens, kvh, d, vd, 16, dtype, g)
    n = sum(q_lens)
    q = (torch.randn(n, heads, d, generator=g) * 2).to(dtype)
    cu, token_req, _ = _batch(q_lens, [0] * 5)
    cl = torch.tensor(ctx_lens, dtype=torch.int32)
    tol = 2e-5 if dtype == torch.float32 else 1.6e-2
    for sink in (None, torch.randn(heads, generator=g) + 1.0, torch.tensor([9.0] * heads), torch.tensor([-40.0] * heads)):
        want = emu.paged_attention(q, k, v, bt, cu, cl, token_req, 0.3, window, max(q_lens), max(ctx_lens), None, None, sink, keep)
        for singles in (0, 2):      # (the single tokens as portions of one, and through the kernels for decoding)
            got = ops.paged_attention(q.to(DEV), k.to(DEV), v.to(DEV), bt.to(DEV), cu.to(DEV), cl.to(DEV), token_req.to(DEV), 0.3, window,
                                      max(q_lens), max(ctx_lens), singles, sink=None if sink is None else sink.to(DEV), keep_first=keep)
            _close(got, want, tol)
        # a step of single tokens only (split over the context and combined, where the matrix-core kernels serve)
        q1 = (torch.randn(5, heads, d, generator=g) * 2).to(dtype)
        cu1, tr1, _ = _batch([1] * 5, [0] * 5)
        want = emu.paged_attention(q1, k, v, bt, cu1, cl, tr1, 0.3, window, 1, max(ctx_lens), None, None, sink, keep)
        got = ops.paged_attention(q1.to(DEV), k.to(DEV), v.to(DEV), bt.to(DEV), cu1.to(DEV), cl.to(DEV), tr1.to(DEV), 0.3, window, 1,
                                  max(ctx_lens), 5, sink=None if sink is None else sink.to(DEV), keep_first=keep)
        _close(got, want, tol)
    if window:
        without = emu.paged_attention(q, k, v, bt, cu, cl, token_req, 0.3, window, max(q_lens), max(ctx_lens), None, None, None, 0)
        kept = emu.paged_attention(q, k, v, bt, cu, cl, token_req, 0.3, window, max(q_lens), max(ctx_lens), None, None, None, keep)
        assert keep == 0 or not torch.allclose(without.float(), kept.float(), atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_key_that_stands_out_at_every_edge(dtype):
    """One query whose score for ONE key is far above the rest: the last kept key, the first key that is not kept, the
    oldest key of the window, the key just outside it, a page's first and last place.  The output is that key's value
    when the query sees it and something else when it does not."""
    ops = _ops()
    g = torch.Generator().manual_seed(3)
    heads, kvh, d, vd, ps, window, keep = 2, 1, 64, 24, 16, 40, 19
    ctx = 200
    k, v, bt = _paged([ctx], kvh, d, vd, ps, dtype, g)
    pos = ctx - 1
    cu, token_req, _ = _batch([1], [0])
    cl = torch.tensor([ctx], dtype=torch.int32)
    sink = torch.tensor([0.5, -1.0])
    for needle, seen in ((keep - 1, True), (keep, False), (0, True), (15, True), (16, True), (pos - window + 1, True), (pos - window, False),
                         (pos, True), (pos - 7, True), (100, False)):
        q = torch.zeros(1, heads, d)
        page, off = int(bt[0, needle // ps]), needle % ps
        q[0, :] = k[page, 0, off].float() * 3.0
        q = q.to(dtype)
        want = emu.paged_attention(q, k, v, bt, cu, cl, token_req, 1.0, window, 1, ctx, None, None, sink, keep)
        got = ops.paged_attention(q.to(DEV), k.to(DEV), v.to(DEV), bt.to(DEV), cu.to(DEV), cl.to(DEV), token_req.to(DEV), 1.0, window, 1, ctx,
                                  1, sink=sink.to(DEV), keep_first=keep)
        _close(got, want, 2e-5 if dtype == torch.float32 else 1.6e-2)
        value = v[page, 0, :, off].float()
        is_value = torch.allclose(want.float().reshape(heads, vd)[0], value, atol=0.05)
        assert is_value == seen, (needle, seen)


def test_norm_per_head_in_place():
    ops = _ops()
    g = torch.Generator().manual_seed(6)
    for H, G, D in ((4, 2, 12), (1, 1, 20), (3, 3, 64), (5, 1, 130), (2, 2, 7)):
        rows = torch.randn(19, 3 + (H + G) * D + 11, generator=g) * 4
        wq, wk = torch.randn(D, generator=g), torch.randn(D, generator=g)
        ref, dev = rows.clone(), rows.to(DEV)
        emu.head_rmsnorm(ref, 3, H, wq, 3 + H * D, G, wk, D, 1e-5)
        ops.head_rmsnorm(dev, 3, H, wq.to(DEV), 3 + H * D, G, wk.to(DEV), D, 1e-5)
        _close(dev, ref, 2e-6)
        assert torch.equal(dev.cpu()[:, :3], rows[:, :3]) and torch.equal(dev.cpu()[:, 3 + (H + G) * D:], rows[:, 3 + (H + G) * D:])
        # queries alone (a call that reads another call's cache)
        ref, dev = rows.clone(), rows.to(DEV)
        emu.head_rmsnorm(ref, 3, H, wq, 3 + H * D, 0, wk, D, 1e-5)
        ops.head_rmsnorm(dev, 3, H, wq.to(DEV), 3 + H * D, 0, wk.to(DEV), D, 1e-5)
        _close(dev, ref, 2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_vector_a_token_into_key_and_value_pages(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(8)
    for dim, ps in ((20, 16), (96, 16), (7, 8), (64, 32)):
        k = torch.randn(9, 1, ps, dim, generator=g).to(dtype)
        v = torch.randn(9, 1, dim, ps, generator=g).to(dtype)
        c = torch.randn(23, dim, generator=g).to(dtype)
        slots = torch.randperm(9 * ps, generator=g)[:23].to(torch.int32)
        kd, vd = k.to(DEV), v.to(DEV)
        emu.vector_store(c, slots, k, v)
        ops.vector_store(c.to(DEV), slots.to(DEV), kd, vd)
        assert torch.equal(kd.cpu(), k) and torch.equal(vd.cpu(), v)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_activations_of_rows_with_a_gate_column(out_dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(2)
    u = torch.randn(37, 45, generator=g) * 2.5
    tol = 2e-6 if out_dtype == torch.float32 else 8e-3
    for kind in ("gelu_erf", "gelu_tanh", "silu"):
        _close(ops.activation(u.to(DEV), kind, out_dtype), emu.activation(u, kind, out_dtype), tol)
        _close(ops.activation(u.to(DEV), kind, out_dtype, 3, 30, 33), emu.activation(u, kind, out_dtype, 3, 30, 33), tol)
        _close(ops.activation(u.to(DEV), kind, out_dtype, 0, 44, None), emu.activation(u, kind, out_dtype, 0, 44, None), tol)
    z = torch.tensor([[-3.0, -0.5, 0.0, 0.7, 4.0]])
    exact = 0.5 * z.double() * (1.0 + torch.erf(z.double() / 2 ** 0.5))
    _close(ops.activation(z.to(DEV), "gelu_erf", torch.float32), exact, 1e-6)


def test_router_with_a_bias_and_a_softmax_over_the_chosen():
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    for E, top in ((6, 2), (16, 3), (4, 1), (5, 5), (130, 4), (3, 3)):
        logits = torch.randn(50, E + 3, generator=g) * 2
        bias = torch.randn(E, generator=g) * 1.5
        want = emu.moe_route(logits, None, E, top, 1, 1, "softmax", 1, True, 0.0, 1.0, bias)
        got = ops.moe_route(logits.to(DEV), None, E, top, 1, 1, score="softmax", normalize=True, sum_eps=0.0, bias=bias.to(DEV))
        assert torch.equal(got[1].cpu(), want[1])
        _close(got[2], want[2], 3e-6)
        _close(got[0], want[0], 3e-6)
        z = (logits[:, :E] + bias).double()
        chosen = torch.gather(z, 1, want[1].long())
        _close(got[2], torch.softmax(chosen, dim=-1), 3e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_scale_bigram_and_learned_positions(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(7)
    vocab, width, buckets = 50, 40, 13
    table, bigram, pos = (torch.randn(r, width, generator=g).to(dtype) for r in (vocab, buckets + 1, 64))
    cu, token_req, slots = _batch([4, 1, 6], [2, 0, 3])
    tokens = torch.randint(0, vocab, (11,), generator=g).to(torch.int32)
    positions = torch.tensor([0, 1, 2, 3, 9, 0, 1, 2, 3, 4, 5], dtype=torch.int32)
    prev = torch.randint(0, vocab, (5, 1), generator=g).to(torch.int32)
    for bg, pt in ((bigram, pos), (bigram, None), (None, pos)):
        p_ref, p_dev = prev.clone(), prev.to(DEV)
        want = emu.embed_bigram(tokens, table, bg, positions, token_req, cu, slots, p_ref, 3, 31, 7, buckets, 2.5, pt)
        got = ops.embed_bigram(tokens.to(DEV), table.to(DEV), None if bg is None else bg.to(DEV), positions.to(DEV), token_req.to(DEV), cu.to(DEV),
                               slots.to(DEV), p_dev, 3, 31, 7, buckets, 2.5, None if pt is None else pt.to(DEV))
        _close(got, want, 1e-6)
        assert torch.equal(p_dev.cpu(), p_ref)


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


@pytest.mark.parametrize("name", ["mix", "one", "wide"])
def test_each_part_alone_matches_its_plain_function(dirs, name):
    import zemarax_mechanisms
    zemarax_mechanisms.check(dirs[name], name, DEV, 3e-5)


@pytest.mark.parametrize("name", ["mix", "wide"])
def test_each_part_alone_in_bfloat16(dirs, name):
    """The parts over the bfloat16 kernels (the matrix-core attention where it serves), every expert used."""
    import zemarax_mechanisms
    zemarax_mechanisms.check(dirs.get(name, "bfloat16"), name, DEV, 6e-2, dtype="bfloat16", cfg=cases.config_json(name, True))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mix", "one", "wide"])
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
        _assert_logits(got[rid], _ref(name, rid, dtype), dtype, f"{name}/{mode}/{dtype}: request {rid}")
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_cutting_changes_rounding_only(dirs):
    """The same request whole, in portions and beside others, in float32: summation order only."""
    reqs = cases.requests("wide")
    lengths = cases.LENGTHS["wide"]
    runs = []
    for steps in (helpers.schedule_whole(lengths), helpers.schedule_portions(lengths, sizes=(2, 9, 33, 2, 16, 5)),
                  helpers.schedule_mixed(lengths, 512, seed=3)):
        runs.append(helpers.run_schedule(_runner(dirs["wide"], "float32", 512), reqs, steps))
    for rid in reqs:
        for other in runs[1:]:
            assert plain.logit_error(other[rid], runs[0][rid]) < 1e-4, rid


@pytest.mark.parametrize("window,keep", [(16, 1), (17, 16), (40, 8), (24, 33)])
def test_the_edges_of_the_window_and_of_the_kept_tokens_on_the_gpu(tmp_path, window, keep, dtype="float32"):
    """Queries many times larger than drawn (a softmax that rests on one or two keys anywhere among those it sees): a
    prompt whole, then in portions that end at and beside page borders with decoding behind them.  The premise first: a
    window or a kept count one longer or one shorter gives other logits.  (float32: in bfloat16 the rounding of q and k
    decides between near-equal keys of such a softmax; the kernels' own tests plant their keys in both types.)"""
    from tempura_amd.engine.runner import StepEntry
    every = dtype == "bfloat16"
    cfg = cases.config_json("wide", every)
    cfg["layers"][2]["mixer"]["mask"] = {"size": window, "keep_first": keep}
    W = cases.make_weights("wide", sharp=6.0)
    folder = cases.write_model("wide", str(tmp_path / "sharp"), weights=W, config=cfg)
    toks = cases.tokens("wide", 200, 5)
    ref = plain.forward(cfg, W, toks)
    first = max(window, keep) + 1
    for w2, k2 in ((window - 1, keep), (window + 1, keep), (window, keep + 1), (window, keep - 1)):
        c2 = copy.deepcopy(cfg)
        c2["layers"][2]["mixer"]["mask"] = {"size": w2, "keep_first": k2}
        assert plain.logit_error(plain.forward(c2, W, toks)[first:], ref[first:]) > 0.05, (w2, k2)
    runner = _runner(folder, dtype, 256 + 128)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", toks, list(range(200)))]).cpu()
    assert plain.logit_error(whole, ref) < SHARP_TOL
    runner.end_request("w")
    runner.add_request("r")
    rows, at = [], 0
    for c in (16, 15, 2, 31, 57, 40, 3):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]).cpu())
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]).cpu() for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < SHARP_TOL


def test_a_far_latent_decides_on_the_gpu(tmp_path, dtype="float32"):
    """Sharp queries over the cached latents, 450 tokens: the borrower reads the lender's pages far back, in a prompt
    cut anywhere, then in decoding."""
    from tempura_amd.engine.runner import StepEntry
    cfg = cases.config_json("wide", dtype == "bfloat16")
    W = cases.make_weights("wide", sharp=6.0)
    folder = cases.write_model("wide", str(tmp_path / "far"), weights=W, config=cfg)
    toks = cases.tokens("wide", 450, 17)
    ref = plain.forward(cfg, W, toks)
    runner = _runner(folder, dtype, 512)
    runner.add_request("r")
    rows, at = [], 0
    for c in (130, 2, 161, 100, 7):
        rows.append(runner.step([StepEntry("r", toks[at: at + c], list(range(c)))]).cpu())
        at += c
    rows += [runner.step([StepEntry("r", [t], [0])]).cpu() for t in toks[at:]]
    assert plain.logit_error(torch.cat(rows), ref) < SHARP_TOL


def test_long_decoding_through_a_captured_step(dirs):
    """Two requests decoded token by token for 150 steps through the graph path: pages, latents, memories and running
    maxima all move along, and the window passes over decoded tokens."""
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


@pytest.mark.parametrize("name", ["mix", "wide"])
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
    toks = cases.tokens("mix", 30, 5)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[11:13], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[13:], "want": [16]}, {"id": "b", "tokens": toks[:4], "want": [3]}], "end": ["a", "b"]}]
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", dirs["mix"], "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = plain.forward(cases.config_json("mix"), cases.make_weights("mix"), toks)
    vocab = ref.shape[1]
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
    assert plain.logit_error(torch.cat([a, c]), torch.stack([ref[0], ref[10], ref[29], ref[3]])) < TOL["float32"]
