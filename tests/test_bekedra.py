"""Bekedra in the engine against the plain implementation (tests/plain_bekedra.py): every way of cutting the work,
on the CPU with plain PyTorch ops (the host side: batching, paging, the order of parts) and, marked ``gpu``, with
the HIP kernels in true float32 and in bfloat16."""
import copy
import json
import os

import pytest
import torch

import bekedra_cases as X
import plain_bekedra as P
import replay_cases as C
from kernel_refs import RefOps

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]
_ops = {}
_plain = {}


def ops_for(device):
    if device == "cpu":
        return RefOps()
    if device not in _ops:
        from yalis_amd.ops.hip import HipOps

        _ops[device] = HipOps(device)
    return _ops[device]


def setup(name):
    cfg = X.CONFIGS[name]
    if name not in _plain:
        weights = X.random_weights(cfg, seed=len(name))
        reqs = X.make_requests(cfg, X.LENGTHS[name], seed=10)
        _plain[name] = (weights, reqs, *X.plain_logits_and_gaps(cfg, weights, reqs))
    return (cfg, *_plain[name])


TRACES = {"whole": C.trace_whole, "tail": C.trace_tail, "one_by_one": lambda r: C.trace_tail(r, tail=1 << 20),
          "portions": C.trace_portions, "mixed": C.trace_mixed, "random": lambda r: C.trace_random(r, 5)}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["odd", "mix", "wide"])
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_modes(backend, name, mode):
    """Whole prompts; a prompt and then its last tokens one by one; every token one by one (prefill against
    decoding); portions down to two tokens; up to four unequal requests a step in a pool so small that pages are
    used again; cuts at random."""
    device, dtype = backend
    if device == "cpu" and (name == "wide" or (name == "mix" and mode not in ("whole", "mixed", "portions"))):
        pytest.skip("the plain ops are slow at this size; the GPU runs every mode")
    cfg, weights, reqs, want, gaps = setup(name)
    steps = TRACES[mode](reqs)
    page = X.PAGE[name]
    n_pages = C.pages_needed(steps, reqs, page)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), page, n_pages)
    got, rp = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/{mode}", gaps)
    runner.pages.audit()
    assert runner.pages.live_requests() == 0
    assert all(runner.pages.free_pages(g) == n_pages for g in range(len(runner.group_shapes)))
    if mode == "mixed":
        owners, reused = {}, False
        for held in rp.page_log:
            for rid, tables in held.items():
                for g, pages in enumerate(tables):
                    for p in pages:
                        if p >= 0:
                            reused |= owners.setdefault((g, p), rid) != rid
        assert reused, "the trace was meant to reuse pages"


def test_memory_plan_and_run_order():
    """Every pass over the looped layers is a run of the same parts with pages of its own; a pass's first entry
    carries its row of the table of steps; layers with equal key and value sizes share a pool."""
    cfg, weights, _, _, _ = setup("odd")
    runner = X.make_runner(cfg, weights, "float32", "cpu", RefOps(), 16, 4)
    m = runner.model
    assert [e.layer for e in m.spec.run_order] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [None if e.added_row is None else e.added_row[:2] for e in m.spec.run_order] == \
        [None, ("loop.step", 0), None, ("loop.step", 1), None, ("loop.step", 2), None, None]
    assert all(s.owns_cache for s in m.sites) and not m.state_needs
    assert m.blocks[m.spec.run_order[3].layer] is m.blocks[m.spec.run_order[1].layer]
    needs = sorted((g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, g.need.window, len(g.entries)) for g in m.cache_groups)
    assert needs == sorted([(3, 10, 10, None, 1), (2, 12, 10, None, 3), (1, 6, 6, None, 3), (2, 8, 8, None, 1)])
    assert m.tensor_specs()["loop.step"].shape == (3, 40)
    no_loop = X.make_runner(X.CONFIGS["mix"], setup("mix")[1], "float32", "cpu", RefOps(), 16, 4).model
    assert [e.layer for e in no_loop.spec.run_order] == [0, 1, 2, 3] and "loop.step" not in no_loop.tensor_specs()
    whole = X.CONFIGS["wide"]
    from yalis_amd.engine.factory import spec_from_config
    order = spec_from_config(whole)[2].run_order
    assert [e.layer for e in order] == [0, 1, 2, 0, 1, 2] and order[0].added_row[:2] == ("loop.step", 0) and order[3].added_row[:2] == ("loop.step", 1)


@pytest.mark.parametrize("backend", BACKENDS)
def test_slots_and_pages_are_used_again(backend):
    """Two slots, six requests one after another in pairs, in a pool that holds two of them: a request that takes
    over pages reads nothing of what the one before left there."""
    device, dtype = backend
    cfg, weights, reqs, want, gaps = setup("odd")
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8, max_seqs=2)
    steps = C.trace_mixed(reqs, max_live=2)
    got, _ = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", "two slots", gaps)
    assert runner.pages.free_slots() == 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    """A short prompt and 200 tokens decoded one by one: every pass's pages grow step by step, the temperature
    steps up every few tokens, the rotation reaches angles far beyond the original context."""
    device, dtype = backend
    cfg = X.CONFIGS["odd"]
    weights = X.random_weights(cfg, seed=21)
    reqs = X.make_requests(cfg, [215], seed=3)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 14, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_tail(reqs, tail=200))
    X.assert_matches(got, want, dtype == "bfloat16", "long decoding", gaps)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["mix", "wide"])
def test_long_prompt_in_one_step(backend, name):
    """A prompt of 450 tokens whole, then a few tokens one by one; and the same prompt in portions whose edges
    fall inside pages and inside the blocks of keys the attention kernels walk (at this length the experts'
    products take their tiles of many rows)."""
    device, dtype = backend
    if device == "cpu":
        pytest.skip("the plain ops are slow at this size; the GPU runs it")
    cfg = X.CONFIGS[name]
    weights = X.random_weights(cfg, seed=31)
    reqs = X.make_requests(cfg, [456], seed=8)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_tail(reqs, tail=6))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt", gaps)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_portions(reqs, sizes=[70, 2, 33, 64, 5, 100]))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt in portions", gaps)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_width_whose_products_come_in_slices(backend):
    """Width 1,024 with heads of 128: for few tokens the projections' products are left as slices that the next
    kernel sums (the mixer's output waits in the library's workspace while nothing else may take it); single tokens
    behind a prompt, and the prompt in portions."""
    device, dtype = backend
    if device == "cpu":
        pytest.skip("the plain ops have no slices; the GPU runs it")
    cfg = X.model(300, 1024, 1e-6, 32.0, [
        (X.sinked(8, 2, 128, 128, 0.09, softcap=30.0, rot=(64, 10000.0, 8.0, 1.0, 4.0, 32)), X.moe(4, 2, 256)),
        (X.tempered(8, 2, 128, 0.09, 0.3, 32), X.moe(4, 2, 256)),
    ], loop=(0, 2, 2))
    weights = X.random_weights(cfg, seed=51)
    reqs = X.make_requests(cfg, [70, 9], seed=5)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    for make in (lambda r: C.trace_tail(r, tail=20), C.trace_portions, C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 64, 4)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "width 1,024", gaps)


def _one_layer(layer, ff, width=32, eps=1e-5, scale=2.0, loop=None, vocab=80):
    return X.model(vocab, width, eps, scale, [(layer, ff)], loop=loop)


MECHANISMS = {
    "tempered": _one_layer(X.tempered(4, 2, 8, 0.3, 0.6, 7), None),
    "tempered_no_temperature_one_head": _one_layer(X.tempered(1, 1, 16, 0.25), None),
    "tempered_steps_every_token_a_key_head_per_head": _one_layer(X.tempered(3, 3, 6, 0.4, 2.0, 1), None),
    "tempered_negative_coefficient": _one_layer(X.tempered(2, 1, 12, 0.3, -0.2, 4), None),
    "sinked": _one_layer(X.sinked(4, 2, 8, 6, 0.3, softcap=4.0, rot=(4, 100.0, 4.0, 1.0, 2.0, 8)), None),
    "sinked_no_cap_no_rotation_wide_values": _one_layer(X.sinked(3, 1, 6, 10, 0.5), None),
    "sinked_whole_head_rotates_no_scaling": _one_layer(X.sinked(2, 2, 8, 8, 0.3, softcap=2.0, rot=(8, 30.0)), None),
    "sinked_every_frequency_in_the_middle_band": _one_layer(X.sinked(2, 1, 8, 8, 0.3, rot=(4, 4.0, 3.0, 0.01, 1000.0, 50)), None),
    "moe_one_of_five": _one_layer(X.tempered(1, 1, 8, 0.3), X.moe(5, 1, 12)),
    "moe_three_of_seven": _one_layer(X.tempered(1, 1, 8, 0.3), X.moe(7, 3, 6)),
    "moe_every_expert": _one_layer(X.tempered(1, 1, 8, 0.3), X.moe(2, 2, 10)),
    "moe_one_expert": _one_layer(X.sinked(1, 1, 8, 8, 0.3), X.moe(1, 1, 20)),
    "loop_of_one_pass": _one_layer(X.tempered(2, 1, 8, 0.3, 0.5, 3), X.moe(3, 2, 8), loop=(0, 1, 1)),
    "loop_of_four_passes_unscaled_embedding": _one_layer(X.sinked(2, 2, 8, 8, 0.3, rot=(8, 30.0)), X.moe(3, 1, 8), scale=1.0, loop=(0, 1, 4)),
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("which", list(MECHANISMS))
def test_each_mechanism_alone(backend, which):
    """One-layer models, each with one mechanism, whole, in portions and with the last tokens one by one."""
    device, dtype = backend
    cfg = MECHANISMS[which]
    weights = X.random_weights(cfg, seed=5)
    reqs = X.make_requests(cfg, [37, 12], seed=1)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    for make in (C.trace_whole, C.trace_portions, lambda r: C.trace_tail(r, tail=9)):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", which, gaps)


@pytest.mark.parametrize("backend", BACKENDS)
def test_residual_stream_after_every_layer_run(backend):
    """The float32 stream the engine holds after each layer run equals the plain one (the pending branches added):
    the embedding's scale, each pass's added row and both branches of a layer show here before a final norm could
    hide a factor.  The engine is made to stop after the first d entries of its run order."""
    device, dtype = backend
    cfg, weights, reqs, _, gaps = setup("odd")
    toks = reqs["r2"]
    streams = []
    P.forward(weights, cfg, toks, streams)
    runs = P.layer_runs(cfg)
    for depth in (1, 2, 4, 5, 8):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        m = runner.model
        m.spec = copy.copy(m.spec)
        object.__setattr__(m.spec, "run_order", m.spec.run_order[:depth])
        captured = {}
        final = m.final_norm
        original = final.gather_add_norm

        def spy(residual, delta, rows, _original=original):
            settled = residual.float().clone()
            if delta is not None:
                parts = getattr(delta, "tensor", None)
                settled += delta.float() if parts is None else parts.float().sum(0)
            captured["x"] = settled.cpu()
            return _original(residual, delta, rows)

        final.gather_add_norm = spy
        C.run_trace(runner, C.trace_whole({"a": toks}))
        want = streams[depth - 1]
        keep = gaps["r2"] >= X.CLOSE_CALL[dtype == "bfloat16"]
        err = (captured["x"].double() - want)[keep].abs().max().item() / want.abs().max().item()
        assert err < (4e-2 if dtype == "bfloat16" else 1e-5), f"stream after layer run {depth - 1} (layer {runs[depth - 1][0]}): relative error {err:.2e}"


def _peaks(cfg, weights, toks):
    P.ATTENTION_PEAKS = seen = []
    try:
        want = P.forward(weights, cfg, toks)
    finally:
        P.ATTENTION_PEAKS = None
    return want, seen


def _differs(a, b):
    return X.relative_error(a.double(), b)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("kind", ["tempered", "sinked"])
def test_sharp_attention_over_a_long_prompt(backend, kind):
    """Scores multiplied so hard that nearly every query gives most of its weight to one key, which lies anywhere
    among the 300 before it: a key lost or misplaced at a page's border, at the border of a block of keys, among the
    first tokens or hundreds of tokens back changes that query's logits outright instead of by a three-hundredth."""
    device, dtype = backend
    layer = X.tempered(2, 1, 8, 14.0, 0.3, 64) if kind == "tempered" else X.sinked(2, 1, 8, 6, 6.0, softcap=60.0, rot=(4, 1000.0, 8.0, 1.0, 4.0, 64))
    cfg = _one_layer(layer, None, vocab=400)
    weights = X.random_weights(cfg, seed=13)
    if kind == "sinked":
        weights["l0.mix.sink"] = weights["l0.mix.sink"] - 3.0  # (a small sink: the keys have the weight)
    # (every token once: a mixer without positions gives equal tokens equal keys, which would share the weight)
    toks = torch.randperm(400, generator=torch.Generator().manual_seed(2))[:300].tolist()
    want, peaks = _peaks(cfg, weights, toks)
    late = [p for p in peaks if p[0] >= 100]
    assert sorted(p[3] for p in late)[len(late) // 2] > 0.5, "the test's attention was meant to be sharp"
    assert any(p[0] >= 200 and p[2] < 100 for p in peaks), "some late query was meant to pick a key far back"
    assert any(p[0] >= 150 and p[2] < 16 for p in peaks), "nor one of the first keys"
    for make in (lambda r: C.trace_tail(r, tail=60), C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 24, max_len=400)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", f"sharp {kind} attention")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_sink_takes_its_share(backend):
    """Sinks large enough to take much of the weight: without them (or with them scaled by the scores' scale, or
    squashed by the cap) the logits are others, which the plain implementation shows; first tokens, where one key
    stands against the sink, included."""
    device, dtype = backend
    cfg = _one_layer(X.sinked(3, 1, 8, 6, 0.3, softcap=2.0, rot=(8, 100.0)), None)
    weights = X.random_weights(cfg, seed=17)
    weights["l0.mix.sink"] = torch.tensor([4.0, 3.0, 5.0])
    reqs = X.make_requests(cfg, [40, 3, 1], seed=6)
    want = X.plain_logits(cfg, weights, reqs)
    without = X.plain_logits(cfg, dict(weights, **{"l0.mix.sink": torch.full((3,), -1e4)}), reqs)
    capped = X.plain_logits(cfg, dict(weights, **{"l0.mix.sink": 2.0 * torch.tanh(weights["l0.mix.sink"] / 2.0)}), reqs)
    for r in reqs:
        for other in (without, capped):
            d = _differs(other[r], want[r])
            assert d.min().item() > 0.01 and d.median().item() > 0.03, "the sinks were meant to matter at every position"
    for make in (C.trace_whole, lambda r: C.trace_tail(r, tail=30), C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "sinks")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("every,page", [(16, 16), (13, 16), (32, 16), (5, 32)])
def test_the_temperature_steps_where_it_says(backend, every, page):
    """A large coefficient, so that the step of the temperature decides how sharp a query is: the queries just
    before a step (position every * k - 2) and just after it (every * k - 1) differ by it, in prompts, portions and
    decoded tokens; stepping a token early or late, or counting positions from 1 twice, gives other logits there
    (shown with the plain implementation)."""
    device, dtype = backend
    cfg = _one_layer(X.tempered(2, 1, 8, 0.8, 3.0, every), None)
    weights = X.random_weights(cfg, seed=every)
    toks = X.make_requests(cfg, [150], seed=4)["r0"]
    want = P.forward(weights, cfg, toks)
    original = P.query_temperature
    late = lambda n, coef, ev: torch.cat([original(n, coef, ev)[:1], original(n, coef, ev)[:-1]])
    early = lambda n, coef, ev: original(n + 1, coef, ev)[1:]
    for wrong, first_edge in ((late, every - 1), (early, every - 2)):
        P.query_temperature = wrong
        try:
            d = _differs(P.forward(weights, cfg, toks), want)
        finally:
            P.query_temperature = original
        edges = [first_edge + k * every for k in range(3)]
        assert all(d[e] > 1e-3 for e in edges), f"a temperature that steps a token {'late' if wrong is late else 'early'} was meant to show"
        assert d[first_edge + 1] < 1e-9 or every == 1  # (and only there)
    for make in (lambda r: C.trace_tail(r, tail=70), lambda r: C.trace_portions(r, sizes=[7, 2, 30, 16, 3]), C.trace_whole):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), page, -(-150 // page) + 1, max_len=256)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", f"temperature every {every}")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_values_are_the_keys_before_the_norm(backend):
    """Biases and norm weights far from 0 and 1, so that keys before and after the norm are different vectors: the
    plain implementation with the normed keys as values, or with values that leave the bias out, gives other
    logits."""
    device, dtype = backend
    cfg = _one_layer(X.tempered(4, 2, 8, 0.3, 0.5, 8), None)
    weights = X.random_weights(cfg, seed=19)
    weights["l0.mix.k.b"] = (weights["l0.mix.k.b"] * 3.0).to(torch.bfloat16).float()
    weights["l0.mix.k.norm"] = (weights["l0.mix.k.norm"] * 2.0 - 1.5).to(torch.bfloat16).float()
    reqs = X.make_requests(cfg, [50, 6], seed=3)
    want = X.plain_logits(cfg, weights, reqs)
    original = P.tempered_attention

    def normed_values(W, p, m, eps, h):
        k = P.rms(h @ W[p + "k"].T + W[p + "k.b"], eps) * W[p + "k.norm"]
        return _with_values(W, p, m, eps, h, k.view(h.shape[0], m["kv_heads"], m["dim"]))

    def _with_values(W, p, m, eps, h, v):
        n, H, G, d = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
        q = P.rms(h @ W[p + "q"].T + W[p + "q.b"], eps) * W[p + "q.norm"]
        k = P.rms(h @ W[p + "k"].T + W[p + "k.b"], eps) * W[p + "k.norm"]
        q = (q * P.query_temperature(n, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]).view(n, H, d)
        k = k.view(n, G, d)
        out = torch.zeros(n, H, d, dtype=P.F)
        for i in range(n):
            for hd in range(H):
                g = hd // (H // G)
                out[i, hd] = torch.softmax((k[: i + 1, g] @ q[i, hd]) * m["scale"], 0) @ v[: i + 1, g]
        return out.reshape(n, H * d) @ W[p + "o"].T

    def unbiased_values(W, p, m, eps, h):
        return _with_values(W, p, m, eps, h, (h @ W[p + "k"].T).view(h.shape[0], m["kv_heads"], m["dim"]))

    for wrong in (normed_values, unbiased_values):
        P.tempered_attention = wrong
        try:
            other = X.plain_logits(cfg, weights, reqs)
        finally:
            P.tempered_attention = original
        assert (_differs(other["r0"], want["r0"]) > 0.05).float().mean().item() > 0.8, "which keys are the values was meant to show"
    for make in (C.trace_whole, lambda r: C.trace_tail(r, tail=20), C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "values from keys")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_norm_spans_all_heads(backend):
    """Heads of very different size (some rows of the projections are multiplied), so that one root mean square
    over all heads and one per head are different norms: the plain implementation with a norm per head gives other
    logits."""
    device, dtype = backend
    cfg = _one_layer(X.tempered(4, 2, 8, 0.5), None)
    weights = X.random_weights(cfg, seed=37)
    weights["l0.mix.q"][:8] *= 8.0
    weights["l0.mix.k"][8:] *= 0.125
    reqs = X.make_requests(cfg, [40, 9], seed=5)
    want = X.plain_logits(cfg, weights, reqs)
    original = P.rms

    def per_head(x, eps):
        if x.shape[-1] in (32, 16):  # the projections: normed head by head instead
            return original(x.view(x.shape[0], -1, 8), eps).reshape(x.shape)
        return original(x, eps)

    P.rms = per_head
    try:
        other = X.plain_logits(cfg, weights, reqs)
    finally:
        P.rms = original
    assert (_differs(other["r0"], want["r0"]) > 0.05).float().mean().item() > 0.7, "what the norm spans was meant to show"
    for make in (C.trace_whole, C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "a norm over all heads")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_rotation_far_beyond_the_original_context(backend):
    """Sharp scores that depend on distance through the rotation alone (the same token everywhere, so content
    says nothing): bands of frequencies scaled wrongly (every frequency divided, or none) give other logits 200
    tokens out, with the original context at 16."""
    device, dtype = backend
    cfg = _one_layer(X.sinked(2, 1, 16, 8, 2.0, rot=(12, 40.0, 6.0, 1.0, 4.0, 16)), None)
    weights = X.random_weights(cfg, seed=41)
    weights["l0.mix.sink"] = weights["l0.mix.sink"] - 2.0
    toks = X.make_requests(cfg, [230], seed=7)["r0"]
    want = P.forward(weights, cfg, toks)
    for change in ({"low": 1e-6, "high": 2e-6}, {"low": 1e5, "high": 2e5}):
        wrong = copy.deepcopy(cfg)
        wrong["layers"][0]["mixer"]["rot"]["scaling"].update(change)
        assert (_differs(P.forward(weights, wrong, toks), want)[100:] > 0.05).float().mean().item() > 0.6, "the bands were meant to show"
    for make in (lambda r: C.trace_tail(r, tail=80), C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 16, max_len=256)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", "rotation")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_routers_bias_and_the_weights_of_the_chosen(backend):
    """A router bias of several units and logits far apart, so that the bias decides who is chosen and the weights
    of the chosen are uneven: the plain implementation without the bias, with a softmax over all experts, or with
    the weight on the expert's input (an expert squares what it reads) gives other logits."""
    device, dtype = backend
    cfg = _one_layer(X.tempered(1, 1, 8, 0.3), X.moe(6, 3, 16))
    weights = X.random_weights(cfg, seed=29)
    weights["l0.mlp.router.b"] = torch.tensor([3.0, -2.0, 0.5, 2.0, -3.0, 1.0])
    weights["l0.mlp.router"] = (weights["l0.mlp.router"] * 0.4).to(torch.bfloat16).float()  # (the experts left out keep some weight)
    for e in range(6):
        weights[f"l0.mlp.e{e}.up"] = (weights[f"l0.mlp.e{e}.up"] * 1.5).to(torch.bfloat16).float()
    reqs = X.make_requests(cfg, [60, 5], seed=12)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    original = P.moe_ff

    def variant(bias=True, over_all=False, on_input=False):
        def ff(W, p, f, h):
            top = f["router"]["top"]
            logits = h @ W[p + "router"].T + (W[p + "router.b"] if bias else 0.0)
            out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=P.F)
            for t in range(h.shape[0]):
                chosen = torch.topk(logits[t], top).indices.tolist()
                weight = torch.softmax(logits[t], 0)[chosen] if over_all else torch.softmax(logits[t][chosen], 0)
                for w, e in zip(weight, chosen):
                    out[t] += P.expert(W, f"{p}e{e}.", (w * h[t])[None])[0] if on_input else w * P.expert(W, f"{p}e{e}.", h[t][None])[0]
            return out
        return ff

    for wrong in (variant(bias=False), variant(over_all=True), variant(on_input=True)):
        P.moe_ff = wrong
        try:
            other = X.plain_logits(cfg, weights, reqs)
        finally:
            P.moe_ff = original
        assert (_differs(other["r0"], want["r0"]) > 3e-3).float().mean().item() > 0.8, "the router's rules were meant to show"
    for make in (C.trace_whole, C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "router", gaps)


@pytest.mark.parametrize("backend", BACKENDS)
def test_each_pass_has_its_own_pages_and_row(backend):
    """Rows of the table of steps that are large and differ, three passes over one layer: passes that shared their
    pages, or took the first pass's row again, would give other logits (the plain implementation with one row for
    all passes shows the second)."""
    device, dtype = backend
    cfg = _one_layer(X.tempered(2, 1, 8, 0.4, 0.5, 8), X.moe(3, 1, 8), loop=(0, 1, 3))
    weights = X.random_weights(cfg, seed=43)
    weights["loop.step"] = (weights["loop.step"] * 4.0).to(torch.bfloat16).float()
    reqs = X.make_requests(cfg, [45, 4, 17], seed=2)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)
    same = dict(weights, **{"loop.step": weights["loop.step"][:1].repeat(3, 1)})
    assert (_differs(X.plain_logits(cfg, same, reqs)["r0"], want["r0"]) > 0.05).float().mean().item() > 0.8
    for make in (C.trace_whole, lambda r: C.trace_tail(r, tail=12), C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 6)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "passes", gaps)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("num_pages", [24, 7])
def test_greedy_generation_through_the_engine(tmp_path, backend, num_pages):
    """``LLMEngine.generate`` with the scheduler under a token budget that cuts prompts into portions, and with so
    few pages that the youngest request is preempted and starts again: greedy tokens are the plain implementation's
    wherever its two best logits are clearly apart."""
    from yalis_amd import EngineConfig, InferenceConfig, LLMEngine, ModelConfig
    from yalis_amd.weights.safetensors_io import write_dict

    device, dtype = backend
    cfg = X.CONFIGS["odd"]
    weights = X.random_weights(cfg, seed=9)
    weights["embed"] = (weights["embed"] * 3.0).to(torch.bfloat16).float()  # (logits far enough apart to call)
    folder = tmp_path / "model"
    os.makedirs(folder)
    with open(folder / "config.json", "w") as f:
        json.dump(cfg, f)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    write_dict(str(folder / "model.safetensors"), {k: v.to(wd).contiguous() for k, v in weights.items()})
    precision = "fp32" if dtype == "float32" else "bf16"
    eng = LLMEngine(
        ModelConfig(model_path=str(folder), precision=precision),
        InferenceConfig(max_batch_size=3, max_length_of_generated_sequences=128, temperature=0.0),
        device=device, ops=RefOps() if device == "cpu" else None,
        engine_config=EngineConfig(page_size=16, num_pages=num_pages, max_num_seqs=3, max_model_len=128, max_num_batched_tokens=24,
                                   dtype=dtype, device=device),
    )
    prompts = list(X.make_requests(cfg, [30, 7, 45], seed=4).values())
    out, metrics = eng.generate(prompts, tokens_to_generate=12)
    assert out.shape == (3, 12)
    if num_pages == 7:
        assert metrics["Preemptions"] > 0, "this pool was meant to force a preemption"
    gap = 0.2 if dtype == "bfloat16" else 1e-3
    compared = 0
    for prompt, row in zip(prompts, out.tolist()):
        toks = list(prompt)
        for t in row:
            logits = P.forward(weights, cfg, toks)[-1]
            top2 = torch.topk(logits, 2).values
            if (top2[0] - top2[1]).item() < gap * logits.abs().max().item():
                break  # too close to call; what follows would compare other sequences
            assert t == int(torch.argmax(logits)), f"generated {row}, the plain implementation differs after {len(toks) - len(prompt)} tokens"
            toks.append(t)
            compared += 1
    assert compared >= 3


def test_config_reader_and_spec():
    """Sizes and constants come from config.json; what cannot run is refused with the key's name; the tensors a
    model asks for are the design's names and shapes."""
    from yalis_amd.config.reader import ConfigError
    from yalis_amd.engine.factory import spec_from_config, tensor_specs_for

    cfg = X.CONFIGS["mix"]
    _, typed, spec = spec_from_config(cfg)
    assert spec.vocab_size == 128 and spec.hidden_size == 64 and len(spec.layers) == 4 and len(spec.run_order) == 4
    assert spec.head.params["tied_to"] == "embed" and spec.embedding.params["scale"] == 1.0
    assert all(layer.block == "parallel" for layer in spec.layers)
    a2 = spec.layers[0].parts["mixer"].params
    assert (a2["num_heads"], a2["num_kv_heads"], a2["head_dim"], a2["value_dim"], a2["softcap"], a2["sink"], a2["gate_per"]) == (4, 1, 16, 24, 30.0, "sink", "element")
    rot = a2["position"].params
    assert rot["rotary_dim"] == 8 and rot["scaling"] == {"kind": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                                         "original_max_position_embeddings": 32.0}
    assert a2["qk_norm"].get("over", "head") == "head"
    a1 = spec.layers[1].parts["mixer"].params
    assert a1["values_from_keys"] and a1["qk_norm"]["over"] == "projection" and a1["query_temperature"] == {"coef": 0.4, "every": 16}
    assert a1["projection_bias"] == {"q": "q.b", "k": "k.b"} and a1["position"] is None
    assert "feed_forward" not in spec.layers[1].parts
    moe = spec.layers[2].parts["feed_forward"].params
    assert (moe["experts"], moe["top"], moe["intermediate_size"], moe["gated"], moe["activation"], moe["scores"], moe["weighs"]) == \
        (6, 3, 16, False, "relu2", "softmax_of_chosen", "output")
    assert spec.layers[0].parts["norm"].params["unit_offset"] is False
    specs = tensor_specs_for(cfg)
    assert specs["embed"].shape == (128, 64) and "head" not in specs and "loop.step" not in specs
    assert specs["l0.mix.q"].shape == (64, 64) and specs["l0.mix.k"].shape == (16, 64) and specs["l0.mix.v"].shape == (24, 64)
    assert specs["l0.mix.q.norm"].shape == (16,) and specs["l0.mix.sink"].shape == (4,) and specs["l0.mix.g"].shape == (96, 64)
    assert specs["l0.mix.o"].shape == (64, 96)
    assert specs["l1.mix.q.norm"].shape == (64,) and specs["l1.mix.k.norm"].shape == (64,) and specs["l1.mix.q.b"].shape == (64,)
    assert "l1.mix.v" not in specs and "l1.mix.g" not in specs and not any(k.startswith("l1.mlp") for k in specs)
    assert specs["l2.mlp.e5.up"].shape == (16, 64) and specs["l2.mlp.e5.down"].shape == (64, 16) and "l2.mlp.e0.gate" not in specs
    assert specs["l2.mlp.router"].shape == (6, 64) and specs["l2.mlp.router.b"].shape == (6,)
    assert not any(k.endswith(("norm2",)) for k in specs)
    for path, value, what in [
        (("layers", 0, "mixer", "kv_heads"), 3, "multiple"), (("layers", 1, "mixer", "vdim"), 16, "vdim"),
        (("layers", 0, "type"), "mamba2", "not one of"), (("layers", 0, "mixer", "rot", "dims"), 18, "dims"),
        (("layers", 0, "mixer", "rot", "dims"), 7, "dims"), (("layers", 2, "mlp", "router", "top"), 7, "top"),
        (("layers", 2, "mlp", "kind"), "dense", "kind"), (("layers", 1, "mixer", "q_temp", "every"), 0, "every"),
        (("loop",), {"start": 2, "stop": 2, "times": 2}, "stretch"), (("loop",), {"start": 0, "stop": 5, "times": 2}, "stretch"),
        (("loop",), {"start": 0, "stop": 2, "times": 0}, "times"),
    ]:
        bad = copy.deepcopy(cfg)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError, match=what):
            spec_from_config(bad)
    unscaled = copy.deepcopy(cfg)
    del unscaled["embedding"]
    assert spec_from_config(unscaled)[2].embedding.params["scale"] == 1.0
    for path in (("embedding", "scale"), ("layers", 0, "mixer", "scale"), ("norm", "eps")):
        missing = copy.deepcopy(cfg)
        node = missing
        for key in path[:-1]:
            node = node[key]
        del node[path[-1]]
        with pytest.raises(ConfigError, match=path[-1]):
            spec_from_config(missing)
