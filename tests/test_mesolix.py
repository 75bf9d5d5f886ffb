"""Mesolix in the engine against the plain implementation (tests/plain_mesolix.py): every way of cutting the
work, on the CPU with plain PyTorch ops (the host side: batching, paging, slots, the order of parts) and,
marked ``gpu``, with the HIP kernels in true float32 and in bfloat16."""
import copy
import json
import os

import pytest
import torch

import mesolix_cases as X
import plain_mesolix as P
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
    decoding); portions down to two tokens; up to four unequal requests a step in a pool so small that pages and
    slots are used again; cuts at random."""
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


def test_memory_plan():
    """A layer that runs another's weights again owns a cache or a state of its own; latent layers keep a row of
    kv_rank numbers a token and no values; the recurrent layers keep a matrix per head and, with more than one tap,
    the convolution's last inputs."""
    cfg, weights, _, _, _ = setup("mix")
    runner = X.make_runner(cfg, weights, "float32", "cpu", RefOps(), 32, 4)
    m = runner.model
    assert len(m.sites) == 7 and [e.layer for e in m.spec.run_order] == [0, 1, 2, 3, 2, 4, 0]
    assert [s.owns_cache for s in m.sites] == [True, False, True, False, True, True, True]
    assert m.blocks[m.spec.run_order[6].layer] is m.blocks[m.spec.run_order[0].layer]
    needs = sorted((g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, g.need.window, len(g.entries)) for g in m.cache_groups)
    assert needs == sorted([(1, 24, 0, None, 2), (1, 16, 16, 40, 2), (1, 48, 0, None, 1)])
    assert sorted(tuple(s.shape) for s in m.state_needs) == sorted([(4, 16, 16), (2, 24, 32), (3, 2 * 32 + 2 * 2 * 24)])


@pytest.mark.parametrize("backend", BACKENDS)
def test_slots_are_used_again_with_clean_state(backend):
    """Two slots, six requests one after another in pairs: a request that takes over a slot starts from a zero
    matrix and an empty convolution, whatever the one before left there."""
    device, dtype = backend
    cfg, weights, reqs, want, gaps = setup("odd")
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 16, max_seqs=2)
    steps = C.trace_mixed(reqs, max_live=2)
    got, _ = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", "two slots", gaps)
    assert runner.pages.free_slots() == 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    """A short prompt and 200 tokens decoded one by one: the states are carried through every step, the window
    slides over decoded tokens and gives pages back, the latent attention reads pages written by hundreds of
    earlier steps."""
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
    fall inside pages, inside the window and inside the blocks of keys the attention kernels walk."""
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


def _one_layer(layer, ff, width=32, eps=1e-5):
    return X.model(80, width, eps, 400, [(layer, ff)])


MECHANISMS = {
    "latent_attention": _one_layer(X.latent(2, 8, 12, 16, 10, 0.4), None),
    "latent_attention_one_head_equal_sizes": _one_layer(X.latent(1, 16, 16, 8, 8, 0.25), None),
    "window": _one_layer(X.window(4, 2, 8, 6, 0.3, 9, 8, 30.0), None),
    "window_every_key_visible_one_kv_head": _one_layer(X.window(3, 1, 6, 10, 0.5, None, 12, 20.0), None),
    "window_of_one_key": _one_layer(X.window(2, 2, 8, 8, 0.3, 1, 4, 16.0), None),
    "window_two_buckets": _one_layer(X.window(2, 1, 4, 4, 0.3, 30, 2, 9.0), None),
    "ssd": _one_layer(X.ssd(4, 6, 8, 2, 4, 2), None),
    "ssd_one_tap_one_group_every_head_normed_alone": _one_layer(X.ssd(3, 8, 5, 1, 1, 3), None),
    "ssd_a_group_per_head_wide_state": _one_layer(X.ssd(2, 4, 70, 2, 2, 1), None),
    "dense": _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.dense(48, 0.6)),
    "dense_wide_limit": _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.dense(20, 7.0)),
    "moe_one_of_five": _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.moe(5, 1, 12)),
    "moe_three_of_seven_with_shared": _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.moe(7, 3, 6, shared=20)),
    "moe_every_expert": _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.moe(2, 2, 10, shared=4)),
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
def test_residual_stream_after_every_layer(backend):
    """The float32 stream the engine holds after each layer run equals the plain one (the pending branch added):
    the learned positions, the norms' weights around zero and every branch show here before a final norm could
    hide a factor."""
    device, dtype = backend
    cfg, weights, reqs, _, gaps = setup("odd")
    toks = reqs["r2"]
    streams = []
    P.forward(weights, cfg, toks, streams)
    for depth in range(1, len(cfg["layers"]) + 1):
        cut = copy.deepcopy(cfg)
        cut["layers"] = cut["layers"][:depth]
        names = X.tensor_specs_for(cut)
        runner = X.make_runner(cut, {k: weights[k] for k in names}, dtype, device, ops_for(device), 16, 8)
        captured = {}
        final = runner.model.final_norm
        original = final.gather_add_norm

        def spy(residual, delta, rows, _original=original):
            settled = residual.float().clone()
            if delta is not None:  # a tensor, or a product's slices that are still to be summed
                parts = getattr(delta, "tensor", None)
                settled += delta.float() if parts is None else parts.float().sum(0)
            captured["x"] = settled.cpu()
            return _original(residual, delta, rows)

        final.gather_add_norm = spy
        C.run_trace(runner, C.trace_whole({"a": toks}))
        want = streams[depth - 1]
        keep = gaps["r2"] >= X.CLOSE_CALL[dtype == "bfloat16"]
        err = (captured["x"].double() - want)[keep].abs().max().item() / want.abs().max().item()
        assert err < (4e-2 if dtype == "bfloat16" else 1e-5), f"stream after layer run {depth - 1}: relative error {err:.2e}"


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
def test_sharp_latent_attention_over_a_long_prompt(backend):
    """Scores multiplied so hard that nearly every query gives most of its weight to one key, which lies anywhere
    among the 300 before it: a key lost or misplaced at a page's border, at the border of a block of keys, among the
    first tokens or hundreds of tokens back changes that query's logits outright instead of by a three-hundredth."""
    device, dtype = backend
    cfg = _one_layer(X.latent(2, 8, 12, 16, 10, 30.0), None)
    weights = X.random_weights(cfg, seed=13)
    weights["l0.mix.sink"] = weights["l0.mix.sink"] - 3.0  # (a small sink: the keys have the weight)
    toks = X.make_requests(cfg, [300], seed=2)["r0"]
    want, peaks = _peaks(cfg, weights, toks)
    late = [p for p in peaks if p[0] >= 100]
    assert sorted(p[3] for p in late)[len(late) // 2] > 0.5, "the test's attention was meant to be sharp"
    assert any(p[0] >= 200 and p[2] < 100 for p in peaks), "some late query was meant to pick a key far back"
    assert any(p[0] >= 250 and p[2] < 8 for p in peaks) or any(p[0] >= 150 and p[2] < 16 for p in peaks), "nor one of the first keys"
    for make in (lambda r: C.trace_tail(r, tail=60), C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 24, max_len=400)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", "sharp latent attention")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_sink_takes_its_share(backend):
    """Sinks large enough to take much of the weight: without them (or with them scaled, or
    counted per key) the logits are others, which the plain implementation without sinks shows; first tokens, where
    one key stands against the sink, included."""
    device, dtype = backend
    cfg = _one_layer(X.latent(3, 8, 6, 12, 10, 0.3), None)
    weights = X.random_weights(cfg, seed=17)
    weights["l0.mix.sink"] = torch.tensor([4.0, 3.0, 5.0])
    reqs = X.make_requests(cfg, [40, 3, 1], seed=6)
    want = X.plain_logits(cfg, weights, reqs)
    without = X.plain_logits(cfg, dict(weights, **{"l0.mix.sink": torch.full((3,), -1e4)}), reqs)
    for r in reqs:
        d = _differs(without[r], want[r])
        assert d.min().item() > 0.01 and d.median().item() > 0.03, "the sinks were meant to matter at every position"
    for make in (C.trace_whole, lambda r: C.trace_tail(r, tail=30), C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "sinks")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("size,page", [(13, 16), (16, 16), (40, 16), (33, 32)])
def test_the_window_ends_where_it_says(backend, size, page):
    """Sharp scores again, now below a window: many queries give their weight to the last key the window keeps,
    and many would give it to the one just outside if they saw it (the plain implementation with a window one key
    longer or shorter gives other logits there), in a prompt, in portions and in tokens decoded one by one while
    pages behind the window are given back."""
    device, dtype = backend
    layer = X.window(2, 1, 8, 6, 4.0, size, 6, 24.0)
    cfg = _one_layer(layer, None)
    weights = X.random_weights(cfg, seed=size)
    weights["l0.mix.rel"] = weights["l0.mix.rel"] * 0.3
    toks = X.make_requests(cfg, [170], seed=4)["r0"]
    want, peaks = _peaks(cfg, weights, toks)
    edge = [p for p in peaks if p[0] - p[2] == size - 1 and p[3] > 0.5]
    assert any(p[0] < 100 for p in edge) and any(p[0] >= 110 for p in edge), "queries were meant to pick the window's last key"
    for other in (size + 1, size - 1):
        if other < 1:
            continue
        wrong_cfg = copy.deepcopy(cfg)
        wrong_cfg["layers"][0]["mixer"]["mask"]["size"] = other
        d = _differs(P.forward(weights, wrong_cfg, toks), want)
        assert (d[:100] > 0.1).any() and (d[110:] > 0.1).any(), f"a window of {other} was meant to show"
    for make in (lambda r: C.trace_tail(r, tail=60), lambda r: C.trace_portions(r, sizes=[7, 2, 30, 16, 3])):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), page, -(-170 // page) + 1, max_len=256)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", f"window of {size}")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("rows,far,size", [(10, 40.0, None), (7, 33.0, 64), (16, 120.0, 96), (4, 3.0, None)])
def test_the_bias_per_distance(backend, rows, far, size):
    """A table with large entries, so that the bias decides where the weight goes: the rows for exact distances,
    the rows that cover growing stretches, the last row for everything beyond ``far``; an odd number of rows; a
    table read by a row off, or a bias multiplied by the scale, gives other logits (shown with the plain
    implementation)."""
    device, dtype = backend
    cfg = _one_layer(X.window(3, 3, 6, 5, 0.2, size, rows, far), None)
    weights = X.random_weights(cfg, seed=rows)
    weights["l0.mix.rel"] = (weights["l0.mix.rel"] * 3.0).to(torch.bfloat16).float()
    reqs = X.make_requests(cfg, [150], seed=7)
    want = X.plain_logits(cfg, weights, reqs)
    shifted = dict(weights, **{"l0.mix.rel": torch.roll(weights["l0.mix.rel"], 1, 0)})
    assert (_differs(X.plain_logits(cfg, shifted, reqs)["r0"], want["r0"]) > 0.05).float().mean().item() > 0.8
    scaled = dict(weights, **{"l0.mix.rel": weights["l0.mix.rel"] * 0.2})
    assert (_differs(X.plain_logits(cfg, scaled, reqs)["r0"], want["r0"]) > 0.05).float().mean().item() > 0.8
    if far > rows:  # (else every row past the exact ones is the last)
        nearer = copy.deepcopy(cfg)
        nearer["layers"][0]["mixer"]["bias_max"] = far * 0.7
        assert (_differs(X.plain_logits(nearer, weights, reqs)["r0"], want["r0"])[rows:] > 0.05).float().mean().item() > 0.3
    for make in (C.trace_whole, lambda r: C.trace_tail(r, tail=70), C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 12, max_len=256)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", f"bias with {rows} rows")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_state_remembers_far_back(backend):
    """Decays so slow that what was written a hundred and more tokens ago still decides the read-out (with the
    learned positions set to zero the plain implementation started 160 tokens late is the same model with its state
    lost there, and gives other logits to the end), next to a head that forgets at once: a state that is lost,
    zeroed or decayed by the wrong step between portions shows at every later token."""
    device, dtype = backend
    cfg = _one_layer(X.ssd(4, 6, 8, 2, 3, 2), None)
    weights = X.random_weights(cfg, seed=23)
    weights["l0.mix.A_log"] = torch.tensor([-6.0, -5.0, 1.5, -7.0])
    weights["l0.mix.dt_bias"] = torch.tensor([0.5, 1.0, 2.0, -0.5])
    weights["l0.mix.D"] = weights["l0.mix.D"] * 0.1
    weights["pos"] = torch.zeros_like(weights["pos"])
    toks = X.make_requests(cfg, [260], seed=9)["r0"]
    want = P.forward(weights, cfg, toks)
    assert _differs(P.forward(weights, cfg, toks[160:]), want[160:])[-20:].min().item() > 0.05, "tokens far back were meant to be remembered"
    for make in (lambda r: C.trace_tail(r, tail=100), lambda r: C.trace_portions(r, sizes=[64, 2, 3, 61, 17]), C.trace_whole):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 4, max_len=400)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, {"a": want}, dtype == "bfloat16", "slow decays")


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_score_weighs_an_experts_input(backend):
    """Experts whose gates are steep, so that an expert is far from linear in its input: the plain implementation with the score on the expert's output instead (which differs because an expert is not
    linear) or with renormalised scores gives other logits; with ``top`` 2 of 4 and no shared expert."""
    device, dtype = backend
    cfg = _one_layer(X.ssd(1, 8, 8, 1, 2, 1), X.moe(4, 2, 16))
    weights = X.random_weights(cfg, seed=29)
    weights["l0.mlp.router"] = (weights["l0.mlp.router"] * 0.5).to(torch.bfloat16).float()
    for e in range(4):
        weights[f"l0.mlp.e{e}.gate"] = (weights[f"l0.mlp.e{e}.gate"] * 6.0).to(torch.bfloat16).float()
    reqs = X.make_requests(cfg, [60, 5], seed=12)
    want, gaps = X.plain_logits_and_gaps(cfg, weights, reqs)

    original = P.moe_ff

    def score_on_the_output(W, p, f, h):
        logits = h @ W[p + "router"].T
        s = torch.sigmoid(logits)
        out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=P.F)
        for t in range(h.shape[0]):
            for e in torch.topk(s[t], f["router"]["top"]).indices.tolist():
                out[t] += s[t, e] * P.silu_expert(W, f"{p}e{e}.", h[t][None])[0]
        return out

    P.moe_ff = score_on_the_output
    try:
        wrong = X.plain_logits(cfg, weights, reqs)
    finally:
        P.moe_ff = original
    assert (_differs(wrong["r0"], want["r0"]) > 0.02).float().mean().item() > 0.8, "the place of the score was meant to show"
    for make in (C.trace_whole, C.trace_mixed):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", "scores on inputs", gaps)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("num_pages", [24, 7])
def test_greedy_generation_through_the_engine(tmp_path, backend, num_pages):
    """``LLMEngine.generate`` with the scheduler under a token budget that cuts prompts into portions, and with so
    few pages that the youngest request is preempted and starts again (its state slot cleared): greedy tokens are
    the plain implementation's wherever its two best logits are clearly apart."""
    from yalis_amd import EngineConfig, InferenceConfig, LLMEngine, ModelConfig
    from yalis_amd.weights.safetensors_io import write_dict

    device, dtype = backend
    cfg = X.CONFIGS["odd"]
    weights = X.random_weights(cfg, seed=9)
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
    for prompt, row in zip(prompts, out.tolist()):
        toks = list(prompt)
        for t in row:
            logits = P.forward(weights, cfg, toks)[-1]
            top2 = torch.topk(logits, 2).values
            if (top2[0] - top2[1]).item() < gap * logits.abs().max().item():
                break  # too close to call; what follows would compare other sequences
            assert t == int(torch.argmax(logits)), f"generated {row}, the plain implementation differs after {len(toks) - len(prompt)} tokens"
            toks.append(t)


def test_config_reader_and_spec():
    """Sizes and constants come from config.json; what cannot run is refused with the key's name; the tensors a
    model asks for are the design's names and shapes; a layer that names another's weights becomes a second run of
    that layer and asks for no tensors."""
    from yalis_amd.config.reader import ConfigError
    from yalis_amd.engine.factory import spec_from_config, tensor_specs_for

    cfg = X.CONFIGS["mix"]
    _, typed, spec = spec_from_config(cfg)
    assert spec.vocab_size == 128 and spec.hidden_size == 64 and len(spec.layers) == 5 and len(spec.run_order) == 7
    assert spec.head.params["tied_to"] is None and spec.embedding.kind == "token_position_embedding"
    assert all(layer.block == "prenorm" for layer in spec.layers)
    lat = spec.layers[0].parts["mixer"].params
    assert (lat["num_heads"], lat["head_dim"], lat["rot_dim"], lat["value_dim"], lat["kv_rank"], lat["q_rank"]) == (2, 32, 0, 16, 24, 40)
    assert lat["sink"] == "sink" and lat["gate_per"] == "element" and lat["position"] is None
    att = spec.layers[2].parts["mixer"].params
    assert (att["window"], att["scale"], att["distance_bias"]["far"], att["num_kv_heads"]) == (40, 0.25, 64.0, 1)
    assert "feed_forward" not in spec.layers[2].parts and "feed_forward_norm" not in spec.layers[2].parts
    assert spec.layers[1].parts["feed_forward"].params["activation"] == ("clamped_swish", 2.5, 1.702)
    moe = spec.layers[0].parts["feed_forward"].params
    assert (moe["experts"], moe["top"], moe["intermediate_size"], moe["shared"]["intermediate_size"]) == (4, 1, 32, 16)
    assert spec.layers[3].parts["feed_forward"].params["shared"] is None
    assert spec.layers[0].parts["mixer_norm"].params["unit_offset"] is True
    specs = tensor_specs_for(cfg)
    assert specs["pos"].shape == (512, 64) and specs["head"].shape == (128, 64)
    assert specs["l0.mix.dkv"].shape == (24, 64) and specs["l0.mix.uq"].shape == (2 * 32, 40) and specs["l0.mix.g"].shape == (2 * 16, 64)
    assert specs["l0.mix.sink"].shape == (2,) and specs["l0.mix.uv"].shape == (2 * 16, 24)
    assert specs["l1.mix.in"].shape == (2 * 64 + 2 * 16 + 4, 64) and specs["l1.mix.conv"].shape == (64 + 32, 1) and specs["l1.mix.norm"].shape == (64,)
    assert specs["l3.mix.in"].shape == (2 * 64 + 2 * 2 * 24 + 2, 64) and specs["l3.mix.conv.b"].shape == (64 + 96,)
    assert specs["l2.mix.rel"].shape == (8, 4) and specs["l2.mix.k"].shape == (16, 64) and specs["l2.mix.g"].shape == (64, 64)
    assert specs["l0.mlp.e3.gate"].shape == (32, 64) and specs["l0.mlp.shared.down"].shape == (64, 16) and specs["l0.mlp.router"].shape == (4, 64)
    assert not any(k.startswith(("l4.", "l6.", "l2.norm2", "l2.mlp")) for k in specs) and "l5.norm2" in specs
    for path, value, what in [
        (("layers", 2, "mixer", "kv_heads"), 3, "multiple"), (("layers", 1, "mixer", "groups"), 3, "multiple"),
        (("layers", 1, "mixer", "norm_groups"), 5, "norm_groups"), (("layers", 0, "type"), "delta", "not one of"),
        (("layers", 4, "weights_of"), 5, "earlier layer"), (("layers", 6, "weights_of"), 4, "earlier layer"),
        (("layers", 4, "mixer", "scale"), 0.5, "again"), (("layers", 0, "mlp", "router", "top"), 5, "top"),
        (("layers", 1, "mlp", "kind"), "glu", "kind"),
    ]:
        bad = copy.deepcopy(cfg)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError, match=what):
            spec_from_config(bad)
    missing = copy.deepcopy(cfg)
    del missing["layers"][2]["mixer"]["bias_max"]
    with pytest.raises(ConfigError, match="bias_max"):
        spec_from_config(missing)


def test_the_bias_tables_rows_come_from_the_checkpoint(tmp_path):
    """Nothing in config.json says how many rows the table of biases has: a folder whose table has another number
    of rows than the random-weights mode would make loads and runs as the plain implementation does."""
    from yalis_amd.config.runtime import EngineConfig
    from yalis_amd.engine.factory import load_runner
    from yalis_amd.weights.safetensors_io import write_dict

    cfg = _one_layer(X.window(2, 1, 8, 6, 0.3, 50, 6, 40.0), None)
    weights = X.random_weights(cfg, seed=3)
    del cfg["layers"][0]["mixer"]["bias_rows"]
    g = torch.Generator().manual_seed(1)
    weights["l0.mix.rel"] = (torch.randn((22, 2), generator=g) * 2.0).to(torch.bfloat16).float()
    folder = tmp_path / "model"
    os.makedirs(folder)
    with open(folder / "config.json", "w") as f:
        json.dump(cfg, f)
    write_dict(str(folder / "model.safetensors"), {k: v.contiguous() for k, v in weights.items()})
    eng = EngineConfig(page_size=16, num_pages=8, max_num_seqs=2, max_model_len=128, max_num_batched_tokens=128, dtype="float32", device="cpu")
    runner = load_runner(str(folder), eng, ops=RefOps())
    toks = X.make_requests(cfg, [90], seed=1)
    got, _ = C.run_trace(runner, C.trace_tail(toks, tail=20))
    X.assert_matches(got, X.plain_logits(cfg, weights, toks), False, "22 rows")
