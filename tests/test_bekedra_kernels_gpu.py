"""What Bekedra added to the kernels, each against plain arithmetic (float64 where the inputs are made by hand,
tests/kernel_refs.py otherwise), at sizes of their own, odd ones included, and with inputs made so that a fault
shows: one key whose score stands out, placed at every edge, against sinks large enough to decide."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import kernel_refs as R
from kernel_refs import tile_cache, untile_cache
from test_nutavik_kernels_gpu import close, context
from yalis_amd.engine.batch import SeqSpan, attention_tiles, build_host_batch

pytestmark = pytest.mark.gpu

_ops = {}


def ops():
    if "o" not in _ops:
        from yalis_amd.ops.hip import HipOps

        _ops["o"] = HipOps("cuda:0")
    return _ops["o"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 320, 4096])
def test_scaled_embedding(dtype, width):
    o = ops()
    g = torch.Generator().manual_seed(width)
    table = torch.randn(90, width, generator=g).to(dtype)
    ids = torch.randint(0, 90, (61,), generator=g, dtype=torch.int32)
    got = o.embed(ids.cuda(), table.cuda(), scale=11.5)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), table.float()[ids.long()] * 11.5)
    pos_table = torch.randn(7, width, generator=g).to(dtype)
    pos = torch.randint(0, 7, (61,), generator=g, dtype=torch.int32)
    got = o.embed(ids.cuda(), table.cuda(), positions=pos.cuda(), position_table=pos_table.cuda(), scale=3.0)
    close(got, table.float()[ids.long()] * 3.0 + pos_table.float()[pos.long()], torch.float32, "scaled, with positions", f32=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,n", [(40, 5), (42, 3), (320, 37), (4096, 9), (8200, 2)])
def test_a_vector_for_every_row_joins_in_the_norm(dtype, width, n):
    """residual += delta + row, then the norm, in one pass: with a delta, with a product's slices, with nothing
    else pending; the residual is written back."""
    o = ops()
    g = torch.Generator().manual_seed(width + n)
    res = torch.randn(n, width, generator=g) * 2
    delta = torch.randn(n, width, generator=g).to(dtype)
    row = torch.randn(width, generator=g) * 3
    w = (torch.randn(width, generator=g) * 0.3 + 1).to(dtype)
    for d in (delta, None):
        r = res.clone().cuda()
        got = o.add_rmsnorm(r, None if d is None else d.cuda(), w.cuda(), 1e-5, False, dtype, row=row.cuda())
        stream = res.double() + (0 if d is None else d.double()) + row.double()
        close(r, stream, torch.float32, "residual", f32=1e-6)
        want = stream / torch.sqrt((stream * stream).mean(-1, keepdim=True) + 1e-5) * w.double()
        close(got, want, dtype, "normed", f32=1e-5, bf16=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,extra", [(4, 2, 8, 0), (3, 3, 10, 6), (16, 4, 64, 16), (32, 8, 128, 0), (5, 0, 12, 4)])
def test_rows_scales(dtype, heads, kv, dim, extra):
    """The inverse root mean square over all query columns and over all key columns of the biased projection, and
    the temperature by position; each alone and both; positions just before and after a step of the temperature."""
    o = ops()
    g = torch.Generator().manual_seed(heads * dim)
    n, nq, nk = 70, heads * dim, kv * dim
    proj = (torch.randn(n, nq + nk + extra, generator=g) * 2).to(dtype)
    bias = torch.randn(nq + nk + extra, generator=g)
    pos = torch.randint(0, 500, (n,), generator=g, dtype=torch.int32)
    pos[:6] = torch.tensor([0, 62, 63, 64, 126, 127], dtype=torch.int32)
    for b in (bias, None):
        for eps in (1e-5, None):
            for temp in ((0.75, 64), (2.0, 1), None):
                if eps is None and temp is None:
                    continue
                got = o.qk_row_scales(proj.cuda(), nq, nk, pos.cuda(), bias=None if b is None else b.cuda(), eps=eps, temperature=temp)
                x = proj.double() + (0 if b is None else b.double())
                want = torch.ones(n, 2, dtype=torch.float64)
                if eps is not None:
                    want[:, 0] = 1 / torch.sqrt((x[:, :nq] ** 2).mean(-1) + eps)
                    if nk:
                        want[:, 1] = 1 / torch.sqrt((x[:, nq: nq + nk] ** 2).mean(-1) + eps)
                if temp is not None:
                    want[:, 0] *= 1 + temp[0] * torch.log(torch.div(pos.long() + 1, temp[1], rounding_mode="floor").double() + 1)
                close(got, want, torch.float32, f"scales (bias {b is not None}, eps {eps}, temperature {temp})", f32=2e-6)
                close(got, R.qk_row_scales(proj, nq, nk, pos, bias=b, eps=eps, temperature=temp), torch.float32, "against the plain counterpart", f32=2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,page,n", [(4, 2, 8, 16, 5), (3, 3, 10, 16, 40), (4, 2, 64, 64, 37), (8, 2, 128, 64, 20), (2, 1, 80, 32, 3)])
def test_prepare_with_biases_a_norm_over_all_heads_and_values_from_keys(dtype, heads, kv, dim, page, n):
    """qkv_prepare with everything the design's first mixer asks of it, for few tokens and for many (the two forms of
    the kernel), plain pages and tiled ones: queries, and what the pages then hold, against the plain counterpart."""
    o = ops()
    g = torch.Generator().manual_seed(heads * dim + n)
    nq, nk = heads * dim, kv * dim
    cols = nq + nk + (-(nq + nk) % 16)
    proj = (torch.randn(n, cols, generator=g)).to(dtype)
    bias = torch.zeros(cols)
    bias[: nq + nk] = torch.randn(nq + nk, generator=g)
    qn, kn = (torch.randn(nq, generator=g) * 0.3 + 1).to(dtype), (torch.randn(nk, generator=g) * 0.3 + 1).to(dtype)
    dev_ctx, cpu_ctx, n_pages = context([(3, n)], page)
    pos, slots = cpu_ctx.arrays["positions"], cpu_ctx.arrays["slots_g0"]
    scales = R.qk_row_scales(proj, nq, nk, pos, bias=bias, eps=1e-5, temperature=(0.7, 4))
    kc, vc = torch.zeros(n_pages, kv, page, dim, dtype=dtype), torch.zeros(n_pages, kv, dim, page, dtype=dtype)
    want_q = R.qkv_prepare(proj, heads, kv, dim, dim, pos, dtype, q_norm=qn, k_norm=kn, qk_eps=1e-5, k_cache=kc, v_cache=vc, slots=slots,
                           page_size=page, bias=bias, row_scales=scales, norm_over_projection=True, values_from_keys=True)
    kd, vd = torch.zeros_like(kc).cuda(), torch.zeros_like(vc).cuda()
    got_q = o.qkv_prepare(proj.cuda(), heads, kv, dim, dim, dev_ctx.arrays["positions"], dtype, q_norm=qn.cuda(), k_norm=kn.cuda(), qk_eps=1e-5,
                          k_cache=kd, v_cache=vd, slots=dev_ctx.arrays["slots_g0"], page_size=page, bias=bias.cuda(),
                          row_scales=scales.cuda(), norm_over_projection=True, values_from_keys=True)
    close(got_q, want_q, dtype, "queries", f32=2e-6, bf16=1e-2)
    kd, vd = kd.cpu(), vd.cpu()
    if o.masked_pages_tiled(dtype, dim, dim, page):
        kd, vd = untile_cache(kd, vd)
    close(kd, kc, dtype, "keys in the pages", f32=2e-6, bf16=1e-2)
    close(vd, vc, dtype, "values in the pages", f32=2e-6, bf16=1e-2)
    # the values are the biased keys as projected: the token's slot holds them before any norm
    t = n - 1
    pg, off = int(slots[t]) // page, int(slots[t]) % page
    raw = (proj[t, nq: nq + nk].float() + bias[nq: nq + nk]).view(kv, dim)
    close(vd[pg, :, :, off], raw.to(dtype), dtype, "a token's values", f32=1e-6, bf16=1e-2)


def sink_attention(q, k, v, positions, heads_per_kv, scale, softcap, sink):
    """q [N, H, d] at ``positions``; k [L, G, d], v [L, G, dv] of one sequence; sink [H]: float64, a dense mask."""
    L = k.shape[0]
    mask = torch.arange(L)[None, :] <= positions[:, None]
    out = torch.empty(q.shape[0], q.shape[1], v.shape[2], dtype=torch.float64)
    for h in range(q.shape[1]):
        g = h // heads_per_kv
        s = (q[:, h].double() @ k[:, g].double().T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = torch.cat([s.masked_fill(~mask, -float("inf")), sink[h].double().expand(q.shape[0], 1)], dim=1)
        out[:, h] = torch.softmax(s, dim=-1)[:, :-1] @ v[:, g].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim,value_dim,heads,kv", [(64, 64, 4, 2), (128, 128, 6, 1), (32, 48, 4, 4), (80, 80, 5, 5), (64, 64, 2, 2)])
@pytest.mark.parametrize("special,softcap", [(0, 0.0), (63, 0.0), (64, 15.0), (127, 15.0), (128, 0.0), (400, 15.0), (599, 0.0), (650, 15.0)])
def test_sinks_at_every_edge(dtype, head_dim, value_dim, heads, kv, special, softcap):
    """One key's score towers over the rest, against sinks of which some take most of the weight and some nothing: a
    prompt's portion at positions 550..699 and single tokens at 599, 600, 64, 63 and 0 (one key against its sink)
    look for it; 63 / 64 and 127 / 128 lie across borders of pages and key blocks.  The general kernel at every size,
    the matrix-core kernels (bfloat16, keys and values of 64 or 128 alike) whole and with their keys split (the
    sink joins once, in the merge)."""
    o = ops()
    H, G, d, dv, page, L = heads, kv, head_dim, value_dim, 64, 700
    scale = 0.2
    gen = torch.Generator().manual_seed(special + heads)
    k = torch.randn(L, G, d, generator=gen) * 0.1
    v = torch.randn(L, G, dv, generator=gen)
    k[special, :, 0] = 40.0
    k, v = k.to(dtype).float(), v.to(dtype).float()
    sink = torch.tensor([7.5, -30.0, 3.0, 9.0, 0.0, 8.0])[:H].contiguous()
    spans_at = [(550, 150), (599, 1), (600, 1), (64, 1), (63, 1), (0, 1)]
    n_pages = sum(-(-(p0 + n) // page) for p0, n in spans_at)
    perm = torch.randperm(n_pages, generator=gen).tolist()
    kc = torch.zeros(n_pages, G, page, d)
    vc = torch.zeros(n_pages, G, dv, page)
    spans, used = [], 0
    for p0, n in spans_at:
        need = -(-(p0 + n) // page)
        table = np.array(perm[used: used + need], dtype=np.int32)
        used += need
        for j in range(p0 + n):
            kc[table[j // page], :, j % page] = k[j]
            vc[table[j // page], :, :, j % page] = v[j]
        spans.append(SeqSpan(tokens=[0] * n, first_position=p0, block_tables=[table], state_slot=len(spans), want=[]))
    hb = build_host_batch(spans, 1, page)
    positions = torch.from_numpy(hb.positions).long()
    q = torch.randn(hb.n_tokens, H, d, generator=gen) * 0.1
    q[:, :, 0] = 1.0
    q = q.to(dtype).float()
    want = sink_attention(q, k, v, positions, H // G, scale, softcap, sink)
    without = sink_attention(q, k, v, positions, H // G, scale, softcap, torch.full((H,), -1e4))
    assert (want - without).abs().max() > 0.05, "the sinks were meant to matter"
    dev = "cuda:0"
    arrays = {"positions": torch.from_numpy(hb.positions).to(dev), "token_seq": torch.from_numpy(hb.token_seq).to(dev),
              "block_table_g0": torch.from_numpy(hb.block_tables[0]).to(dev)}
    ctx = SimpleNamespace(arrays=arrays, max_ctx=hb.max_ctx, host=hb)
    kc_d, vc_d = kc.to(dtype), vc.to(dtype)
    if o.masked_pages_tiled(dtype, d, dv, page):
        kc_d, vc_d = tile_cache(kc_d, vc_d)
    kc_d, vc_d = kc_d.to(dev).contiguous(), vc_d.to(dev).contiguous()
    qd = q.to(dtype).reshape(hb.n_tokens, H * d).to(dev)
    sink_d = sink.to(dev)
    tol = 2e-4 if dtype == torch.float32 else 4e-2
    got = o.attention_masked(qd, H, G, d, dv, kc_d, vc_d, page, scale, ctx, 0, softcap=softcap, sink=sink_d)
    err = (got.float().cpu().view(-1, H, dv).double() - want).abs().max(dim=2).values.max(dim=1).values
    assert err.max() < tol, f"general kernel: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"
    if dtype == torch.bfloat16 and d == dv and d in (64, 128):
        assert o.attention_takes_sink(dtype, d)
        tpt, big = o.attention_tokens_per_tile(H, G), o.attention_long_span_tile(H, G)
        tiles = torch.from_numpy(attention_tiles(hb, tpt, 1, big)).to(dev)
        long_tiles = torch.from_numpy(attention_tiles(hb, big, big + 1, longest_first=True)).to(dev)
        for plan, long_plan in ((None, None), ((4, 3), 2), ((1, 1), 1), ((1, 5), 3)):
            got = o.attention(qd, H, G, d, kc_d, vc_d, page, scale, 0, ctx, 0, tiles, long_tiles, plan=plan, long_plan=long_plan,
                              softcap=softcap, sink=sink_d)
            err = (got.float().cpu().view(-1, H, d).double() - want).abs().max(dim=2).values.max(dim=1).values
            assert err.max() < tol, f"matrix cores, plan {plan}/{long_plan}: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"


@pytest.mark.parametrize("n,experts,top,padded", [(1, 2, 1, 16), (37, 5, 2, 16), (200, 8, 8, 8), (64, 40, 3, 48), (9, 130, 6, 144)])
def test_router_with_bias_and_weights_of_the_chosen(n, experts, top, padded):
    """The ``top`` largest of logits + bias (padding columns are no experts; among equals the lower number), and the
    softmax over the chosen alone; a bias that changes who is chosen."""
    o = ops()
    g = torch.Generator().manual_seed(n + experts)
    logits = torch.randn(n, padded, generator=g) * 2
    logits[:, experts:] = 50.0
    bias = torch.randn(experts, generator=g) * 3
    if experts >= 3 and n > 2:
        logits[2, 1], logits[2, 2] = 40.0 - float(bias[1]), 40.0 - float(bias[2])
    choice, weights = o.moe_router_topk(logits.cuda(), None, top, experts=experts, bias=bias.cuda(), scores="softmax_of_chosen")
    z = logits[:, :experts] + bias
    want_choice = torch.sort(z, dim=1, descending=True, stable=True).indices[:, :top]
    tie = experts >= 3 and n > 2 and abs(float(z[2, 1]) - float(z[2, 2])) > 0  # (float32 sums of the made tie may differ by a bit)
    rows = [t for t in range(n) if not (tie and t == 2)]
    assert torch.equal(torch.sort(choice.cpu().long(), dim=1).values[rows], torch.sort(want_choice, dim=1).values[rows])
    assert not torch.equal(want_choice, torch.sort(logits[:, :experts], dim=1, descending=True, stable=True).indices[:, :top]) or n == 1
    want_w = torch.softmax(torch.gather(z.double(), 1, choice.cpu().long()), dim=1)
    close(weights, want_w, torch.float32, "weights", f32=2e-6)
    assert (weights.sum(1).cpu() - 1).abs().max() < 1e-5
    c2, w2 = R.moe_router_topk(logits, None, top, experts=experts, bias=bias, scores="softmax_of_chosen")
    assert torch.equal(c2[rows], choice.cpu()[rows])


@pytest.mark.parametrize("n,top,width", [(1, 1, 40), (37, 3, 320), (200, 8, 2048)])
def test_rows_summed_with_their_weights(n, top, width):
    o = ops()
    g = torch.Generator().manual_seed(n)
    rows = torch.randn(n * top, width, generator=g)
    w = torch.rand(n, top, generator=g)
    dense = torch.randn(n, width, generator=g).to(torch.bfloat16)
    got = o.moe_combine(dense.cuda(), rows.cuda(), top, 1.0, row_weights=w.cuda())
    close(got, dense.double() + (rows.view(n, top, width).double() * w.double()[:, :, None]).sum(1), torch.float32, "with the mixer's output", f32=1e-6)
    got = o.moe_combine(None, rows.cuda(), top, 1.0, row_weights=w.cuda())
    close(got, (rows.view(n, top, width).double() * w.double()[:, :, None]).sum(1), torch.float32, "rows alone", f32=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,hidden,ff,experts,top", [(1, 64, 32, 4, 1), (40, 96, 24, 5, 2), (300, 128, 64, 12, 1), (700, 256, 128, 16, 4),
                                                     (130, 64, 48, 3, 3), (2048, 256, 96, 8, 2)])
def test_experts_without_gates(dtype, n, hidden, ff, experts, top):
    """down(relu(up x)^2) through the grouped products with a row of x per token, every way the library runs them (a
    token alone, few tokens, tiles of tokens sorted by expert, the tiles of many rows), against each expert's plain
    feed-forward."""
    o = ops()
    g = torch.Generator().manual_seed(n + ff)
    x = torch.randn(n, hidden, generator=g).to(dtype)
    logits = torch.randn(n, experts + (-experts % 16), generator=g) * 1.5
    w_u = (torch.randn(experts, 1, ff, hidden, generator=g) / hidden ** 0.5).to(dtype)
    w_d = (torch.randn(experts, hidden, ff, generator=g) / ff ** 0.5).to(dtype)
    choice, _ = o.moe_router_topk(logits.cuda(), None, top, experts=experts, scores="softmax_of_chosen")
    got = o.moe_experts(x.cuda(), None, choice, w_u.cuda(), w_d.cuda(), "relu2", input_per_token=True)
    assert tuple(got.shape) == (n * top, hidden) and got.dtype == torch.float32
    c = choice.cpu().long().reshape(-1)
    xs = x.double().repeat_interleave(top, 0)
    want = torch.empty(n * top, hidden, dtype=torch.float64)
    for e in range(experts):
        mine = torch.nonzero(c == e)[:, 0]
        if len(mine):
            a = torch.relu(xs[mine] @ w_u[e, 0].double().T)
            want[mine] = (a * a) @ w_d[e].double().T
    close(got, want, dtype, "experts", f32=5e-5, bf16=2e-2)
