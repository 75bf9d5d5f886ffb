"""What Mesolix added to the kernels, each against plain arithmetic (float64 where the inputs are made by hand,
tests/kernel_refs.py otherwise), at sizes of their own, odd ones included, and with inputs made so that a fault
shows: one key or page row whose score stands out, placed at every edge; sinks and biases large enough to decide."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import kernel_refs as R
from kernel_refs import tile_cache
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
@pytest.mark.parametrize("width,n_pos", [(40, 50), (320, 700), (4096, 33)])
def test_embedding_with_learned_positions(dtype, width, n_pos):
    o = ops()
    g = torch.Generator().manual_seed(width)
    table = torch.randn(90, width, generator=g).to(dtype)
    pos_table = torch.randn(n_pos, width, generator=g).to(dtype)
    ids = torch.randint(0, 90, (61,), generator=g, dtype=torch.int32)
    pos = torch.randint(0, n_pos, (61,), generator=g, dtype=torch.int32)
    pos[0], pos[1] = 0, n_pos - 1
    got = o.embed(ids.cuda(), table.cuda(), positions=pos.cuda(), position_table=pos_table.cuda())
    want = table.float()[ids.long()] + pos_table.float()[pos.long()]
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), want)


def biased_attention(q, k, v, positions, heads_per_kv, scale, window, bias):
    """q [N, H, d] at ``positions``; k [L, G, d], v [L, G, dv] of one sequence; bias [distances, H] (the last row for
    everything farther): float64, a dense mask."""
    L = k.shape[0]
    j = torch.arange(L)[None, :]
    p = positions[:, None]
    mask = (j <= p) & ((p - j < window) if window else torch.ones_like(j <= p))
    dist = (p - j).clamp(0, bias.shape[0] - 1)
    out = torch.empty(q.shape[0], q.shape[1], v.shape[2], dtype=torch.float64)
    for h in range(q.shape[1]):
        g = h // heads_per_kv
        s = (q[:, h].double() @ k[:, g].double().T) * scale + bias[:, h].double()[dist]
        out[:, h] = torch.softmax(s.masked_fill(~mask, -float("inf")), dim=-1) @ v[:, g].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim,value_dim,heads,kv", [(64, 64, 4, 2), (128, 128, 6, 1), (32, 48, 4, 4), (64, 32, 4, 2), (64, 64, 2, 2)])
@pytest.mark.parametrize("special,window,rows", [(400, 200, 200), (401, 200, 200), (399, 200, 37), (0, 0, 64), (63, 0, 700), (64, 0, 5), (127, 0, 128),
                                                  (128, 700, 1), (536, 64, 64), (537, 64, 30), (599, 1, 4)])
def test_biased_attention_at_every_edge(dtype, head_dim, value_dim, heads, kv, special, window, rows):
    """One key's score towers over the rest, under a table of biases with entries of several units (a table
    shorter than the window, as long, longer, of one row): a prompt's portion at positions 550..699 and single
    tokens at 599, 600, 269 and 270 look for it.  With a window of 200, key 400 leaves it between 599 and 600 and
    key 401 a token later; 63 / 64 and 127 / 128 lie across borders of pages and key blocks; a window of 64 ends at
    keys 536 and 537 for the tokens at 599 and 600; a window of one key sees itself alone.  The general kernel at
    every size, the matrix-core kernels (bfloat16, keys and values of 64 or 128 alike) whole and with their keys
    split."""
    o = ops()
    H, G, d, dv, page, L = heads, kv, head_dim, value_dim, 64, 700
    scale = 0.2
    gen = torch.Generator().manual_seed(special + rows)
    k = torch.randn(L, G, d, generator=gen) * 0.1
    v = torch.randn(L, G, dv, generator=gen)
    k[special, :, 0] = 150.0
    k, v = k.to(dtype).float(), v.to(dtype).float()
    bias = torch.randn(rows, H, generator=gen) * 2.5
    spans_at = [(550, 150), (599, 1), (600, 1), (269, 1), (270, 1)]
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
    want = biased_attention(q, k, v, positions, H // G, scale, window, bias)
    dev = "cuda:0"
    arrays = {"positions": torch.from_numpy(hb.positions).to(dev), "token_seq": torch.from_numpy(hb.token_seq).to(dev),
              "block_table_g0": torch.from_numpy(hb.block_tables[0]).to(dev)}
    ctx = SimpleNamespace(arrays=arrays, max_ctx=hb.max_ctx, host=hb)
    kc_d, vc_d = kc.to(dtype), vc.to(dtype)
    if o.masked_pages_tiled(dtype, d, dv, page):
        kc_d, vc_d = tile_cache(kc_d, vc_d)
    kc_d, vc_d = kc_d.to(dev).contiguous(), vc_d.to(dev).contiguous()
    qd = q.to(dtype).reshape(hb.n_tokens, H * d).to(dev)
    bias_d = bias.to(dev)
    tol = 2e-4 if dtype == torch.float32 else 4e-2
    got = o.attention_masked(qd, H, G, d, dv, kc_d, vc_d, page, scale, ctx, 0, window=window, distance_bias=bias_d)
    err = (got.float().cpu().view(-1, H, dv).double() - want).abs().max(dim=2).values.max(dim=1).values
    assert err.max() < tol, f"general kernel: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"
    if dtype == torch.bfloat16 and d == dv and d in (64, 128):
        tpt, big = o.attention_tokens_per_tile(H, G), o.attention_long_span_tile(H, G)
        tiles = torch.from_numpy(attention_tiles(hb, tpt, 1, big)).to(dev)
        long_tiles = torch.from_numpy(attention_tiles(hb, big, big + 1, longest_first=True)).to(dev)
        for plan, long_plan in ((None, None), ((4, 3), 2), ((1, 1), 1)):
            got = o.attention(qd, H, G, d, kc_d, vc_d, page, scale, window, ctx, 0, tiles, long_tiles, plan=plan, long_plan=long_plan,
                              distance_bias=bias_d)
            err = (got.float().cpu().view(-1, H, d).double() - want).abs().max(dim=2).values.max(dim=1).values
            assert err.max() < tol, f"matrix cores, plan {plan}/{long_plan}: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"
    visible = [t for t in range(hb.n_tokens) if special <= int(positions[t]) and (not window or int(positions[t]) - special < window)]
    if visible and dv == d:  # where the key is visible it carries nearly all the weight: its own value comes back
        back = got.float().cpu().view(-1, H, d)[visible]
        assert (back - v[special].repeat_interleave(H // G, 0)).abs().max() < 0.1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_rank,page", [(2, 64, 32), (5, 20, 16), (16, 512, 64), (3, 128, 32), (1, 130, 16), (20, 256, 32)])
@pytest.mark.parametrize("special", [0, 31, 32, 63, 64, 399, 400])
def test_latent_rows_alone_with_sinks(dtype, heads, kv_rank, page, special):
    """Page rows that are the latent alone (no rotated part) and a sink per head, some so large that they take most
    of the weight, some negligible: the towering row of the other tests at borders of pages and key blocks; a
    prompt's portion at 380..449 and single tokens at 399, 400, 699, 16 and 0 (one key against its sink).  The
    general kernel, and for bfloat16 latents of 64, 128, 256 and 512 the matrix-core form whole, split in three
    and split as the library decides."""
    if kv_rank >= 256 and special not in (0, 63, 64, 400):
        pytest.skip("the largest sizes run a few of the borders")
    o = ops()
    L = 700
    g = torch.Generator().manual_seed(special + heads)
    rows = torch.randn(L, kv_rank, generator=g) * 0.2
    rows[special, 0] = 12.0
    rows = rows.to(dtype).float()
    sink = torch.randn(heads, generator=g) * 3.0 + 4.0
    sink[0] = 9.0
    spans_at = [(380, 70), (399, 1), (400, 1), (699, 1), (16, 1), (0, 1)]
    n_tok = sum(n for _, n in spans_at)
    q = torch.randn(n_tok, heads, kv_rank, generator=g) * 0.3
    q[:, :, 0] = 1.0
    q = q.to(torch.bfloat16).float()
    scale = 0.7
    want = None
    on_cores = dtype == torch.bfloat16 and o.latent_attention_on_matrix_cores(dtype, kv_rank, 0, page)
    assert on_cores == (dtype == torch.bfloat16 and kv_rank in (64, 128, 256, 512))
    for cores in ([False, True] if on_cores else [False]):
        tile = o.latent_tile_tokens(heads, cores)
        dev, cpu, n_pages = context(spans_at, page, tile_tokens=tile)
        pages = torch.full((n_pages, 1, page, kv_rank), 7.0)
        bt = cpu.arrays["block_table_g0"]
        for s, (p0, n) in enumerate(spans_at):
            for j in range(p0 + n):
                pages[int(bt[s, j // page]), 0, j % page] = rows[j]
        if want is None:
            pos = cpu.arrays["positions"]
            want = torch.empty(n_tok, heads, kv_rank, dtype=torch.float64)
            for t in range(n_tok):
                keys = rows[: int(pos[t]) + 1].double()
                s = q[t].double() @ keys.T * scale
                top = torch.maximum(s.max(dim=-1).values, sink.double())
                e = torch.exp(s - top[:, None])
                want[t] = (e / (e.sum(-1) + torch.exp(sink.double() - top))[:, None]) @ keys
        values = pages.transpose(2, 3).contiguous().to(dtype).cuda() if cores else None
        for splits in ([1, 3, None] if cores else [None]):
            got = o.latent_attention(q.reshape(n_tok, -1).cuda(), pages.to(dtype).cuda(), heads, kv_rank, 0, scale, dev, 0, page,
                                     tiles=dev.arrays[f"latent_tiles_{tile}"], values=values, splits=splits, sink=sink.cuda())
            close(got, want.reshape(n_tok, -1), torch.bfloat16 if cores else torch.float32, f"row {special}, matrix cores {cores}, splits {splits}",
                  f32=3e-5, bf16=1e-2)
    # the sinks took their share: head 0's sink outweighs every key but the towering one
    alone = n_tok - 1  # the token at position 0
    if special != 0:
        assert want[alone, 0].abs().max() < 0.05 * rows[0].abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,groups,state,vdim", [(4, 2, 12, 10), (3, 3, 24, 9), (2, 1, 64, 32), (6, 2, 48, 32), (4, 1, 128, 64), (1, 1, 200, 5), (2, 2, 16, 300)])
def test_state_scan_as_state_space_duality(dtype, heads, groups, state, vdim):
    """The write by the step (u = dt x with dt the softplus behind the head's decay), the skip per head, and columns
    laid out as [x | B | C] with B and C shared by groups of heads: spans of one token and of several staged chunks
    behind states that are not zero; a span cut in two gives the same state and outputs bit for bit."""
    o = ops()
    spans_at = [(0, 37), (5, 1), (9, 18)]
    dev, cpu, _ = context(spans_at, 16, slots=[1, 3, 0])
    n = sum(k for _, k in spans_at)
    g = torch.Generator().manual_seed(state + vdim)
    inner, bc = heads * vdim, groups * state
    u = torch.randn(n, inner + 2 * bc, generator=g).to(dtype)
    memory = torch.randn(4, heads, state, vdim, generator=g) * 0.5
    dt = torch.randn(n, heads + 3, generator=g)
    a_log, dt_bias, skip = torch.randn(heads, generator=g) * 0.5, torch.randn(heads, generator=g) * 0.5, torch.randn(heads, generator=g)
    args = lambda f: dict(q_scale=1.0, unit_eps=None, decay=("head", f(dt), 2, f(a_log), f(dt_bias)), beta="step",
                          columns=(inner + bc, inner, 0), skip=f(skip))
    s_ref = memory.clone()
    want = R.linear_state_scan(u, heads, groups, state, vdim, s_ref, cpu, **args(lambda t: t))
    # and against the recurrence written out, for the first request
    x = u[:37, :inner].double().view(37, heads, vdim)
    B = u[:37, inner: inner + bc].double().view(37, groups, state)
    C = u[:37, inner + bc:].double().view(37, groups, state)
    step = torch.nn.functional.softplus(dt[:37, 2: 2 + heads].double() + dt_bias.double())
    S = memory[1].double().clone()
    for t in range(37):
        for h in range(heads):
            gi = h // (heads // groups)
            S[h] = torch.exp(-torch.exp(a_log[h].double()) * step[t, h]) * S[h] + step[t, h] * torch.outer(B[t, gi], x[t, h])
            y = S[h].T @ C[t, gi] + skip[h].double() * x[t, h]
            assert (y - want[t].double().view(heads, vdim)[h]).abs().max() < 1e-3 * max(1.0, y.abs().max().item())
    s_dev = memory.clone().cuda()
    got = o.linear_state_scan(u.cuda(), heads, groups, state, vdim, s_dev, dev, **args(lambda t: t.cuda()))
    close(got, want, torch.float32, "read-outs", f32=5e-5)
    close(s_dev, s_ref, torch.float32, "states", f32=5e-5)
    s_two = memory.clone().cuda()
    outs = []
    for p0, cnt, lo in ((0, 20, 0), (20, 17, 20)):
        d2, _, _ = context([(p0, cnt)], 16, slots=[1])
        part = lambda t, lo=lo, cnt=cnt: t[lo: lo + cnt].contiguous().cuda() if t.dim() == 2 and t.shape[0] == n else t.cuda()
        outs.append(o.linear_state_scan(part(u), heads, groups, state, vdim, s_two, d2, **args(part)))
    assert torch.equal(torch.cat(outs), got[:37]) and torch.equal(s_two[1], s_dev[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("parts,size", [(1, 40), (2, 96), (4, 10), (3, 200), (1, 2048)])
def test_gate_before_the_norm(dtype, parts, size):
    """rms(o silu(gate)) * weight in equal parts, the weight as wide as the row: not the norm gated afterwards."""
    o = ops()
    g = torch.Generator().manual_seed(size)
    n = 21
    x = torch.randn(n, parts * size, generator=g) * 4
    w = (torch.randn(parts * size, generator=g) * 0.3 + 1).to(dtype)
    gate = torch.randn(n, parts * size + 9, generator=g).to(dtype)
    got = o.gated_head_norm(x.cuda(), w.cuda(), 1e-5, gate.cuda(), 9, parts, size, dtype, gate_first=True)
    z = gate[:, 9:].double()
    y = (x.double() * z * torch.sigmoid(z)).view(n, parts, size)
    want = (y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-5)).reshape(n, -1) * w.double()
    close(got, want, dtype, "gate first", bf16=1e-2)
    after = R.gated_head_norm(x, w, 1e-5, gate, 9, parts, size, dtype)
    assert (after.double() - want).abs().max() > 0.1, "the two orders were meant to differ"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,in_dim,out_dim,n", [(3, 10, 20, 7), (8, 128, 32, 150), (2, 64, 16, 33), (5, 512, 128, 77)])
def test_a_gate_per_element_behind_the_heads_products(dtype, heads, in_dim, out_dim, n):
    o = ops()
    g = torch.Generator().manual_seed(n)
    w = (torch.randn(heads, in_dim, out_dim, generator=g) / in_dim ** 0.5).to(dtype)
    x = torch.randn(n, heads * in_dim, generator=g)
    gate = (torch.randn(n, heads * out_dim + 16, generator=g) * 2).to(dtype)
    w_t = o.head_weights_transposed(w.cuda()) if dtype == torch.bfloat16 else None
    got = o.head_linear(x.cuda(), w.cuda(), heads, in_dim, out_dim, dtype, gate=gate.cuda(), gate_col=16, w_t=w_t, gate_elems=out_dim)
    want = torch.einsum("nhi,hio->nho", x.double().view(n, heads, in_dim), w.double()).reshape(n, -1) * torch.sigmoid(gate[:, 16:].double())
    close(got, want, dtype, "gated per element", f32=3e-5, bf16=1.5e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,experts,top,padded", [(1, 5, 1, 16), (50, 12, 1, 16), (33, 7, 3, 16), (200, 64, 8, 64), (9, 2, 2, 2), (17, 70, 64, 80)])
def test_router_choice_and_scaled_rows(dtype, n, experts, top, padded):
    """The ``top`` largest of each row's first ``experts`` logits (padding columns, however large, are no experts;
    among equals the lower number), and the token's row once per chosen expert times sigmoid(logit)."""
    o = ops()
    g = torch.Generator().manual_seed(n + experts)
    logits = torch.randn(n, padded, generator=g) * 2
    logits[:, experts:] = 50.0
    if experts >= 3 and n > 2:
        logits[2, 1] = logits[2, 2] = 40.0  # equals: the lower number first
    x = torch.randn(n, 40, generator=g).to(dtype)
    choice, rows = o.moe_router_topk(logits.cuda(), x.cuda(), top, experts=experts)
    want_choice = torch.sort(logits[:, :experts], dim=1, descending=True, stable=True).indices[:, :top]
    assert torch.equal(torch.sort(choice.cpu().long(), dim=1).values, torch.sort(want_choice, dim=1).values)
    if experts >= 3 and n > 2 and top >= 1:
        assert 1 in choice[2].tolist() and (top == 1) == (2 not in choice[2].tolist())
    score = torch.sigmoid(torch.gather(logits, 1, choice.cpu().long()))
    want_rows = (x.float()[:, None, :] * score[:, :, None]).reshape(n * top, -1)
    close(rows, want_rows, dtype, "scaled rows", f32=1e-6, bf16=4e-3)


@pytest.mark.parametrize("n,top,width", [(1, 1, 40), (37, 3, 320), (200, 8, 2048)])
def test_rows_summed_per_token(n, top, width):
    o = ops()
    g = torch.Generator().manual_seed(n)
    rows = torch.randn(n * top, width, generator=g)
    dense = torch.randn(n, width, generator=g).to(torch.bfloat16)
    got = o.moe_combine(dense.cuda(), rows.cuda(), top, 1.0)
    close(got, dense.float() + rows.view(n, top, width).sum(1), torch.float32, "with a dense part", f32=1e-6)
    got = o.moe_combine(None, rows.cuda(), top, 0.5)
    close(got, 0.5 * rows.view(n, top, width).sum(1), torch.float32, "rows alone", f32=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,hidden,ff,experts,top", [(1, 64, 32, 4, 1), (40, 96, 24, 5, 2), (300, 128, 64, 12, 1), (700, 256, 128, 16, 4), (130, 64, 48, 3, 3)])
def test_experts_on_a_routers_choice(dtype, n, hidden, ff, experts, top):
    """The grouped products with a choice per token as their table and an input row per (token, choice): every way
    the library runs them (a token alone, few tokens, tiles of tokens sorted by expert), against each expert's
    plain feed-forward on its rows."""
    o = ops()
    g = torch.Generator().manual_seed(n + ff)
    x = torch.randn(n, hidden, generator=g).to(dtype)
    logits = torch.randn(n, experts + (-experts % 16), generator=g) * 1.5
    w_gu = (torch.randn(experts, 2, ff, hidden, generator=g) / hidden ** 0.5).to(dtype)
    w_d = (torch.randn(experts, hidden, ff, generator=g) / ff ** 0.5).to(dtype)
    choice, scaled = o.moe_router_topk(logits.cuda(), x.cuda(), top, experts=experts)
    got = o.moe_experts(scaled, None, choice, w_gu.cuda(), w_d.cuda(), "silu")
    assert tuple(got.shape) == (n * top, hidden) and got.dtype == torch.float32
    s, c = scaled.float().cpu().double(), choice.cpu().long().reshape(-1)
    want = torch.empty(n * top, hidden, dtype=torch.float64)
    for e in range(experts):
        mine = torch.nonzero(c == e)[:, 0]
        if len(mine):
            gg, uu = s[mine] @ w_gu[e, 0].double().T, s[mine] @ w_gu[e, 1].double().T
            want[mine] = (gg * torch.sigmoid(gg) * uu) @ w_d[e].double().T
    close(got, want, dtype, "experts", f32=5e-5, bf16=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("limit", [0.5, 7.0])
def test_the_clamped_gated_pair(dtype, limit):
    """min(g, limit) sigmoid(1.702 min(g, limit)) (clamp(u, -limit, limit) + 1) behind the stacked product."""
    o = ops()
    g = torch.Generator().manual_seed(int(limit * 10))
    n, hidden, ff = 45, 96, 80
    x = (torch.randn(n, hidden, generator=g) * 2).to(dtype)
    wg, wu = ((torch.randn(ff, hidden, generator=g) / hidden ** 0.5).to(dtype) for _ in range(2))
    packed, group = o.pack_gate_up(wg.cuda(), wu.cuda())
    got = o.gate_up_act(x.cuda(), packed, group, ("clamped_swish", limit, 1.702), dtype)
    gg = torch.clamp(x.double() @ wg.double().T, max=limit)
    uu = torch.clamp(x.double() @ wu.double().T, -limit, limit)
    want = gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)
    assert (x.double() @ wg.double().T).max() > limit and (x.double() @ wu.double().T).min() < -limit, "the clamps were meant to bite"
    close(got, want, dtype, "clamped pair", f32=3e-5, bf16=2e-2)
