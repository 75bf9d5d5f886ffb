"""Plain PyTorch counterparts of the HIP kernels, one function per kernel, with the
same call signatures as ``yalis_amd.ops.hip.HipOps``.

Two uses: the GPU tests compare each kernel with its counterpart here at sizes of
their own; and ``RefOps`` lets the CPU tests run the framework's host logic (batching,
paging, scheduling) without a GPU.  It is test equipment: the framework never imports
it.  Everything is computed in float32 and rounded once to the output dtype.
"""
from __future__ import annotations

import math

import torch


def embed(token_ids, table, positions=None, position_table=None, scale=1.0):
    x = table[token_ids.long()].to(torch.float32)
    if scale != 1.0:
        x = x * torch.tensor(scale, dtype=torch.float32)
    if position_table is not None:
        x = x + position_table[positions.long()].to(torch.float32)
    return x


def add_rmsnorm(residual, delta, weight, eps, unit_offset, out_dtype, row=None):
    """residual += delta (+ row, one vector for every token) in place (float32); returns the normalised rows."""
    if delta is not None:
        residual += delta.to(torch.float32)
    if row is not None:
        residual += row.to(torch.float32)
    return _rmsnorm(residual, weight, eps, unit_offset).to(out_dtype)


def gather_add_rmsnorm(residual, delta, rows, weight, eps, unit_offset, out_dtype):
    v = residual[rows.long()]
    if delta is not None:
        v = v + delta[rows.long()].to(torch.float32)
    return _rmsnorm(v, weight, eps, unit_offset).to(out_dtype)


def _rmsnorm(x, weight, eps, unit_offset):
    ms = (x * x).mean(dim=-1, keepdim=True)
    w = weight.to(torch.float32)
    if unit_offset:
        w = w + 1.0
    return x * torch.rsqrt(ms + eps) * w


def rmsnorm(x, weight, eps, unit_offset, out_dtype):
    """The norm of rows that are no residual stream."""
    return _rmsnorm(x.to(torch.float32), weight, eps, unit_offset).to(out_dtype)


def linear(x, w, out_dtype, partial_ok=False, bias=None):
    y = x.to(torch.float32) @ w.to(torch.float32).T
    if bias is not None:  # added to the float32 product, one rounding (torch's addmm, the reference's biased Linear)
        y = y + bias.to(torch.float32)
    return y.to(out_dtype)


def rope_append(qkv, n_heads, n_kv, head_dim, positions, cos, sin, rotary_dim, interleaved,
                k_cache, v_cache, slots, page_size):
    """Rotates the query heads of ``qkv`` in place; rotates the key heads and stores
    them, and the value heads transposed, at each token's slot of the pages.  Returns the
    tensor whose rows start with the rotated queries."""
    n = qkv.shape[0]
    x = qkv.view(n, n_heads + 2 * n_kv, head_dim)
    rot = x[:, : n_heads + n_kv].to(torch.float32)
    if rotary_dim:
        c = cos[positions.long()][:, None, :]
        s = sin[positions.long()][:, None, :]
        if interleaved:
            a = rot[..., 0:rotary_dim:2]
            b = rot[..., 1:rotary_dim:2]
        else:
            a = rot[..., : rotary_dim // 2]
            b = rot[..., rotary_dim // 2 : rotary_dim]
        ra = a * c - b * s
        rb = b * c + a * s
        rot = rot.clone()
        if interleaved:
            rot[..., 0:rotary_dim:2] = ra
            rot[..., 1:rotary_dim:2] = rb
        else:
            rot[..., : rotary_dim // 2] = ra
            rot[..., rotary_dim // 2 : rotary_dim] = rb
    rot = rot.to(qkv.dtype)
    x[:, :n_heads] = rot[:, :n_heads]
    if n_kv:
        page = (slots // page_size).long()
        off = (slots % page_size).long()
        k_cache[page, :, off, :] = rot[:, n_heads:]
        v_cache[page, :, :, off] = x[:, n_heads + n_kv :]
    return qkv


def attention_paged(q, k_cache, v_cache, positions, token_seq, block_table, page_size, scale, window):
    """q: [N, H, D]; pages as in the framework (keys [pages, G, page, D], values
    [pages, G, D, page]).  Gathers each token's visible keys through its request's
    block table and runs a float32 softmax."""
    n, n_heads, d = q.shape
    n_kv = k_cache.shape[1]
    qpk = n_heads // n_kv
    out = torch.empty((n, n_heads, d), dtype=torch.float32, device=q.device)
    for t in range(n):
        pos = int(positions[t])
        lo = max(0, pos - window + 1) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t])][(keys // page_size).long()].long()
        offs = (keys % page_size).long()
        k = k_cache[pages, :, offs, :].to(torch.float32)  # [keys, G, D]
        v = v_cache[pages, :, :, offs].to(torch.float32)  # [keys, G, D]
        for h in range(n_heads):
            g = h // qpk
            s = (k[:, g, :] @ q[t, h].to(torch.float32)) * scale
            p = torch.softmax(s, dim=0)
            out[t, h] = p @ v[:, g, :]
    return out


def attention(qkv, n_heads, n_kv, head_dim, k_cache, v_cache, page_size, scale,
              window, ctx, group, tiles, long_tiles=None, plan=None, long_plan=None, long_col_tiles=1, token_cols=None):
    n = qkv.shape[0]
    q = qkv.view(n, -1, head_dim)[:, :n_heads]
    out = attention_paged(
        q, k_cache, v_cache, ctx.arrays["positions"], ctx.arrays["token_seq"],
        ctx.arrays[f"block_table_g{group}"], page_size, scale, window,
    )
    return out.reshape(n, n_heads * head_dim).to(qkv.dtype)


def gated_act(gu, activation, out_dtype=None, group=0):
    inter = gu.shape[1] // 2
    if group:
        pairs = gu.reshape(gu.shape[0], inter // group, 2, group)
        g = pairs[:, :, 0, :].reshape(gu.shape[0], inter).to(torch.float32)
        u = pairs[:, :, 1, :].reshape(gu.shape[0], inter).to(torch.float32)
    else:
        g = gu[:, :inter].to(torch.float32)
        u = gu[:, inter:].to(torch.float32)
    if activation == "silu":
        a = g * torch.sigmoid(g)
    elif activation == "gelu_tanh":
        a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g**3)))
    else:
        raise ValueError(activation)
    return (a * u).to(out_dtype or gu.dtype)


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)


class RefOps:
    """The kernel library's interface over the functions above (CPU or GPU tensors)."""

    def check_attention_sizes(self, n_heads, n_kv, head_dim, page_size):
        assert n_heads % n_kv == 0 and head_dim % 16 == 0 and page_size % 16 == 0

    def attention_tokens_per_tile(self, n_heads, n_kv):
        return 16 // min(n_heads // n_kv, 16)

    def attention_long_span_tile(self, n_heads, n_kv, col_tiles=1):
        return 4 * col_tiles * self.attention_tokens_per_tile(n_heads, n_kv)

    @staticmethod
    def attention_long_col_tiles(workgroups, fewest_keys):
        return 1

    embed = staticmethod(embed)
    add_rmsnorm = staticmethod(add_rmsnorm)
    gather_add_rmsnorm = staticmethod(gather_add_rmsnorm)
    rmsnorm = staticmethod(rmsnorm)
    linear = staticmethod(linear)
    rope_append = staticmethod(rope_append)
    attention = staticmethod(attention)
    gated_act = staticmethod(gated_act)
    argmax = staticmethod(argmax)

    @staticmethod
    def pack_gate_up(w_gate, w_up):
        return torch.cat([w_gate, w_up], dim=0).contiguous(), 0

    @staticmethod
    def gate_up_act(x, w_gate_up, group, activation, out_dtype):
        return gated_act(linear(x, w_gate_up, out_dtype), activation, out_dtype, group)

    def sample(self, logits, temperature, top_k, top_p, seeds, draws, whole_row=False):
        from plain_llama import sample_token

        out = []
        for i in range(logits.shape[0]):
            k = int(top_k[i])
            out.append(
                sample_token(logits[i].cpu(), float(temperature[i]), k if k > 0 else None, float(top_p[i]), int(seeds[i]), int(draws[i]))
            )
        return torch.tensor(out, dtype=torch.int32, device=logits.device)


# ------------------------------------------------------------------ tiled cache pages
# The matrix-core attention keeps bfloat16 pages of a multiple of 64 tokens (head sizes 64 and
# 128) in the order its loads take them.  Written out here once more, from the layout's
# description (yalis_amd/csrc/common.h), so that tests can fill pages and read them back:
#   keys:   within a block of 64 slots, piece (((u*2 + sb) * D/32 + ks) * 4 + g) * 16 + r holds
#           dims 32ks + 8g .. +7 of slot 32u + 8(r/4) + 4sb + r%4;
#   values: piece ((u * D/16 + dt) * 4 + g) * 16 + r holds slots 32u + 8g .. +7 of dim 16dt + r.
def _tiled_indices(page, d):
    import numpy as np

    slot = np.arange(page)[:, None]
    dim = np.arange(d)[None, :]
    j = slot % 64
    u, a, sb, b = j // 32, (j % 32) // 8, (j % 8) // 4, j % 4
    piece_k = (((u * 2 + sb) * (d // 32) + dim // 32) * 4 + (dim % 32) // 8) * 16 + 4 * a + b
    k_at = (slot // 64) * 64 * d + piece_k * 8 + dim % 8            # [slot, dim] -> offset in the slab
    piece_v = ((u * (d // 16) + dim // 16) * 4 + (j % 32) // 8) * 16 + dim % 16
    v_at = (slot // 64) * 64 * d + piece_v * 8 + j % 8              # [slot, dim] -> offset in the slab
    assert sorted(k_at.ravel()) == list(range(page * d)) and sorted(v_at.ravel()) == list(range(page * d))
    return torch.from_numpy(k_at.ravel()), torch.from_numpy(v_at.T.copy().ravel())  # in the plain slabs' element order


def tile_cache(k_plain, v_plain):
    """Plain pages ([pages, kv, page, D] keys, [pages, kv, D, page] values) -> the same shapes
    holding the tiled order."""
    n, g, page, d = k_plain.shape
    k_at, v_at = _tiled_indices(page, d)
    k = torch.empty_like(k_plain).view(n, g, page * d)
    v = torch.empty_like(v_plain).view(n, g, page * d)
    k[:, :, k_at] = k_plain.reshape(n, g, page * d)
    v[:, :, v_at] = v_plain.reshape(n, g, page * d)
    return k.view(n, g, page, d), v.view(n, g, d, page)


def untile_cache(k_tiled, v_tiled):
    n, g, page, d = k_tiled.shape
    k_at, v_at = _tiled_indices(page, d)
    k = k_tiled.reshape(n, g, page * d)[:, :, k_at]
    v = v_tiled.reshape(n, g, page * d)[:, :, v_at]
    return k.reshape(n, g, page, d), v.reshape(n, g, d, page)


# ------------------------------------------------------------- parts beyond the plain decoder
# Counterparts of the kernels for branch norms, prepared / masked / finished attention heads,
# the short convolution with its gated linear recurrence, and the mixture of experts.
def round_rows(x, out_dtype):
    return x if out_dtype == torch.float32 else x.to(out_dtype)


def norm_add(residual, branch, weight, eps, unit_offset, out_dtype, expert_rows=None, expert_weight=1.0):
    n, width = residual.shape
    v = torch.zeros((n, width), dtype=torch.float32, device=residual.device)
    if branch is not None:
        v = v + branch.to(torch.float32)
    if expert_rows is not None:
        v = v + expert_weight * expert_rows.view(n, -1, width).sum(1)
    residual += _rmsnorm(v, weight, eps, unit_offset)
    return round_rows(residual, out_dtype)


def gated_kind(activation):
    name, consts = (activation, ()) if isinstance(activation, str) else (activation[0], tuple(activation[1:]))
    if name not in ("silu", "gelu_tanh", "clamped_swish"):
        raise ValueError(f"unknown activation {name!r}")
    return name, consts


def gated_pair(g, u, activation):
    name, consts = gated_kind(activation)
    if name == "silu":
        return g * torch.sigmoid(g) * u
    if name == "gelu_tanh":
        return 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g**3))) * u
    limit, slope = consts
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(slope * g) * (u + 1.0)


def gated_act_general(gu, activation, out_dtype=None, group=0):
    inter = gu.shape[1] // 2
    if group:
        pairs = gu.reshape(gu.shape[0], inter // group, 2, group)
        g = pairs[:, :, 0, :].reshape(gu.shape[0], inter).to(torch.float32)
        u = pairs[:, :, 1, :].reshape(gu.shape[0], inter).to(torch.float32)
    else:
        g, u = gu[:, :inter].to(torch.float32), gu[:, inter:].to(torch.float32)
    return gated_pair(g, u, activation).to(out_dtype or gu.dtype)


def _turn(x, cos, sin, rot, interleaved, sign=1.0):
    """x [..., d] float32; cos/sin [..., rot/2] broadcastable; the first rot elements turn."""
    x = x.clone()
    if interleaved:
        a, b = x[..., 0:rot:2].clone(), x[..., 1:rot:2].clone()
        x[..., 0:rot:2] = a * cos - b * sign * sin
        x[..., 1:rot:2] = b * cos + a * sign * sin
    else:
        a, b = x[..., : rot // 2].clone(), x[..., rot // 2: rot].clone()
        x[..., : rot // 2] = a * cos - b * sign * sin
        x[..., rot // 2: rot] = b * cos + a * sign * sin
    return x


def query_temperature(positions, coef, every):
    """float32 1 + coef ln(floor((p + 1) / every) + 1)."""
    steps = torch.div(positions.long() + 1, int(every), rounding_mode="floor").to(torch.float32)
    return 1.0 + torch.tensor(coef, dtype=torch.float32) * torch.log(steps + 1.0)


def qk_row_scales(proj, n_q_cols, n_k_cols, positions, bias=None, eps=None, temperature=None):
    """float32 [N, 2]: what a token's queries (column 0) and keys (column 1) are multiplied with as wholes: with
    ``eps`` the inverse root mean square over all the query columns (all the key columns) of the biased projection,
    with ``temperature`` = (coef, every) the queries' factor by position on top."""
    x = proj.to(torch.float32)
    if bias is not None:
        x = x + bias[: x.shape[1]]
    out = torch.ones((x.shape[0], 2), dtype=torch.float32, device=x.device)
    if eps is not None:
        q, k = x[:, :n_q_cols], x[:, n_q_cols: n_q_cols + n_k_cols]
        out[:, 0] = torch.rsqrt((q * q).mean(-1) + eps)
        if n_k_cols:
            out[:, 1] = torch.rsqrt((k * k).mean(-1) + eps)
    if temperature is not None:
        out[:, 0] = out[:, 0] * query_temperature(positions, *temperature)
    return out


def qkv_prepare(qkv, n_heads, n_kv, head_dim, value_dim, positions, act_dtype, q_norm=None, k_norm=None, qk_eps=0.0,
                rotation=None, value_norm_eps=None, value_rotation=None, k_cache=None, v_cache=None, slots=None, page_size=0,
                bias=None, row_scales=None, norm_over_projection=False, values_from_keys=False):
    n = qkv.shape[0]
    x = qkv.to(torch.float32)
    if bias is not None:
        x = x + bias[: x.shape[1]]
    hd = n_heads * head_dim
    q = x[:, :hd].reshape(n, n_heads, head_dim)
    k = x[:, hd: hd + n_kv * head_dim].reshape(n, n_kv, head_dim)
    if values_from_keys:
        v = k
    else:
        v = x[:, hd + n_kv * head_dim: hd + n_kv * (head_dim + value_dim)].reshape(n, n_kv, value_dim)
    pos = positions.long()
    if norm_over_projection:  # the inverse root mean square comes with the row scales; the weights span the projection
        q = q * q_norm.to(torch.float32).view(1, n_heads, head_dim)
        if n_kv:
            k = k * k_norm.to(torch.float32).view(1, n_kv, head_dim)
    elif q_norm is not None:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + qk_eps) * q_norm.to(torch.float32)
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + qk_eps) * k_norm.to(torch.float32)
    if row_scales is not None:
        q = q * row_scales[:, 0].view(n, 1, 1)
        k = k * row_scales[:, 1].view(n, 1, 1)
    if rotation is not None:
        c, s = rotation.cos[pos][:, None, :], rotation.sin[pos][:, None, :]
        q = _turn(q, c, s, rotation.rotary_dim, rotation.interleaved)
        k = _turn(k, c, s, rotation.rotary_dim, rotation.interleaved)
    if n_kv:
        if value_norm_eps is not None:
            v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + value_norm_eps)
        if value_rotation is not None:
            v = _turn(v, value_rotation.cos[pos][:, None, :], value_rotation.sin[pos][:, None, :], value_dim, value_rotation.interleaved)
        page, off = (slots // page_size).long(), (slots % page_size).long()
        k_cache[page, :, off, :] = k.to(k_cache.dtype)
        v_cache[page, :, :, off] = v.to(v_cache.dtype)
    return q.reshape(n, hd).to(act_dtype)


def attention_masked(q, n_heads, n_kv, head_dim, value_dim, k_cache, v_cache, page_size, scale, ctx, group, window=0,
                     keep_first=0, softcap=0.0, value_rotation=None, gate=None, gate_col=0, gate_elems=1, distance_bias=None, sink=None):
    n = q.shape[0]
    positions, token_seq = ctx.arrays["positions"], ctx.arrays["token_seq"]
    bt = ctx.arrays[f"block_table_g{group}"]
    qh = q.view(n, n_heads, head_dim).to(torch.float32)
    qpk = n_heads // n_kv
    out = torch.empty((n, n_heads, value_dim), dtype=torch.float32, device=q.device)
    for t in range(n):
        pos = int(positions[t])
        j = torch.arange(pos + 1, device=q.device)
        if window:
            j = j[(pos - j < window) | (j < keep_first)]
        pages = bt[int(token_seq[t])][(j // page_size).long()].long()
        offs = (j % page_size).long()
        k = k_cache[pages, :, offs, :].to(torch.float32)
        v = v_cache[pages, :, :, offs].to(torch.float32)
        for h in range(n_heads):
            g = h // qpk
            s = (k[:, g, :] @ qh[t, h]) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if distance_bias is not None:
                s = s + distance_bias[(pos - j).clamp(max=distance_bias.shape[0] - 1).long(), h]
            if sink is not None:  # one more term in the denominator, with no value
                w = torch.softmax(torch.cat([s, sink[h].to(torch.float32).view(1)]), dim=0)[:-1]
            else:
                w = torch.softmax(s, dim=0)
            out[t, h] = w @ v[:, g, :]
    out = attention_finish(out, positions, n_heads, value_dim, value_rotation, gate, gate_col, gate_elems)
    return out.reshape(n, n_heads * value_dim).to(q.dtype)


def attention_finish(out, positions, n_heads, value_dim, value_rotation=None, gate=None, gate_col=0, gate_elems=1):
    shape = out.shape
    o = out.reshape(out.shape[0], n_heads, value_dim).to(torch.float32)
    if value_rotation is not None:
        pos = positions.long()
        o = _turn(o, value_rotation.cos[pos][:, None, :], value_rotation.sin[pos][:, None, :], value_dim, value_rotation.interleaved, -1.0)
    if gate is not None and gate_elems > 1:
        o = o * torch.sigmoid(gate[:, gate_col: gate_col + n_heads * value_dim].to(torch.float32)).view(-1, n_heads, value_dim)
    elif gate is not None:
        o = o * torch.sigmoid(gate[:, gate_col: gate_col + n_heads].to(torch.float32))[:, :, None]
    return o.reshape(shape).to(out.dtype)


def causal_conv(x, weight, bias, state, ctx):
    n, channels = x.shape
    taps = weight.shape[1]
    a = ctx.arrays
    out = torch.empty((n, channels), dtype=torch.float32, device=x.device)
    for t in range(n):
        seq = int(a["token_seq"][t])
        local = t - int(a["seq_qstart"][seq])
        acc = bias.to(torch.float32).clone() if bias is not None else torch.zeros(channels)
        for j in range(taps):
            back = taps - 1 - j
            if local - back >= 0:
                v = x[t - back].to(torch.float32)
            else:
                v = state[int(a["state_slots"][seq]), taps - 1 + local - back].to(torch.float32)
            acc = acc + weight[:, j].to(torch.float32) * v
        out[t] = acc
    return out.to(x.dtype)


def rglru(u, y, x, wa_t, ba, wi_t, bi, lam, rate, s_state, conv_state, taps, ctx, wa=None, wi=None, chunks=None, seq_chunk0=None):
    n, channels = u.shape
    blocks = wa_t.shape[0]
    a = ctx.arrays
    uf = u.to(torch.float32).view(n, blocks, -1)
    r = torch.sigmoid(torch.einsum("tbi,bio->tbo", uf, wa_t.to(torch.float32)).reshape(n, channels) + ba.to(torch.float32))
    i = torch.sigmoid(torch.einsum("tbi,bio->tbo", uf, wi_t.to(torch.float32)).reshape(n, channels) + bi.to(torch.float32))
    log_a = -rate * r * torch.nn.functional.softplus(lam.to(torch.float32))
    av = torch.exp(log_a)
    bv = torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.to(torch.float32)
    yf = y.to(torch.float32)
    gelu = 0.5 * yf * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (yf + 0.044715 * yf**3)))
    out = torch.empty((n, channels), dtype=torch.float32, device=u.device)
    for s in range(a["seq_qstart"].numel()):
        q0, ql, slot = int(a["seq_qstart"][s]), int(a["seq_qlen"][s]), int(a["state_slots"][s])
        S = s_state[slot].clone()
        for t in range(q0, q0 + ql):
            S = av[t] * S + bv[t]
            out[t] = S * gelu[t]
        s_state[slot] = S
        if taps > 1:
            hist = torch.cat([conv_state[slot], x[q0: q0 + ql].to(conv_state.dtype)], dim=0)
            conv_state[slot] = hist[-(taps - 1):]
    return out.to(u.dtype)


def plain_kind(activation):
    return {"silu": 0, "gelu_tanh": 1, "relu2": 2}[activation]


def plain_act(u, activation):
    if activation == "relu2":
        r = torch.relu(u)
        return r * r
    if activation == "silu":
        return u * torch.sigmoid(u)
    k = math.sqrt(2.0 / math.pi)
    return 0.5 * u * (1.0 + torch.tanh(k * (u + 0.044715 * u * u * u)))


def moe_experts(x, token_ids, table, w_gate_up, w_down, activation, input_per_token=False):
    """``token_ids`` None: ``table`` has a row per token and ``x`` a row per (token, choice), or, with
    ``input_per_token``, a row per token.  ``w_gate_up`` [experts, 1, ff, hidden]: experts without a gate,
    down(act(up x)) with a plain activation."""
    top = table.shape[1]
    hidden = x.shape[1]
    n = x.shape[0] if token_ids is not None else table.shape[0]
    rows = torch.empty((n * top, hidden), dtype=torch.float32, device=x.device)
    xf = x.to(torch.float32)
    gated = w_gate_up.shape[1] == 2
    for t in range(n):
        for k in range(top):
            e = int(table[int(token_ids[t]) if token_ids is not None else t, k])
            xin = xf[t] if (token_ids is not None or input_per_token) else xf[t * top + k]
            if gated:
                g = w_gate_up[e, 0].to(torch.float32) @ xin
                u = w_gate_up[e, 1].to(torch.float32) @ xin
                yv = gated_pair(g, u, activation).to(x.dtype).to(torch.float32)
            else:
                yv = plain_act(w_gate_up[e, 0].to(torch.float32) @ xin, activation).to(x.dtype).to(torch.float32)
            rows[t * top + k] = w_down[e].to(torch.float32) @ yv
    return rows


RefOps.round_rows = staticmethod(round_rows)
RefOps.norm_add = staticmethod(norm_add)
RefOps.gated_kind = staticmethod(gated_kind)
RefOps.gated_act = staticmethod(gated_act_general)
RefOps.gate_up_act = staticmethod(lambda x, w, group, activation, out_dtype: gated_act_general(linear(x, w, out_dtype), activation, out_dtype, group))
RefOps.qkv_prepare = staticmethod(qkv_prepare)
RefOps.attention_masked = staticmethod(attention_masked)
RefOps.attention_finish = staticmethod(attention_finish)
RefOps.causal_conv = staticmethod(causal_conv)
RefOps.rglru = staticmethod(rglru)
RefOps.moe_experts = staticmethod(moe_experts)
RefOps.plain_kind = staticmethod(plain_kind)
RefOps.qk_row_scales = staticmethod(qk_row_scales)


# ------------------------------------------------- norms on both sides of a branch, plain feed-forward
def _norm_rows(x, constants):
    weight, bias, eps, center = constants
    if center:
        x = x - x.mean(dim=-1, keepdim=True)
    y = x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight.to(torch.float32)
    return y if bias is None else y + bias.to(torch.float32)


def sandwich_norm(residual, branch, post, scale, pre, rows, out_dtype):
    """residual (float32, in place unless ``rows`` picks some) += scale * post(branch); returns
    pre(residual) in ``out_dtype`` (None without ``pre``).  Without a residual: pre(branch)."""
    b = None if branch is None else branch.float()
    if residual is None:
        return _norm_rows(b, pre).to(out_dtype)
    if rows is not None:
        idx = rows.long()
        r = residual[idx]
        if b is not None:
            r = r + scale * (_norm_rows(b[idx], post) if post is not None else b[idx])
    else:
        if b is not None:
            residual += scale * (_norm_rows(b, post) if post is not None else b)
        r = residual
    return None if pre is None else _norm_rows(r, pre).to(out_dtype)


def activation(x, kind, out_dtype):
    x = x.float()
    if kind == "relu2":
        y = torch.relu(x) ** 2
    elif kind == "silu":
        y = x * torch.sigmoid(x)
    else:
        y = 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x**3)))
    return y.to(out_dtype)


def scale_rows(x, s):
    x *= s
    return x


# ------------------------------------------------------------- attention over one latent per token
def latent_prepare(proj, q_rank, q_norm, eps, act_dtype, kv_col=0, kv_rank=0, rot_dim=0, kv_norm=None, rotation=None,
                   positions=None, pages=None, slots=None, page_size=0, values=None):
    p = proj.float()
    c_q = _rmsnorm(p[:, :q_rank], q_norm, eps, False).to(act_dtype)
    if kv_rank:
        c = _rmsnorm(p[:, kv_col: kv_col + kv_rank], kv_norm, eps, False)
        pos = positions.long()
        row = c
        if rot_dim:
            r = _turn(p[:, kv_col + kv_rank: kv_col + kv_rank + rot_dim], rotation.cos[pos], rotation.sin[pos], rot_dim, rotation.interleaved)
            row = torch.cat([c, r], dim=1)
        row = row.to(pages.dtype)
        s = slots.long()
        pages[s // page_size, 0, s % page_size, :] = row
        if values is not None:  # the latent once more, transposed
            values[s // page_size, 0, :, s % page_size] = c.to(values.dtype)
    return c_q


def head_linear(x, w, n_heads, in_dim, out_dim, out_dtype, tail=0, rotation=None, positions=None, gate=None, gate_col=0, w_t=None,
                gate_elems=1):
    """Per head, out[n, h, :out_dim] = x[n, h, :in_dim] . w[h] (w [heads, in, out]); ``tail`` more elements of
    every head of x follow the product, turned by the token's position; ``gate``: the head's output times
    the sigmoid of column gate_col + h of ``gate``."""
    n = x.shape[0]
    xh = x.float().reshape(n, n_heads, in_dim + tail)
    out = torch.einsum("nhi,hio->nho", xh[..., :in_dim], w.float())
    if tail:
        pos = positions.long()
        t = _turn(xh[..., in_dim:], rotation.cos[pos][:, None, :], rotation.sin[pos][:, None, :], tail, rotation.interleaved)
        out = torch.cat([out, t], dim=-1)
    if gate is not None and gate_elems > 1:
        out = out * torch.sigmoid(gate[:, gate_col: gate_col + n_heads * out_dim].float()).view(n, n_heads, out_dim)
    elif gate is not None:
        out = out * torch.sigmoid(gate[:, gate_col: gate_col + n_heads].float())[:, :, None]
    return out.reshape(n, -1).to(out_dtype)


def latent_attention(q_lat, pages, n_heads, kv_rank, rot_dim, scale, ctx, group, page_size, tiles=None, values=None, sink=None):
    a = ctx.arrays
    n = q_lat.shape[0]
    width = kv_rank + rot_dim
    q = q_lat.float().view(n, n_heads, width)
    out = torch.zeros((n, n_heads, kv_rank), dtype=torch.float32, device=q_lat.device)
    bt = a[f"block_table_g{group}"]
    for t in range(n):
        seq, p = int(a["token_seq"][t]), int(a["positions"][t])
        idx = torch.arange(p + 1)
        rows = pages[bt[seq, idx // page_size].long(), 0, idx % page_size, :].float()
        scores = (q[t] @ rows.T) * scale
        if sink is not None:  # a score with no key and no value
            scores = torch.cat([scores, sink.float()[:, None]], dim=1)
        prob = torch.softmax(scores, dim=-1)[:, : rows.shape[0]]
        out[t] = prob @ rows[:, :kv_rank]
    return out.view(n, n_heads * kv_rank)


# ---------------------------------------------------------------- a matrix per head as the memory
def causal_conv_act(x, weight, bias, state, ctx, act=None):
    y = causal_conv(x, weight, bias, state, ctx)
    return y if act is None else activation(y, act, y.dtype)


def conv_state_push(x, state, ctx):
    a = ctx.arrays
    keep = state.shape[1]
    for s in range(a["seq_qstart"].numel()):
        q0, ql, slot = int(a["seq_qstart"][s]), int(a["seq_qlen"][s]), int(a["state_slots"][s])
        state[slot] = torch.cat([state[slot], x[q0: q0 + ql].to(state.dtype)], dim=0)[-keep:]


def linear_state_scan(qkv, n_heads, n_kv, dim, vdim, state, ctx, q_scale=1.0, unit_eps=None, decay=None, beta=None, columns=None,
                      skip=None):
    a = ctx.arrays
    n = qkv.shape[0]
    x = qkv.float()
    kd = n_kv * dim
    qc, kc, vc = columns if columns is not None else (0, kd, 2 * kd)
    q, k, v = x[:, qc: qc + kd].reshape(n, n_kv, dim), x[:, kc: kc + kd].reshape(n, n_kv, dim), x[:, vc: vc + n_heads * vdim].reshape(n, n_heads, vdim)
    if unit_eps is not None:
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps)
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)
    q = q * q_scale
    if decay[0] == "head":
        _, src, col, a_log, dt_bias = decay
        step = torch.nn.functional.softplus(src[:, col: col + n_heads].float() + dt_bias.float())
        g = torch.exp(-torch.exp(a_log.float()) * step)
        g = g[:, :, None].expand(n, n_heads, dim)
    else:
        _, src, col, bias, tau = decay
        z = src[:, col: col + n_heads * dim].float() + bias.float()
        g = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(n, n_heads, dim)
    by_step = isinstance(beta, str)  # "step": u = dt v, no delta rule
    b = None if beta is None or by_step else torch.sigmoid(beta[0][:, beta[1]: beta[1] + n_heads].float())
    out = torch.empty((n, n_heads, vdim), dtype=torch.float32, device=qkv.device)
    per = n_heads // n_kv
    for s in range(a["seq_qstart"].numel()):
        q0, ql, slot = int(a["seq_qstart"][s]), int(a["seq_qlen"][s]), int(a["state_slots"][s])
        S = state[slot].clone()
        for t in range(q0, q0 + ql):
            for h in range(n_heads):
                kk, qq = k[t, h // per], q[t, h // per]
                Sh = g[t, h][:, None] * S[h]
                u = v[t, h] if b is None else b[t, h] * (v[t, h] - Sh.T @ kk)
                if by_step:
                    u = step[t, h] * v[t, h]
                Sh = Sh + torch.outer(kk, u)
                out[t, h] = Sh.T @ qq
                if skip is not None:
                    out[t, h] += skip[h].float() * v[t, h]
                S[h] = Sh
        state[slot] = S
    return out.view(n, n_heads * vdim)


def gated_head_norm(o, weight, eps, gate, gate_col, n_heads, vdim, out_dtype, gate_first=False):
    n = o.shape[0]
    g = gate[:, gate_col: gate_col + n_heads * vdim].float()
    w = weight.float() if weight.numel() == vdim else weight.float().view(n_heads, vdim)
    if gate_first:
        return _rmsnorm((o.float() * g * torch.sigmoid(g)).view(n, n_heads, vdim), w, eps, False).reshape(n, -1).to(out_dtype)
    y = _rmsnorm(o.float().view(n, n_heads, vdim), w, eps, False).reshape(n, -1)
    return (y * g * torch.sigmoid(g)).to(out_dtype)


def moe_router_topk(logits, x, top, experts=None, bias=None, scores="sigmoid"):
    """``scores`` "sigmoid": (choice, x's rows once per chosen expert times sigmoid(logit)); "softmax_of_chosen":
    (choice, float32 weights [N, top], the softmax over the chosen logits alone); ``bias`` joins the logits first."""
    experts = logits.shape[1] if experts is None else experts
    z = logits[:, :experts].float()
    if bias is not None:
        z = z + bias.float()
    n = z.shape[0]
    choice = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    for t in range(n):
        left = z[t].clone()
        for k in range(top):
            e = int(torch.argmax(left))  # (the first of equals)
            choice[t, k] = e
            left[e] = -math.inf
    chosen = torch.gather(z, 1, choice.long())
    if scores == "softmax_of_chosen":
        return choice, torch.softmax(chosen, dim=1)
    xs = (x.float()[:, None, :] * torch.sigmoid(chosen)[:, :, None]).to(x.dtype).reshape(n * top, x.shape[1])
    return choice, xs


def moe_combine(dense, rows, top, weight=1.0, row_weights=None):
    r = rows.view(rows.shape[0] // top, top, rows.shape[1])
    if row_weights is not None:
        r = r * row_weights.view(-1, top, 1)
    out = r.sum(1) * weight
    return out if dense is None else out + dense.float()


RefOps.sandwich_norm = staticmethod(sandwich_norm)
RefOps.activation = staticmethod(activation)
RefOps.scale_rows = staticmethod(scale_rows)
RefOps.latent_prepare = staticmethod(latent_prepare)
RefOps.head_linear = staticmethod(head_linear)
RefOps.latent_attention = staticmethod(latent_attention)
RefOps.latent_tile_tokens = staticmethod(lambda n_heads, matrix_cores=False: 16 // min(n_heads, 4))
RefOps.latent_attention_on_matrix_cores = staticmethod(lambda act_dtype, kv_rank, rot_dim, page_size: False)
RefOps.causal_conv = staticmethod(causal_conv_act)
RefOps.conv_state_push = staticmethod(conv_state_push)
RefOps.linear_state_scan = staticmethod(linear_state_scan)
RefOps.gated_head_norm = staticmethod(gated_head_norm)
RefOps.moe_router_topk = staticmethod(moe_router_topk)
RefOps.moe_combine = staticmethod(moe_combine)
RefOps.moe_experts = staticmethod(moe_experts)
