"""Zetunex on the GPU against the plain implementation (``plain_zetunex.py``): each new kernel
alone, then small models of several shapes stepped whole, decoded token by token, in portions
down to two tokens, and in mixed batches whose pages and state slots are used again."""

import pytest
import torch

import helpers
import plain_zetunex as plain
import zetunex_models

pytestmark = pytest.mark.gpu

F64 = torch.float64
# |engine - plain| <= TOLERANCE * max|plain logits|
TOLERANCE = {"float32": 5e-5, "bfloat16": 3e-2}


def _kernels():
    from pagedserve_amd.ops import kernels

    return kernels


def _gpu(tensor, dtype=torch.float32):
    return tensor.to(dtype).cuda().contiguous()


def _ints(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("width", [40, 256, 1100])
def test_stream_step_adds_norms_and_clears(width):
    kernels = _kernels()
    g = torch.Generator().manual_seed(width)
    tokens = 6
    h = torch.randn((tokens, width), generator=g, dtype=F64)
    y = torch.randn((tokens, width), generator=g, dtype=F64)
    bias = torch.randn(width, generator=g, dtype=F64)
    gamma = 1 + 0.2 * torch.randn(width, generator=g, dtype=F64)
    eps, factor = 1e-5, 0.35
    for dtype in (torch.float32, torch.bfloat16):
        dh, dy = _gpu(h), _gpu(y)
        normed = torch.full((tokens, width), float("nan"), dtype=dtype, device="cuda")
        kernels.stream_step(dh, tokens, width, add=(dy, factor), bias=_gpu(bias),
                            norm=(_gpu(gamma), eps, normed), zero=dy)
        summed = h + factor * y + bias
        assert torch.allclose(dh.double().cpu(), summed, atol=1e-5)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(normed.double().cpu(), plain.rms_norm(summed, gamma, eps), atol=tol, rtol=tol)
        assert float(dy.abs().max()) == 0.0
    # a norm alone leaves the stream as it is; an add alone writes no norm; fewer rows than the buffer has
    dh = _gpu(h)
    normed = torch.zeros((tokens, width), device="cuda")
    kernels.stream_step(dh, tokens - 2, width, norm=(_gpu(gamma), eps, normed))
    assert torch.equal(dh.cpu(), h.float())
    assert torch.allclose(normed[:tokens - 2].double().cpu(), plain.rms_norm(h[:tokens - 2], gamma, eps), atol=1e-5)
    assert float(normed[tokens - 2:].abs().max()) == 0.0
    kernels.stream_step(dh, tokens, width, add=(_gpu(y), -2.0))
    assert torch.allclose(dh.double().cpu(), h - 2 * y, atol=1e-5)


def test_gate_product_and_pair_of_norms():
    kernels = _kernels()
    g = torch.Generator().manual_seed(3)
    tokens, inner, width = 5, 300, 72
    both = torch.randn((tokens, 2 * inner), generator=g, dtype=F64) * 3
    expected = plain.silu(both[:, :inner]) * both[:, inner:]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        out = torch.empty((tokens, inner), dtype=dtype, device="cuda")
        kernels.silu_gate(_gpu(both), out)
        assert torch.allclose(out.double().cpu(), expected, atol=tol, rtol=tol)
    a = torch.randn((tokens, width), generator=g, dtype=F64) * 5
    b = torch.randn((tokens, width), generator=g, dtype=F64) * 0.01
    wa, wb = torch.randn(width, generator=g, dtype=F64), torch.randn(width, generator=g, dtype=F64)
    y = torch.randn((tokens, width), generator=g, dtype=F64)
    da, db, dy = _gpu(a), _gpu(b), _gpu(y)
    kernels.pair_norm_mix(da, db, _gpu(wa), _gpu(wb), 1e-5, 0.5, dy, tokens, width)
    want = y + 0.5 * (plain.rms_norm(a, wa, 1e-5) + plain.rms_norm(b, wb, 1e-5))
    assert torch.allclose(dy.double().cpu(), want, atol=1e-5)
    assert float(da.abs().max()) == 0.0 and float(db.abs().max()) == 0.0


@pytest.mark.parametrize("experts,groups,keep,top", [(8, 4, 2, 3), (18, 3, 1, 4), (6, 1, 1, 6), (12, 6, 3, 1),
                                                     (5, 5, 2, 2), (64, 8, 4, 8), (128, 8, 4, 6), (66, 3, 2, 30)])
def test_router_chooses_within_the_best_groups(experts, groups, keep, top):
    kernels = _kernels()
    g = torch.Generator().manual_seed(experts * 10 + top)
    tokens, width = 33, 48
    x = torch.randn((tokens, width), generator=g)
    router = torch.randn((experts, width), generator=g) * 0.5
    # one row whose best expert sits in a group that is otherwise poor, next to a group of good ones
    logits = x.double() @ router.double().T
    chosen, weights = plain.route(logits, groups, keep, top, 1.75)
    ids = torch.full((tokens, top), -1, dtype=torch.int32, device="cuda")
    got = torch.zeros((tokens, top), device="cuda")
    kernels.moe_route(x.cuda(), router.cuda(), groups, keep, top, 1.75, ids, got)
    ids, got = ids.cpu(), got.double().cpu()
    for t in range(tokens):
        assert sorted(ids[t].tolist()) == sorted(chosen[t]), t
        by_id = dict(zip(chosen[t], weights[t]))
        for e, weight in zip(ids[t].tolist(), got[t].tolist()):
            assert abs(weight - by_id[e]) <= 1e-5
    if keep < groups and top > keep:
        # the limit bites (the best `keep` experts always lie in open groups, the next need not)
        free = [sorted(range(experts), key=lambda e: -float(logits[t, e]))[:top] for t in range(tokens)]
        assert any(sorted(free[t]) != sorted(chosen[t]) for t in range(tokens))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,inner,experts,top", [(48, 20, 5, 2), (128, 96, 4, 3), (72, 130, 3, 1), (44, 24, 5, 2)])
def test_experts_of_every_token(dtype, width, inner, experts, top):
    kernels = _kernels()
    g = torch.Generator().manual_seed(width + inner)
    tokens = 19
    x = torch.randn((tokens, width), generator=g).to(dtype)
    w1 = (torch.randn((experts, 2 * inner, width), generator=g) / width ** 0.5).to(dtype)
    w2 = (torch.randn((experts, width, inner), generator=g) / inner ** 0.5).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand((tokens, top), generator=g)
    y0 = torch.randn((tokens, width), generator=g)
    y = y0.clone().cuda()
    hidden = torch.empty((tokens * top + 3, inner), dtype=dtype, device="cuda")
    kernels.moe_experts(x.cuda(), w1.cuda(), w2.cuda(), ids.cuda(), weights.cuda(), hidden, y)
    expected = y0.double().clone()
    for t in range(tokens):
        for j in range(top):
            e = int(ids[t, j])
            expected[t] += float(weights[t, j]) * plain.gated(
                x[t:t + 1].double(), w1[e, :inner].double(), w1[e, inner:].double(), w2[e].double())[0]
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert torch.allclose(y.double().cpu(), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("width,inner,experts,top,tokens", [(64, 40, 5, 2, 150), (128, 96, 4, 3, 70), (72, 136, 7, 1, 333),
                                                            (256, 200, 3, 2, 64)])
def test_experts_of_many_tokens_sorted_onto_the_matrix_cores(width, inner, experts, top, tokens):
    """The path for many rows: pairs sorted by expert into tiles (experts with a few pairs,
    with more than a tile, and one with none), against the plain sum and the path for few rows."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(width + inner)
    dtype = torch.bfloat16
    x = torch.randn((tokens, width), generator=g).to(dtype)
    w1 = (torch.randn((experts, 2 * inner, width), generator=g) / width ** 0.5).to(dtype)
    w2 = (torch.randn((experts, width, inner), generator=g) / inner ** 0.5).to(dtype)
    # the last expert gets nothing, the first most
    ids = torch.stack([torch.randperm(experts - 1, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    ids[: tokens // 2, 0] = 0
    for row in range(tokens // 2):
        if top > 1 and int(ids[row, 1]) == 0:
            ids[row, 1] = 1 if int(ids[row, min(2, top - 1)]) != 1 or top == 2 else experts - 2
    weights = torch.rand((tokens, top), generator=g)
    y0 = torch.randn((tokens, width), generator=g)
    y = y0.clone().cuda()
    pairs = tokens * top
    tiles = kernels.moe_grouped_tiles(pairs, experts)
    hidden = torch.empty((pairs, inner), dtype=dtype, device="cuda")
    out = torch.empty((pairs, width), device="cuda")
    order = torch.empty(tiles * kernels.MOE_TILE, dtype=torch.int32, device="cuda")
    tile_expert = torch.empty(tiles, dtype=torch.int32, device="cuda")
    assert kernels.moe_grouped_supported(dtype, width, inner)
    kernels.moe_experts_grouped(x.cuda(), w1.cuda(), w2.cuda(), ids.cuda(), weights.cuda(), hidden, out, order,
                                tile_expert, y)
    # every pair has one place, in a tile of its expert
    placed = order.cpu()
    assert sorted(placed[placed >= 0].tolist()) == list(range(pairs))
    owners = tile_expert.cpu()
    flat_ids = ids.reshape(-1)
    for place in range(0, tiles * kernels.MOE_TILE, 7):
        if int(placed[place]) >= 0:
            assert int(owners[place // kernels.MOE_TILE]) == int(flat_ids[int(placed[place])])
    rowwise = y0.clone().cuda()
    kernels.moe_experts(x.cuda(), w1.cuda(), w2.cuda(), ids.cuda(), weights.cuda(), torch.empty_like(hidden), rowwise)
    expected = y0.double().clone()
    for t in range(0, tokens, 3):
        for j in range(top):
            e = int(ids[t, j])
            expected[t] += float(weights[t, j]) * plain.gated(
                x[t:t + 1].double(), w1[e, :inner].double(), w1[e, inner:].double(), w2[e].double())[0]
    assert torch.allclose(y.double().cpu()[::3], expected[::3], atol=3e-2, rtol=3e-2)
    assert torch.allclose(y, rowwise, atol=2e-2, rtol=2e-2)


def _scan_inputs(g, total, channels, states, rank):
    proj = torch.randn((total, 2 * channels + 3), generator=g)
    low = torch.randn((total, rank + 2 * states + 2), generator=g)
    return proj, low


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,states,rank,taps", [(48, 8, 3, 4), (40, 5, 1, 2), (24, 130, 2, 1),
                                                       (256, 16, 8, 4), (70, 32, 4, 3), (9, 3, 2, 7)])
def test_selective_scan_in_one_go_in_pieces_and_in_reused_slots(dtype, channels, states, rank, taps):
    """Convolution, step sizes and recurrence of several requests of unequal length in one launch
    each against the plain ones; the same tokens cut into pieces (also shorter than the
    convolution) give the same outputs and state; a slot that no request holds stays as it is."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(channels + states)
    lengths, slots = [45, 1, 9, 100], [2, 0, 3, 1]
    total = sum(lengths)
    u_col, z_col = 1, 1 + channels
    b_col, c_col = rank + 1, rank + 1 + states
    proj, low = _scan_inputs(g, total, channels, states, rank)
    conv_w = torch.randn((channels, taps), generator=g) / taps ** 0.5
    conv_b = torch.randn(channels, generator=g) * 0.1
    dt_w = (torch.randn((channels, rank), generator=g) / rank ** 0.5).to(dtype)
    dt_b = torch.randn(channels, generator=g) - 3
    a_log = torch.log(torch.arange(1, states + 1).float()).repeat(channels, 1) + 0.1 * torch.randn((channels, states), generator=g)
    skip = torch.randn(channels, generator=g)
    row = states + taps - 1
    state = torch.zeros((5, channels, row), device="cuda")
    state[4] = 7.0
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    tok_item = _ints([n for n, length in enumerate(lengths) for _ in range(length)])

    def run(rows, state, cu_list, slot_list, items, pieces=False, own_steps=False):
        count = rows.stop - rows.start
        dproj, dlow = proj[rows].cuda(), low[rows].cuda()
        x = torch.empty((count, channels), dtype=dtype, device="cuda")
        kernels.conv_silu(dproj, u_col, conv_w.cuda(), conv_b.cuda(), state, states, x, items,
                          _ints(cu_list), _ints(slot_list))
        dt = torch.empty((count, channels), device="cuda")
        kernels.step_size(dlow[:, 1:1 + rank], dt_w.cuda(), dt_b.cuda(), dt)
        y = torch.full((count, channels), float("nan"), dtype=dtype, device="cuda")
        scratch = None
        if pieces:
            sizes = kernels.selective_scan_records(count, len(slot_list), channels, states)
            scratch = tuple(torch.full((size,), float("nan"), device="cuda") for size in sizes)
        # (own_steps: the launch works the step sizes out itself instead of reading them)
        kernels.selective_scan(x, None if own_steps else dt, dlow, b_col, c_col, dproj, u_col, z_col,
                               a_log.cuda(), skip.cuda(), state, y, _ints(cu_list), _ints(slot_list), taps,
                               scratch=scratch,
                               step_weights=(1, dt_w.cuda(), dt_b.cuda()) if own_steps else None)
        return x, dt, y

    x, dt, y = run(slice(0, total), state, cu, slots, tok_item)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    a = -torch.exp(a_log.double())
    for n, length in enumerate(lengths):
        rows = slice(cu[n], cu[n + 1])
        raw = proj[rows, u_col:u_col + channels].double()
        want_x = plain.silu(plain.causal_conv(raw, conv_w.double(), conv_b.double()))
        assert torch.allclose(x[rows].double().cpu(), want_x, atol=tol, rtol=tol)
        want_dt = plain.softplus(low[rows, 1:1 + rank].double() @ dt_w.double().T + dt_b.double())
        assert torch.allclose(dt[rows].double().cpu(), want_dt, atol=1e-5, rtol=1e-5)
        # the recurrence from the engine's own rounded inputs
        got_x = x[rows].double().cpu()
        want_y, last = plain.selective_recurrence(
            got_x, dt[rows].double().cpu(), a, low[rows, b_col:b_col + states].double(),
            low[rows, c_col:c_col + states].double(), skip.double())
        want_y = want_y * plain.silu(proj[rows, z_col:z_col + channels].double())
        assert torch.allclose(y[rows].double().cpu(), want_y, atol=tol, rtol=tol)
        kept = state[slots[n]].double().cpu()
        assert torch.allclose(kept[:, :states], last, atol=2e-4, rtol=2e-4)
        before = torch.cat([torch.zeros((taps - 1, channels), dtype=F64), raw])[-(taps - 1):] if taps > 1 else raw[:0]
        assert torch.allclose(kept[:, states:], before.T, atol=1e-6)
    assert float((state[4] - 7.0).abs().max()) == 0.0
    # the same step cut into pieces that run side by side (the shape for long portions), from
    # states that are not zero: the whole step once more on top of what the first run left
    again = state.clone()
    _, _, y_twice = run(slice(0, total), state, cu, slots, tok_item)
    _, _, y_pieces = run(slice(0, total), again, cu, slots, tok_item, pieces=True)
    assert torch.allclose(y_pieces.float(), y_twice.float(), atol=tol, rtol=tol)
    assert torch.allclose(again, state, atol=2e-4, rtol=2e-4)
    state.zero_()
    state[4] = 7.0
    _, _, y_pieces = run(slice(0, total), state, cu, slots, tok_item, pieces=True)
    assert torch.allclose(y_pieces.float(), y.float(), atol=tol, rtol=tol)
    assert float((state[4] - 7.0).abs().max()) == 0.0
    # the first request again, in pieces, in a slot that held another request before
    reference_state = state[slots[0]].clone()
    state[0].zero_()
    cursor, pieces = 0, []
    for size in (1, 2, 1, 7, 16, 17, 1):
        _, _, piece = run(slice(cursor, cursor + size), state, [0, size], [0], _ints([0] * size),
                          own_steps=size != 7)
        pieces.append(piece)
        cursor += size
    assert cursor == lengths[0]
    assert torch.allclose(torch.cat(pieces).float(), y[:cursor].float(), atol=tol / 10, rtol=tol / 10)
    assert torch.allclose(state[0], reference_state, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 24), (1, 40, 72), (3, 8, 8), (2, 64, 64)])
def test_recurrence_with_a_decay_per_head_and_activated_inputs(heads, dim, vdim):
    """The matrix-state recurrence with one decay per head and silu on queries, keys and values:
    several requests at once, then one of them in pieces in a slot that is used again.  One key
    far back is long, and the query that matches it comes hundreds of tokens later."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(heads * 100 + dim)
    lengths, slots = [307, 1, 9], [2, 0, 3]
    total = sum(lengths)
    q_col, k_col, v_col = 2, 2 + heads * dim, 2 + 2 * heads * dim
    proj = torch.randn((total, v_col + heads * vdim + 3), generator=g)
    proj[5, k_col:k_col + heads * dim] = 6.0
    proj[300, q_col:q_col + heads * dim] = 6.0
    decay = torch.tensor([0.999, 0.9, 0.97][:heads])
    state = torch.zeros((4, heads, dim, vdim), device="cuda")
    state[1] = 7.0
    out = torch.full((total, heads * vdim), float("nan"), device="cuda")
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    kernels.gla_scan(proj.cuda(), (q_col, k_col, v_col), None, state, out, _ints(cu), _ints(slots), heads, dim,
                     vdim, 1.0, head_decay=decay.cuda(), silu_inputs=True)
    finals = []
    for n, length in enumerate(lengths):
        rows = slice(cu[n], cu[n + 1])
        q = plain.silu(proj[rows, q_col:q_col + heads * dim].double()).view(length, heads, dim)
        k = plain.silu(proj[rows, k_col:k_col + heads * dim].double()).view(length, heads, dim)
        v = plain.silu(proj[rows, v_col:v_col + heads * vdim].double()).view(length, heads, vdim)
        o, final = plain.decayed_recurrence(q, k, v, decay.double())
        finals.append(final)
        scale = float(o.abs().max())
        assert float((out[rows].double().cpu().view(length, heads, vdim) - o).abs().max()) <= 2e-5 * scale
        assert torch.allclose(state[slots[n]].double().cpu(), final, atol=1e-3, rtol=2e-4)
    assert float((state[1] - 7.0).abs().max()) == 0.0
    state[0].zero_()
    cursor, pieces = 0, []
    for size, longest in ((1, 1), (7, 0), (8, 8), (2, 0), (33, 0), (32, 0), (17, 0), (207, 0)):
        rows = slice(cursor, cursor + size)
        piece = torch.empty((size, heads * vdim), device="cuda")
        kernels.gla_scan(proj[rows].cuda(), (q_col, k_col, v_col), None, state, piece, _ints([0, size]),
                         _ints([0]), heads, dim, vdim, 1.0, longest=longest, head_decay=decay.cuda(),
                         silu_inputs=True)
        pieces.append(piece)
        cursor += size
    assert cursor == lengths[0]
    scale = float(out[:cursor].abs().max())
    assert float((torch.cat(pieces) - out[:cursor]).abs().max()) <= 1e-5 * scale
    assert torch.allclose(state[0].double().cpu(), finals[0], atol=1e-3, rtol=2e-4)


@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 24), (3, 64, 64)])
def test_recurrence_with_a_decay_per_head_in_pieces_side_by_side(heads, dim, vdim):
    """The mixer's way with long portions (every piece of 128 tokens an item of its own, joined in
    order) against the walk of one block per item: items of unequal length, one shorter than a
    piece, one of a whole number of pieces, from states that are not zero."""
    import types

    from pagedserve_amd.parts import Workspace
    from pagedserve_amd.parts.linear_attention import LightningAttention

    kernels = _kernels()
    g = torch.Generator().manual_seed(dim)
    lengths, slots = [300, 40, 256, 1], [3, 0, 1, 4]
    total = sum(lengths)
    k_col, v_col = heads * dim, 2 * heads * dim
    proj = (torch.randn((total, v_col + heads * vdim), generator=g) * 0.5).cuda()
    decay = [0.999, 0.9, 0.97][:heads]
    mixer = LightningAttention(64, torch.float32, heads, dim, vdim, decay, 1e-5)
    mixer.head_decay = torch.tensor(decay, device="cuda")
    start = torch.randn((5, heads, dim, vdim), generator=g).cuda()
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    whole_state, whole_out = start.clone(), torch.empty((total, heads * vdim), device="cuda")
    kernels.gla_scan(proj, (0, k_col, v_col), None, whole_state, whole_out, _ints(cu), _ints(slots), heads, dim,
                     vdim, 1.0, head_decay=mixer.head_decay)
    ctx = types.SimpleNamespace(workspace=Workspace(total + 50, "cuda"), cu_tokens=_ints(cu), slots=_ints(slots))
    cache = types.SimpleNamespace(state=start.clone())
    out = torch.full((total, heads * vdim), float("nan"), device="cuda")
    for _ in range(2):      # (the second time the scratch holds what the first left)
        cache.state.copy_(start)
        mixer._scan_in_pieces(proj, (0, k_col, v_col), out, ctx, cache, total, len(lengths))
        scale = float(whole_out.abs().max())
        assert float((out - whole_out).abs().max()) <= 2e-5 * scale
        assert torch.allclose(cache.state, whole_state, atol=1e-3, rtol=2e-4)
    assert torch.equal(cache.state[2], start[2])      # a slot that no item holds


def test_norm_over_all_heads_with_a_sigmoid_gate():
    kernels = _kernels()
    g = torch.Generator().manual_seed(9)
    tokens, columns = 5, 216
    o = torch.randn((tokens, columns), generator=g)
    wide = torch.randn((tokens, columns + 4), generator=g)
    weight = 1 + 0.2 * torch.randn(columns, generator=g)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        out = torch.empty((tokens, columns), dtype=dtype, device="cuda")
        kernels.row_norm_gate(o.cuda(), weight.cuda(), 1e-5, wide.cuda()[:, 4:], out)
        expected = plain.rms_norm(o.double(), weight.double(), 1e-5) * torch.sigmoid(wide[:, 4:].double())
        assert torch.allclose(out.double().cpu(), expected, atol=tol, rtol=tol)


# ---------------------------------------------------------------- whole models
def _close(rows, reference, dtype):
    """float32: every position within the tolerance.  bfloat16: a router's close call or a norm
    over a nearly empty state at a request's first tokens can turn on a rounding, so the bulk of
    the positions must be within the tolerance and only a few per cent may lie beyond it (a wrong
    key, page, window or state shows at every later position, not at a few)."""
    worst, scale, where = helpers.max_error(rows, reference)
    if dtype == "float32" or worst <= TOLERANCE[dtype] * scale:
        return worst <= TOLERANCE[dtype] * scale, (worst / scale, where)
    errors = sorted(float((row - reference[rid][position]).abs().max()) / scale
                    for (rid, position), row in rows.items())
    beyond = sum(error > TOLERANCE[dtype] for error in errors)
    return (beyond <= max(1, len(errors) // 25) and errors[len(errors) // 2] <= TOLERANCE[dtype] / 3,
            (worst / scale, where, beyond))


def _requests(raw, lengths, seed):
    return {f"r{index}": helpers.random_tokens(length, raw["vocab"], seed + index)
            for index, length in enumerate(lengths)}


def _reference(raw, tensors, requests):
    return {rid: plain.forward(raw, tensors, tokens)[0] for rid, tokens in requests.items()}


def _engine(folder, dtype, page_size, steps, max_requests=4, graphs=True):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    model, _ = load_model(folder, dtype=dtype, device="cuda")
    budget = helpers.live_token_budget(steps, round_to=page_size)
    longest = max(sum(len(e["tokens"]) for e in step["entries"]) for step in steps)
    return Engine(model, num_pages=-(-budget // page_size), page_size=page_size, max_requests=max_requests,
                  max_step_tokens=max(longest, page_size), use_graphs=graphs)


LENGTHS = (45, 1, 19, 33, 7, 2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(zetunex_models.MODELS))
def test_model_whole_decoded_in_portions_and_mixed(tmp_path, which, dtype):
    folder, raw, tensors, page_size = zetunex_models.folder_of(tmp_path, which)
    requests = _requests(raw, LENGTHS, 11)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("whole", helpers.trace_whole(requests)),
                        ("decoded", helpers.trace_tail_decoded(requests, tail=12)),
                        ("portions", helpers.trace_portions(requests)),
                        ("mixed", helpers.trace_mixed(requests, max_live=3))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=3)
        holders = {}
        rows = helpers.replay_in_process(engine, steps, page_holders=holders)
        assert len(rows) == sum(LENGTHS)
        good, what = _close(rows, reference, dtype)
        assert good, (which, name, what)
        engine.cache.check_invariants()
        assert not engine.cache.requests and len(engine.cache.free_slots) == 3
        if name == "mixed":
            # six requests went through three slots and a pool made for the live ones only
            assert any(len(who) > 1 for who in holders.values())


def test_the_stream_after_every_layer_run(tmp_path):
    """The stream after each call of the run order (a looped layer counts each time), read from
    the engine's workspace while every block folds its sum into the stream itself."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model

    folder, raw, tensors, page_size = zetunex_models.folder_of(tmp_path, "A")
    tokens = helpers.random_tokens(13, raw["vocab"], 4)
    _, after = plain.forward(raw, tensors, tokens)
    model, _ = load_model(folder, dtype="float32", device="cuda")
    caught = []
    for block in model.blocks:
        block.takes_stream_write = False      # the model then asks every block to finish at once

        def finish(h, ctx, inner=block.finish):
            inner(h, ctx)
            caught.append(h[:ctx.tokens].double().cpu())
        block.finish = finish
    engine = Engine(model, num_pages=8, page_size=page_size, max_requests=2, max_step_tokens=16, use_graphs=False)
    engine.step([StepEntry("a", tokens, [])])
    assert len(caught) == len(after) == 8
    for index, (got, want) in enumerate(zip(caught, after)):
        assert torch.allclose(got, want, atol=2e-4), (index, float((got - want).abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [6, 16, 19])
def test_a_loud_key_just_inside_and_just_outside_the_window(tmp_path, window, dtype):
    """One key that takes nearly all the weight of the queries that match it: queries at every
    distance around the window's edge (a page holds 8 tokens), inside a prompt, at the start of a
    portion, and decoded one by one; the recurrent layer meets the same key from far away."""
    folder, raw, tensors = zetunex_models.loud_key_model(tmp_path, window, 0.999)
    loud, ask = zetunex_models.LOUD, zetunex_models.ASK
    g = torch.Generator().manual_seed(window)

    def filler(count):
        return (torch.randint(3, raw["vocab"], (count,), generator=g)).tolist()

    requests = {}
    for place in (0, 3, 7, 8):              # where the loud key lies: first token, a page's last and first place
        tokens = filler(place) + [loud] + filler(window - 3) + [ask] * 5 + filler(170) + [ask]
        requests[f"p{place}"] = tokens
    reference = _reference(raw, tensors, requests)
    # the effect is there: the logits of the query at the edge differ from those one step outside
    edge = requests["p3"]
    inside, outside = 3 + window - 1, 3 + window
    assert edge[inside] == ask and edge[outside] == ask
    assert float((reference["p3"][inside] - reference["p3"][outside]).abs().max()) > 0.05 * float(reference["p3"].abs().max())
    traces = {"whole": helpers.trace_whole(requests),
              "decoded": helpers.trace_tail_decoded(requests, tail=190),
              "portions": helpers.trace_portions(requests, sizes=(window + 1, 2, 3, 2, 64, 5)),
              "mixed": helpers.trace_mixed(requests, max_live=3, decode_tail=180)}
    for name, steps in traces.items():
        engine = _engine(folder, dtype, 8, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        worst, scale, where = helpers.max_error(rows, reference)
        assert worst <= TOLERANCE[dtype] * scale, (name, worst / scale, where)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "C"])
def test_long_portions_whose_recurrences_run_in_pieces(tmp_path, which, dtype):
    """Prompts of several hundred tokens whole and in long portions beside a short one: the
    recurrent mixers cut such steps into pieces that run side by side."""
    folder, raw, tensors, page_size = zetunex_models.folder_of(tmp_path, which)
    requests = _requests(raw, (520, 300, 9), 23)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("whole", helpers.trace_whole(requests)),
                        ("portions", helpers.trace_portions(requests, sizes=(260, 2, 131, 300))),
                        ("mixed", helpers.trace_mixed(requests, max_live=3, portion=(270, 129), decode_tail=3))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (which, name, what)
        engine.cache.check_invariants()


def test_a_recorded_step_of_a_long_portion_replays_right(tmp_path):
    """A step of one long prompt is recorded as a graph once its layout keeps coming back; every
    replay (pieces, joins, sorted experts and cleared scratch inside it) gives what the plain
    implementation gives for that request's own tokens."""
    folder, raw, tensors, page_size = zetunex_models.folder_of(tmp_path, "A")
    requests = _requests(raw, (300,) * 7, 61)
    reference = _reference(raw, tensors, requests)
    steps = helpers.trace_whole(requests)
    engine = _engine(folder, "float32", page_size, steps, max_requests=2)
    engine.record_after = 2
    rows = helpers.replay_in_process(engine, steps)
    assert engine.graph_summary()["graph_replays"] >= 3
    for rid in requests:
        mine = {key: row for key, row in rows.items() if key[0] == rid}
        worst, scale, where = helpers.max_error(mine, reference)
        assert worst <= TOLERANCE["float32"] * scale, (rid, worst / scale, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_many_pages_and_graph_replays(tmp_path, dtype):
    folder, raw, tensors, _ = zetunex_models.folder_of(tmp_path, "A")
    requests = _requests(raw, (150, 131), 5)
    reference = _reference(raw, tensors, requests)
    # two requests decoded side by side from their third token on, pages of four tokens
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": tokens[:3], "want": [0, 1, 2]}
                                      for rid, tokens in requests.items()], "end": []}]
    for index in range(3, 150):
        entries = [{"id": rid, "tokens": [tokens[index]], "want": [0]}
                   for rid, tokens in requests.items() if index < len(tokens)]
        steps.append({"step": len(steps), "entries": entries, "end": []})
    steps[-1]["end"] = list(requests)
    engine = _engine(folder, dtype, 4, steps)
    rows = helpers.replay_in_process(engine, steps)
    good, what = _close(rows, reference, dtype)
    assert good, what
    assert engine.graph_summary()["graph_replays"] > 50      # decode steps ran as recorded graphs


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_scheduler(tmp_path, which):
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    folder, raw, tensors, page_size = zetunex_models.folder_of(tmp_path, which)
    prompts = [helpers.random_tokens(length, raw["vocab"], 40 + length) for length in (9, 1, 21, 5, 14)]
    count = 10
    expected = [plain.greedy_generate(raw, tensors, prompt, count) for prompt in prompts]
    llm = LLM(folder, dtype="float32", num_kv_pages=40, block_size=page_size, max_batch_size=3,
              eos_token_id=None, prefill_chunk_size=6, scheduling_strategy="sarathi")
    outputs = llm.generate(prompts, SamplingParams(max_new_tokens=count))
    assert [output.token_ids for output in outputs] == expected
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests
