"""Kosesun on the GPU against the plain implementation (``plain_kosesun.py``): each new
kernel alone, then small models of several shapes stepped whole, decoded token by token, in
portions down to two tokens, and in mixed batches whose pages and state slots are used again."""

import math

import pytest
import torch

import helpers
import kosesun_models
import plain_kosesun as plain

pytestmark = pytest.mark.gpu

F64 = torch.float64
# |engine - plain| <= TOLERANCE * max|plain logits|
TOLERANCE = {"float32": 5e-5, "bfloat16": 3e-2}


def _kernels():
    from pagedserve_amd.ops import kernels

    return kernels


def _gpu(tensor, dtype=torch.float32):
    return tensor.to(dtype).cuda().contiguous()


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("streams,width", [(1, 48), (2, 64), (4, 200), (8, 1100), (3, 4104)])
def test_stream_copies_write_and_read(streams, width):
    kernels = _kernels()
    g = torch.Generator().manual_seed(streams * 1000 + width)
    tokens = 5
    x = torch.randn((tokens, streams, width), generator=g, dtype=F64)
    y = torch.randn((tokens, width), generator=g, dtype=F64)
    mix = torch.eye(streams, dtype=F64) + 0.3 * torch.randn((streams, streams), generator=g, dtype=F64)
    out_w = torch.randn(streams, generator=g, dtype=F64)
    in_w = torch.randn(streams, generator=g, dtype=F64)
    gamma = 1 + 0.2 * torch.randn(width, generator=g, dtype=F64)
    eps = 1e-5
    copies = [x[:, s] for s in range(streams)]
    written = plain.hyper_write(copies, y, mix, out_w)
    # write, then read, in one launch; the buffer of y is cleared behind it
    dx, dy = _gpu(x.reshape(tokens, -1)), _gpu(y)
    for dtype in (torch.float32, torch.bfloat16):
        dx, dy = _gpu(x.reshape(tokens, -1)), _gpu(y)
        normed = torch.full((tokens, width), float("nan"), dtype=dtype, device="cuda")
        kernels.hyper_step(dx, tokens, width, streams, write=(dy, _gpu(mix.reshape(-1)), _gpu(out_w)),
                           read=(_gpu(in_w), _gpu(gamma), eps, normed), zero=dy)
        expected = plain.rms_norm(plain.hyper_read(written, in_w), gamma, eps)
        assert torch.allclose(dx.double().cpu().view(tokens, streams, width), torch.stack(written, 1), atol=1e-5)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(normed.double().cpu(), expected, atol=tol, rtol=tol)
        assert float(dy.abs().max()) == 0.0
    # a read alone leaves the copies as they are; a write alone writes no norm
    dx = _gpu(x.reshape(tokens, -1))
    normed = torch.empty((tokens, width), dtype=torch.float32, device="cuda")
    kernels.hyper_step(dx, tokens, width, streams, read=(_gpu(in_w), _gpu(gamma), eps, normed))
    assert torch.equal(dx.cpu(), x.reshape(tokens, -1).float())
    assert torch.allclose(normed.double().cpu(), plain.rms_norm(plain.hyper_read(copies, in_w), gamma, eps), atol=1e-5)
    kernels.hyper_step(dx, tokens, width, streams, write=(_gpu(y), _gpu(mix.reshape(-1)), _gpu(out_w)))
    assert torch.allclose(dx.double().cpu().view(tokens, streams, width), torch.stack(written, 1), atol=1e-5)
    # all copies from one row, and their sum for chosen rows
    e = _gpu(y)
    kernels.streams_expand(e, dx, tokens, width, streams)
    assert torch.equal(dx.view(tokens, streams, width)[:, streams - 1], e)
    rows = torch.tensor([3, 0], dtype=torch.int32, device="cuda")
    summed = torch.empty((2, width), dtype=torch.float32, device="cuda")
    kernels.streams_collapse(_gpu(x.reshape(tokens, -1)), rows, summed, width, streams)
    assert torch.allclose(summed.double().cpu(), x[[3, 0]].sum(1), atol=1e-5)


def _paged(contexts, kv_heads, head_dim, page_size, g, dtype):
    """Keys and values of several requests in scattered pages; returns pools, tables, dense copies."""
    pages_per = [-(-length // page_size) for length in contexts]
    total = sum(pages_per) + 2
    order = (torch.randperm(total, generator=g)).tolist()
    tables = torch.full((len(contexts), max(pages_per) + 1), -1, dtype=torch.int32)
    k_pool = torch.full((total, kv_heads, page_size, head_dim), float("nan"))
    v_pool = torch.full((total, kv_heads, page_size, head_dim), float("nan"))
    dense = []
    cursor = 0
    for index, (count, length) in enumerate(zip(pages_per, contexts)):
        k = torch.randn((length, kv_heads, head_dim), generator=g).to(dtype).float()
        v = torch.randn((length, kv_heads, head_dim), generator=g).to(dtype).float()
        dense.append((k, v))
        for logical in range(count):
            page = order[cursor + logical]
            tables[index, logical] = page
            rows = slice(logical * page_size, min(length, (logical + 1) * page_size))
            filled = rows.stop - rows.start
            k_pool[page, :, :filled] = k[rows].transpose(0, 1)
            v_pool[page, :, :filled] = v[rows].transpose(0, 1)
        cursor += count
    return k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda(), tables.cuda(), dense


def _attend_plain(q, k, v, scale, sink, position):
    """One query at ``position`` over keys 0..position (grouped heads), with a sink."""
    heads, kv_heads = q.shape[0], k.shape[1]
    out = torch.zeros((heads, v.shape[2]), dtype=F64)
    for h in range(heads):
        kv = h // (heads // kv_heads)
        scores = (k[: position + 1, kv].double() @ q[h].double()) * scale
        top = torch.maximum(scores.max(), sink[h].double()) if sink is not None else scores.max()
        weights = torch.exp(scores - top)
        total = weights.sum() + (torch.exp(sink[h].double() - top) if sink is not None else 0.0)
        out[h] = (weights / total) @ v[: position + 1, kv].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim,heads,kv_heads,page_size", [(64, 4, 2, 16), (32, 6, 1, 8), (48, 2, 2, 16)])
def test_sink_in_every_attention_kernel(dtype, head_dim, heads, kv_heads, page_size):
    """Single queries (row-wise, split-KV with one and several ranges) and prompt portions (tiled
    kernels, and both kinds in one launch) with a sink per head: a large sink takes nearly all
    the weight, a very negative one none.  One query of every request is aimed at a single far
    key (at a page's first or last place, or the very first token), whose value must come out."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(head_dim + heads)
    contexts = [300, 17, 1, 2 * page_size, 2 * page_size + 1]
    k_pool, v_pool, tables, dense = _paged(contexts, kv_heads, head_dim, page_size, g, dtype)
    scale = head_dim ** -0.5
    sink = torch.tensor([8.0, -30.0, 0.5, -1.0, 2.0, 0.0][:heads])
    count = len(contexts)
    q = torch.randn((count, heads, head_dim), generator=g)
    targets = [page_size - 1, page_size, 0, page_size, page_size - 1]
    for n, target in enumerate(targets):
        if target < contexts[n]:
            key = dense[n][0][target, 0]
            q[n, 1 % heads] = key * (40.0 / scale / float(key @ key))    # score 40 at the target (head of kv head 0)
    q = q.to(dtype)
    tok_item = torch.arange(count, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda")
    # a gate per token and head (columns of a wider tensor): the kernels multiply a head's output by its sigmoid
    wide = torch.randn((count, heads + 3), generator=g)
    dgate = wide.cuda()[:, 2:2 + heads]
    expected = torch.stack([_attend_plain(q[n].float(), dense[n][0], dense[n][1], scale, sink, contexts[n] - 1)
                            for n in range(count)]) * torch.sigmoid(wide[:, 2:2 + heads].double())[:, :, None]
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    dq = q.reshape(count, -1).cuda()
    dsink = sink.cuda()

    def check(out, what):
        got = out.double().cpu().view(count, heads, head_dim)
        assert torch.allclose(got, expected, atol=tol, rtol=tol), (what, float((got - expected).abs().max()))

    out = torch.empty_like(dq)
    kernels.attention_rowwise(dq, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, sink=dsink,
                              gate=dgate)
    check(out, "row-wise")
    # the far key's value came out where the sink is very negative, and nearly nothing where it is large
    head = 1 % heads
    if kv_heads * (head // (heads // kv_heads)) == 0:
        got = out.double().cpu().view(count, heads, head_dim)[0, head] / torch.sigmoid(wide[0, 2 + head].double())
        assert torch.allclose(got, dense[0][1][targets[0], 0].double(), atol=5e-2)
    assert float(out.double().cpu().view(count, heads, head_dim)[1:, 0].abs().max()) < 0.2
    for splits in (1, 3):
        for waves in (4, 16):
            partial = torch.full((count * heads * splits * (head_dim + 2),), float("nan"), device="cuda")
            out = torch.full_like(dq, float("nan"))
            kernels.attention_decode(dq, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits,
                                     partial=partial, waves=waves, sink=dsink, gate=dgate)
            check(out, f"split-KV {splits} x {waves}")
    # the same queries as the last tokens of prompt portions (every request brings all its tokens)
    if head_dim % 16 == 0 or dtype == torch.float32:
        lengths = contexts
        total = sum(lengths)
        big_q = torch.randn((total, heads * head_dim), generator=g).to(dtype)
        cu = [0]
        for length in lengths:
            cu.append(cu[-1] + length)
        for n in range(count):
            big_q[cu[n + 1] - 1] = q[n].reshape(-1)
        big_q = big_q.cuda()
        big_gate = torch.randn((total, heads), generator=g)
        for n in range(count):
            big_gate[cu[n + 1] - 1] = wide[n, 2:2 + heads]
        big_gate = big_gate.cuda()
        tile = kernels.PREFILL_TILE
        items, firsts = [], []
        for n, length in enumerate(lengths):
            if length > 1:
                items += [n] * -(-length // tile)
                firsts += list(range(0, length, tile))
        singles = [cu[n] for n, length in enumerate(lengths) if length == 1]
        tile_item = torch.tensor(items, dtype=torch.int32, device="cuda")
        tile_q0 = torch.tensor(firsts, dtype=torch.int32, device="cuda")
        cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
        kv_lens = torch.tensor(lengths, dtype=torch.int32, device="cuda")
        item_of = torch.tensor([n for n, length in enumerate(lengths) for _ in range(length)],
                               dtype=torch.int32, device="cuda")
        position_of = torch.tensor([p for length in lengths for p in range(length)], dtype=torch.int32, device="cuda")
        single_list = torch.tensor(singles, dtype=torch.int32, device="cuda")
        last_rows = [cu[n + 1] - 1 for n in range(count)]

        def check_rows(out, what):
            got = out[last_rows].double().cpu().view(count, heads, head_dim)
            keep = [n for n, length in enumerate(lengths) if length > 1 or what == "mixed"]
            assert torch.allclose(got[keep], expected[keep], atol=tol, rtol=tol), (
                what, float((got[keep] - expected[keep]).abs().max()))

        out = torch.full_like(big_q, float("nan"))
        if dtype == torch.float32:
            kernels.attention_tiled_f32(big_q, k_pool, v_pool, out, tile_item, tile_q0, cu_t, kv_lens, tables,
                                        heads, scale, sink=dsink, gate=big_gate)
            check_rows(out, "tiled 32-bit")
        else:
            kernels.attention_prefill(big_q, k_pool, v_pool, out, tile_item, tile_q0, cu_t, kv_lens, tables,
                                      heads, scale, sink=dsink, gate=big_gate)
            check_rows(out, "tiled")
            if kernels.mixed_supported(dtype, head_dim, tables.shape[1]):
                out = torch.full_like(big_q, float("nan"))
                kernels.attention_mixed(big_q, k_pool, v_pool, out, single_list, item_of, position_of,
                                        tile_item, tile_q0, cu_t, kv_lens, tables, heads, scale, sink=dsink,
                                        gate=big_gate)
                check_rows(out, "mixed")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 32, 8), (3, 1, 8, 40, 4), (2, 2, 24, 24, 24),
                                                          (2, 1, 64, 32, 0)])
def test_prepare_norms_rotates_mixes_and_stores(dtype, heads, kv_heads, dim, vdim, rot):
    kernels = _kernels()
    g = torch.Generator().manual_seed(dim * 7 + vdim)
    page_size, pages = 4, 12
    positions = [0, 1, 3, 4, 7, 33, 2]            # of two requests: 0, 1, 3, 4, 7, 33 and 2
    items = [0, 0, 0, 0, 0, 0, 1]
    tokens = len(positions)
    cache_dim = dim if dim == vdim else -(-max(dim, vdim) // 16) * 16
    q_cols, k_cols, v_cols = heads * dim, kv_heads * dim, kv_heads * vdim
    proj = torch.randn((tokens, q_cols + k_cols + v_cols + 5), generator=g)   # (other columns behind)
    q_gamma = 1 + 0.3 * torch.randn(q_cols, generator=g)
    k_gamma = 1 + 0.3 * torch.randn(k_cols, generator=g)
    eps, base, lam = 1e-5, 777.0, 0.37
    first = torch.randn((tokens, kv_heads * vdim), generator=g).to(dtype)
    tables = torch.full((2, 10), -1, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()
    for logical in range(9):
        tables[0, logical] = order[logical]
    tables[1, 0] = order[9]
    pos_t = torch.tensor(positions)
    q_ref = plain.rms_norm(proj[:, :q_cols].double(), q_gamma.double(), eps).view(tokens, heads, dim)
    k_ref = plain.rms_norm(proj[:, q_cols:q_cols + k_cols].double(), k_gamma.double(), eps).view(tokens, kv_heads, dim)
    if rot:
        q_ref = plain.rotate_pairs(q_ref, pos_t, rot, base)
        k_ref = plain.rotate_pairs(k_ref, pos_t, rot, base)
    v_own = proj[:, q_cols + k_cols:q_cols + k_cols + v_cols].double()
    freqs = None
    if rot:
        freqs = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32).cuda()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for mode in (0, 1, 2):
        k_pool = torch.full((pages, kv_heads, page_size, cache_dim), float("nan"), dtype=dtype, device="cuda")
        v_pool = torch.full_like(k_pool, float("nan"))
        q_out = torch.full((tokens, heads * cache_dim), float("nan"), dtype=dtype, device="cuda")
        v_first = first.clone().cuda()
        kernels.attention_prepare(
            proj.cuda(), (0, q_cols, q_cols + k_cols), q_out, k_pool, v_pool,
            torch.tensor(items, dtype=torch.int32, device="cuda"),
            torch.tensor(positions, dtype=torch.int32, device="cuda"), tables.cuda(), heads, dim, vdim,
            q_gamma=q_gamma.cuda(), k_gamma=k_gamma.cuda(), eps=eps, freqs=freqs, rot_dims=rot,
            v_first=v_first if mode else None, v_lambda=torch.tensor([lam], device="cuda") if mode == 2 else None,
            v_mode=mode)
        got_q = q_out.double().cpu().view(tokens, heads, cache_dim)
        assert torch.allclose(got_q[:, :, :dim], q_ref, atol=tol, rtol=tol)
        assert float(got_q[:, :, dim:].abs().sum()) == 0.0
        v_ref = v_own if mode < 2 else (1 - lam) * v_own + lam * first.double()
        for t in range(tokens):
            page = int(tables[items[t], positions[t] // page_size])
            slot = positions[t] % page_size
            got_k = k_pool[page, :, slot].double().cpu()
            got_v = v_pool[page, :, slot].double().cpu()
            assert torch.allclose(got_k[:, :dim], k_ref[t], atol=tol, rtol=tol)
            assert torch.allclose(got_v[:, :vdim], v_ref[t].view(kv_heads, vdim), atol=tol, rtol=tol)
            assert float(got_k[:, dim:].abs().sum()) == 0.0 and float(got_v[:, vdim:].abs().sum()) == 0.0
        # nothing else was written
        written = {(int(tables[items[t], positions[t] // page_size]), positions[t] % page_size) for t in range(tokens)}
        untouched = torch.isnan(k_pool.float()).all(dim=(1, 3)).cpu()
        assert int((~untouched).sum()) == len(written)
        if mode == 1:
            assert torch.allclose(v_first.double().cpu(), v_own, atol=tol, rtol=tol)


def test_head_gate_softcap_and_squared_relu():
    kernels = _kernels()
    g = torch.Generator().manual_seed(5)
    context = torch.randn((7, 3 * 10), generator=g)
    wide = torch.randn((7, 9), generator=g)
    gate = wide[:, 4:7]
    got = context.clone().cuda()
    kernels.head_gate(got, wide.cuda()[:, 4:7], 3, 10)
    expected = (context.view(7, 3, 10).double() * torch.sigmoid(gate.double())[:, :, None]).view(7, 30)
    assert torch.allclose(got.double().cpu(), expected, atol=1e-6)
    logits = 60 * torch.randn((4, 50), generator=g)
    buffer = torch.zeros((4, 56), device="cuda")
    buffer[:, :50] = logits.cuda()
    kernels.softcap(buffer[:, :50], 15.0)
    assert torch.allclose(buffer[:, :50].double().cpu(), plain.softcap(logits.double(), 15.0), atol=1e-5)
    assert float(buffer[:, 50:].abs().max()) == 0.0
    for dtype, rows, n, k in ((torch.float32, 5, 33, 20), (torch.bfloat16, 3, 128, 64), (torch.bfloat16, 100, 256, 128)):
        a = torch.randn((rows, k), generator=g).to(dtype)
        w = (torch.randn((n, k), generator=g) / math.sqrt(k)).to(dtype)
        out = torch.empty((rows, n), dtype=dtype, device="cuda")
        kernels.linear(a.cuda(), w.cuda(), None, out, epilogue="relu2", packed=kernels.pack_decode_weight(w.cuda()))
        expected = torch.relu(a.double() @ w.double().T) ** 2
        tol = 1e-5 if dtype == torch.float32 else 3e-2
        assert torch.allclose(out.double().cpu(), expected, atol=tol, rtol=tol)


def test_decay_is_right_at_both_ends():
    kernels = _kernels()
    g = torch.Generator().manual_seed(2)
    tokens, rank, channels, tau = 6, 5, 37, 16.0
    proj = torch.randn((tokens, 3 + rank), generator=g)
    proj[0, 3:] = 40.0            # sigmoid -> 1
    proj[1, 3:] = -40.0           # sigmoid -> tiny: the power must not lose it
    w = torch.ones((channels, rank)) + 0.1 * torch.randn((channels, rank), generator=g)
    bias = torch.randn(channels, generator=g)
    alpha = torch.empty((tokens, channels), device="cuda")
    kernels.gla_decay(proj.cuda(), 3, w.cuda(), bias.cuda(), tau, alpha)
    z = proj[:, 3:].double() @ w.double().T + bias.double()
    expected = plain.decay_of(z, tau)
    assert torch.allclose(alpha.double().cpu(), expected, rtol=2e-5, atol=1e-12)
    assert float(alpha[1].max()) < 1e-3 and float(alpha[0].min()) > 0.999999


@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 24), (1, 40, 72), (3, 8, 8), (2, 64, 64), (1, 130, 20)])
def test_recurrence_in_one_go_in_pieces_and_in_reused_slots(heads, dim, vdim):
    """Several requests of unequal length in one launch against the plain recurrence; the same
    tokens cut into pieces (around the 8 and the 32 tokens that the kernel stages at a time) give the same
    state and outputs; a slot that is cleared and used again carries nothing over."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(heads * 100 + dim)
    lengths = [107, 1, 9]
    slots = [2, 0, 3]
    total = sum(lengths)
    q_col, k_col, v_col = 2, 2 + heads * dim, 2 + 2 * heads * dim
    width = v_col + heads * vdim + 3
    proj = torch.randn((total, width), generator=g)
    alpha = torch.rand((total, heads * dim), generator=g) * 0.5 + 0.5
    scale = dim ** -0.5
    state = torch.zeros((4, heads, dim, vdim), device="cuda")
    state[1] = 7.0      # a slot that no request of the step holds stays as it is
    out = torch.full((total, heads * vdim), float("nan"), device="cuda")
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    kernels.gla_scan(proj.cuda(), (q_col, k_col, v_col), alpha.cuda(), state, out,
                     torch.tensor(cu, dtype=torch.int32, device="cuda"),
                     torch.tensor(slots, dtype=torch.int32, device="cuda"), heads, dim, vdim, scale)
    finals = []
    for n, length in enumerate(lengths):
        rows = slice(cu[n], cu[n + 1])
        q = proj[rows, q_col:q_col + heads * dim].double().view(length, heads, dim) * scale
        k = proj[rows, k_col:k_col + heads * dim].double().view(length, heads, dim)
        v = proj[rows, v_col:v_col + heads * vdim].double().view(length, heads, vdim)
        o, final = plain.gated_recurrence(q, k, v, alpha[rows].double().view(length, heads, dim))
        finals.append(final)
        assert torch.allclose(out[rows].double().cpu().view(length, heads, vdim), o, atol=2e-4, rtol=2e-4)
        assert torch.allclose(state[slots[n]].double().cpu(), final, atol=2e-4, rtol=2e-4)
    assert float((state[1] - 7.0).abs().max()) == 0.0
    # the first request again, in pieces, in a slot that held another request before
    state[0].zero_()
    cursor = 0
    pieces = []
    for size, longest in ((1, 1), (7, 0), (8, 8), (9, 0), (33, 0), (32, 0), (17, 0)):
        rows = slice(cursor, cursor + size)
        piece = torch.empty((size, heads * vdim), device="cuda")
        kernels.gla_scan(proj[rows].cuda(), (q_col, k_col, v_col), alpha[rows].cuda(), state, piece,
                         torch.tensor([0, size], dtype=torch.int32, device="cuda"),
                         torch.tensor([0], dtype=torch.int32, device="cuda"), heads, dim, vdim, scale,
                         longest=longest)
        pieces.append(piece)
        cursor += size
    assert cursor == lengths[0]
    assert torch.allclose(torch.cat(pieces), out[:cursor], atol=1e-5, rtol=1e-5)
    assert torch.allclose(state[0].double().cpu(), finals[0], atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("heads,dim,vdim", [(3, 24, 64), (2, 100, 144)])
def test_recurrence_of_many_requests_at_once(heads, dim, vdim):
    """So many (request, head, column block) triples that the kernel takes its wide blocks."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(dim)
    count = 2 * kernels.compute_units() // (heads * -(-vdim // 16)) + 1
    lengths = [1 + (n * 5) % 11 for n in range(count)]
    total = sum(lengths)
    q_col, k_col, v_col = 0, heads * dim, 2 * heads * dim
    proj = torch.randn((total, v_col + heads * vdim), generator=g)
    alpha = torch.rand((total, heads * dim), generator=g) * 0.6 + 0.4
    initial = torch.randn((count + 1, heads, dim, vdim), generator=g)
    state = initial.clone().cuda()
    slots = torch.randperm(count, generator=g).tolist()
    out = torch.full((total, heads * vdim), float("nan"), device="cuda")
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    kernels.gla_scan(proj.cuda(), (q_col, k_col, v_col), alpha.cuda(), state, out,
                     torch.tensor(cu, dtype=torch.int32, device="cuda"),
                     torch.tensor(slots, dtype=torch.int32, device="cuda"), heads, dim, vdim, 0.5)
    got, final = out.double().cpu(), state.double().cpu()
    for n in range(0, count, 7):
        rows, length = slice(cu[n], cu[n + 1]), lengths[n]
        o, last = plain.gated_recurrence(
            proj[rows, :k_col].double().view(length, heads, dim) * 0.5,
            proj[rows, k_col:v_col].double().view(length, heads, dim),
            proj[rows, v_col:].double().view(length, heads, vdim),
            alpha[rows].double().view(length, heads, dim), initial[slots[n]].double())
        assert torch.allclose(got[rows].view(length, heads, vdim), o, atol=5e-4, rtol=5e-4)
        assert torch.allclose(final[slots[n]], last, atol=5e-4, rtol=5e-4)
    assert torch.equal(final[count].float(), initial[count])


def test_recurrent_output_norm_and_gate():
    kernels = _kernels()
    g = torch.Generator().manual_seed(9)
    tokens, heads, vdim = 5, 3, 72
    o = torch.randn((tokens, heads * vdim), generator=g)
    wide = torch.randn((tokens, heads * vdim + 4), generator=g)
    weight = 1 + 0.2 * torch.randn(vdim, generator=g)
    for dtype in (torch.float32, torch.bfloat16):
        out = torch.empty((tokens, heads * vdim), dtype=dtype, device="cuda")
        kernels.gla_output(o.cuda(), weight.cuda(), 1e-5, wide.cuda()[:, 4:], out, heads, vdim)
        gate = wide[:, 4:].double()
        expected = (plain.rms_norm(o.double().view(tokens, heads, vdim), weight.double(), 1e-5).view(tokens, -1)
                    * gate * torch.sigmoid(gate))
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(out.double().cpu(), expected, atol=tol, rtol=tol)


# ---------------------------------------------------------------- whole models
def _close(rows, reference, dtype):
    """float32: every position within the tolerance.  bfloat16: the recurrent mixer norms each
    head's output, which at a request's first tokens is a product of one or two small dot
    products, so a rounding there can turn a whole head round; the bulk of the positions must
    be within the tolerance and only a few per cent may lie beyond it (a wrong key, page or
    state shows at every later position, not at a few early ones)."""
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
@pytest.mark.parametrize("which", sorted(kosesun_models.MODELS))
def test_model_whole_decoded_in_portions_and_mixed(tmp_path, which, dtype):
    folder, raw, tensors, page_size = kosesun_models.folder_of(tmp_path, which)
    requests = _requests(raw, LENGTHS, 11)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("whole", helpers.trace_whole(requests)),
                        ("decoded", helpers.trace_tail_decoded(requests, tail=12)),
                        ("portions", helpers.trace_portions(requests)),
                        ("mixed", helpers.trace_mixed(requests, max_live=3))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=3)
        holders = {}
        rows = helpers.replay_in_process(engine, steps, page_holders=holders if engine.cache.groups else None)
        assert len(rows) == sum(LENGTHS)
        good, what = _close(rows, reference, dtype)
        assert good, (which, name, what)
        engine.cache.check_invariants()
        assert not engine.cache.requests and len(engine.cache.free_slots) == 3
        if name == "mixed" and holders:
            # six requests went through three slots and a pool made for the live ones only
            assert any(len(who) > 1 for who in holders.values())


def test_the_first_layer_outputs_of_a_short_prompt(tmp_path):
    """The summed stream after every layer, read from the engine's workspace after a step that
    stops there (a model cut after each layer in turn)."""
    import copy
    import json
    import os

    from safetensors.torch import save_file

    folder, raw, tensors, page_size = kosesun_models.folder_of(tmp_path, "A")
    tokens = helpers.random_tokens(13, raw["vocab"], 4)
    _, after = plain.forward(raw, tensors, tokens)
    for depth in range(1, len(raw["layers"]) + 1):
        cut = copy.deepcopy(raw)
        cut["layers"] = cut["layers"][:depth]
        cut.pop("logit_softcap")
        kept = {name: tensor for name, tensor in tensors.items()
                if not name.startswith("l") or int(name[1:name.index(".")]) < depth}
        # identity head over the first columns and a unit final norm make the logits the normed stream
        kept["final.norm"] = torch.zeros(raw["width"])
        kept["head"] = torch.eye(raw["vocab"], raw["width"])
        where = os.path.join(str(tmp_path), f"cut{depth}")
        os.makedirs(where, exist_ok=True)
        save_file({k: v.contiguous() for k, v in kept.items()}, os.path.join(where, "model.safetensors"))
        with open(os.path.join(where, "config.json"), "w") as handle:
            json.dump(cut, handle)
        steps = helpers.trace_whole({"a": tokens})
        rows = helpers.replay_in_process(_engine(where, "float32", page_size, steps), steps)
        expected = plain.rms_norm(after[depth - 1], None, raw["norm"]["eps"])[:, :raw["width"]]
        got = torch.stack([rows[("a", p)] for p in range(len(tokens))])[:, :raw["width"]]
        assert torch.allclose(got, expected, atol=2e-4), (depth, float((got - expected).abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_many_pages_and_graph_replays(tmp_path, dtype):
    folder, raw, tensors, _ = kosesun_models.folder_of(tmp_path, "A")
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
    worst, scale, where = helpers.max_error(rows, reference)
    assert worst <= TOLERANCE[dtype] * scale, (worst / scale, where)
    assert engine.graph_summary()["graph_replays"] > 50      # decode steps ran as recorded graphs


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_scheduler(tmp_path, which):
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    folder, raw, tensors, page_size = kosesun_models.folder_of(tmp_path, which)
    prompts = [helpers.random_tokens(length, raw["vocab"], 40 + length) for length in (9, 1, 21, 5, 14)]
    count = 10
    expected = [plain.greedy_generate(raw, tensors, prompt, count) for prompt in prompts]
    llm = LLM(folder, dtype="float32", num_kv_pages=40, block_size=page_size, max_batch_size=3,
              eos_token_id=None, prefill_chunk_size=6, scheduling_strategy="sarathi")
    outputs = llm.generate(prompts, SamplingParams(max_new_tokens=count))
    assert [output.token_ids for output in outputs] == expected
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests
