"""Rezelix on the GPU against the plain implementation (``plain_rezelix.py``): each new kernel
alone, then small models of several shapes stepped whole, decoded token by token, in portions
down to two tokens, and in mixed batches whose pages and state slots are used again."""

import pytest
import torch

import helpers
import plain_rezelix as plain
import rezelix_models

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


def _bf16(tensor):
    return tensor.to(torch.bfloat16).to(tensor.dtype)


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("width", [40, 256, 1100])
def test_stream_step_with_a_factor_per_column(width):
    kernels = _kernels()
    g = torch.Generator().manual_seed(width)
    tokens = 5
    h = torch.randn((tokens, width), generator=g, dtype=F64)
    y = torch.randn((tokens, width), generator=g, dtype=F64)
    column = torch.randn(width, generator=g, dtype=F64)
    gamma = 1 + 0.2 * torch.randn(width, generator=g, dtype=F64)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        dh, dy = _gpu(h), _gpu(y)
        normed = torch.full((tokens, width), float("nan"), dtype=dtype, device="cuda")
        kernels.stream_step(dh, tokens, width, add=(dy, 1.0, _gpu(column)), norm=(_gpu(gamma), 1e-5, normed),
                            zero=dy)
        summed = h + column * y
        assert torch.allclose(dh.double().cpu(), summed, atol=1e-5)
        assert torch.allclose(normed.double().cpu(), plain.rms_norm(summed, gamma, 1e-5), atol=tol, rtol=tol)
        assert float(dy.abs().max()) == 0.0


@pytest.mark.parametrize("blocks,n,k,x_step,out_step,tokens", [(3, 16, 16, 16, 16, 7), (1, 30, 30, 30, 30, 1),
                                                               (5, 80, 40, 40, 80, 37), (2, 20, 24, 72, 32, 19),
                                                               (4, 200, 70, 70, 200, 130)])
def test_block_diagonal_product(blocks, n, k, x_step, out_step, tokens):
    kernels = _kernels()
    g = torch.Generator().manual_seed(blocks * 100 + n)
    x = torch.randn((tokens, (blocks - 1) * x_step + k + 3), generator=g)
    w = torch.randn((blocks, n, k), generator=g) / k ** 0.5
    bias = torch.randn(blocks * n, generator=g)
    gate = torch.randn((tokens, blocks * n), generator=g) * 2
    for x_dtype, w_dtype, out_dtype in ((torch.float32, torch.float32, torch.float32),
                                        (torch.float32, torch.bfloat16, torch.float32),
                                        (torch.float32, torch.bfloat16, torch.bfloat16),
                                        (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                        (torch.bfloat16, torch.bfloat16, torch.float32)):
        xs, ws = x.to(x_dtype), w.to(w_dtype)
        for with_gate in (False, True):
            expected = torch.zeros((tokens, (blocks - 1) * out_step + n), dtype=F64)
            for b in range(blocks):
                part = xs[:, b * x_step:b * x_step + k].double() @ ws[b].double().T + bias[b * n:(b + 1) * n].double()
                if with_gate:
                    part = part * torch.sigmoid(gate[:, b * n:(b + 1) * n].double())
                expected[:, b * out_step:b * out_step + n] = part
            out = torch.zeros((tokens + 2, (blocks - 1) * out_step + n), dtype=out_dtype, device="cuda")
            kernels.block_linear(xs.cuda(), x_step, ws.cuda(), bias.cuda(), out, out_step,
                                 gate=gate.cuda() if with_gate else None)
            tol = 2e-5 if out_dtype == torch.float32 else 2e-2
            assert torch.allclose(out[:tokens].double().cpu(), expected, atol=tol, rtol=tol)
            assert float(out[tokens:].abs().max()) == 0.0


def _recurrence_inputs(g, total, channels, blocks):
    size = channels // blocks
    proj = torch.randn((total, 2 * channels + 3), generator=g)
    u = torch.randn((total, channels), generator=g)
    gates = torch.randn((total, 2 * channels), generator=g) * 2
    # decays between slow and fast; one channel that barely forgets
    decay = torch.rand(channels, generator=g) * 0.3 + 0.69
    decay[0] = 0.99999
    lam = torch.log(torch.expm1(-torch.log(decay) / 8.0))
    r = torch.zeros((total, channels), dtype=F64)
    i = torch.zeros((total, channels), dtype=F64)
    for b in range(blocks):
        r[:, b * size:(b + 1) * size] = torch.sigmoid(gates[:, 2 * b * size:(2 * b + 1) * size].double())
        i[:, b * size:(b + 1) * size] = torch.sigmoid(gates[:, (2 * b + 1) * size:(2 * b + 2) * size].double())
    return proj, u, gates, lam, r, i


@pytest.mark.parametrize("channels,blocks,taps", [(48, 3, 4), (30, 1, 1), (200, 5, 2), (128, 2, 3)])
def test_gated_recurrence_per_item_and_in_pieces(channels, blocks, taps):
    """Items of unequal length from states that are not zero (one of several hundred tokens, which
    runs sixteen runs side by side; one of a single token), a slot that nobody holds, and then one
    item's tokens again in pieces of every kind, each piece from the state the piece before left."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(channels + taps)
    lengths, slots = [333, 1, 40, 128], [3, 0, 4, 1]
    total = sum(lengths)
    proj, u, gates, lam, r, i = _recurrence_inputs(g, total, channels, blocks)
    y_col, x_col = 3, 3 + channels
    start = torch.randn((6, channels, taps), generator=g)
    state = start.clone().cuda()
    out = torch.full((total, channels), float("nan"), device="cuda")
    cu = [0]
    for length in lengths:
        cu.append(cu[-1] + length)
    kernels.lru_scan(proj.cuda(), y_col, x_col, u.cuda(), gates.cuda(), channels // blocks, lam.cuda(), 8.0,
                     state, out, _ints(cu), _ints(slots), taps)
    finals = []
    for n, length in enumerate(lengths):
        rows = slice(cu[n], cu[n + 1])
        states, final = plain.gated_recurrence(u[rows].double(), r[rows], i[rows], lam.double(), 8.0,
                                               start[slots[n], :, 0].double())
        finals.append(final)
        expected = states * plain.gelu_tanh(proj[rows, y_col:y_col + channels].double())
        assert torch.allclose(out[rows].double().cpu(), expected, atol=2e-5, rtol=2e-5), n
        assert torch.allclose(state[slots[n], :, 0].double().cpu(), final, atol=2e-5, rtol=2e-5)
        # the convolution's last inputs: what the slot held, then this step's, oldest first
        history = torch.cat([start[slots[n], :, 1:].T, proj[rows, x_col:x_col + channels]])
        assert torch.equal(state[slots[n], :, 1:].cpu(), history[history.shape[0] - (taps - 1):].T.contiguous())
    for idle in (2, 5):
        assert torch.equal(state[idle].cpu(), start[idle])
    # the first item again, in pieces
    state[3].copy_(start[3])
    cursor, pieces = 0, []
    for size in (1, 2, 7, 1, 64, 3, 100, 2, 153):
        rows = slice(cursor, cursor + size)
        piece = torch.empty((size, channels), device="cuda")
        kernels.lru_scan(proj[rows].cuda(), y_col, x_col, u[rows].cuda(), gates[rows].cuda(), channels // blocks,
                         lam.cuda(), 8.0, state, piece, _ints([0, size]), _ints([3]), taps)
        pieces.append(piece)
        cursor += size
    assert cursor == lengths[0]
    assert torch.allclose(torch.cat(pieces), out[:cursor], atol=2e-5, rtol=2e-5)
    assert torch.allclose(state[3, :, 0].double().cpu(), finals[0], atol=2e-5, rtol=2e-5)
    # the engine's 16-bit output type
    half = torch.empty((total, channels), dtype=torch.bfloat16, device="cuda")
    state = start.clone().cuda()
    kernels.lru_scan(proj.cuda(), y_col, x_col, u.cuda(), gates.cuda(), channels // blocks, lam.cuda(), 8.0,
                     state, half, _ints(cu), _ints(slots), taps)
    assert torch.allclose(half.float(), out, atol=2e-2, rtol=2e-2)


def test_a_channel_that_barely_forgets_keeps_what_it_was_given():
    """A decay next to one: ``sqrt(1 - a^2)`` must not be lost to cancellation, and what the first
    token wrote is still there five hundred tokens on."""
    kernels = _kernels()
    channels, total = 64, 500
    proj = torch.ones((total, 2 * channels))
    u = torch.zeros((total, channels))
    u[0] = 3.0
    gates = torch.zeros((total, 2 * channels))
    decay = torch.full((channels,), 0.9999999)
    lam = torch.log(torch.expm1(-torch.log(decay.double()) / 8.0)).float()
    state = torch.zeros((1, channels, 1), device="cuda")
    out = torch.empty((total, channels), device="cuda")
    kernels.lru_scan(proj.cuda(), 0, channels, u.cuda(), gates.cuda(), channels, lam.cuda(), 8.0, state, out,
                     _ints([0, total]), _ints([0]), 1)
    half = torch.full((total, channels), 0.5, dtype=F64)
    states, _ = plain.gated_recurrence(u.double(), half, half, lam.double())
    expected = states * plain.gelu_tanh(torch.ones((), dtype=F64))
    assert float(expected[-1, 0]) > 1e-4
    assert torch.allclose(out.double().cpu(), expected, rtol=1e-3, atol=0)


@pytest.mark.parametrize("channels,taps", [(48, 4), (30, 1), (200, 2)])
def test_convolution_without_activation_into_float_rows(channels, taps):
    kernels = _kernels()
    g = torch.Generator().manual_seed(channels)
    lengths, slots = [9, 1, 2], [2, 0, 1]
    total = sum(lengths)
    proj = torch.randn((total, channels + 5), generator=g)
    weight = torch.randn((channels, taps), generator=g)
    bias = torch.randn(channels, generator=g)
    start = torch.randn((3, channels, taps), generator=g)
    state = start.clone().cuda()
    out = torch.empty((total, channels), device="cuda")
    cu, items = [0], []
    for n, length in enumerate(lengths):
        cu.append(cu[-1] + length)
        items += [n] * length
    kernels.conv_silu(proj.cuda(), 5, weight.cuda(), bias.cuda(), state, 1, out, _ints(items), _ints(cu),
                      _ints(slots), activation=False)
    for n in range(len(lengths)):
        rows = slice(cu[n], cu[n + 1])
        expected = plain.causal_convolution(proj[rows, 5:].double(), weight.double(), bias.double(),
                                            before=start[slots[n], :, 1:].T.double())
        assert torch.allclose(out[rows].double().cpu(), expected, atol=1e-5), n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,rot,scaling,norm", [(4, 2, 16, 8, (4.0, 16, 8.0, 1.0), True),
                                                                (3, 3, 12, 12, None, True),
                                                                (2, 1, 64, 64, (6.0, 64, 24.0, 1.0), False),
                                                                (2, 2, 128, 0, None, True),
                                                                (5, 1, 96, 32, (2.0, 40, 16.0, 2.0), True)])
def test_heads_rotated_in_halves_normed_and_stored_with_the_keys_as_values(dtype, heads, kv_heads, dim, rot,
                                                                           scaling, norm):
    from pagedserve_amd.parts.position import rotary_frequencies

    kernels = _kernels()
    g = torch.Generator().manual_seed(dim + heads)
    page_size, pages = 4, 14
    positions = [0, 1, 3, 4, 7, 40, 2]
    items = [0, 0, 0, 0, 0, 0, 1]
    tokens = len(positions)
    cache_dim = -(-dim // 16) * 16
    q_cols, k_cols = heads * dim, kv_heads * dim
    proj = torch.randn((tokens, q_cols + k_cols + 3), generator=g)
    tables = torch.full((2, 11), -1, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()
    for logical in range(11):
        tables[0, logical] = order[logical]
    tables[1, 0] = order[11]
    eps, base = 1e-5, 500.0
    raw_rot = None
    freqs, magnitude = None, 1.0
    if rot:
        raw_rot = {"dims": rot, "base": base}
        if scaling:
            raw_rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        freqs, magnitude = rotary_frequencies(rot, base, scaling)
        plain_freqs, plain_magnitude = plain.stretched_frequencies(raw_rot)
        assert torch.allclose(freqs.double(), plain_freqs, rtol=1e-12) and abs(magnitude - plain_magnitude) < 1e-12
        freqs = freqs.to(torch.float32).cuda()
    q_ref = plain.rotate_halves(proj[:, :q_cols].double().view(tokens, heads, dim), positions, raw_rot)
    k_raw = proj[:, q_cols:q_cols + k_cols].double().view(tokens, kv_heads, dim)
    k_ref = plain.rotate_halves(k_raw, positions, raw_rot)
    if norm:
        q_ref, k_ref = plain.rms_norm(q_ref, None, eps), plain.rms_norm(k_ref, None, eps)
    k_pool = torch.full((pages, kv_heads, page_size, cache_dim), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full_like(k_pool, float("nan"))
    q_out = torch.full((tokens, heads * cache_dim), float("nan"), dtype=dtype, device="cuda")
    kernels.attention_prepare_heads(proj.cuda(), (0, q_cols, q_cols), q_out, k_pool, v_pool, _ints(items),
                                    _ints(positions), tables.cuda(), heads, dim, dim, freqs=freqs, rot_dims=rot,
                                    halves=True, magnitude=magnitude, head_norm=norm, eps=eps)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    scale = 1.0 if norm else float(q_ref.abs().max())
    got_q = q_out.double().cpu().view(tokens, heads, cache_dim)
    assert torch.allclose(got_q[:, :, :dim], q_ref, atol=tol * scale, rtol=tol)
    assert float(got_q[:, :, dim:].abs().sum()) == 0.0
    for t in range(tokens):
        page, place = int(tables[items[t], positions[t] // page_size]), positions[t] % page_size
        got_k, got_v = k_pool[page, :, place].double().cpu(), v_pool[page, :, place].double().cpu()
        assert torch.allclose(got_k[:, :dim], k_ref[t], atol=tol * scale, rtol=tol)
        assert torch.allclose(got_v[:, :dim], k_raw[t], atol=tol * float(k_raw.abs().max()), rtol=tol)
        assert float(got_k[:, dim:].abs().sum()) == 0.0 and float(got_v[:, dim:].abs().sum()) == 0.0
    written = {(int(tables[items[t], positions[t] // page_size]), positions[t] % page_size) for t in range(tokens)}
    untouched = torch.isnan(k_pool.float()).all(dim=(1, 3)).cpu()
    assert int((~untouched).sum()) == len(written)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rot,rank,scaling", [(3, 8, 4, 20, (2.0, 8, 4.0, 0.5)), (1, 5, 2, 9, None),
                                                       (4, 32, 32, 96, (2.0, 32, 16.0, 2.0)), (2, 24, 48, 200, None),
                                                       (2, 16, 0, 16, None)])
def test_latent_row_normed_rotated_and_stored_and_the_queries_rotated_part(dtype, heads, dim, rot, rank, scaling):
    from pagedserve_amd.parts.position import rotary_frequencies

    kernels = _kernels()
    g = torch.Generator().manual_seed(rank)
    page_size, pages = 4, 14
    positions = [0, 1, 3, 4, 7, 40, 2]
    items = [0, 0, 0, 0, 0, 0, 1]
    tokens = len(positions)
    cache_dim = -(-(rank + rot) // 16) * 16
    q_cols = heads * (dim + rot)
    proj = torch.randn((tokens, 2 + q_cols + rank + rot + 3), generator=g)
    q_col, kv_col = 2, 2 + q_cols
    gamma = 1 + 0.3 * torch.randn(rank, generator=g)
    tables = torch.full((2, 11), -1, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()
    for logical in range(11):
        tables[0, logical] = order[logical]
    tables[1, 0] = order[11]
    eps, base = 1e-6, 250.0
    raw_rot, freqs, magnitude = None, None, 1.0
    if rot:
        raw_rot = {"dims": rot, "base": base}
        if scaling:
            raw_rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        freqs, magnitude = rotary_frequencies(rot, base, scaling)
        freqs = freqs.to(torch.float32).cuda()
    q = proj[:, q_col:q_col + q_cols].double().view(tokens, heads, dim + rot)
    q_turned = plain.rotate_halves(q[:, :, dim:], positions, raw_rot)
    down = proj[:, kv_col:kv_col + rank + rot].double()
    latent = plain.rms_norm(down[:, :rank], gamma.double(), eps)
    k_turned = plain.rotate_halves(down[:, rank:].view(tokens, 1, rot), positions, raw_rot)[:, 0]
    k_pool = torch.full((pages, 1, page_size, cache_dim), float("nan"), dtype=dtype, device="cuda")
    marker = 7.0
    q_out = torch.full((tokens, heads * cache_dim), marker, dtype=dtype, device="cuda")
    kernels.latent_prepare(proj.cuda(), q_col, kv_col, q_out, k_pool, gamma.cuda(), eps, _ints(items),
                           _ints(positions), tables.cuda(), heads, dim, rank, freqs=freqs, rot_dims=rot,
                           halves=True, magnitude=magnitude)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    got_q = q_out.double().cpu().view(tokens, heads, cache_dim)
    assert float((got_q[:, :, :rank] - marker).abs().max()) == 0.0        # left to the caller
    assert torch.allclose(got_q[:, :, rank:rank + rot], q_turned, atol=tol * 4, rtol=tol)
    assert float(got_q[:, :, rank + rot:].abs().sum()) == 0.0
    for t in range(tokens):
        page, place = int(tables[items[t], positions[t] // page_size]), positions[t] % page_size
        row = k_pool[page, 0, place].double().cpu()
        assert torch.allclose(row[:rank], latent[t], atol=tol * 4, rtol=tol)
        assert torch.allclose(row[rank:rank + rot], k_turned[t], atol=tol * 4, rtol=tol)
        assert float(row[rank + rot:].abs().sum()) == 0.0
    written = {(int(tables[items[t], positions[t] // page_size]), positions[t] % page_size) for t in range(tokens)}
    untouched = torch.isnan(k_pool.float()).all(dim=(1, 3)).cpu()
    assert int((~untouched).sum()) == len(written)


def _scores_capped(scores, cap):
    return scores if not cap else cap * torch.tanh(scores / cap)


@pytest.mark.parametrize("heads,kv_heads,dim,same,cap,window", [(12, 1, 256, True, 0.0, 0), (6, 1, 80, True, 0.0, 0),
                                                              (16, 2, 64, False, 5.0, 0), (40, 2, 32, False, 0.0, 0),
                                                              (7, 1, 128, False, 3.0, 37), (12, 2, 16, True, 0.0, 0)])
def test_single_queries_whose_heads_share_a_tile_of_keys(heads, kv_heads, dim, same, cap, window):
    """Requests of unequal length (one key, a tile's last and first key, hundreds) over pages in
    any order, every number of ranges; one loud key far back that takes most of a head's weight."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(heads * dim)
    page_size, lengths = 8, [1, 64, 65, 300, 7, 129]
    count = len(lengths)
    width = max(-(-n // page_size) for n in lengths)
    pages = count * width
    order = torch.randperm(pages, generator=g).tolist()
    tables = torch.full((count, width), -1, dtype=torch.int32)
    for n, length in enumerate(lengths):
        for logical in range(-(-length // page_size)):
            tables[n, logical] = order.pop()
    k_pool = torch.randn((pages, kv_heads, page_size, dim), generator=g).to(torch.bfloat16)
    v_pool = k_pool if same else torch.randn((pages, kv_heads, page_size, dim), generator=g).to(torch.bfloat16)
    q = torch.randn((count, heads * dim), generator=g).to(torch.bfloat16)
    # request 3: head 1 points along its third key, long
    loud_page, loud_place = int(tables[3, 0]), 2
    q.view(count, heads, dim)[3, 1] = (k_pool[loud_page, 1 // (heads // kv_heads), loud_place].float() * 3).to(torch.bfloat16)
    gate = torch.randn((count, heads), generator=g)
    scale = dim ** -0.5
    expected = torch.zeros((count, heads, dim), dtype=F64)
    for n, length in enumerate(lengths):
        first = max(0, length - window) if window else 0
        rows = [(int(tables[n, p // page_size]), p % page_size) for p in range(first, length)]
        for h in range(heads):
            kv = h // (heads // kv_heads)
            keys = torch.stack([k_pool[page, kv, place] for page, place in rows]).double()
            values = torch.stack([v_pool[page, kv, place] for page, place in rows]).double()
            scores = _scores_capped((keys @ q.view(count, heads, dim)[n, h].double()) * scale, cap)
            weights = torch.softmax(scores, 0)
            if n == 3 and h == 1 and not window and not cap:
                assert float(weights[2]) > 0.5
            expected[n, h] = (weights @ values) * torch.sigmoid(gate[n, h].double())
    dk = k_pool.cuda()
    dv = dk if same else v_pool.cuda()
    positions = _ints([length - 1 for length in lengths])
    scale_of = float(expected.abs().max())
    for splits in (1, 2, 3, 5, 64):
        out = torch.full((count, heads * dim), float("nan"), dtype=torch.bfloat16, device="cuda")
        partial = torch.full((count * heads * splits * (dim + 2),), float("nan"), device="cuda")
        for direct in (True, False):
            kernels.attention_decode_shared(q.cuda(), dk, dv, out, None if direct else _ints(list(range(count))),
                                            positions, tables.cuda(), heads, scale, splits, partial, window=window,
                                            gate=gate.cuda(), softcap=cap)
            got = out.double().cpu().view(count, heads, dim)
            assert float((got - expected).abs().max()) <= 2e-2 * scale_of, (splits, direct)
    # a list of some of the tokens: the others' rows stay as they are
    out = torch.full((count, heads * dim), 7.0, dtype=torch.bfloat16, device="cuda")
    partial = torch.empty((2 * heads * 2 * (dim + 2),), device="cuda")
    kernels.attention_decode_shared(q.cuda(), dk, dv, out, _ints(list(range(count))), positions, tables.cuda(),
                                    heads, scale, 2, partial, window=window, tok_list=_ints([3, 1]),
                                    gate=gate.cuda(), softcap=cap)
    got = out.double().cpu().view(count, heads, dim)
    for n in range(count):
        if n in (1, 3):
            assert float((got[n] - expected[n]).abs().max()) <= 2e-2 * scale_of
        else:
            assert float((got[n] - 7.0).abs().max()) == 0.0


# ---------------------------------------------------------------- whole models
def _close(rows, reference, dtype):
    """float32: every position within the tolerance.  bfloat16: the bulk of the positions within
    the tolerance and only a few per cent beyond it (a wrong key, page or state shows at every
    later position, not at a few)."""
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
@pytest.mark.parametrize("which", sorted(rezelix_models.MODELS))
def test_model_whole_decoded_in_portions_and_mixed(tmp_path, which, dtype):
    folder, raw, tensors, page_size = rezelix_models.folder_of(tmp_path, which)
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(rezelix_models.EDGE_MODELS))
def test_models_of_one_kind_of_layer_and_sizes_at_their_ends(tmp_path, which, dtype):
    folder, raw, tensors = rezelix_models.edge_folder(tmp_path, which)
    requests = _requests(raw, (70, 1, 23, 130, 2), 3)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("decoded", helpers.trace_tail_decoded(requests, tail=40)),
                        ("mixed", helpers.trace_mixed(requests, max_live=3))):
        engine = _engine(folder, dtype, 16, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        worst, scale, where = helpers.max_error(rows, reference)
        assert worst <= TOLERANCE[dtype] * scale, (which, name, worst / scale, where)
        engine.cache.check_invariants()


@pytest.mark.parametrize("which", ["A", "D"])
def test_the_stream_after_every_layer(tmp_path, which):
    """The stream after each layer, read from the engine's workspace while every block folds its
    sum into the stream itself."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model

    folder, raw, tensors, page_size = rezelix_models.folder_of(tmp_path, which)
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
    assert len(caught) == len(after) == len(raw["layers"])
    for index, (got, want) in enumerate(zip(caught, after)):
        assert torch.allclose(got, want, atol=2e-4), (index, float((got - want).abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_a_loud_key_far_back_and_at_page_borders(tmp_path, kind, dtype):
    """One key that takes nearly all the weight of the queries that match it, hundreds of tokens
    back: at a sequence's first place, at a page's last and first place (a page holds 8 tokens)
    and further in; asked for inside a prompt, at the start of a portion, and decoded one by one."""
    folder, raw, tensors = rezelix_models.loud_key_model(tmp_path, kind)
    loud, ask = rezelix_models.LOUD, rezelix_models.ASK
    g = torch.Generator().manual_seed(len(kind))

    def filler(count):
        return (torch.randint(3, raw["vocab"], (count,), generator=g)).tolist()

    requests = {}
    for place in (0, 7, 8, 21):
        requests[f"p{place}"] = filler(place) + [loud] + filler(40) + [ask] * 2 + filler(300) + [ask] + filler(4) + [ask]
    # the same tokens without the loud one: what a lost key would give
    quiet = list(requests["p7"])
    quiet[7] = 5
    reference = _reference(raw, tensors, requests)
    without = plain.forward(raw, tensors, quiet)[0]
    last = len(quiet) - 1
    assert float((reference["p7"][last] - without[last]).abs().max()) > 0.05 * float(reference["p7"].abs().max())
    traces = {"whole": helpers.trace_whole(requests),
              "decoded": helpers.trace_tail_decoded(requests, tail=320),
              "portions": helpers.trace_portions(requests, sizes=(9, 2, 3, 2, 64, 5, 200, 2, 61, 2)),
              "mixed": helpers.trace_mixed(requests, max_live=3, decode_tail=20)}
    for name, steps in traces.items():
        engine = _engine(folder, dtype, 8, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        worst, scale, where = helpers.max_error(rows, reference)
        assert worst <= TOLERANCE[dtype] * scale, (name, worst / scale, where)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "C"])
def test_long_portions_whose_recurrences_run_side_by_side(tmp_path, which, dtype):
    """Prompts of several hundred tokens whole and in long portions beside a short one: the
    recurrent layers walk such items in sixteen runs at once, the attention layers on tiles."""
    folder, raw, tensors, page_size = rezelix_models.folder_of(tmp_path, which)
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
    folder, raw, tensors, page_size = rezelix_models.folder_of(tmp_path, "C")
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
@pytest.mark.parametrize("which", ["A", "D"])
def test_long_decoding_over_many_pages_and_graph_replays(tmp_path, which, dtype):
    folder, raw, tensors, _ = rezelix_models.folder_of(tmp_path, which)
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


@pytest.mark.parametrize("which", ["A", "B", "D"])
def test_greedy_generation_through_the_scheduler(tmp_path, which):
    from pagedserve_amd.engine.llm import LLM
    from pagedserve_amd.sampling import SamplingParams

    folder, raw, tensors, page_size = rezelix_models.folder_of(tmp_path, which)
    prompts = [helpers.random_tokens(length, raw["vocab"], 40 + length) for length in (9, 1, 21, 5, 14)]
    count = 10
    expected = [plain.greedy_generate(raw, tensors, prompt, count) for prompt in prompts]
    llm = LLM(folder, dtype="float32", num_kv_pages=40, block_size=page_size, max_batch_size=3,
              eos_token_id=None, prefill_chunk_size=6, scheduling_strategy="sarathi")
    outputs = llm.generate(prompts, SamplingParams(max_new_tokens=count))
    assert [output.token_ids for output in outputs] == expected
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests
