"""Kozapel on the GPU against the plain implementation (``plain_kozapel.py``): each new kernel
or kernel option alone, then small models of several shapes stepped whole, decoded token by
token, in portions down to two tokens, and in mixed batches whose pages and slots are used again;
a key that stands out just inside and just outside a window, and far back through a latent."""

import pytest
import torch

import helpers
import kozapel_models
import plain_kozapel as plain

pytestmark = pytest.mark.gpu

F64 = torch.float64
# |engine - plain| <= TOLERANCE * max|plain logits|
TOLERANCE = {"float32": 5e-5, "bfloat16": 3e-2}


def _kernels():
    from pagedserve_amd.ops import kernels

    return kernels


def _ints(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("map_major", [True, False])
@pytest.mark.parametrize("heads,vdim,cache_dim,gated", [(4, 64, 64, True), (3, 20, 32, True), (2, 130, 144, False),
                                                        (1, 8, 16, True), (5, 256, 256, True)])
def test_difference_of_the_maps_normed_scaled_and_gated(dtype, heads, vdim, cache_dim, gated, map_major):
    kernels = _kernels()
    g = torch.Generator().manual_seed(heads * vdim)
    tokens = 11
    context = torch.randn((tokens, 2 * heads * cache_dim), generator=g).to(dtype)
    gate_rows = torch.randn((tokens, 3 + heads * vdim + 2), generator=g)
    lam, diff, eps = 0.37, 0.4, 1e-5
    out = torch.full((tokens, heads * vdim), 9.0, dtype=dtype, device="cuda")
    gate = gate_rows.cuda()[:, 3:3 + heads * vdim] if gated else None
    kernels.differential_combine(context.cuda(), torch.tensor([lam], device="cuda"), 1.0 - diff, eps, gate, out,
                                 heads, vdim, cache_dim, map_major=map_major)
    if map_major:
        maps = context.double().view(tokens, 2, heads, cache_dim)[..., :vdim]
    else:
        maps = context.double().view(tokens, heads, 2, cache_dim)[..., :vdim].transpose(1, 2)
    expected = plain.rms_norm(maps[:, 0] - lam * maps[:, 1], None, eps) * (1.0 - diff)
    if gated:
        expected = expected * torch.sigmoid(gate_rows[:, 3:3 + heads * vdim].double().view(tokens, heads, vdim))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(out.double().cpu().view(tokens, heads, vdim), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("map_major", [True, False])
@pytest.mark.parametrize("heads,vdim,cache_dim,splits", [(4, 64, 64, 5), (3, 20, 32, 1), (2, 130, 144, 64), (1, 8, 16, 9)])
def test_ranges_of_both_maps_merged_and_combined_in_one_launch(dtype, heads, vdim, cache_dim, splits, map_major):
    """Records per (token, head, key range) as the split-KV kernels leave them (accumulators, the
    running maximum in units of log 2, the sum; a range that saw no key has minus infinity and
    zeros), for a list of tokens of a larger step."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(heads + splits)
    rows, tok_list = 9, [7, 0, 3, 4]
    count = len(tok_list)
    acc = torch.randn((count, 2 * heads, splits, cache_dim), generator=g)
    top = torch.randn((count, 2 * heads, splits), generator=g) * 3
    total = torch.rand((count, 2 * heads, splits), generator=g) + 0.5
    if splits > 1:
        acc[:, :, 1], top[:, :, 1], total[:, :, 1] = 0.0, float("-inf"), 0.0
    records = torch.cat([acc, top[..., None], total[..., None]], dim=-1).contiguous()
    gate_rows = torch.randn((rows, heads * vdim + 5), generator=g)
    lam, diff, eps = 0.61, 0.3, 1e-5
    out = torch.full((rows, heads * vdim), 9.0, dtype=dtype, device="cuda")
    kernels.differential_merge(records.cuda().reshape(-1), count, splits, torch.tensor([lam], device="cuda"),
                               1.0 - diff, eps, gate_rows.cuda()[:, 2:2 + heads * vdim], out, heads, vdim,
                               cache_dim, map_major=map_major, tok_list=_ints(tok_list))
    weight = torch.exp2(top.double() - top.double().max(-1, keepdim=True).values)
    merged = ((acc.double() * weight[..., None]).sum(2) / (total.double() * weight).sum(-1)[..., None])[..., :vdim]
    maps = merged.view(count, 2, heads, vdim) if map_major else merged.view(count, heads, 2, vdim).transpose(1, 2)
    expected = plain.rms_norm(maps[:, 0] - lam * maps[:, 1], None, eps) * (1.0 - diff)
    expected = expected * torch.sigmoid(gate_rows[tok_list, 2:2 + heads * vdim].double().view(count, heads, vdim))
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    got = out.double().cpu()
    assert torch.allclose(got[tok_list].view(count, heads, vdim), expected, atol=tol, rtol=tol)
    untouched = [row for row in range(rows) if row not in tok_list]
    assert float((got[untouched] - 9.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,store", [(4, 2, 16, 24, True), (3, 3, 12, 20, True),
                                                           (4, 1, 64, 32, True), (2, 1, 8, 8, False)])
def test_two_maps_of_keys_stored_over_one_set_of_values(dtype, heads, kv_heads, dim, vdim, store):
    """The prepare launch with fewer value heads than key heads (key/value head j caches value
    head j mod the value heads), and for a layer that stores nothing."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(dim + vdim)
    page_size, pages = 4, 9
    positions, items = [0, 1, 5, 2, 11], [0, 0, 0, 1, 0]
    tokens = len(positions)
    cache_dim = -(-max(dim, vdim) // 16) * 16
    seen_heads, seen_kv = 2 * heads, 2 * kv_heads
    q_col = 1
    k_col = q_col + seen_heads * dim
    v_col = k_col + (seen_kv * dim if store else 0)
    total = v_col + (kv_heads * vdim if store else 0) + 2
    proj = torch.randn((tokens, total), generator=g)
    tables = torch.full((2, 4), -1, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()
    tables[0, :3] = torch.tensor(order[:3], dtype=torch.int32)
    tables[1, 0] = order[3]
    k_pool = torch.full((pages, seen_kv, page_size, cache_dim), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full_like(k_pool, float("nan"))
    q_out = torch.full((tokens, seen_heads * cache_dim), 5.0, dtype=dtype, device="cuda")
    kernels.attention_prepare(proj.cuda(), (q_col, k_col, v_col), q_out, k_pool, v_pool, _ints(items),
                              _ints(positions), tables.cuda(), seen_heads, dim, vdim,
                              value_heads=kv_heads, store=store)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    got_q = q_out.double().cpu().view(tokens, seen_heads, cache_dim)
    want_q = proj[:, q_col:q_col + seen_heads * dim].double().view(tokens, seen_heads, dim)
    assert torch.allclose(got_q[..., :dim], want_q, atol=tol, rtol=tol)
    assert float(got_q[..., dim:].abs().sum()) == 0.0
    if not store:
        assert bool(torch.isnan(k_pool.float()).all()) and bool(torch.isnan(v_pool.float()).all())
        return
    _two_maps_side_by_side(dtype, heads, kv_heads, dim, vdim, proj, q_col, k_col, v_col, tables, items, positions)
    keys = proj[:, k_col:k_col + seen_kv * dim].double().view(tokens, seen_kv, dim)
    values = proj[:, v_col:v_col + kv_heads * vdim].double().view(tokens, kv_heads, vdim)
    for t in range(tokens):
        page, place = int(tables[items[t], positions[t] // page_size]), positions[t] % page_size
        for head in range(seen_kv):
            row_k, row_v = k_pool[page, head, place].double().cpu(), v_pool[page, head, place].double().cpu()
            assert torch.allclose(row_k[:dim], keys[t, head], atol=tol, rtol=tol)
            assert torch.allclose(row_v[:vdim], values[t, head % kv_heads], atol=tol, rtol=tol)
            assert float(row_k[dim:].abs().sum()) == 0.0 and float(row_v[vdim:].abs().sum()) == 0.0


def _two_maps_side_by_side(dtype, heads, kv_heads, dim, vdim, proj, q_col, k_col, v_col, tables, items, positions):
    """The same projection cached the other way: a key/value head's two maps side by side in one
    cached head, every query at the places of its own map and zeros elsewhere."""
    kernels = _kernels()
    tokens, page_size, pages = len(positions), 4, 9
    cache_dim = -(-max(2 * dim, vdim) // 16) * 16
    k_pool = torch.full((pages, kv_heads, page_size, cache_dim), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full_like(k_pool, float("nan"))
    q_out = torch.full((tokens, 2 * heads * cache_dim), 5.0, dtype=dtype, device="cuda")
    kernels.attention_prepare(proj.cuda(), (q_col, k_col, v_col), q_out, k_pool, v_pool, _ints(items),
                              _ints(positions), tables.cuda(), 2 * heads, 2 * dim, vdim, query_maps=2)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    got_q = q_out.double().cpu().view(tokens, heads, 2, cache_dim)
    want_q = proj[:, q_col:q_col + 2 * heads * dim].double().view(tokens, heads, 2, dim)
    for m in range(2):
        assert torch.allclose(got_q[:, :, m, m * dim:(m + 1) * dim], want_q[:, :, m], atol=tol, rtol=tol)
        assert float(got_q[:, :, m, :m * dim].abs().sum()) == 0.0
        assert float(got_q[:, :, m, (m + 1) * dim:].abs().sum()) == 0.0
    keys = proj[:, k_col:k_col + 2 * kv_heads * dim].double().view(tokens, kv_heads, 2 * dim)
    values = proj[:, v_col:v_col + kv_heads * vdim].double().view(tokens, kv_heads, vdim)
    for t in range(tokens):
        page, place = int(tables[items[t], positions[t] // page_size]), positions[t] % page_size
        for head in range(kv_heads):
            row_k, row_v = k_pool[page, head, place].double().cpu(), v_pool[page, head, place].double().cpu()
            assert torch.allclose(row_k[:2 * dim], keys[t, head], atol=tol, rtol=tol)
            assert torch.allclose(row_v[:vdim], values[t, head], atol=tol, rtol=tol)
            assert float(row_k[2 * dim:].abs().sum()) == 0.0 and float(row_v[vdim:].abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,groups,keep", [(6, 2, 3, 2), (8, 3, 4, 3), (4, 4, 1, 1), (4, 2, 4, 2),
                                                     (72, 5, 8, 3), (64, 8, 8, 4), (130, 3, 5, 2), (3, 1, 3, 1)])
def test_sigmoid_router_with_corrections_groups_by_their_two_best_and_normed_weights(dtype, experts, top, groups, keep):
    kernels = _kernels()
    g = torch.Generator().manual_seed(experts + top)
    tokens, width = 37, 40
    x = torch.randn((tokens, width), generator=g).to(dtype)
    router = torch.randn((experts, width), generator=g) * 0.5
    correction = torch.randn(experts, generator=g) * 0.6 - 0.8      # choice scores of both signs
    spec = {"experts": experts, "top": top, "scale": 2.5, "groups": {"count": groups, "keep": keep}}
    w = {"r.router": router.double(), "r.correction": correction.double()}
    chosen, weights = plain.route(x.double(), w, "r.", spec)
    ids = torch.full((tokens, top), -1, dtype=torch.int32, device="cuda")
    got = torch.zeros((tokens, top), device="cuda")
    kernels.moe_route(x.cuda(), router.cuda(), groups, keep, top, 2.5, ids, got, sigmoid=True,
                      correction=correction.cuda(), group_top=2, normalise=True)
    ids, got = ids.cpu(), got.double().cpu()
    for t in range(tokens):
        assert sorted(ids[t].tolist()) == sorted(chosen[t]), t
        by_id = dict(zip(chosen[t], weights[t].tolist()))
        for e, weight in zip(ids[t].tolist(), got[t].tolist()):
            assert abs(weight - by_id[e]) <= 1e-5
        assert abs(float(got[t].sum()) - 2.5) <= 1e-5
    if keep < groups and top > keep:
        # the groups' limit bites, and the two best of a group decide, not its best alone
        size = experts // groups
        scores = torch.sigmoid(x.double() @ router.double().T) + correction.double()
        free = [sorted(torch.topk(scores[t], top).indices.tolist()) for t in range(tokens)]
        assert any(free[t] != sorted(chosen[t]) for t in range(tokens))
        if size > 2 and experts >= 64:
            by_best = [set(torch.topk(scores[t].view(groups, size).max(1).values, keep).indices.tolist())
                       for t in range(tokens)]
            assert any(not {e // size for e in chosen[t]} <= by_best[t] for t in range(tokens))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,inner,experts,top,tokens", [(48, 20, 5, 2, 19), (128, 96, 4, 3, 7), (44, 24, 5, 2, 3),
                                                            (64, 40, 5, 2, 150), (72, 136, 7, 1, 333),
                                                            (24, 16, 3, 2, 100), (200, 8, 2, 2, 70)])
def test_squared_relu_experts_by_rows_and_sorted_onto_the_matrix_cores(dtype, width, inner, experts, top, tokens):
    kernels = _kernels()
    g = torch.Generator().manual_seed(width + inner)
    x = torch.randn((tokens, width), generator=g).to(dtype)
    w1 = (torch.randn((experts, inner, width), generator=g) / width ** 0.5).to(dtype)
    w2 = (torch.randn((experts, width, inner), generator=g) / inner ** 0.5).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand((tokens, top), generator=g)
    y0 = torch.randn((tokens, width), generator=g)
    expected = y0.double().clone()
    for t in range(tokens):
        for j in range(top):
            e = int(ids[t, j])
            expected[t] += float(weights[t, j]) * (plain.relu2(x[t].double() @ w1[e].double().T) @ w2[e].double().T)
    tol = 1e-4 if dtype == torch.float32 else 4e-2
    y = y0.clone().cuda()
    hidden = torch.empty((tokens * top + 3, inner), dtype=dtype, device="cuda")
    kernels.moe_experts(x.cuda(), w1.cuda(), w2.cuda(), ids.cuda(), weights.cuda(), hidden, y, gated=False)
    assert torch.allclose(y.double().cpu(), expected, atol=tol, rtol=tol)
    if dtype == torch.bfloat16 and tokens * top >= kernels.MOE_GROUPED_FROM:
        assert kernels.moe_grouped_supported(dtype, width, inner)
        pairs = tokens * top
        tiles = kernels.moe_grouped_tiles(pairs, experts)
        sorted_y = y0.clone().cuda()
        kernels.moe_experts_grouped(
            x.cuda(), w1.cuda(), w2.cuda(), ids.cuda(), weights.cuda(), torch.empty_like(hidden),
            torch.empty((pairs, width), device="cuda"),
            torch.empty(tiles * kernels.MOE_TILE, dtype=torch.int32, device="cuda"),
            torch.empty(tiles, dtype=torch.int32, device="cuda"), sorted_y, gated=False)
        assert torch.allclose(sorted_y.double().cpu(), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,inner,experts,top,pieces", [(48, 20, 5, 2, 2), (128, 64, 8, 3, 1), (44, 24, 70, 2, 3)])
def test_a_shared_expert_cut_into_experts_that_every_token_uses(dtype, width, inner, experts, top, pieces):
    """The router names the pieces behind its own choices with the weight one, and the row
    kernels find them in tensors of their own: the sum is the routed experts' plus one dense
    squared-ReLU expert of ``pieces * inner`` hidden columns."""
    kernels = _kernels()
    g = torch.Generator().manual_seed(width + experts)
    tokens = 6
    x = torch.randn((tokens, width), generator=g).to(dtype)
    router = torch.randn((experts, width), generator=g) * 0.5
    correction = torch.randn(experts, generator=g) * 0.2
    w1 = (torch.randn((experts, inner, width), generator=g) / width ** 0.5).to(dtype)
    w2 = (torch.randn((experts, width, inner), generator=g) / inner ** 0.5).to(dtype)
    shared_up = (torch.randn((pieces * inner, width), generator=g) / width ** 0.5).to(dtype)
    shared_down = (torch.randn((width, pieces * inner), generator=g) / inner ** 0.5).to(dtype)
    spec = {"experts": experts, "top": top, "scale": 1.3, "groups": {"count": 1, "keep": 1}}
    chosen, weights = plain.route(x.double(), {"r.router": router.double(), "r.correction": correction.double()}, "r.", spec)
    ids = torch.full((tokens, top + pieces), -1, dtype=torch.int32, device="cuda")
    got = torch.zeros((tokens, top + pieces), device="cuda")
    kernels.moe_route(x.cuda(), router.cuda(), 1, 1, top, 1.3, ids, got, sigmoid=True, correction=correction.cuda(),
                      group_top=2, normalise=True, fixed=pieces)
    assert ids[:, top:].cpu().tolist() == [list(range(experts, experts + pieces))] * tokens
    assert torch.equal(got[:, top:].cpu(), torch.ones(tokens, pieces))
    assert [sorted(row) for row in ids[:, :top].cpu().tolist()] == [sorted(row) for row in chosen]
    y0 = torch.randn((tokens, width), generator=g)
    expected = y0.double() + plain.relu2(x.double() @ shared_up.double().T) @ shared_down.double().T
    for t in range(tokens):
        for e, weight in zip(chosen[t], weights[t].tolist()):
            expected[t] += weight * (plain.relu2(x[t].double() @ w1[e].double().T) @ w2[e].double().T)
    extra = (shared_up.cuda().view(pieces, inner, width),
             shared_down.cuda().view(width, pieces, inner).transpose(0, 1).contiguous())
    y = y0.clone().cuda()
    hidden = torch.empty((tokens * (top + pieces), inner), dtype=dtype, device="cuda")
    kernels.moe_experts(x.cuda(), w1.cuda(), w2.cuda(), ids, got, hidden, y, gated=False, extra=extra)
    tol = 1e-4 if dtype == torch.float32 else 4e-2
    assert torch.allclose(y.double().cpu(), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_with_the_tanh_form_of_gelu(dtype):
    kernels = _kernels()
    g = torch.Generator().manual_seed(2)
    both = torch.randn((9, 2 * 70), generator=g) * 2
    out = torch.empty((9, 70), dtype=dtype, device="cuda")
    kernels.silu_gate(both.cuda(), out, "gelu_tanh")
    expected = plain.gelu_tanh(both[:, :70].double()) * both[:, 70:].double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(out.double().cpu(), expected, atol=tol, rtol=tol)
    with pytest.raises(Exception):
        kernels.silu_gate(both.cuda(), out, "relu")


def test_latent_prepare_reads_queries_from_rows_of_their_own():
    kernels = _kernels()
    g = torch.Generator().manual_seed(8)
    heads, dim, rot, rank, page_size = 3, 8, 4, 20, 4
    cache_dim = 32
    positions, items = [0, 3, 4, 9], [0, 0, 0, 0]
    proj = torch.randn((4, rank + rot + 1), generator=g)
    queries = torch.randn((4, heads * (dim + rot)), generator=g)
    gamma = 1 + 0.2 * torch.randn(rank, generator=g)
    freqs = torch.tensor([70.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32)
    tables = _ints([[2, 0, 1]])
    k_pool = torch.zeros((3, 1, page_size, cache_dim), device="cuda")
    q_out = torch.zeros((4, heads * cache_dim), device="cuda")
    kernels.latent_prepare(proj.cuda(), 0, 0, q_out, k_pool, gamma.cuda(), 1e-5, _ints(items), _ints(positions),
                           tables, heads, dim, rank, freqs=freqs.cuda(), rot_dims=rot, halves=False,
                           queries=queries.cuda())
    turned = plain.rotate_neighbours(queries.double().view(4, heads, dim + rot)[..., dim:],
                                     torch.tensor(positions), rot, 70.0)
    got = q_out.double().cpu().view(4, heads, cache_dim)[..., rank:rank + rot]
    assert torch.allclose(got, turned, atol=1e-4)


# ---------------------------------------------------------------- whole models
def _close(rows, reference, dtype):
    """float32: every position within the tolerance; that pins the arithmetic.  bfloat16: a
    router's close call may go to another expert than in float64 (one position far off, the
    later ones that read its keys slightly), and the difference of two attention maps, divided
    by its own root mean square, passes rounding on enlarged.  So the bulk of the positions
    must be within a third of the tolerance, few beyond it, and very few far beyond: a wrong
    key, page or slot shows at nearly every later position, not at a few."""
    worst, scale, where = helpers.max_error(rows, reference)
    if dtype == "float32" or worst <= TOLERANCE[dtype] * scale:
        return worst <= TOLERANCE[dtype] * scale, (worst / scale, where)
    errors = sorted(float((row - reference[rid][position]).abs().max()) / scale
                    for (rid, position), row in rows.items())
    beyond = sum(error > TOLERANCE[dtype] for error in errors)
    far = sum(error > 5 * TOLERANCE[dtype] for error in errors)
    good = (errors[len(errors) // 2] <= TOLERANCE[dtype] / 3 and beyond <= max(1, len(errors) * 15 // 100)
            and far <= max(1, len(errors) // 20))
    return good, (worst / scale, where, beyond, far, len(errors))


def _requests(raw, lengths, seed):
    return {f"r{index}": helpers.random_tokens(length, raw["vocab"], seed + index)
            for index, length in enumerate(lengths)}


def _reference(raw, tensors, requests):
    return {rid: plain.forward(raw, tensors, tokens) for rid, tokens in requests.items()}


def _engine(folder, dtype, page_size, steps, max_requests=4, graphs=True):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    model, _ = load_model(folder, dtype=dtype, device="cuda")
    budget = helpers.live_token_budget(steps, round_to=page_size)
    longest = max(sum(len(e["tokens"]) for e in step["entries"]) for step in steps)
    return Engine(model, num_pages=-(-budget // page_size), page_size=page_size, max_requests=max_requests,
                  max_step_tokens=max(longest, page_size), use_graphs=graphs)


LENGTHS = (58, 1, 19, 33, 7, 2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(kozapel_models.MODELS))
def test_model_whole_decoded_in_portions_and_mixed(tmp_path, which, dtype):
    folder, raw, tensors, page_size = kozapel_models.folder_of(tmp_path, which)
    requests = _requests(raw, LENGTHS, 11)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("whole", helpers.trace_whole(requests)),
                        ("decoded", helpers.trace_tail_decoded(requests, tail=40)),
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


@pytest.mark.parametrize("which", ["A", "C", "D"])
def test_the_stream_after_every_layer(tmp_path, which):
    """The sum of the stream's copies after each layer, read from the engine's workspace while
    every block writes its last result back itself."""
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import load_model

    folder, raw, tensors, page_size = kozapel_models.folder_of(tmp_path, which)
    tokens = helpers.random_tokens(13, raw["vocab"], 4)
    _, after = plain.forward(raw, tensors, tokens, return_layers=True)
    model, _ = load_model(folder, dtype="float32", device="cuda")
    streams, width = max(raw.get("streams", 0), 1), raw["width"]
    caught = []

    def catch(h, ctx):
        caught.append(h[:ctx.tokens].double().cpu().view(ctx.tokens, streams, width).sum(1))
    for block in model.blocks:
        if hasattr(block, "finish"):
            block.takes_stream_write = False      # the model then asks every block to finish at once

            def finish(h, ctx, inner=block.finish):
                inner(h, ctx)
                catch(h, ctx)
            block.finish = finish
        else:
            def forward(h, ctx, cache, inner=block.forward):
                out = inner(h, ctx, cache)
                catch(h, ctx)
                return out
            block.forward = forward
    engine = Engine(model, num_pages=8, page_size=page_size, max_requests=2, max_step_tokens=16, use_graphs=False)
    engine.step([StepEntry("a", tokens, [])])
    assert len(caught) == len(after) == len(raw["layers"])
    for index, (got, want) in enumerate(zip(caught, after)):
        assert torch.allclose(got, want, atol=3e-4, rtol=1e-5), (index, float((got - want).abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_loud_key_just_inside_and_just_outside_the_window(tmp_path, dtype):
    """One key that takes nearly all the weight of the queries that see it.  The queries that
    match it stand at the window's last place (heard), one further (not heard), and, for the
    layer that reads the same keys under a narrower window, at that window's edge; in a prompt,
    at the start of a portion, and decoded one by one; with the key at a page's first and last
    place (a page holds 8 tokens)."""
    window = 24
    folder, raw, tensors = kozapel_models.loud_key_model(tmp_path, "attention", window=window)
    loud, ask = kozapel_models.LOUD, kozapel_models.ASK
    g = torch.Generator().manual_seed(5)

    def filler(count):
        return (torch.randint(3, raw["vocab"], (count,), generator=g)).tolist()

    requests = {}
    for place in (0, 7, 8, 21):
        # asks at distances window - 4 (inside both), window - 3 (outside the reader's),
        # window - 1 (the writer's last place), window (outside)
        tokens = filler(place) + [loud] + filler(window + 8)
        for distance in (window - 4, window - 3, window - 1, window):
            tokens[place + distance] = ask
        requests[f"p{place}"] = tokens + filler(9)
    reference = _reference(raw, tensors, requests)
    # the loud key matters where it is seen and not where it is not
    quiet = list(requests["p7"])
    quiet[7] = 5
    without = plain.forward(raw, tensors, quiet)
    scale = float(reference["p7"].abs().max())
    inside, outside = 7 + window - 1, 7 + window
    assert float((reference["p7"][inside] - without[inside]).abs().max()) > 0.05 * scale
    # (what the first layer heard travels on through the stream of later tokens only; at the
    # first place outside, the token itself sees nothing of it in the first layer)
    traces = {"whole": helpers.trace_whole(requests),
              "decoded": helpers.trace_tail_decoded(requests, tail=window + 14),
              "portions": helpers.trace_portions(requests, sizes=(9, 2, 3, 2, 11, 5, 2, 7)),
              "mixed": helpers.trace_mixed(requests, max_live=3, decode_tail=20)}
    for name, steps in traces.items():
        engine = _engine(folder, dtype, 8, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (name, what)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_loud_key_far_back_through_the_latent(tmp_path, dtype):
    folder, raw, tensors = kozapel_models.loud_key_model(tmp_path, "latent_attention")
    loud, ask = kozapel_models.LOUD, kozapel_models.ASK
    g = torch.Generator().manual_seed(6)

    def filler(count):
        return (torch.randint(3, raw["vocab"], (count,), generator=g)).tolist()

    requests = {}
    for place in (0, 7, 8):
        requests[f"p{place}"] = filler(place) + [loud] + filler(30) + [ask] * 2 + filler(260) + [ask] + filler(4) + [ask]
    quiet = list(requests["p7"])
    quiet[7] = 5
    reference = _reference(raw, tensors, requests)
    without = plain.forward(raw, tensors, quiet)
    last = len(quiet) - 1
    assert float((reference["p7"][last] - without[last]).abs().max()) > 0.05 * float(reference["p7"].abs().max())
    traces = {"whole": helpers.trace_whole(requests),
              "decoded": helpers.trace_tail_decoded(requests, tail=280),
              "portions": helpers.trace_portions(requests, sizes=(9, 2, 3, 2, 64, 5, 200, 2, 61, 2)),
              "mixed": helpers.trace_mixed(requests, max_live=3, decode_tail=20)}
    for name, steps in traces.items():
        engine = _engine(folder, dtype, 8, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (name, what)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "C"])
def test_long_prompts_whole_and_in_long_portions(tmp_path, which, dtype):
    """Prompts of several hundred tokens: the attention layers on tiles over many pages that the
    window has passed and given back, the experts sorted onto the matrix cores."""
    folder, raw, tensors, page_size = kozapel_models.folder_of(tmp_path, which)
    requests = _requests(raw, (330, 200, 9), 23)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("whole", helpers.trace_whole(requests)),
                        ("portions", helpers.trace_portions(requests, sizes=(160, 2, 131, 300))),
                        ("mixed", helpers.trace_mixed(requests, max_live=3, portion=(170, 129), decode_tail=3))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (which, name, what)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "D"])
def test_long_decoding_over_many_pages_and_graph_replays(tmp_path, which, dtype):
    folder, raw, tensors, _ = kozapel_models.folder_of(tmp_path, which)
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

    folder, raw, tensors, page_size = kozapel_models.folder_of(tmp_path, which)
    prompts = [helpers.random_tokens(length, raw["vocab"], 40 + length) for length in (9, 1, 21, 5, 14)]
    count = 10
    expected = [plain.greedy_generate(raw, tensors, prompt, count) for prompt in prompts]
    llm = LLM(folder, dtype="float32", num_kv_pages=48, block_size=page_size, max_batch_size=3,
              eos_token_id=None, prefill_chunk_size=6, scheduling_strategy="sarathi")
    outputs = llm.generate(prompts, SamplingParams(max_new_tokens=count))
    assert [output.token_ids for output in outputs] == expected
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.requests


def _drawn_configuration(seed):
    """A configuration whose every size and constant comes from a seeded generator: widths and
    vocabularies that are multiples of nothing, one to six heads on one to as many key/value
    heads, maps of 4 to 136, values of 4 to 200, windows of one token to none, readers of earlier
    layers, latents of 7 to 200, 2 to 66 experts in any grouping, no copies of the stream to five."""
    import random

    rng = random.Random(seed)
    width = rng.choice([24, 40, 72, 136, 200])
    layers, writers = [], []
    for index in range(rng.randint(2, 5)):
        kind = rng.choice(["attention", "attention", "latent_attention"])
        if kind == "attention":
            if writers and rng.random() < 0.4:
                source = rng.choice(writers)
                m = dict(layers[source]["mixer"])
                m.update(kv_from=source, diff=round(rng.uniform(0.1, 0.9), 3),
                         scale=round(m["scale"] * rng.uniform(0.7, 1.3), 4))
            else:
                kv_heads = rng.choice([1, 1, 2, 3])
                dim = rng.choice([4, 6, 8, 20, 32, 64, 100, 136])
                m = {"heads": kv_heads * rng.choice([1, 1, 2, 3]), "kv_heads": kv_heads, "dim": dim,
                     "vdim": rng.choice([4, 10, 16, 40, 64, 128, 200]),
                     "scale": round(dim ** -0.5 * rng.uniform(0.5, 2.0), 4), "diff": round(rng.uniform(0.1, 0.9), 3)}
                writers.append(index)
            window = rng.choice([1, 2, 3, 5, 8, 16, 17, 40, None])
            m.pop("mask", None)
            if window is not None:
                m["mask"] = {"size": window}
        else:
            rot_dim = rng.choice([0, 2, 8, 32])
            dim = rng.choice([3, 8, 16, 40])
            m = {"heads": rng.choice([1, 2, 5]), "dim": dim, "rot_dim": rot_dim, "vdim": rng.choice([5, 16, 48]),
                 "kv_rank": rng.choice([7, 24, 64, 200]), "q_rank": rng.choice([5, 16, 48]),
                 "scale": round((dim + rot_dim) ** -0.5 * rng.uniform(0.5, 2.0), 4)}
            if rot_dim:
                m["rot"] = {"dims": rot_dim, "base": rng.choice([10.0, 500.0, 10000.0, 1e6])}
        what = rng.choice(["none", "dense", "moe", "moe"])
        mlp = None
        if what == "dense":
            mlp = {"kind": "dense", "ff": rng.choice([10, 48, 100])}
        elif what == "moe":
            experts = rng.choice([2, 4, 6, 8, 12, 64, 66])
            count = rng.choice([g for g in (1, 2, 3, 4, 6, 8, 11) if experts % g == 0])
            keep = rng.randint(1, count)
            top = rng.randint(1, min(8, (experts // count) * keep))
            ff = rng.choice([6, 16, 40])
            mlp = {"kind": "moe", "expert": {"ff": ff},
                   "router": {"experts": experts, "top": top, "scale": round(rng.uniform(0.5, 3.0), 3),
                              "groups": {"count": count, "keep": keep}}}
            shared = rng.choice([None, ff, 2 * ff, ff + 3])
            if shared:
                mlp["shared"] = {"ff": shared}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    raw = {"architecture": "Kozapel", "vocab": rng.randint(30, 300), "width": width,
           "norm": {"eps": rng.choice([1e-5, 1e-6])}, "embedding": {"scale": round(rng.uniform(0.3, 3.0), 3)},
           "layers": layers}
    streams = rng.choice([0, 1, 2, 3, 4, 5])
    if streams:
        raw["streams"] = streams
    return raw, rng.choice([4, 8, 16])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations_in_mixed_batches(tmp_path, seed, dtype):
    """Sixteen configurations drawn from seeds, each stepped as a mixed trace of five requests
    through three slots, and its longest request decoded over a tail that passes every window,
    against the plain implementation: in 32-bit at every position, in bfloat16 (with routers
    that make no close calls) by the criterion of ``_close``."""
    import os

    raw, page_size = _drawn_configuration(seed)
    folder = os.path.join(str(tmp_path), f"drawn_{seed}")
    weights = plain.random_checkpoint(raw, 100 + seed)
    if dtype == "bfloat16":
        # a router whose choice hangs on a close call goes one way in float64 and the other in
        # bfloat16, and the position is then off by a whole expert: here the corrections lie
        # three apart (in an order of their own per layer), so that no call is close; the 32-bit
        # runs keep the drawn routers
        for name in weights:
            if name.endswith("mlp.correction"):
                order = torch.randperm(weights[name].numel(), generator=torch.Generator().manual_seed(seed))
                weights[name] = order.float() * 3.0
    tensors = kozapel_models.write_folder(folder, raw, weights)
    requests = _requests(raw, (61, 1, 17, 30, 2), 7 + seed)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("mixed", helpers.trace_mixed(requests, max_live=3, seed=seed)),
                        ("decoded", helpers.trace_tail_decoded({"r0": requests["r0"]}, tail=50))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=3)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (seed, name, what, raw)
        engine.cache.check_invariants()


def test_the_trace_program_replays_a_mixed_trace(tmp_path):
    """``bin/trace_run`` as a user calls it, on a Kozapel folder: JSON lines in, ``<step>.f32``
    files and ``done`` lines out, a pool made for the live requests only."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    folder, raw, tensors, _ = kozapel_models.folder_of(tmp_path, "C")
    requests = _requests(raw, (70, 1, 23, 40, 9), 31)
    reference = _reference(raw, tensors, requests)
    steps = helpers.trace_mixed(requests, max_live=4, seed=3)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out_dir = tmp_path / "out"
    process = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
         "--out", str(out_dir), "--max-tokens", str(helpers.live_token_budget(steps))],
        input="\n".join(json.dumps(step) for step in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert process.returncode == 0, process.stderr[-2000:]
    done = [line for line in process.stdout.splitlines() if line.startswith("done ")]
    assert done == [f"done {step['step']}" for step in steps]
    held, rows = {}, {}
    for step in steps:
        wanted = sum(len(entry["want"]) for entry in step["entries"])
        values = np.fromfile(out_dir / f"{step['step']}.f32", dtype="<f4").reshape(wanted, raw["vocab"])
        row = 0
        for entry in step["entries"]:
            start = held.get(entry["id"], 0)
            for place in entry["want"]:
                rows[(entry["id"], start + place)] = torch.from_numpy(values[row]).double()
                row += 1
            held[entry["id"]] = start + len(entry["tokens"])
    worst, scale, where = helpers.max_error(rows, reference)
    assert len(rows) == sum(len(tokens) for tokens in requests.values())
    assert worst <= TOLERANCE["float32"] * scale, (worst / scale, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(30, 44))
def test_drawn_configurations_with_long_prompts(tmp_path, seed, dtype):
    """More drawn configurations under prompts of a few hundred tokens, whole and in long
    portions beside decoded tokens of four live requests: the tiled attention kernels over windows
    of a few tokens, experts sorted onto the matrix cores at inner widths under one k tile (whose
    stand-in loads once reached behind the last expert's last row), a prompt of 70 tokens and then
    decoding."""
    import os

    raw, page_size = _drawn_configuration(seed)
    folder = os.path.join(str(tmp_path), f"drawn_{seed}")
    weights = plain.random_checkpoint(raw, 100 + seed)
    if dtype == "bfloat16":
        for name in weights:      # (no close calls: see above)
            if name.endswith("mlp.correction"):
                order = torch.randperm(weights[name].numel(), generator=torch.Generator().manual_seed(seed))
                weights[name] = order.float() * 3.0
    tensors = kozapel_models.write_folder(folder, raw, weights)
    requests = _requests(raw, (230, 130, 64, 3, 1), 7 + seed)
    reference = _reference(raw, tensors, requests)
    for name, steps in (("mixed", helpers.trace_mixed(requests, max_live=4, portion=(70, 2, 150, 9),
                                                      decode_tail=12, seed=seed)),
                        ("whole", helpers.trace_whole(requests)),
                        ("decoded", helpers.trace_tail_decoded({"r1": requests["r1"]}, tail=60))):
        engine = _engine(folder, dtype, page_size, steps, max_requests=4)
        rows = helpers.replay_in_process(engine, steps)
        good, what = _close(rows, reference, dtype)
        assert good, (seed, name, what, raw)
        engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixteen_requests_decoding_together_over_long_contexts(tmp_path, dtype):
    """Sixteen requests of two heads (four maps) decode side by side over 150 to 200 keys without
    a window: a (token, head) pair per quarter compute unit, where the split-KV kernel runs blocks
    of sixteen waves, here leaving records that the merge of both maps reads."""
    folder, raw, tensors, page_size = kozapel_models.folder_of(tmp_path, "D")
    requests = _requests(raw, tuple(150 + 3 * index for index in range(16)), 71)
    reference = _reference(raw, tensors, requests)
    tail = 6
    steps = [{"step": index, "entries": [{"id": rid, "tokens": tokens[:-tail], "want": [len(tokens) - tail - 1]}],
              "end": []} for index, (rid, tokens) in enumerate(requests.items())]
    for back in range(tail, 0, -1):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [tokens[-back]], "want": [0]}
                                                      for rid, tokens in requests.items()], "end": []})
    steps[-1]["end"] = list(requests)
    engine = _engine(folder, dtype, page_size, steps, max_requests=16)
    rows = helpers.replay_in_process(engine, steps)
    assert len(rows) == 16 * (tail + 1)
    good, what = _close(rows, reference, dtype)
    assert good, what
    engine.cache.check_invariants()
