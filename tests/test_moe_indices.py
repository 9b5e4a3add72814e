"""Expert-grouping index generation: the oracle against the reference's own test cases and a brute force
(CPU), the HIP kernels against the oracle (GPU, bit-exact: integer work)."""
import pytest
import torch

from oracle import moe_oracle as MO


def test_oracle_reference_self_test_cases():
    # cosmos_rl/policy/kernel/moe/indices.py:225-261: 4 ranks x 4 experts, 4 tokens each, alignment 32
    idx, m_sizes, m_offsets = MO.generate_permute_indices(torch.full((16,), 4, dtype=torch.int32), 4, 4, 32)
    assert m_sizes.tolist() == [32] * 4 and m_offsets.tolist() == [32, 64, 96, 128]
    assert bool((m_sizes % 32 == 0).all())
    for e in range(4):
        want = [r * 16 + e * 4 + k for r in range(4) for k in range(4)]
        assert idx[e * 32:e * 32 + 16].tolist() == want and bool((idx[e * 32 + 16:(e + 1) * 32] == -1).all())
    # :264-330: zero-token experts, alignment 8
    counts = torch.tensor([4, 0, 2, 3, 1, 0, 0, 5], dtype=torch.int32)
    idx, m_sizes, m_offsets = MO.generate_permute_indices(counts, 4, 2, 8)
    total = counts.view(2, -1).sum(0)
    assert bool((m_sizes % 8 == 0).all()) and bool((m_sizes[total == 0] >= 8).all())
    for e in range(4):
        sl = idx[int(m_offsets[e] - m_sizes[e]):int(m_offsets[e])]
        if total[e] == 0:
            assert bool((sl == -1).all()) and sl.numel() >= 8
    assert idx.tolist() == MO.brute_force(counts.tolist(), 4, 2, 8)


def test_oracle_docstring_example_and_brute_force():
    # indices.py:166-171: rank 0 [4,2,1,3], rank 1 [1,2,3,4]
    counts = [4, 2, 1, 3, 1, 2, 3, 4]
    idx, m_sizes, m_offsets = MO.generate_permute_indices(torch.tensor(counts), 4, 2, 1)
    assert m_sizes.tolist() == [5, 4, 4, 7]
    assert idx.tolist() == [0, 1, 2, 3, 10, 4, 5, 11, 12, 6, 13, 14, 15, 7, 8, 9, 16, 17, 18, 19]
    g = torch.Generator().manual_seed(0)
    for E, R, al in [(1, 1, 1), (3, 5, 4), (8, 2, 16), (128, 1, 128), (16, 8, 128)]:
        c = torch.randint(0, 40, (E * R,), generator=g)
        c[torch.rand(E * R, generator=g) < 0.3] = 0
        idx, m_sizes, m_offsets = MO.generate_permute_indices(c, E, R, al)
        assert idx.tolist() == MO.brute_force(c.tolist(), E, R, al)
        valid = idx[idx >= 0]
        assert sorted(valid.tolist()) == list(range(int(c.sum())))           # every incoming row exactly once
        assert torch.equal(m_offsets, torch.cumsum(m_sizes, 0).to(torch.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("E,R,al,hi", [(4, 4, 32, 5), (4, 2, 8, 6), (1, 1, 1, 10), (128, 1, 128, 900), (16, 8, 128, 300),
                                       (300, 7, 16, 50), (2000, 3, 8, 12)])
def test_generate_permute_indices_gpu(dev, E, R, al, hi):
    from cosmos_rl_amd.policy.kernel.moe.indices import generate_permute_indices
    g = torch.Generator().manual_seed(E * 31 + R)
    c = torch.randint(0, hi, (E * R,), generator=g, dtype=torch.int32)
    c[torch.rand(E * R, generator=g) < 0.25] = 0
    if (E, R, al) == (4, 2, 8):
        c = torch.tensor([4, 0, 2, 3, 1, 0, 0, 5], dtype=torch.int32)
    want, ws, wo = MO.generate_permute_indices(c, E, R, al)
    got, ms, mo = generate_permute_indices(c.to(dev), E, R, al)
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), want)
    assert torch.equal(ms.cpu(), ws) and torch.equal(mo.cpu(), wo)
    # with a capacity bound: no read-back, -1 past the end
    cap = int(c.sum()) + E * al + 7
    got2, _, _ = generate_permute_indices(c.to(dev), E, R, al, max_len=cap)
    assert torch.equal(got2.cpu()[:want.numel()], want) and bool((got2.cpu()[want.numel():] == -1).all())
    with pytest.raises(RuntimeError):
        generate_permute_indices(c, E, R, al, use_cpu=True)


@pytest.mark.gpu
def test_permute_tokens_feeds_the_grouped_layout(dev):
    from cosmos_rl_amd.policy.kernel.moe.indices import generate_permute_indices, permute_tokens
    E, R, al, H = 8, 2, 128, 2048
    g = torch.Generator().manual_seed(3)
    c = torch.randint(0, 200, (E * R,), generator=g, dtype=torch.int32)
    x = torch.randn(int(c.sum()), H, generator=g).to(torch.bfloat16)
    idx, m_sizes, m_offsets = generate_permute_indices(c.to(dev), E, R, al)
    out = permute_tokens(x.to(dev), idx).cpu()
    want_idx, _, _ = MO.generate_permute_indices(c, E, R, al)
    want = torch.zeros(want_idx.numel(), H, dtype=torch.bfloat16)
    want[want_idx >= 0] = x[want_idx[want_idx >= 0].long()]
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


# ---------------------------------------------------------------------------------------------
# weighted combine of expert outputs (the output side of GroupedExperts.forward)
# ---------------------------------------------------------------------------------------------
def _same_bf16(a, b):
    """bit-equal, except that a NaN matches any NaN: inf - inf has an unspecified sign and payload (x86 gives a
    negative quiet NaN, the GPU a positive one, and torch's vector and scalar casts disagree as well)"""
    a, b = a.cpu(), b.cpu()
    na, nb = torch.isnan(a), torch.isnan(b)
    return bool((na == nb).all()) and torch.equal(a.view(torch.int16)[~na], b.view(torch.int16)[~nb])


def _routing_case(seed, T, K, E, H, mask_p=0.2):
    g = torch.Generator().manual_seed(seed)
    indices = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])      # distinct experts per token
    token_mask = torch.rand(T, generator=g) >= mask_p
    weights = torch.rand(T, K, generator=g).to(torch.bfloat16)
    expert_rows = []
    for i in range(E):
        n = int(((indices == i) & token_mask[:, None]).sum())
        r = torch.randn(n, H, generator=g)
        r[torch.rand(n, H, generator=g) < 0.01] *= 1e-39                               # bf16 subnormals
        r[torch.rand(n, H, generator=g) < 0.01] *= 3e38                                # overflow to infinity
        expert_rows.append(r.to(torch.bfloat16))
    return indices, token_mask, weights, expert_rows


def _row_map_by_loops(indices, token_mask, expert_rows):
    """rows of all experts stacked in expert order; row_map[t] = the token's rows by ascending expert, -1 filled"""
    T, K = indices.shape
    starts, n = [], 0
    for r in expert_rows:
        starts.append(n)
        n += r.shape[0]
    seen = [0] * len(expert_rows)
    row_of = {}
    for t in range(T):                      # tokens ascending inside an expert: the order torch.where gives
        if not token_mask[t]:
            continue
        for k in range(K):
            e = int(indices[t, k])
            row_of[(t, k)] = starts[e] + seen[e]
            seen[e] += 1
    row_map = torch.full((T, K), -1, dtype=torch.int32)
    w_order = torch.zeros((T, K), dtype=torch.int64)
    for t in range(T):
        slots = sorted(range(K), key=lambda k: int(indices[t, k]))
        for j, k in enumerate(slots):
            row_map[t, j] = row_of.get((t, k), -1)
            w_order[t, j] = k
    return torch.cat(expert_rows) if expert_rows else None, row_map, w_order


def test_combine_oracle_pinned_by_scalar_restatement():
    from oracle import c_oracle as CO
    for seed, (T, K, E, H) in enumerate([(40, 4, 8, 16), (17, 8, 16, 24), (5, 1, 3, 8), (30, 2, 2, 8)]):
        indices, token_mask, weights, expert_rows = _routing_case(seed, T, K, E, H)
        want = MO.grouped_experts_combine(expert_rows, token_mask, weights, indices, H)
        rows, row_map, w_order = _row_map_by_loops(indices, token_mask, expert_rows)
        w = torch.gather(weights, 1, w_order)
        got = CO.combine_rows(rows.view(torch.int16).numpy().view("uint16"), row_map.numpy(),
                              w.view(torch.int16).numpy().view("uint16"), mode=0)
        assert _same_bf16(torch.from_numpy(got.view("int16")).view(torch.bfloat16), want), seed


def test_combine_closed_forms():
    from oracle import c_oracle as CO
    bf = lambda v: torch.tensor(v, dtype=torch.float32).to(torch.bfloat16)
    one = bf([[1.0] * 8])
    # one expert, weight 1: the row itself
    rows = torch.randn(3, 8, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    y = MO.grouped_experts_combine([rows], torch.ones(3, dtype=torch.bool), torch.ones(3, 1, dtype=torch.bfloat16),
                                   torch.zeros(3, 1, dtype=torch.int64), 8)
    assert torch.equal(y, rows)
    # the order of accumulation is the expert order: 1 + 2^-8 ties to 1 (twice), 2^-8 + 2^-8 + 1 = 1 + 2^-7
    small = bf([[2.0 ** -8] * 8])
    idx = torch.tensor([[0, 1, 2]])
    m, w = torch.ones(1, dtype=torch.bool), torch.ones(1, 3, dtype=torch.bfloat16)
    assert MO.grouped_experts_combine([one, small, small], m, w, idx, 8)[0, 0].item() == 1.0
    assert MO.grouped_experts_combine([small, small, one], m, w, idx, 8)[0, 0].item() == 1.0 + 2.0 ** -7
    # and the slot order of `indices` does not matter, only the expert ids do
    assert MO.grouped_experts_combine([small, small, one], m, w, torch.tensor([[2, 0, 1]]), 8)[0, 0].item() == 1.0 + 2.0 ** -7
    # the product is rounded before it is added: 1.5 * (1 + 2^-7) = 1.51171875 -> bf16 1.5078125 (tie to even)... checked in C
    r = CO.combine_rows(bf([[1.0 + 2.0 ** -7] * 8]).view(torch.int16).numpy().view("uint16"), torch.tensor([[0]], dtype=torch.int32).numpy(),
                        bf([[1.5]]).view(torch.int16).numpy().view("uint16"), mode=0)
    want = (bf([1.0 + 2.0 ** -7]) * bf([1.5]))
    assert int(r[0, 0]) == int(want.view(torch.int16).item()) & 0xFFFF
    # fp32 mode: nothing is rounded until the end -> 1 + 2^-8 + 2^-8 = 1 + 2^-7 whatever the order
    rows3 = torch.cat([one, small, small]).view(torch.int16).numpy().view("uint16")
    r = CO.combine_rows(rows3, torch.tensor([[0, 1, 2]], dtype=torch.int32).numpy(),
                        torch.ones(1, 3, dtype=torch.float32).numpy(), mode=1)
    assert r[0, 0] == int(bf([1.0 + 2.0 ** -7]).view(torch.int16).item())
    # a masked token stays zero
    y = MO.grouped_experts_combine([one[:0], one[:0]], torch.zeros(1, dtype=torch.bool), torch.ones(1, 2, dtype=torch.bfloat16),
                                   torch.tensor([[0, 1]]), 8)
    assert torch.equal(y, torch.zeros(1, 8, dtype=torch.bfloat16))


@pytest.mark.gpu
@pytest.mark.parametrize("T,K,E,H", [(300, 8, 16, 2048), (77, 4, 32, 264), (1, 1, 1, 8), (513, 6, 64, 7168), (64, 8, 8, 520)])
def test_combine_rows_gpu_bit_exact(dev, T, K, E, H):
    from oracle import c_oracle as CO
    from cosmos_rl_amd.policy.kernel.moe.moe import TokenRouting, combine_expert_outputs
    indices, token_mask, weights, expert_rows = _routing_case(T + H, T, K, E, H)
    want = MO.grouped_experts_combine(expert_rows, token_mask, weights, indices, H)
    rows, row_map, w_order = _row_map_by_loops(indices, token_mask, expert_rows)
    routing = TokenRouting(None, row_map.to(dev), w_order.to(dev), None, None)
    got = combine_expert_outputs(rows.to(dev), routing, weights.to(dev))
    assert _same_bf16(got, want) and bool(torch.isnan(want).any()) == (H >= 264)  # the big cases do hit inf - inf
    # fp32 accumulation, against the scalar restatement (small cases) and an fp64 sum (all)
    for w in (weights, weights.float() * 1.37):
        got32 = combine_expert_outputs(rows.to(dev), routing, w.to(dev), accumulate="fp32").cpu()
        ws = torch.gather(w, 1, w_order)
        if T * H <= 300 * 2048:
            wn = ws.numpy() if ws.dtype == torch.float32 else ws.view(torch.int16).numpy().view("uint16")
            ref = CO.combine_rows(rows.view(torch.int16).numpy().view("uint16"), row_map.numpy(), wn, mode=1)
            assert _same_bf16(got32, torch.from_numpy(ref.view("int16")).view(torch.bfloat16))
        safe = row_map.clamp_min(0).long()
        terms = rows.double()[safe] * ws.double()[:, :, None] * (row_map >= 0)[:, :, None]
        exact = terms.nan_to_num(0.0, 0.0, 0.0).sum(1)
        fin = torch.isfinite(got32.double()) & torch.isfinite(terms).all(1) & (exact.abs() < 1e30)
        err = (got32.double() - exact).abs()[fin]
        assert bool((err <= exact.abs()[fin] * 2.0 ** -8 + terms.nan_to_num(0.0, 0.0, 0.0).abs().sum(1)[fin] * 2.0 ** -22).all())


@pytest.mark.gpu
def test_grouped_experts_forward_routes_and_combines(dev):
    from cosmos_rl_amd.policy.kernel.moe.moe import grouped_experts_forward, route_tokens
    T, K, E, H, al = 500, 4, 12, 256, 32
    indices, token_mask, weights, _ = _routing_case(9, T, K, E, 8)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)

    class PerExpertScale:  # stands for the expert MLP: expert e multiplies its rows by (e + 2) / 4
        def execute(self, contig, m_sizes, m_offsets, module):
            ends = m_offsets.cpu().tolist()
            out = contig.clone()
            for e in range(E):
                s = ends[e] - int(m_sizes[e])
                out[s:ends[e]] = contig[s:ends[e]] * ((e + 2) / 4)
            return out

    got = grouped_experts_forward(x.to(dev), token_mask.to(dev), weights.to(dev), indices.to(dev), PerExpertScale(), None, E, al)
    expert_rows = []
    for e in range(E):
        idx, _top = torch.where((indices == e) & token_mask[:, None])
        expert_rows.append(x[idx] * ((e + 2) / 4))
    want = MO.grouped_experts_combine(expert_rows, token_mask, weights, indices, H)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    # the layout itself: every routed (token, expert) pair owns exactly one row of the expert's group
    r = route_tokens(indices.to(dev), token_mask.to(dev), E, al)
    ends = r.m_offsets.cpu().tolist()
    sizes = r.m_sizes.cpu().tolist()
    rt = r.row_tokens.cpu()
    for e in range(E):
        grp = rt[ends[e] - sizes[e]:ends[e]]
        idx, _ = torch.where((indices == e) & token_mask[:, None])
        assert grp[:idx.numel()].tolist() == idx.tolist() and bool((grp[idx.numel():] == -1).all())
        assert sizes[e] % al == 0 and sizes[e] >= al
    assert bool((rt[ends[-1]:] == -1).all())
    # nobody routed: zeros
    none = grouped_experts_forward(x.to(dev), torch.zeros(T, dtype=torch.bool, device=dev), weights.to(dev), indices.to(dev),
                                   PerExpertScale(), None, E, al)
    assert not bool(none.any())


@pytest.mark.gpu
def test_combine_rows_slot_limits(dev):
    """64 slots per token (the most the kernel takes), no slot at all (zeros), and indices no source row has"""
    from cosmos_rl_amd import _lib
    from cosmos_rl_amd.policy.kernel.moe.moe import TokenRouting, combine_expert_outputs
    from oracle import c_oracle as CO
    g = torch.Generator().manual_seed(5)
    T, K, H, R = 9, 64, 72, 700
    rows = torch.randn(R, H, generator=g).to(torch.bfloat16)
    row_map = torch.randint(-1, R, (T, K), generator=g, dtype=torch.int32)
    w = torch.rand(T, K, generator=g).to(torch.bfloat16)
    order = torch.arange(K).expand(T, K).contiguous()
    want = CO.combine_rows(rows.view(torch.int16).numpy().view("uint16"), row_map.numpy(), w.view(torch.int16).numpy().view("uint16"), 0)
    got = combine_expert_outputs(rows.to(dev), TokenRouting(None, row_map.to(dev), order.to(dev), None, None), w.to(dev))
    assert _same_bf16(got, torch.from_numpy(want.view("int16")).view(torch.bfloat16))
    # rows >= the number of source rows count as padding
    rm2 = row_map.clone()
    rm2[0, :5] = R + 3
    want2 = row_map.clone()
    want2[0, :5] = -1
    ref2 = CO.combine_rows(rows.view(torch.int16).numpy().view("uint16"), want2.numpy(), w.view(torch.int16).numpy().view("uint16"), 0)
    got2 = combine_expert_outputs(rows.to(dev), TokenRouting(None, rm2.to(dev), order.to(dev), None, None), w.to(dev))
    assert _same_bf16(got2, torch.from_numpy(ref2.view("int16")).view(torch.bfloat16))
    # no slot: zeros, and no pointer is needed for what is not read
    out = torch.full((T, H), 3.0, dtype=torch.bfloat16, device=dev)
    _lib.check(_lib.load().cfp8_combine_rows(None, H, 0, None, None, _lib.IN_BF16, T, 0, H, 0, out.data_ptr(), H,
                                             torch.cuda.current_stream().cuda_stream))
    assert not bool(out.any())


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,R", [(300, 2048, 1000), (50, 264, 333), (8, 128, 1), (1000, 7168, 513)])
def test_permute_quantize_tokens_is_gather_then_quant(dev, T, H, R):
    from cosmos_rl_amd import ops
    from cosmos_rl_amd.policy.kernel.moe.indices import permute_quantize_tokens, permute_tokens
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    x[3 % T, 5] = 300.0
    idx = torch.randint(-1, T, (R,), generator=g, dtype=torch.int32)
    idx[0] = -1
    xd = torch.zeros(T, H + 8, dtype=torch.bfloat16, device=dev)[:, :H]      # a row pitch larger than H
    xd.copy_(x)
    q1, s1 = permute_quantize_tokens(xd, idx.to(dev))
    q0, s0 = ops.groupwise_activation_quant(permute_tokens(x.to(dev), idx.to(dev)))
    assert torch.equal(q1.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(s1.view(torch.int32), s0.view(torch.int32))
    from oracle import fp8_oracle as O
    xs = torch.zeros(R, H, dtype=torch.bfloat16)
    xs[idx >= 0] = x[idx[idx >= 0].long()]
    qo, so = O.quant_group128(xs)
    assert torch.equal(q1.view(torch.uint8).cpu(), qo) and torch.equal(s1.cpu().view(torch.int32), so.view(torch.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,E,K,masked", [(512, 2048, 16, 8, False), (300, 264, 7, 3, True), (64, 128, 40, 12, True), (1000, 7168, 8, 2, False),
                                            (5, 1024, 4, 1, False)])
def test_scatter_quantize_equals_gather_quantize(dev, T, H, E, K, masked):
    """The token-side form (every token quantised once, stored to all its rows) against the row-side form and the
    oracle: same bytes and scales on every row, padding rows included; untouched where neither index names a row."""
    from cosmos_rl_amd import _lib
    from cosmos_rl_amd.policy.kernel.moe.indices import permute_quantize_tokens
    from cosmos_rl_amd.policy.kernel.moe.moe import route_tokens
    from oracle import fp8_oracle as O
    g = torch.Generator().manual_seed(T * 7 + H + K)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    x[T // 2, 3] = 250.0
    x[0] = 0
    indices = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    mask = (torch.rand(T, generator=g) > 0.2) if masked else None
    routing = route_tokens(indices.to(dev), None if mask is None else mask.to(dev), E)
    xd = torch.zeros(T, H + 16, dtype=torch.bfloat16, device=dev)[:, :H]
    xd.copy_(x)
    q1, s1 = permute_quantize_tokens(xd, routing.row_tokens, routing.row_map)
    q0, s0 = permute_quantize_tokens(xd, routing.row_tokens)
    assert torch.equal(q1.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(s1.view(torch.int32), s0.view(torch.int32))
    rt = routing.row_tokens.cpu()
    xs = torch.zeros(rt.numel(), H, dtype=torch.bfloat16)
    xs[rt >= 0] = x[rt[rt >= 0].long()]
    qo, so = O.quant_group128(xs)
    assert torch.equal(q1.view(torch.uint8).cpu(), qo) and torch.equal(s1.cpu().view(torch.int32), so.view(torch.int32))
    assert int((rt >= 0).sum()) == (T * K if mask is None else int(mask.sum()) * K)
    # straight through the C ABI with an output pitch of its own and rows that no index names: they keep their bytes
    lib = _lib.load()
    rows = rt.numel()
    src = routing.row_tokens.clone()
    rm = routing.row_map.clone()
    victim = int(torch.nonzero(rt >= 0)[0])                 # drop one routed row from both indices
    tok = int(rt[victim])
    rm[tok][rm[tok] == victim] = -1
    src[victim] = 10 ** 6                                   # neither padding nor listed by its token
    qb = torch.full((rows, H + 8), 0x5A, dtype=torch.uint8, device=dev)
    sb = torch.full((rows, (H + 127) // 128), -3.0, device=dev)
    _lib.check(lib.cfp8_scatter_quant_group128(xd.data_ptr(), xd.stride(0), T, H, rm.data_ptr(), K, src.data_ptr(), rows,
                                               qb.data_ptr(), H + 8, sb.data_ptr(), torch.cuda.current_stream().cuda_stream))
    keep = torch.ones(rows, dtype=torch.bool)
    keep[victim] = False
    assert torch.equal(qb[:, :H].cpu()[keep], qo[keep]) and torch.equal(sb.cpu().view(torch.int32)[keep], so.view(torch.int32)[keep])
    assert bool((qb[victim] == 0x5A).all()) and bool((sb[victim] == -3.0).all()) and bool((qb[:, H:] == 0x5A).all())
