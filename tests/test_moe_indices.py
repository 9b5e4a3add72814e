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
