"""Pins the torch oracle (oracle/fp8_oracle.py) without any GPU: known answers, closed forms,
brute force and invariants chosen so that a dropped term, a wrong index or a transposed operand
fails at least one of them."""
import math

import pytest
import torch

from oracle import fp8_oracle as O


def all_bf16():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


E4M3_VALUES = None


def e4m3_table():
    """All 256 codes decoded from first principles (bias 7, 3 mantissa bits, subnormal step 2^-9)."""
    global E4M3_VALUES
    if E4M3_VALUES is None:
        vals = []
        for b in range(256):
            e, m = (b >> 3) & 0xF, b & 7
            if (b & 0x7F) == 0x7F:
                v = float("nan")
            elif e == 0:
                v = m * 2.0 ** -9
            else:
                v = (8 + m) * 2.0 ** (e - 10)
            vals.append(-v if b & 0x80 else v)
        E4M3_VALUES = torch.tensor(vals, dtype=torch.float64)
    return E4M3_VALUES


def test_decode_table_matches_torch():
    tab = e4m3_table()
    got = O.e4m3_to_f32(torch.arange(256, dtype=torch.uint8)).double()
    ok = (got == tab) | (got.isnan() & tab.isnan())
    assert bool(ok.all())
    assert float(tab[0x7E]) == 448.0 and float(tab[0x01]) == 2.0 ** -9 and float(tab[0x08]) == 2.0 ** -6


KAT = [(0.0, 0x00), (-0.0, 0x80), (2.0 ** -9, 0x01), (2.0 ** -10, 0x00), (1.5 * 2.0 ** -10, 0x01),
       (3 * 2.0 ** -10, 0x02), (15 * 2.0 ** -10, 0x08), (2.0 ** -6, 0x08), (1.0, 0x38), (1.0625, 0x38),
       (1.125, 0x39), (1.1875, 0x3A), (240.0, 0x77), (416.0, 0x7D), (432.0, 0x7E), (448.0, 0x7E),
       (-448.0, 0xFE), (float("nan"), 0x7F), (float("inf"), 0x7F), (-float("inf"), 0x7F)]


def test_cast_known_answers():
    x = torch.tensor([v for v, _ in KAT], dtype=torch.float32)
    want = torch.tensor([b for _, b in KAT], dtype=torch.uint8)
    assert torch.equal(O.e4m3_bytes(x), want)


def test_cast_is_nearest_even_exhaustive():
    """Every finite bf16 pattern within +-448: the cast picks the nearest code; on a tie, the one
    with an even mantissa - checked by brute force against the decoded table."""
    x = all_bf16().float()
    x = x[torch.isfinite(x) & (x.abs() <= 448)]
    got = O.e4m3_bytes(x)
    tab = e4m3_table()
    finite_codes = torch.tensor([b for b in range(256) if (b & 0x7F) != 0x7F])
    d = (x.double()[:, None] - tab[finite_codes][None, :]).abs()
    best = d.min(dim=1).values
    gv = tab[got.long()]
    assert bool(((x.double() - gv).abs() == best).all()), "not a nearest value"
    # ties: both neighbours at the same distance -> even code chosen
    ties = (d == best[:, None]).sum(dim=1) > 1
    nz = ties & (x != 0)
    assert int(nz.sum()) > 100
    assert bool((got[nz] & 1 == 0).all()), "tie not broken to even"
    # sign preserved, including on zero results
    assert bool((((got & 0x80) != 0) == torch.signbit(x)).all())


def test_scale_closed_forms():
    s = O.scale_from_amax(torch.tensor([0.0, 1e-13, 1e-12, 448.0, 1.0, float("nan")]))
    bits = s.view(torch.int32).tolist()
    assert bits[0] == 0x2720D7C5 and bits[1] == 0x2720D7C5 and bits[2] == 0x2720D7C5
    assert float(s[3]) == 1.0
    assert bits[4] == torch.tensor(1.0 / 448.0, dtype=torch.float32).view(torch.int32).item()
    assert bits[5] == 0x7FC00000


def brute_rowwise(x):
    """Pure-python restatement on tiny inputs (independent of tensor ops)."""
    import struct
    rows = []
    scales = []
    f32 = lambda v: struct.unpack("f", struct.pack("f", v))[0]
    for r in x.float().tolist():
        amax = max(abs(v) for v in r) if r else 0.0
        sc = f32(max(amax, f32(1e-12)) / 448.0)
        scales.append(sc)
        rows.append([min(448.0, max(-448.0, f32(v / sc))) for v in r])
    return torch.tensor(rows, dtype=torch.float32), torch.tensor(scales, dtype=torch.float32)


def test_rowwise_brute_force_tiny():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(9, 24, generator=g) * torch.tensor([1e-6, 1e-3, 0.02, 1, 7, 300, 1e5, 1e20, 0]).view(9, 1)).to(torch.bfloat16)
    q, s = O.quant_rowwise(x)
    y, sc = brute_rowwise(x)
    assert torch.equal(s.view(-1).view(torch.int32), sc.view(torch.int32))
    assert torch.equal(q, O.e4m3_bytes(y))


def test_quantizer_invariants():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(2000, 256, generator=g) * torch.exp(torch.randn(2000, 1, generator=g) * 4)).to(torch.bfloat16)
    q, s = O.quant_rowwise(x)
    # every non-zero row holds a +-448 byte
    assert bool((((q & 0x7F) == 0x7E).any(dim=1)).all())
    # error at most half an e4m3 ulp of the scaled value (in units of the scale)
    y = (x.float() / s).double()
    deq = O.e4m3_to_f32(q).double()
    ulp = torch.where(deq.abs() < 2.0 ** -6, torch.full_like(deq, 2.0 ** -9),
                      2.0 ** (torch.floor(torch.log2(deq.abs().clamp_min(2.0 ** -6))) - 3))
    assert bool(((y - deq).abs() <= 0.5 * ulp * (1 + 1e-6)).all())
    # quantising the dequantised values with the same scales reproduces the bytes
    assert torch.equal(O._cast_with_scale(deq.float() * s, s), q)
    # commutes with row permutation
    perm = torch.randperm(2000, generator=g)
    qp, sp = O.quant_rowwise(x[perm])
    assert torch.equal(qp, q[perm]) and torch.equal(sp, s[perm])


def test_tensorwise_is_rowwise_of_flattened():
    x = O.make_weight((48, 80), seed=3)
    q, s = O.quant_tensorwise(x)
    q1, s1 = O.quant_rowwise(x.reshape(1, -1))
    assert torch.equal(q.reshape(1, -1), q1) and torch.equal(s, s1.reshape(1))


def test_block128_layout_and_reduction_to_tensorwise():
    """Each 128x128 block equals a tensorwise quantisation of that block alone; the scale of block
    (i, j) sits at s[i, j] - the layout weight_dequant (the in-tree inverse) reads."""
    w = O.make_weight((300, 260), seed=5)
    w = (w.float() * torch.linspace(0.1, 10, 260)[None, :]).to(torch.bfloat16)
    q, s = O.quant_block128(w)
    assert tuple(s.shape) == (3, 3)
    for i in range(3):
        for j in range(3):
            blk = w[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128]
            qb, sb = O.quant_tensorwise(blk.contiguous())
            assert torch.equal(q[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128], qb)
            assert torch.equal(s[i, j].reshape(1), sb)
    # batched form equals per-matrix form
    w3 = torch.stack([w, w.flip(0)])
    q3, s3 = O.quant_block128(w3)
    qf, sf = O.quant_block128(w.flip(0).contiguous())
    assert torch.equal(q3[0], q) and torch.equal(q3[1], qf) and torch.equal(s3[1], sf)
    # round trip through the in-tree inverse: error <= half ulp of the top binade * scale
    y = O.weight_dequant(q, s)
    se = s.repeat_interleave(128, 0).repeat_interleave(128, 1)[:300, :260]
    assert bool(((y - w.float()).abs() <= se * 16 * 1.0001).all())
    # commutes with a permutation of whole blocks
    wp = torch.cat([w[128:256], w[:128], w[256:]])
    qp, sp = O.quant_block128(wp)
    assert torch.equal(qp[:128], q[128:256]) and torch.equal(sp[0], s[1])


def test_group128_reduces_to_rowwise_per_group():
    x = O.make_activation(6, 300, seed=8)
    q, s = O.quant_group128(x)
    assert tuple(s.shape) == (6, 3)
    for g in range(3):
        sl = x[:, g * 128:(g + 1) * 128].contiguous()
        qg, sg = O.quant_rowwise(sl)
        assert torch.equal(q[:, g * 128:(g + 1) * 128], qg) and torch.equal(s[:, g:g + 1], sg)


def test_deepep_formula_matches_in_tree_statement():
    """group128_cast_deepep against a literal transcription of the expression in the reference's
    tests/test_deepep.py:75-85 evaluated step by step, and a round trip through the in-tree
    per_token_cast_back semantics."""
    x = O.make_activation(5, 200, seed=9)
    x[0] = 0
    q, s = O.group128_cast_deepep(x)
    xp = torch.zeros(5, 256, dtype=torch.bfloat16)
    xp[:, :200] = x
    v = xp.view(5, 2, 128)
    amax = v.abs().float().amax(dim=2).clamp(1e-4)
    mul = amax.reciprocal() * 448.0
    want = O.e4m3_bytes(v.float() * mul.unsqueeze(2)).view(5, 256)[:, :200]
    assert torch.equal(q, want)
    assert torch.equal(s, amax / 448.0)
    assert float(s[0, 0]) == pytest.approx(1e-4 / 448.0, rel=1e-6)
    back = O.group128_dequant(q, s)
    assert bool(((back - x.float()).abs() <= s.repeat_interleave(128, 1)[:, :200] * 16 * 1.01).all())


def test_per_token_cast_back_closed_forms():
    """per_token_cast_back (tests/test_deepep.py:86-108) pinned without retyping it: element by element against
    python floats (decode table x scale, one rounding to bf16 through struct), the E8M0 bytes against math.ldexp,
    the byte order of the packed int32 scales against an explicit little-endian pack, a ragged last group, and
    the empty case."""
    import math
    import struct
    g = torch.Generator().manual_seed(3)
    m, n = 3, 200                                     # two groups, the second 72 columns wide
    q = torch.randint(0, 256, (m, n), generator=g, dtype=torch.uint8)
    q[q == 0x7F] = 0x10
    q[q == 0xFF] = 0x90                               # no NaN bytes in the closed-form comparison
    table = [float(v) for v in O.e4m3_to_f32(torch.arange(256, dtype=torch.uint8))]

    def f32(v):                                       # a python float rounded to fp32 (overflow gives infinity)
        try:
            return struct.unpack("<f", struct.pack("<f", v))[0]
        except OverflowError:
            return math.copysign(math.inf, v)

    def bf16_rne(f):                                  # round an fp32 value to bf16, ties to even, as a python float
        if math.isinf(f):
            return f
        u = struct.unpack("<I", struct.pack("<f", f))[0]
        u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
        return struct.unpack("<f", struct.pack("<I", u))[0]

    # fp32 scales
    sc = torch.rand(m, 2, generator=g) * 0.01 + 1e-4
    got = O.per_token_cast_back(q, sc)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    for i in range(m):
        for j in range(0, n, 7):
            prod = f32(table[int(q[i, j])] * float(sc[i, j // 128]))
            assert float(got[i, j]) == bf16_rne(prod), (i, j)
    assert torch.equal(got.float(), O.group128_dequant(q, sc).to(torch.bfloat16).float())
    # packed E8M0 scales: int32 [m, 1] holds the bytes of groups 0..3, lowest byte first (the reference's view
    # needs as many scales as groups, so four groups here, the last one 72 columns wide)
    n = 456
    q = torch.randint(0, 120, (m, n), generator=g, dtype=torch.uint8)
    e = torch.tensor([[120, 131, 90, 140], [127, 100, 127, 126], [1, 254, 3, 200]], dtype=torch.uint8)
    packed = torch.tensor([[int.from_bytes(bytes(row.tolist()), "little", signed=True)] for row in e], dtype=torch.int32)
    got8 = O.per_token_cast_back(q, packed)
    for i in range(m):
        for j in range(0, n, 11):
            want = bf16_rne(f32(table[int(q[i, j])] * math.ldexp(1.0, int(e[i, j // 128]) - 127)))
            assert float(got8[i, j]) == want, (i, j)
    assert O.per_token_cast_back(torch.empty(0, 16, dtype=torch.uint8), torch.empty(0, 1)).shape == (0, 16)


def test_nan_and_inf_policy():
    x = torch.zeros(3, 16, dtype=torch.bfloat16)
    x[0, 1] = float("nan"); x[0, 2] = 1.0
    x[1, 1] = float("inf"); x[1, 2] = -5.0; x[1, 3] = -float("inf")
    q, s = O.quant_rowwise(x)
    assert int(s.view(torch.int32)[0]) == 0x7FC00000 and set(q[0].tolist()) == {0x7F}
    assert math.isinf(float(s[1])) and int(q[1, 1]) == 0x7F and int(q[1, 3]) == 0x7F
    assert int(q[1, 2]) == 0x80 and int(q[1, 0]) == 0x00      # finite / inf = signed zero
    assert int(s.view(torch.int32)[2]) == 0x2720D7C5


def test_scaled_mm_rowwise_closed_forms():
    g = torch.Generator().manual_seed(2)
    M, N, K = 5, 7, 128
    qa = torch.randint(0, 0x7E, (M, K), generator=g, dtype=torch.uint8)
    qb = torch.randint(0x80, 0xFE, (N, K), generator=g, dtype=torch.uint8)
    sa = torch.rand(M, 1, generator=g) + 0.5
    sb = torch.rand(N, 1, generator=g) + 0.5
    out = O.scaled_mm_rowwise(qa, sa, qb, sb, accum=torch.float64)
    # brute-force triple loop in python floats
    tab = e4m3_table()
    for m in (0, 4):
        for n in (0, 6):
            acc = sum(float(tab[int(qa[m, k])]) * float(tab[int(qb[n, k])]) for k in range(K))
            assert float(out[m, n]) == pytest.approx(acc * float(sa[m]) * float(sb[n]), rel=1e-6)
    # transposed-operand mistake would break this asymmetric case
    assert out.shape == (M, N) and bool((out <= 0).all())
    # fp8 linear = quant + mm
    x = O.make_activation(4, 128, seed=1)
    qx, sx = O.quant_rowwise(x)
    assert torch.equal(O.fp8_linear_rowwise(x, qb, sb), O.scaled_mm_rowwise(qx, sx, qb, sb))


def test_block_and_grouped_mm_against_loops():
    g = torch.Generator().manual_seed(4)
    M, N, K, E = 6, 256, 256, 3
    qa = torch.randint(0, 0x70, (M, K), generator=g, dtype=torch.uint8)
    sa = torch.rand(M, 2, generator=g) + 0.5
    qb = torch.randint(0, 0x70, (E, N, K), generator=g, dtype=torch.uint8)
    sb = torch.rand(E, 2, 2, generator=g) + 0.5
    tab = e4m3_table()
    out = O.scaled_mm_block128(qa, sa, qb[1], sb[1], accum=torch.float64)
    m, n = 3, 200
    acc = 0.0
    for kb in range(2):
        part = sum(float(tab[int(qa[m, k])]) * float(tab[int(qb[1, n, k])]) for k in range(kb * 128, kb * 128 + 128))
        acc += part * float(sa[m, kb]) * float(sb[1, n // 128, kb])
    assert float(out[m, n]) == pytest.approx(acc, rel=1e-6)
    idx = torch.tensor([0, 0, 2, 2, -1, 1], dtype=torch.int32)
    outg = O.grouped_mm_block128(qa, sa, qb, sb, idx, accum=torch.float64)
    for r in range(M):
        e = int(idx[r])
        want = torch.zeros(N) if e < 0 else O.scaled_mm_block128(qa[r:r + 1], sa[r:r + 1], qb[e], sb[e], accum=torch.float64)[0]
        assert torch.allclose(outg[r], want, rtol=1e-6, atol=0)


def test_routing_helper():
    g = torch.Generator().manual_seed(6)
    logits = torch.rand(50, 5, generator=g)
    logits[:, 2] = -1
    tok, idx, sizes, offs = O.route_topk_contiguous(logits, 2, 16)
    assert int(sizes[2]) == 16 and int((idx == 2).sum()) == 0       # empty expert clamped up to the alignment
    assert bool((sizes % 16 == 0).all()) and int(offs[-1]) == tok.numel()
    assert int((tok >= 0).sum()) == 100
    for e in range(5):
        rows = (idx == e).nonzero().flatten()
        if rows.numel():
            assert int(rows[0]) == int(offs[e] - sizes[e])         # valid rows first in the group
            assert bool((torch.topk(logits[tok[rows]], 2).indices == e).any(dim=1).all())


def test_qwen_shapes_total():
    assert O.qwen25_7b_numel() == 7_070_285_824
    assert sum(n for _, _, n in O.QWEN25_7B_LINEAR_SHAPES) == 197


def test_calc_diff_closed_forms():
    """tests/test_deepep.py:62-67: zero for identical tensors, symmetric, and 1 - 2ab/(a^2+b^2) for constants."""
    x = torch.tensor([0.5, -2.0, 3.0])
    assert O.calc_diff(x, x) == 0.0
    y = torch.tensor([0.25, -1.0, 2.0])
    assert O.calc_diff(x, y) == O.calc_diff(y, x)
    a, b = torch.full((4,), 1.0), torch.full((4,), 3.0)     # shifted to 2 and 4
    assert abs(O.calc_diff(a, b) - (1 - 2 * 2 * 4 / (4 + 16))) < 1e-15
