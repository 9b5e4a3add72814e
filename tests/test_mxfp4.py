"""MXFP4 weight quantisation.  The oracle restates the published algorithm of triton_kernels'
downcast_to_mxfp (the package itself is absent: parity with the reference is unpinned); what is checked
here is the oracle against the mathematics (CPU) and the HIP kernel against the oracle, bit for bit (GPU)."""
import math

import numpy as np
import pytest
import torch

from oracle import mxfp4_oracle as MX


def _nearest_ties_away(v: float) -> int:
    """code of the e2m1 value nearest to v, ties to the larger magnitude, saturating: brute force"""
    a = min(abs(v), 6.0)
    best, best_d = 0, None
    for code, val in enumerate(MX.E2M1_VALUES.tolist()):
        d = abs(a - val)
        if best_d is None or d < best_d or (d == best_d and val > MX.E2M1_VALUES[best]):
            best, best_d = code, d
    return best | (8 if math.copysign(1.0, v) < 0 else 0)


def test_e2m1_rounding_against_brute_force():
    g = np.random.default_rng(0)
    ties = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    vals = [0.0, -0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, 7.0, 100.0, 1e-30, 0.1249, 0.125, 0.2499999]
    vals += ties + [np.nextafter(np.float32(t), np.float32(0)) for t in ties] + [np.nextafter(np.float32(t), np.float32(9)) for t in ties]
    vals += g.uniform(0, 6.5, 4000).tolist() + (2.0 ** g.uniform(-20, 3, 2000)).tolist()
    v = np.array(vals + [-x for x in vals], dtype=np.float32)
    got = MX.e2m1_codes(v)
    want = np.array([_nearest_ties_away(float(x)) for x in v], dtype=np.uint8)
    assert np.array_equal(got, want)
    assert MX.e2m1_codes(np.array([2.5, -2.5, 0.25], np.float32)).tolist() == [5, 13, 1]   # ties go up: 3, -3, 0.5


def test_scale_is_the_next_power_of_two_of_amax_over_6():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(64, 32, generator=g) * torch.exp(torch.randn(64, 1, generator=g) * 8)).to(torch.bfloat16)
    x[0] = 0                                    # an all-zero block: scale byte 0, all codes 0
    x[1, :] = 0.0
    x[1, 3] = 6.0                               # amax / 6 = 1 exactly: exponent 0, no rounding up
    x[2, 5] = -3.0 * 2 ** 10
    x[2, :5] = 0
    x[2, 6:] = 0                                # amax / 6 = 2^9 exactly
    q, s = MX.downcast(x)
    assert s.shape == (64, 1) and q.shape == (64, 16)
    assert s[0].item() == 0 and not bool(q[0].any())
    assert s[1].item() == 127 and s[2].item() == 127 + 9
    for r in range(3, 64):
        amax = float(x[r].float().abs().max())
        m, e = math.frexp(amax / 6.0)           # amax / 6 = m * 2^e, 0.5 <= m < 1; float64 is exact enough off the powers of two
        want = e - 1 if m == 0.5 else e
        assert s[r].item() - 127 == want, (r, amax)
    # by construction nothing saturates, and the largest element of a block lands on code 4..7 (|q| in (3, 6])
    codes = torch.stack([q & 0xF, q >> 4], -1).reshape(64, 32) & 7
    assert bool((codes[3:].max(dim=1).values >= 5).all())


def test_packing_order_and_round_trip_bound():
    x = torch.zeros(1, 32, dtype=torch.bfloat16)
    x[0, 0], x[0, 1], x[0, 31] = 6.0, -1.0, 0.5
    q, s = MX.downcast(x)
    assert s.item() == 127 and q[0, 0].item() == (7 | (0xA << 4)) and q[0, 15].item() == (1 << 4)  # even element low
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(37, 96, generator=g) * 0.02).to(torch.bfloat16)
    q, s = MX.downcast(x)
    y = MX.upcast(q, s)
    scale = torch.from_numpy(np.ldexp(1.0, s.numpy().astype(np.int64) - 127)).repeat_interleave(32, dim=1)
    # neighbouring e2m1 values are at most 2 apart (4 -> 6): error <= 1 in units of the scale, 0.25 below 2
    err = (y.double() - x.double()).abs() / scale
    assert float(err.max()) <= 1.0 and float(err[(x.double().abs() / scale) <= 2].max()) <= 0.25


def _cases(dev):
    g = torch.Generator().manual_seed(3)
    yield (torch.randn(3, 64, 96, generator=g) * 0.02).to(torch.bfloat16)
    w = torch.randn(130, 2880, generator=g) * torch.exp(torch.randn(130, 1, generator=g) * 4)
    w[5] = 0
    w[6, :32] = 0
    yield w.to(torch.bfloat16)
    # every multiple of 1/16 up to 6 (all the ties and all the representable values) and its two bf16 neighbours,
    # both signs, in blocks whose first element 6 * 2^k fixes the scale at 2^k
    base = torch.arange(0, 97, dtype=torch.float32) / 16
    bits = base.to(torch.bfloat16).view(torch.int16).to(torch.int32)
    near = torch.cat([bits, bits + 1, (bits - 1).clamp_min(0)]).to(torch.int16).view(torch.bfloat16).float()
    near = near[near <= 6.0]
    vals = torch.cat([near, -near])
    vals = torch.cat([vals, torch.zeros((-vals.numel()) % 31)]).reshape(-1, 31)
    rows = [torch.cat([torch.full((vals.shape[0], 1), 6.0), vals], 1) * 2.0 ** k for k in (-130, -126, -20, -1, 0, 3, 60, 120)]
    yield torch.cat(rows).to(torch.bfloat16)
    yield (torch.randn(1, 32, generator=g)).to(torch.bfloat16)


@pytest.mark.gpu
def test_quant_mxfp4_gpu_bit_exact(dev):
    from cosmos_rl_amd import ops
    for x in _cases(dev):
        q, s = ops.quant_mxfp4(x.to(dev))
        wq, ws = MX.downcast(x)
        assert torch.equal(s.cpu(), ws), tuple(x.shape)
        bad = (q.cpu() != wq).nonzero()
        assert bad.numel() == 0, (tuple(x.shape), bad[:5].tolist())


@pytest.mark.gpu
def test_mxfp4_mirrors_and_pitches(dev):
    from cosmos_rl_amd import _lib, ops
    from cosmos_rl_amd.rollout.vllm_rollout.monkey_patch_for_mxfp4 import mxfp4_quantization, quantize_mx4
    g = torch.Generator().manual_seed(4)
    w = (torch.randn(4, 48, 64, generator=g) * 0.05).to(torch.bfloat16)           # [experts, out, in]
    q, s = mxfp4_quantization(w.to(dev))
    wq, ws = MX.downcast(w)
    assert torch.equal(q.cpu(), wq) and torch.equal(s.cpu(), ws)
    # the reference's call shape: [experts, in, out] quantised along axis 1
    q1, s1 = quantize_mx4(w.transpose(1, 2).contiguous().to(dev))
    assert torch.equal(q1.cpu(), wq.transpose(1, 2)) and torch.equal(s1.cpu(), ws.transpose(1, 2))
    # padded pitches through the C ABI: bytes outside the rows stay untouched
    x = w.reshape(-1, 64).to(dev)
    xp = torch.zeros(x.shape[0], 72, dtype=torch.bfloat16, device=dev)
    xp[:, :64] = x
    qp = torch.full((x.shape[0], 40), 0xEE, dtype=torch.uint8, device=dev)
    sp = torch.full((x.shape[0], 5), 0xEE, dtype=torch.uint8, device=dev)
    _lib.check(_lib.load().cfp8_quant_mxfp4(xp.data_ptr(), x.shape[0], 64, 72, qp.data_ptr(), 40, sp.data_ptr(), 5,
                                            torch.cuda.current_stream().cuda_stream))
    assert torch.equal(qp[:, :32].cpu(), wq.reshape(-1, 32)) and bool((qp[:, 32:] == 0xEE).all())
    assert torch.equal(sp[:, :2].cpu(), ws.reshape(-1, 2)) and bool((sp[:, 2:] == 0xEE).all())
    with pytest.raises(ValueError):
        ops.quant_mxfp4(torch.zeros(4, 48, dtype=torch.bfloat16, device=dev))


def test_gemm_oracle_against_loops():
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(16, 64, generator=g) * 0.1).to(torch.bfloat16)
    wq, ws = MX.downcast(w)
    xq = (torch.randn(3, 64, generator=g) * 40).to(torch.float8_e4m3fn)
    sx = torch.tensor([0.5, 0.013, 3.0])
    got = MX.gemm(xq, sx, wq, ws)
    vals = MX.E2M1_VALUES.tolist()
    for m in range(3):
        for n in range(16):
            acc = 0.0
            for k in range(64):
                byte = int(wq[n, k // 2])
                code = (byte >> 4) if k % 2 else (byte & 0xF)
                v = vals[code & 7] * (-1.0 if code & 8 else 1.0) * 2.0 ** (int(ws[n, k // 32]) - 127)
                acc += float(xq[m, k].float()) * v
            assert got[m, n].item() == pytest.approx(acc * float(sx[m]), rel=1e-12, abs=1e-300)


def _mx_weights(g, *shape, spread=2.0):
    w = torch.randn(*shape, generator=g) * 0.05 * torch.exp(torch.randn(*shape[:-1], 1, generator=g) * spread)
    return MX.downcast(w.to(torch.bfloat16))


def _fp8_rows(g, M, K):
    x = torch.randn(M, K, generator=g) * torch.exp(torch.randn(M, 1, generator=g))
    amax = x.abs().amax(dim=1, keepdim=True).clamp_min(1e-12)
    s = (amax / 448.0).float()
    return (x / s).to(torch.float8_e4m3fn), s.reshape(-1)


def _rel(got, want):
    return float((got.double() - want).norm() / want.norm().clamp_min(1e-300))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 16, 32), (5, 48, 96), (16, 64, 128), (17, 80, 160), (33, 128, 2880), (64, 256, 512),
                                   (100, 272, 896), (128, 128, 128), (129, 144, 64), (300, 512, 2880), (1000, 400, 1056),
                                   (16, 80, 2880), (2, 528, 4256), (9, 2064, 3584),
                                   (17, 96, 128), (24, 8400, 2880), (31, 176, 6304), (50, 8272, 896), (64, 320, 4096), (64, 18944, 3584), (4096, 8192, 288), (4000, 8208, 160),
                                   (2048, 4096, 384), (4096, 8192, 128), (2048, 4096, 256), (2560, 3328, 1152),
                                   (2000, 2064, 2880), (1025, 4112, 160), (8192, 272, 128), (130, 16400, 416), (1024, 4096, 3552),
                                   (4000, 4112, 160), (8192, 2544, 416), (4100, 4096, 2880),
                                   (100, 10480, 2880), (128, 16400, 160), (17, 12272, 4256), (65, 10256, 128), (90, 18944, 3584), (40, 20016, 1184),
                                   # 272 and 320 tiles of 256 x 256: one full round, the last tile-columns as a second launch
                                   (4096, 4352, 256), (2048, 10240, 384)])
def test_gemm_mxfp4_against_oracle(dev, M, N, K):
    """fp32 output within 1e-4 (relative Frobenius; the fp32 accumulation of the matrix pipe) of the exact sum, bf16 output within 1e-3 of the bf16-rounded
    exact sum; rows and columns beyond M and N of a padded output stay untouched."""
    from cosmos_rl_amd import ops
    g = torch.Generator().manual_seed(M * 7919 + N * 31 + K)
    wq, ws = _mx_weights(g, N, K)
    xq, sx = _fp8_rows(g, M, K)
    want = MX.gemm(xq, sx, wq, ws)
    got = ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), torch.float32)
    assert _rel(got.cpu(), want) <= 1e-4
    got16 = ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), torch.bfloat16)
    assert _rel(got16.cpu().float(), want.float().to(torch.bfloat16).double()) <= 1e-3
    assert torch.equal(got.to(torch.bfloat16), got16)          # the two epilogues round the same accumulators


@pytest.mark.gpu
def test_gemm_mxfp4_random_shapes_every_kernel_form(dev):
    """Seeded random shapes across the dispatch boundaries (1..16 tokens, 17..64, small register-staged tiles, ragged
    and aligned direct-to-LDS tiles, K with and without a partial last step), fp32 output against the exact sum."""
    from cosmos_rl_amd import ops
    rng = np.random.default_rng(11)
    shapes = []
    for _ in range(8):
        shapes.append((int(rng.integers(1, 17)), 16 * int(rng.integers(1, 600)), 32 * int(rng.integers(1, 140))))
        shapes.append((int(rng.integers(17, 65)), 16 * int(rng.integers(1, 600)), 32 * int(rng.integers(1, 140))))
        shapes.append((int(rng.integers(65, 700)), 16 * int(rng.integers(1, 80)), 32 * int(rng.integers(1, 100))))
        shapes.append((int(rng.integers(700, 5000)), 16 * int(rng.integers(100, 400)), 32 * int(rng.integers(4, 40))))
    shapes += [(256 * int(rng.integers(8, 20)), 256 * int(rng.integers(16, 30)), 128 * int(rng.integers(1, 8))) for _ in range(3)]
    g = torch.Generator().manual_seed(12)
    for M, N, K in shapes:
        wq, ws = _mx_weights(g, N, K)
        xq, sx = _fp8_rows(g, M, K)
        got = ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), torch.float32)
        assert _rel(got.cpu(), MX.gemm(xq, sx, wq, ws)) <= 1e-4, (M, N, K)


@pytest.mark.gpu
@pytest.mark.parametrize("M", [8, 160])
def test_gemm_mxfp4_one_hot_is_exact(dev, M):
    """Row m of the activations is 1.0 at k = m (mod K): the output is the weight value itself, so the nibble
    order, the lane that owns each block of 32 and the scale byte it is paired with are all pinned bit for bit."""
    from cosmos_rl_amd import ops
    K, N = 160, 192
    g = torch.Generator().manual_seed(6)
    wq, ws = _mx_weights(g, N, K, spread=6.0)
    x = torch.zeros(M, K)
    ks = [(m * 37) % K for m in range(M)]
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    xq = x.to(torch.float8_e4m3fn)
    sx = torch.ones(M)
    got = ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), torch.float32).cpu()
    want = MX.upcast(wq, ws)[:, ks].t().contiguous()
    assert torch.equal(got, want)


@pytest.mark.gpu
def test_gemm_mxfp4_grouped(dev):
    """Groups of 128-aligned rows, one of them empty, padding rows (index -1) left untouched."""
    from cosmos_rl_amd import ops
    g = torch.Generator().manual_seed(7)
    E, N, K = 4, 208, 352
    counts = [200, 0, 128, 77]
    wq, ws = _mx_weights(g, E, N, K)
    idx, rows = [], 0
    for e, c in enumerate(counts):
        padded = -(-c // 128) * 128
        idx += [e] * c + [-1] * (padded - c)
        rows += padded
    m_indices = torch.tensor(idx, dtype=torch.int32)
    xq, sx = _fp8_rows(g, rows, K)
    out = torch.full((rows, N), 7.0, dtype=torch.bfloat16, device=dev)
    ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), m_indices=m_indices.to(dev), out=out)
    out = out.cpu()
    for e in range(E):
        sel = m_indices == e
        if not bool(sel.any()):
            continue
        want = MX.gemm(xq[sel], sx[sel], wq[e], ws[e])
        assert _rel(out[sel].float(), want.float().to(torch.bfloat16).double()) <= 1e-3, e
    assert bool((out[m_indices < 0] == 7.0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("N,K,counts", [(1040, 2880, [300, 0, 128, 77, 1000, 513]),          # 128 x 256 tiles
                                        (1520, 1120, [3000, 0, 128, 77, 5000, 2600])])       # 128 x 512 tiles
def test_gemm_mxfp4_grouped_large(dev, N, K, counts):
    """Enough tiles for the direct-to-LDS grouped kernels: a last K step of 64 or 96, N with a ragged last tile,
    an empty expert, experts whose last 128 rows are partly padding; the padding keeps its bytes, bf16 and fp32."""
    from cosmos_rl_amd import ops
    g = torch.Generator().manual_seed(10)
    E = len(counts)
    wq, ws = _mx_weights(g, E, N, K)
    idx, rows = [], 0
    for e, c in enumerate(counts):
        padded = -(-c // 128) * 128
        idx += [e] * c + [-1] * (padded - c)
        rows += padded
    m_indices = torch.tensor(idx, dtype=torch.int32)
    xq, sx = _fp8_rows(g, rows, K)
    for dt, tol in ((torch.bfloat16, 1e-3), (torch.float32, 1e-4)):
        out = torch.full((rows, N), 7.0, dtype=dt, device=dev)
        ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev), ws.to(dev)), m_indices=m_indices.to(dev), out=out)
        out = out.cpu()
        for e in range(E):
            sel = m_indices == e
            if not bool(sel.any()):
                continue
            want = MX.gemm(xq[sel], sx[sel], wq[e], ws[e])
            ref = want.float().to(torch.bfloat16).double() if dt == torch.bfloat16 else want
            assert _rel(out[sel].float(), ref) <= tol, (e, dt)
        assert bool((out[m_indices < 0] == 7.0).all())


@pytest.mark.gpu
def test_gemm_mxfp4_pitches_and_errors(dev):
    from cosmos_rl_amd import _lib, ops
    g = torch.Generator().manual_seed(8)
    M, N, K = 70, 96, 224
    wq, ws = _mx_weights(g, N, K)
    xq, sx = _fp8_rows(g, M, K)
    want = MX.gemm(xq, sx, wq, ws)
    # padded pitches of every operand; the output's padding columns keep their bytes
    xp = torch.zeros(M, 256, dtype=torch.uint8, device=dev); xp[:, :K] = xq.view(torch.uint8).to(dev)
    wp = torch.full((N, 128), 0x77, dtype=torch.uint8, device=dev); wp[:, :K // 2] = wq.to(dev)
    sp = torch.full((N, 9), 0xFF, dtype=torch.uint8, device=dev); sp[:, :K // 32] = ws.to(dev)
    out = torch.full((M, 100), -3.0, dtype=torch.float32, device=dev)
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.cfp8_gemm_mxfp4(xp.data_ptr(), 256, sx.to(dev).data_ptr(), wp.data_ptr(), 128, sp.data_ptr(), 9, None, 0,
                                   out.data_ptr(), 100, _lib.OUT_F32, M, N, K, st))
    assert _rel(out[:, :N].cpu(), want) <= 1e-4 and bool((out[:, N:] == -3.0).all())
    ptr = out.data_ptr()
    assert lib.cfp8_gemm_mxfp4(ptr, 64, ptr, ptr, 32, ptr, 2, None, 0, ptr, 16, _lib.OUT_F32, 4, 16, 48, st) == _lib.EINVAL    # K % 32
    assert lib.cfp8_gemm_mxfp4(ptr, 64, ptr, ptr, 32, ptr, 2, None, 0, ptr, 24, _lib.OUT_F32, 4, 24, 64, st) == _lib.EINVAL    # N % 16
    assert lib.cfp8_gemm_mxfp4(ptr, 64, ptr, ptr, 24, ptr, 2, None, 0, ptr, 16, _lib.OUT_F32, 4, 16, 64, st) == _lib.EINVAL    # ld_w
    assert lib.cfp8_gemm_mxfp4(ptr, 64, ptr, ptr, 32, ptr, 2, None, 3, ptr, 16, _lib.OUT_F32, 4, 16, 64, st) == _lib.EINVAL    # groups without indices
    assert lib.cfp8_gemm_mxfp4(ptr, 64, ptr, ptr, 32, ptr, 2, ptr, 2, ptr, 16, _lib.OUT_F32, 100, 16, 64, st) == _lib.EINVAL   # grouped M % 128
    assert lib.cfp8_gemm_mxfp4(None, 64, None, None, 32, None, 2, None, 0, None, 16, _lib.OUT_F32, 0, 16, 64, st) == 0
    with pytest.raises(ValueError):
        ops.gemm_mxfp4((xq.to(dev), sx.to(dev)), (wq.to(dev)[:, :-1], ws.to(dev)))


@pytest.mark.gpu
def test_linear_mxfp4_end_to_end(dev):
    """bf16 activations -> per-token FP8 -> MXFP4 product, against the same chain in the oracles."""
    from cosmos_rl_amd import ops
    from oracle import fp8_oracle as O
    g = torch.Generator().manual_seed(9)
    w = (torch.randn(320, 2880, generator=g) * 0.03).to(torch.bfloat16)
    x = (torch.randn(2, 45, 2880, generator=g)).to(torch.bfloat16)
    wq, ws = ops.quant_mxfp4(w.to(dev))
    y = ops.linear_mxfp4(x.to(dev), (wq, ws))
    assert y.shape == (2, 45, 320) and y.dtype == torch.bfloat16
    xq, sx = O.quant_rowwise(x.reshape(-1, 2880))
    want = MX.gemm(xq.view(torch.float8_e4m3fn), sx.reshape(-1), *MX.downcast(w)).reshape(2, 45, 320)
    assert _rel(y.cpu().float(), want.float().to(torch.bfloat16).double()) <= 1e-3
    # and the quantisation error of the whole chain against the unquantised product stays at MXFP4's level
    exact = x.double() @ w.double().t()
    assert _rel(y.cpu().float(), exact) < 0.15


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 96, 96), (1, 18944, 3584), (2, 320, 2880), (3, 5760, 2880), (4, 528, 4096), (4, 64, 32),
                                   (5, 320, 2880), (2, 272, 4128), (40, 528, 2880), (300, 512, 1056)])
def test_linear_mxfp4_equals_quantise_then_gemm(dev, M, N, K):
    """The entry point that starts from bf16 activations - one launch up to 4 tokens and K <= 4096, the rowwise
    quantiser into the workspace otherwise - gives the bits of the two separate calls, bf16 and fp32 output."""
    from cosmos_rl_amd import ops
    from oracle import fp8_oracle as O
    g = torch.Generator().manual_seed(M * 131 + N + K)
    wq, ws = _mx_weights(g, N, K)
    x = (torch.randn(M, K, generator=g) * torch.exp(torch.randn(M, 1, generator=g))).to(torch.bfloat16)
    x[0, : min(K, 40)] = 0
    xd, wd, sd = x.to(dev), wq.to(dev), ws.to(dev)
    q, s = ops.quant_rowwise(xd)
    oq, os_ = O.quant_rowwise(x)
    assert torch.equal(q.view(torch.uint8).cpu(), oq) and torch.equal(s.cpu(), os_)
    for dt in (torch.bfloat16, torch.float32):
        want = ops.gemm_mxfp4((q, s), (wd, sd), dt)
        got = ops.linear_mxfp4(xd, (wd, sd), dt)
        assert torch.equal(got, want), dt
    assert _rel(ops.linear_mxfp4(xd, (wd, sd), torch.float32).cpu(), MX.gemm(oq.view(torch.float8_e4m3fn), os_.reshape(-1), wq, ws)) <= 1e-4


@pytest.mark.gpu
def test_linear_mxfp4_errors(dev):
    from cosmos_rl_amd import _lib
    lib = _lib.load()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
    ptr, st = buf.data_ptr(), torch.cuda.current_stream().cuda_stream
    assert lib.cfp8_linear_mxfp4(ptr, 64, ptr, 32, ptr, 2, ptr, 16, _lib.OUT_BF16, 2, 16, 48, None, 0, st) == _lib.EINVAL      # K % 32
    assert lib.cfp8_linear_mxfp4(ptr, 60, ptr, 32, ptr, 2, ptr, 16, _lib.OUT_BF16, 2, 16, 64, None, 0, st) == _lib.EINVAL      # ld_x
    assert lib.cfp8_linear_mxfp4(ptr, 64, ptr, 32, ptr, 2, ptr, 16, _lib.OUT_BF16, 8, 16, 64, None, 0, st) == _lib.EWORKSPACE  # 8 tokens need one
    assert lib.cfp8_linear_mxfp4(ptr, 64, ptr, 32, ptr, 2, ptr, 16, _lib.OUT_BF16, 2, 16, 64, None, 0, st) == 0                # 2 tokens do not
    assert lib.cfp8_linear_mxfp4(None, 64, None, 32, None, 2, None, 16, _lib.OUT_BF16, 0, 16, 64, None, 0, st) == 0

