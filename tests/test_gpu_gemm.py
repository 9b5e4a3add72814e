"""Parity of the FP8 MFMA GEMMs with the oracle (dequantised matmul of the same quantised
operands, accumulated in fp64).  Tolerance: relative Frobenius error <= 1e-3 (TOL) on the
fp32-epilogue output, and bf16(kernel) against bf16(oracle) to the same bar.  The matrix core
sums the 128 products of one instruction with less than fp32 precision (observed ~2e-5
relative), so TIGHT = 1e-4 is asserted as a regression bar well inside TOL.  All calls go
through the C ABI."""
import pytest
import torch

from oracle import fp8_oracle as O
from cosmos_rl_amd import ops

pytestmark = pytest.mark.gpu
TOL = 1e-3
TIGHT = 1e-4


def f8(t_u8, dev):
    return t_u8.to(dev).view(torch.float8_e4m3fn)


def check_bf16(out_bf16, ref_f32, what):
    """bf16(kernel) against bf16(oracle): relative Frobenius error <= 1e-3, and no entry further
    than 2 bf16 ulps of the reference magnitude."""
    ref = ref_f32.to(torch.bfloat16).float()
    got = out_bf16.float().cpu()
    err = O.rel_frobenius(got, ref)
    assert err <= TOL, f"{what}: bf16 rel Frobenius {err:.3e}"
    tol = ref.abs() * 2 ** -6 + ref_f32.abs().max() * 2 ** -12
    assert bool(((got - ref).abs() <= tol).all()), f"{what}: bf16 outlier"


def rowwise_operands(M, N, K, seed, dev):
    x = O.make_activation(M, K, seed=seed, chan_outlier_frac=0.005, outlier_mul=30.0)
    w = O.make_weight((N, K), seed=seed + 1)
    qx, sx = O.quant_rowwise(x)
    qw, sw = O.quant_rowwise(w)
    return x, w, qx, sx, qw, sw


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (16, 64, 256), (17, 80, 384), (64, 128, 512), (100, 272, 896),
                                   (128, 128, 128), (200, 272, 384), (256, 512, 256), (300, 1024, 1024), (513, 528, 640),
                                   (1024, 768, 3584),
                                   # full 256x256 tiles: the four-wave pipelined kernel (two activation and three weight
                                   # stages in LDS), K of 1, 2, 3, 4, 5 and 7 steps
                                   (768, 256, 128), (1024, 512, 384), (2048, 1280, 896), (768, 512, 512), (1024, 256, 640),
                                   # 256 x 128 tiles of the same pipeline: 256 and 512 tokens, few tiles, N not a multiple of 256;
                                   # K of 1, 2, 3, 4, 5 and 7 steps
                                   (256, 128, 128), (512, 256, 256), (256, 2176, 384), (768, 384, 512), (1024, 1152, 640), (1024, 3584, 896),
                                   # more 256 x 256 tiles than CUs: every workgroup walks several tiles and loads the next
                                   # one under the current one; 408 tiles and K of 3 steps, 405 tiles and 4 steps (a second
                                   # round that not every workgroup takes part in), 512 tiles (+ 16 as quarter tiles behind them) and 5 steps
                                   (4352, 6144, 384), (2304, 11520, 512), (2048, 16896, 640),
                                   # 8 x 33 tiles = one full round of 256 + 8: the last tile-column runs as a second launch
                                   (2048, 8448, 256),
                                   # a last round of 16 tiles as quarter tiles inside the walking kernel; with rows beyond a multiple of 256
                                   (2048, 8704, 384), (2100, 8704, 384),
                                   # M not a multiple of 256: aligned body on the 256x256 kernel + the last rows as their own launch
                                   (1000, 512, 384), (520, 256, 256),
                                   # 17..64 tokens: the strip kernel with 32 or 80 weight rows per workgroup (chosen from
                                   # N), ragged last workgroup, K of 1, 3, 8 and 9 steps (fewer and more than the ring holds)
                                   (40, 528, 1152), (20, 8208, 128), (64, 12272, 384), (33, 16400, 1024), (64, 20016, 128),
                                   (18, 24592, 256), (50, 28688, 128), (32, 40976, 128),
                                   # 65..128 tokens: its 128-row form, ring of five stages, K of 1, 3, 5, 9 and 28 steps
                                   (65, 12272, 384), (128, 16400, 1152), (100, 20016, 128), (127, 10480, 640), (96, 18944, 3584),
                                   (128, 4608, 896),
                                   # 512 tokens on a wide weight: one round of 256 x 256 tiles of the direct-to-LDS kernel
                                   (512, 16640, 384)])
def test_scaled_mm_rowwise(dev, M, N, K):
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=M + N + K, dev=dev)
    ref = O.scaled_mm_rowwise(qx, sx, qw, sw, accum=torch.float64)
    a, b = f8(qx, dev), f8(qw, dev)
    out32 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    err = O.rel_frobenius(out32.cpu(), ref)
    assert err <= TOL, f"fp32 epilogue rel Frobenius {err:.3e}"
    assert err <= TIGHT, f"fp32 epilogue rel Frobenius {err:.3e} above the regression bar"
    out16 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.bfloat16)
    check_bf16(out16, ref, f"rowwise {M}x{N}x{K}")


def test_scaled_mm_one_element_scales(dev):
    """Scales of one element - the tensorwise form of ``torch._scaled_mm`` that the converted linear of the tensorwise
    recipe uses - give the bits of the same call with the scale repeated for every row and column."""
    M, N, K = 96, 528, 384
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=5, dev=dev)
    a, b = f8(qx, dev), f8(qw, dev)
    s1, s2 = sx[3].to(dev), sw[7].to(dev)
    for dt in (torch.float32, torch.bfloat16):
        one = ops.scaled_mm(a, b.t(), s1, s2.reshape(1, 1), out_dtype=dt)
        rep = ops.scaled_mm(a, b.t(), s1.expand(M, 1).contiguous(), s2.expand(1, N).contiguous(), out_dtype=dt)
        assert torch.equal(one, rep)
    with pytest.raises(ValueError):
        ops.scaled_mm(a, b.t(), sx[:2].to(dev), sw.to(dev).t())


@pytest.mark.parametrize("M,N,K", [(1, 16, 16), (5, 48, 80), (16, 64, 144), (17, 200 * 16, 1200), (64, 96, 2880), (100, 528, 1200),
                                   (300, 272, 80), (513, 1024, 2192), (2, 18944, 3600)])
def test_rowwise_k_not_a_multiple_of_128(dev, M, N, K):
    """K = 16 k (what module_filter_fn lets through, cosmos_rl/utils/fp8/fp8_util.py:62-87) with a last K step shorter
    than 128: scaled mm and the fused linear against the oracle; operands in pitched buffers whose bytes beyond K are
    NaN patterns, which a kernel that read past K would turn into NaN outputs."""
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=M + N + K, dev=dev)
    ref = O.scaled_mm_rowwise(qx, sx, qw, sw, accum=torch.float64)
    kp = (K + 127) // 128 * 128 + 128
    abuf = torch.full((M, kp), 0x7F, dtype=torch.uint8, device=dev)
    bbuf = torch.full((N, kp), 0x7F, dtype=torch.uint8, device=dev)
    abuf[:, :K] = qx.to(dev)
    bbuf[:, :K] = qw.to(dev)
    a, b = abuf.view(torch.float8_e4m3fn)[:, :K], bbuf.view(torch.float8_e4m3fn)[:, :K]
    out32 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    assert bool(torch.isfinite(out32).all())
    assert O.rel_frobenius(out32.cpu(), ref) <= TIGHT
    same = ops.scaled_mm(f8(qx, dev), f8(qw, dev).t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    assert torch.equal(out32, same)
    out16 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.bfloat16)
    check_bf16(out16, ref, f"rowwise {M}x{N}x{K}")
    lin = ops.fp8_linear(x.to(dev), b.t(), sw.to(dev), out_dtype=torch.float32)
    assert O.rel_frobenius(lin.cpu(), O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)) <= TIGHT
    # a NaN weight byte in column 0 of row 1 reaches output column 1 only
    if N > 2:
        bbuf[1, 0] = 0x7F
        out = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
        assert bool(torch.isnan(out[:, 1]).all()) and torch.equal(out[:, 2:], out32[:, 2:]) and torch.equal(out[:, 0], out32[:, 0])


@pytest.mark.parametrize("M,N,K", [(768, 512, 384), (1024, 768, 1024), (2048, 8704, 384)])  # (the last: walking kernel + quarter tiles)
def test_scaled_mm_rowwise_pitched_operands(dev, M, N, K):
    """The 256x256 kernel fetches its tiles with per-lane addresses built from the leading dimensions: operands that are
    column slices of wider buffers (row pitch K + 128 and K + 256, data pointers offset into the buffer) give the
    same result as contiguous ones."""
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=M + N + K + 7, dev=dev)
    ref = O.scaled_mm_rowwise(qx, sx, qw, sw, accum=torch.float64)
    abuf = torch.full((M, K + 128), 0x7E, dtype=torch.uint8, device=dev)   # neighbours hold 448.0: a wrong pitch shows
    bbuf = torch.full((N, K + 256), 0x7E, dtype=torch.uint8, device=dev)
    abuf[:, 64:64 + K] = qx.to(dev)
    bbuf[:, 128:128 + K] = qw.to(dev)
    a = abuf.view(torch.float8_e4m3fn)[:, 64:64 + K]
    b = bbuf.view(torch.float8_e4m3fn)[:, 128:128 + K]
    assert a.stride(0) == K + 128 and b.stride(0) == K + 256
    out32 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    assert O.rel_frobenius(out32.cpu(), ref) <= TIGHT
    same = ops.scaled_mm(f8(qx, dev), f8(qw, dev).t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    assert torch.equal(out32, same)
    out16 = ops.scaled_mm(a, b.t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.bfloat16)
    check_bf16(out16, ref, f"pitched rowwise {M}x{N}x{K}")


def test_scaled_mm_one_hot_and_pow2(dev):
    """One-hot activation rows reproduce single weight entries exactly; power-of-two scales make
    the epilogue exact, so the fp32 output must equal the oracle bit for bit."""
    M, N, K = 32, 64, 256
    g = torch.Generator().manual_seed(3)
    qw = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    qw[(qw & 0x7F) == 0x7F] = 0x3F
    qx = torch.zeros(M, K, dtype=torch.uint8)
    ks = torch.randint(0, K, (M,), generator=g)
    qx[torch.arange(M), ks] = 0x38  # 1.0
    sx = (2.0 ** torch.randint(-6, 6, (M, 1), generator=g)).float()
    sw = (2.0 ** torch.randint(-6, 6, (N, 1), generator=g)).float()
    out = ops.scaled_mm(f8(qx, dev), f8(qw, dev).t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32).cpu()
    want = O.e4m3_to_f32(qw)[:, ks].t() * sx * sw.t()
    assert torch.equal(out, want)
    # dense exact case: small integers, power-of-two scales -> every partial sum is exact in fp32
    qa = torch.randint(0x30, 0x48, (M, K), generator=g, dtype=torch.uint8)
    ref = O.scaled_mm_rowwise(qa, sx, qw & 0x3F | 0x20, sw, accum=torch.float64)
    out = ops.scaled_mm(f8(qa, dev), f8(qw & 0x3F | 0x20, dev).t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
    assert O.rel_frobenius(out.cpu(), ref) <= TIGHT


@pytest.mark.parametrize("M", [1, 64, 1024])
def test_fp8_linear_cfg3_shapes(dev, M):
    """benchmark config 3 at reduced N (the full N runs in the property test below): per-token
    activation quantisation inside the call, bytes of the intermediate checked through the result."""
    N, K = 2048, 3584
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=1236 + M, dev=dev)
    ref = O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)
    out32 = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32)
    err = O.rel_frobenius(out32.cpu(), ref)
    assert err <= TIGHT, f"M={M}: {err:.3e}"
    out16 = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev))
    assert out16.dtype == torch.bfloat16 and tuple(out16.shape) == (M, N)
    check_bf16(out16, ref, f"linear M={M}")
    # leading batch dims and bias
    if M == 64:
        bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
        o3 = ops.fp8_linear(x.to(dev).view(4, 16, K), f8(qw, dev).t(), sw.to(dev), bias=bias.to(dev))
        assert tuple(o3.shape) == (4, 16, N)
        assert torch.equal(o3.view(M, N), out16 + bias.to(dev))


@pytest.mark.parametrize("M,N,K", [(64, 3584, 18944), (17, 4096, 1792), (40, 528, 7168), (33, 2064, 3584), (64, 1024, 896)])
def test_fp8_linear_split_k(dev, M, N, K):
    """Few weight rows, long K, 17..64 tokens: with the larger workspace the call cuts K into slices (fp32 partial
    sums, summed in slice order by a second launch); with the minimal workspace it does not.  Both meet the GEMM
    bar, and they agree to fp32 summation order."""
    from cosmos_rl_amd import _lib
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=7 + M + N, dev=dev)
    ref = O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)
    lib = _lib.load()
    small = torch.empty(lib.cfp8_linear_workspace_bytes(M, K), dtype=torch.uint8, device=dev)
    big_n = lib.cfp8_linear_workspace_bytes_split(M, N, K)
    assert (big_n > small.numel()) == (K >= 1792)
    y_split = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32)          # allocates the larger one
    y_plain = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32, workspace=small)
    for y in (y_split, y_plain):
        assert O.rel_frobenius(y.cpu(), ref) <= TIGHT
    assert O.rel_frobenius(y_split.cpu(), y_plain.cpu()) <= 1e-6
    if K >= 1792:
        assert not torch.equal(y_split, y_plain) or K == 1792   # a different summation order shows in the last bits
    check_bf16(ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev)), ref, f"split-K linear {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (2, 272, 896), (3, 1024, 3584), (4, 48, 8320), (4, 18944, 3584), (1, 18944, 3584),
                                   (2, 528, 4096), (4, 64, 4224), (5, 272, 896), (1, 16, 2048)])
def test_fp8_linear_small_m(dev, M, N, K):
    """Decode shapes: cfp8_linear_rowwise equals cfp8_scaled_mm_rowwise on separately quantised activations bit
    for bit - up to 4 tokens and K <= 4096 it is one launch that quantises the tokens inside the GEMM kernel,
    otherwise two; K > 4096 walks the K loop of the M <= 16 kernel more than once; a NaN token stays a NaN row
    and leaves the others alone."""
    x, w, qx, sx, qw, sw = rowwise_operands(M, N, K, seed=99 + M + N, dev=dev)
    y = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32)
    qxd, sxd = ops.quant_rowwise(x.to(dev))
    y2 = ops.scaled_mm(qxd, f8(qw, dev).t(), sxd, sw.to(dev).t(), out_dtype=torch.float32)
    assert torch.equal(y, y2)
    ref = O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)
    assert O.rel_frobenius(y.cpu(), ref) <= TIGHT
    # a row pitch larger than K, and the bf16 epilogue
    xp = torch.zeros(M, K + 64, dtype=torch.bfloat16, device=dev)
    xp[:, :K] = x.to(dev)
    assert torch.equal(ops.fp8_linear(xp[:, :K], f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32), y)
    y16 = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev))
    assert torch.equal(y16, ops.scaled_mm(qxd, f8(qw, dev).t(), sxd, sw.to(dev).t(), out_dtype=torch.bfloat16))
    if M > 1:
        xn = x.clone()
        xn[0, 5] = float("nan")
        yn = ops.fp8_linear(xn.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32)
        assert bool(torch.isnan(yn[0]).all()) and torch.equal(yn[1:], y[1:])


def test_fp8_linear_full_cfg3_properties(dev):
    """Full Qwen2.5-7B MLP shape [8192, 3584] x [18944, 3584]^T on the GPU only.  Linearity in the
    weight scales (doubling sw doubles the fp32 output exactly), row-subset consistency with an
    M=64 call (different tile configuration, same numbers), and a sampled block against fp64."""
    M, N, K = 8192, 18944, 3584
    g = torch.Generator(device=dev).manual_seed(21)
    x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    qw, sw = ops.quant_rowwise(w)
    out = ops.fp8_linear(x, qw.t(), sw, out_dtype=torch.float32)
    out2 = ops.fp8_linear(x, qw.t(), sw * 2, out_dtype=torch.float32)
    assert torch.equal(out2, out * 2)
    sub = ops.fp8_linear(x[4096:4160], qw.t(), sw, out_dtype=torch.float32)
    assert O.rel_frobenius(sub.cpu(), out[4096:4160].cpu()) <= TIGHT
    rows = torch.arange(0, M, 257, device=dev)[:24]
    cols = torch.arange(0, N, 601, device=dev)[:32]
    qx, sx = ops.quant_rowwise(x[rows])
    ref = (qx.double() @ qw[cols].double().t()) * sx.double() * sw[cols].double().t()
    got = out[rows][:, cols].double()
    assert O.rel_frobenius(got.cpu(), ref.cpu()) <= TIGHT


# ---------------------------------------------------------------------------- block-scaled
def block_operands(M, N, K, seed):
    x = O.make_activation(M, K, seed=seed)
    w = O.make_weight((N, K), seed=seed + 1)
    qx, sx = O.quant_group128(x)
    qw, sw = O.quant_block128(w)
    return qx, sx, qw, sw


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (16, 128, 256), (70, 208, 384), (128, 256, 1024), (300, 512, 768),
                                   (640, 1536, 2048), (1000, 12288, 384), (1024, 12288, 512),
                                   # full 256 x 128 tiles, >= 384 of them (the eight-wave kernel): K of 5, 1, 9 and 17 steps
                                   (1024, 12288, 640), (768, 16384, 128), (1024, 12416, 1152), (1280, 10240, 2176),
                                   # the same with 16-byte scale loads: K of 8 and 12 steps (one group of eight steps, one and
                                   # a half); 516 tiles (two full rounds of one tile per CU and a short one) with K of 3 steps
                                   (1024, 12288, 1024), (1024, 12288, 1536), (768, 22016, 384),
                                   # a token count that is no multiple of 256: full tiles for the first 768 / 1024 rows, the
                                   # last 232 / 1 as a launch of their own
                                   (1000, 16384, 640), (1025, 12288, 384)])
def test_gemm_block128(dev, M, N, K):
    # the last two shapes have >= 384 tiles of 256 x 128 and take the 8-wave 256 x 128 kernel: one with a
    # ragged last tile-row and K/128 not a multiple of 4 (scalar scale loads), one with 16-byte scale loads
    qx, sx, qw, sw = block_operands(M, N, K, seed=M * 3 + N + K)
    ref = O.scaled_mm_block128(qx, sx, qw, sw, accum=torch.float64)
    out32 = torch.empty(M, N, dtype=torch.float32, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out32)
    err = O.rel_frobenius(out32.cpu(), ref)
    assert err <= TIGHT, f"block fp32 {err:.3e}"
    assert O.calc_diff(out32.cpu(), ref) < 1e-8  # the reference's own metric (tests/test_deepep.py:62-67)
    out16 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out16)
    check_bf16(out16, ref, f"block {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(4096, 4096, 2048), (4096, 4352, 2176), (2048, 8192, 2560)])
def test_gemm_block128_256x256_tiles(dev, M, N, K):
    """The 256 x 256 block-scaled kernel (16 K steps or more, at least 256 such tiles; 4096 x 4352 also cuts the last
    tile-column off for the 256 x 128 kernel).  It keeps a row's accumulators in the units of the running step's scale,
    so the scales are made to jump: activation groups that are zero, tiny or a thousand times the rest, a zero and a
    large weight block."""
    g = torch.Generator().manual_seed(M + N + K)
    x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
    x[:, :128] *= 1000.0
    x[100:300, 128:256] = 0.0
    x[:, 384:512] *= 1e-6
    x[700:900, K - 128:] = 0.0
    w[256:384, 256:384] = 0.0
    w[:128, 512:640] *= 300.0
    w[N - 128:, :128] = 0.0
    qx, sx = O.quant_group128(x)
    qw, sw = O.quant_block128(w)
    ref = O.scaled_mm_block128(qx, sx, qw, sw, accum=torch.float64)
    out32 = torch.empty(M, N, dtype=torch.float32, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out32)
    assert bool(torch.isfinite(out32).all())
    err = O.rel_frobenius(out32.cpu(), ref)
    assert err <= TIGHT, f"fp32 epilogue rel Frobenius {err:.3e}"
    # row by row as well: a row whose scales jump must be as good as the others
    row_err = (out32.cpu().double() - ref).norm(dim=1) / ref.norm(dim=1).clamp_min(1e-30)
    assert float(row_err.max()) <= 10 * TIGHT, f"worst row {int(row_err.argmax())}: {float(row_err.max()):.3e}"
    out16 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out16)
    check_bf16(out16, ref, f"block 256x256 {M}x{N}x{K}")
    again = torch.empty_like(out32)
    ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), again)
    assert torch.equal(again, out32)


def test_gemm_block128_kn_weight_layout(dev):
    """Config 4 layout: weight given [K, N], quantised with the transposing quantiser; scales stay
    [K/128, N/128].  y = x @ W."""
    M, K, N = 192, 512, 384
    x = O.make_activation(M, K, seed=40)
    w = O.make_weight((K, N), seed=41)
    qx, sx = ops.groupwise_activation_quant(x.to(dev))
    qwt, sw = ops.per_block_cast_to_fp8(w.to(dev), transpose_out=True)  # [N, K], scales [K/128, N/128]
    assert tuple(qwt.shape) == (N, K) and tuple(sw.shape) == (K // 128, N // 128)
    out = torch.empty(M, N, dtype=torch.float32, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((qx, sx), (qwt, sw), out, rhs_scale_kn=True)
    qxo, sxo = O.quant_group128(x)
    qwo, swo = O.quant_block128(w)
    ref = (O.group128_dequant(qxo, sxo).double() @ O.weight_dequant(qwo, swo).double())
    assert O.rel_frobenius(out.cpu(), ref) <= TIGHT


def test_gemm_block128_cfg4_properties(dev):
    """Config 4 at full size [4096, 7168] x [7168, 18432]: sampled rows/cols against fp64 and
    exact linearity in a power-of-two rescale of one activation K-block's scales."""
    M, K, N = 4096, 7168, 18432
    g = torch.Generator(device=dev).manual_seed(44)
    x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(K, N, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    qx, sx = ops.groupwise_activation_quant(x)
    qwt, sw = ops.per_block_cast_to_fp8(w, transpose_out=True)
    out = torch.empty(M, N, dtype=torch.float32, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((qx, sx), (qwt, sw), out, rhs_scale_kn=True)
    out2 = torch.empty_like(out)
    ops.gemm_fp8_fp8_bf16_nt((qx, sx * 4), (qwt, sw * 0.5), out2, rhs_scale_kn=True)
    assert torch.equal(out2, out * 2)
    rows = torch.arange(0, M, 173, device=dev)[:20]
    cols = torch.arange(0, N, 577, device=dev)[:30]
    a = qx[rows].double() * sx[rows].double().repeat_interleave(128, dim=1)
    swn = sw.t().contiguous()  # [N/128, K/128]
    b = qwt[cols].double() * swn[cols // 128].double().repeat_interleave(128, dim=1)
    ref = a @ b.t()
    assert O.rel_frobenius(out[rows][:, cols].double().cpu(), ref.cpu()) <= TIGHT


# ---------------------------------------------------------------------------- grouped
@pytest.mark.parametrize("T,E,K,I,topk", [(300, 7, 512, 256, 2), (3300, 7, 1152, 1024, 2), (700, 5, 128, 128, 3), (2000, 9, 1024, 384, 2),
                                          # K of 12 and 17 steps, more tiles than CUs: the form in which a workgroup walks several tiles
                                          (3300, 7, 1536, 1024, 2), (3300, 7, 2176, 1024, 2)])
def test_grouped_swiglu_epilogue_bit_exact(dev, T, E, K, I, topk):
    """Grouped gate_up GEMM with SwiGLU + 1x128 requantisation as its epilogue (interleaved weights) against the
    grouped GEMM on the concatenated weights followed by the SwiGLU quantiser: same bytes, same scales; padding rows
    untouched."""
    g = torch.Generator().manual_seed(T + I)
    logits = torch.rand(T, E, generator=g)
    logits[:, 2] = -1.0  # an expert without tokens
    token_of_row, m_indices, m_sizes, m_offsets = O.route_topk_contiguous(logits, topk, 128)
    x = O.make_activation(T, K, seed=5)
    xs = torch.zeros(token_of_row.numel(), K, dtype=torch.bfloat16)
    valid = token_of_row >= 0
    xs[valid] = x[token_of_row[valid]]
    qx, sx = ops.groupwise_activation_quant(xs.to(dev))
    qg, sg = ops.per_block_cast_to_fp8(O.make_weight((E, I, K), seed=6, std=0.05).to(dev))
    qu, su = ops.per_block_cast_to_fp8(O.make_weight((E, I, K), seed=7, std=0.05).to(dev))
    mi = m_indices.to(dev)
    gu = torch.zeros(xs.shape[0], 2 * I, dtype=torch.bfloat16, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (torch.cat([qg, qu], 1), torch.cat([sg, su], 1)), gu, mi)
    q0, s0 = ops.swiglu_quant(gu[:, :I], gu[:, I:])
    qi, si = ops.interleave_gate_up((qg, sg), (qu, su))
    # rows alternate in units of 16: gate 0-15, up 0-15, gate 16-31, ...; scale rows alternate per block of 128
    assert torch.equal(qi.view(torch.uint8)[:, 16:32], qu.view(torch.uint8)[:, :16]) and torch.equal(qi.view(torch.uint8)[:, 32:48], qg.view(torch.uint8)[:, 16:32])
    assert torch.equal(si[:, 0], sg[:, 0]) and torch.equal(si[:, 1], su[:, 0])
    q1 = torch.full((xs.shape[0], I), 0x55, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s1 = torch.full((xs.shape[0], I // 128), -1.0, dtype=torch.float32, device=dev)
    from cosmos_rl_amd import _lib
    _lib.check(_lib.load().cfp8_gemm_grouped_swiglu_quant(qx.data_ptr(), K, sx.data_ptr(), qi.data_ptr(), si.data_ptr(), mi.data_ptr(),
                                                         q1.data_ptr(), I, s1.data_ptr(), xs.shape[0], I, K, E,
                                                         torch.cuda.current_stream().cuda_stream))
    v = valid.to(dev)
    assert torch.equal(q1.view(torch.uint8)[v], q0.view(torch.uint8)[v]) and torch.equal(s1[v].view(torch.int32), s0[v].view(torch.int32))
    assert bool((q1.view(torch.uint8)[~v] == 0x55).all()) and bool((s1[~v] == -1.0).all())
    q2, s2 = ops.grouped_gemm_swiglu_quant((qx, sx), (qi, si), mi)
    assert torch.equal(q2.view(torch.uint8)[v], q0.view(torch.uint8)[v]) and torch.equal(s2[v], s0[v])


def test_grouped_cfg5_full_size_properties(dev):
    """Config 5 at full size: 8192 tokens routed top-8 over 128 experts (65536 rows, groups padded to 128), expert MLP
    shapes [1536, 2048] and [2048, 768], through the host path of the reference (route -> gather -> DSGroupGEMM-style
    chain -> combine).  Size-independent checks: padding rows stay untouched, sampled rows of both GEMMs against
    the fp64 dequantised product, the fused SwiGLU quantiser against the unfused torch chain's bytes on a slice,
    permuting the tokens of one expert permutes its output rows, and the combined output of a token whose 8 weights
    are zero except one equals that expert's row times the weight."""
    from cosmos_rl_amd.policy.kernel.moe.indices import permute_tokens
    from cosmos_rl_amd.policy.kernel.moe.moe import combine_expert_outputs, route_tokens
    E, T, TOPK, H, I = 128, 8192, 8, 2048, 768
    g = torch.Generator(device=dev).manual_seed(55)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    wgu = (torch.randn(E, 2 * I, H, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    wd = (torch.randn(E, H, I, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    qgu, sgu = ops.per_block_cast_to_fp8(wgu)
    qd, sd = ops.per_block_cast_to_fp8(wd)
    top = torch.topk(torch.rand(T, E, generator=g, device=dev), TOPK, dim=1)
    r = route_tokens(top.indices.to(torch.int32), None, E, 128)
    total = int(r.m_offsets[-1])
    assert total % 128 == 0 and int((r.row_tokens >= 0).sum()) == T * TOPK
    contig = permute_tokens(x, r.row_tokens)[:total]
    m_idx = ops.create_indices_from_offsets_nosync(r.m_offsets, total)
    m_idx = torch.where(r.row_tokens[:total] >= 0, m_idx, torch.full_like(m_idx, -1))
    qx, sx = ops.groupwise_activation_quant(contig)
    gu = torch.full((total, 2 * I), 7.0, dtype=torch.bfloat16, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qgu, sgu), gu, m_idx)
    pad = m_idx < 0
    assert bool(pad.any()) and bool((gu[pad] == 7.0).all()), "padding rows were written"
    rows = (~pad).nonzero().flatten()[::977][:40]

    def ref_rows(qa, sa, qb, sb, rows_):
        e = m_idx[rows_].long()
        a = qa[rows_].double() * sa[rows_].double().repeat_interleave(128, dim=1)
        b = qb[e].double() * sb[e].double().repeat_interleave(128, dim=1).repeat_interleave(128, dim=2)[:, :qb.shape[1]]
        return torch.einsum("rk,rnk->rn", a, b)

    check_bf16(gu[rows], ref_rows(qx, sx, qgu, sgu, rows).float().cpu(), "cfg5 gate_up rows")
    gu[pad] = 0
    qh, sh = ops.swiglu_quant(gu[:, :I], gu[:, I:])
    sl = slice(0, 4096)
    h = torch.nn.functional.silu(gu[sl, :I]) * gu[sl, I:]
    qh2, sh2 = ops.groupwise_activation_quant(h)
    same = (qh[sl].view(torch.uint8) == qh2.view(torch.uint8)).float().mean().item()
    assert same > 0.99, same  # torch's silu differs from the library's fixed exp sequence by a bf16 ulp on a few elements
    dn = torch.zeros(total, H, dtype=torch.bfloat16, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qh, sh), (qd, sd), dn, m_idx)
    check_bf16(dn[rows], ref_rows(qh, sh, qd, sd, rows).float().cpu(), "cfg5 down rows")
    # the configuration the benchmark times: the gate_up GEMM on interleaved weights with the SwiGLU + 1x128
    # requantisation as its epilogue, at this size in the form where a workgroup walks several tiles - bytes and
    # scales equal the unfused chain's on every valid row, padding rows untouched
    qgi, sgi = ops.interleave_gate_up((qgu[:, :I], sgu[:, :I // 128]), (qgu[:, I:], sgu[:, I // 128:]))
    qf = torch.full((total, I), 0x55, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sf = torch.full((total, I // 128), -1.0, dtype=torch.float32, device=dev)
    from cosmos_rl_amd import _lib
    _lib.check(_lib.load().cfp8_gemm_grouped_swiglu_quant(qx.data_ptr(), H, sx.data_ptr(), qgi.data_ptr(), sgi.data_ptr(), m_idx.data_ptr(),
                                                         qf.data_ptr(), I, sf.data_ptr(), total, I, H, E,
                                                         torch.cuda.current_stream().cuda_stream))
    ok = ~pad
    assert torch.equal(qf.view(torch.uint8)[ok], qh.view(torch.uint8)[ok]), "fused SwiGLU epilogue: bytes differ from the unfused chain"
    assert torch.equal(sf[ok].view(torch.int32), sh[ok].view(torch.int32)), "fused SwiGLU epilogue: scales differ"
    assert bool((qf.view(torch.uint8)[pad] == 0x55).all()) and bool((sf[pad] == -1.0).all()), "fused epilogue wrote padding rows"
    # ... and the strategy object on top of it, straight from the token matrix (gather + quantise in one pass,
    # fused gate_up + SwiGLU GEMM, down GEMM), against the chain above
    import torch.nn as nn
    from cosmos_rl_amd.policy.kernel.group_gemms import DSGroupGEMM
    mod = nn.Module()
    for name, qq, ss in (("gate_proj", qgu[:, :I].contiguous(), sgu[:, :I // 128].contiguous()),
                         ("up_proj", qgu[:, I:].contiguous(), sgu[:, I // 128:].contiguous()), ("down_proj", qd, sd)):
        mod.register_parameter(f"{name}_fp8", nn.Parameter(qq, requires_grad=False))
        mod.register_parameter(f"{name}_scales", nn.Parameter(ss, requires_grad=False))
    mod.register_parameter("gate_proj_weight", nn.Parameter(torch.empty(E, I, 0, device=dev), requires_grad=False))
    mod.register_parameter("down_proj_weight", nn.Parameter(torch.empty(E, H, 0, device=dev), requires_grad=False))
    out_ft = DSGroupGEMM(torch.nn.functional.silu, fuse_gate_up=True).execute_from_tokens(x, r.row_tokens, r.m_sizes, r.m_offsets, mod)
    assert out_ft.shape[0] == r.row_tokens.numel() and torch.equal(out_ft[:total][ok], dn[ok])
    assert bool((out_ft[:total][pad] == 0).all()) and bool((out_ft[total:] == 0).all())
    # permutation inside expert 3's group
    rows3 = (m_idx == 3).nonzero().flatten()
    perm = rows3[torch.randperm(rows3.numel(), generator=torch.Generator().manual_seed(1)).to(dev)]
    qh_p, sh_p = qh.clone(), sh.clone()
    qh_p[rows3], sh_p[rows3] = qh[perm], sh[perm]
    dn_p = torch.zeros_like(dn)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qh_p, sh_p), (qd, sd), dn_p, m_idx)
    assert torch.equal(dn_p[rows3], dn[perm])
    # combine: one-hot weights pick one expert row, scaled
    wts = torch.zeros(T, TOPK, dtype=torch.bfloat16, device=dev)
    wts[:, 2] = 0.5
    y = combine_expert_outputs(dn, r, wts)
    slot_pos = (r.slot_order == 2).float().argmax(dim=1)
    src = r.row_map.gather(1, slot_pos[:, None]).flatten().long()
    assert torch.equal(y, (dn[src].float() * 0.5).to(torch.bfloat16))


@pytest.mark.parametrize("T,E,K,N,topk", [(300, 7, 512, 384, 2), (2600, 7, 384, 2048, 2), (3300, 7, 1152, 2048, 2), (3300, 7, 1024, 1792, 2),
                                          (3300, 7, 128, 2048, 2), (3300, 7, 1536, 2048, 2), (3300, 7, 2176, 2048, 2)])
def test_grouped_gemm(dev, T, E, K, N, topk):
    """Ragged groups: top-2 routing over 6 experts plus an empty expert, groups padded to 128 rows;
    padding rows (index -1) must be left untouched.  The shapes with 3300 tokens have >= 384 tiles of
    128 x 256 (the eight-wave kernel): K of 9 steps (more than one group of 8 activation-scale steps, scalar
    scale loads), 8 steps (16-byte scale loads) with N = 7 * 256, and a single step; K of 12 and 17 steps take the
    form of that kernel in which a workgroup walks several tiles (it has to step over the empty expert's padding tile
    and leave padding rows unwritten through masked stores)."""
    g = torch.Generator().manual_seed(77)
    logits = torch.rand(T, E, generator=g)
    logits[:, 3] = -1.0  # expert 3 gets no token
    token_of_row, m_indices, m_sizes, m_offsets = O.route_topk_contiguous(logits, topk, 128)
    assert int(m_sizes[3]) == 128 and int((m_indices == 3).sum()) == 0
    x = O.make_activation(T, K, seed=78)
    xs = torch.zeros(token_of_row.numel(), K, dtype=torch.bfloat16)
    valid = token_of_row >= 0
    xs[valid] = x[token_of_row[valid]]
    w = O.make_weight((E, N, K), seed=79)
    qx, sx = O.quant_group128(xs)
    qw, sw = O.quant_block128(w)
    ref = O.grouped_mm_block128(qx, sx, qw, sw, m_indices, accum=torch.float64)
    out = torch.full((xs.shape[0], N), 7.0, dtype=torch.float32, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out,
                                                  m_indices.to(dev))
    out = out.cpu()
    assert bool((out[~valid] == 7.0).all()), "padding rows were written"
    assert O.rel_frobenius(out[valid], ref[valid]) <= TIGHT
    out16 = torch.zeros((xs.shape[0], N), dtype=torch.bfloat16, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out16,
                                                  m_indices.to(dev))
    check_bf16(out16, ref, "grouped")
    # permuting tokens inside one expert's group permutes the output rows and nothing else
    rows0 = (m_indices == 0).nonzero().flatten()
    perm = rows0[torch.randperm(rows0.numel(), generator=g)]
    qx2, sx2 = qx.clone(), sx.clone()
    qx2[rows0], sx2[rows0] = qx[perm], sx[perm]
    out2 = torch.zeros((xs.shape[0], N), dtype=torch.float32, device=dev)
    ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((f8(qx2, dev), sx2.to(dev)), (f8(qw, dev), sw.to(dev)), out2,
                                                  m_indices.to(dev))
    assert torch.equal(out2.cpu()[rows0], out[perm])


def test_walking_kernels_repeatable(dev):
    """The kernels in which one workgroup walks several tiles keep loads of the next tile in flight across the
    epilogue of the current one; a missing wait or barrier there would show as run-to-run differences.  The same
    call five times gives the same bits, rowwise and block-scaled, fp32 and bf16 output."""
    g = torch.Generator(device=dev).manual_seed(5)
    for mode, (M, N, K) in (("row", (2304, 11520, 512)), ("row", (8192, 4864, 896)), ("blk", (1024, 12288, 1536)), ("blk", (2048, 6400, 640))):
        qx = torch.randint(0, 256, (M, K), generator=g, device=dev, dtype=torch.uint8)
        qw = torch.randint(0, 256, (N, K), generator=g, device=dev, dtype=torch.uint8)
        qx[(qx & 0x7F) == 0x7F] = 0x30
        qw[(qw & 0x7F) == 0x7F] = 0x30
        a, b = qx.view(torch.float8_e4m3fn), qw.view(torch.float8_e4m3fn)
        for dt in (torch.float32, torch.bfloat16):
            runs = []
            for _ in range(5):
                if mode == "row":
                    if not runs:
                        sx = torch.rand(M, 1, generator=g, device=dev) + 0.5
                        sw = torch.rand(N, 1, generator=g, device=dev) + 0.5
                    runs.append(ops.scaled_mm(a, b.t(), sx, sw.t(), out_dtype=dt))
                else:
                    if not runs:
                        sx = torch.rand(M, K // 128, generator=g, device=dev) + 0.5
                        sw = torch.rand(N // 128, K // 128, generator=g, device=dev) + 0.5
                    o = torch.empty(M, N, dtype=dt, device=dev)
                    ops.gemm_fp8_fp8_bf16_nt((a, sx), (b, sw), o)
                    runs.append(o)
            assert all(torch.equal(runs[0], r) for r in runs[1:]), f"{mode} {M}x{N}x{K} {dt}: runs differ"


def _grouped_problem(dev, T, E, K, topk, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.rand(T, E, generator=g)
    logits[:, 1] = -1.0                                   # an expert without tokens: a tile of padding to step over
    token_of_row, m_indices, _, _ = O.route_topk_contiguous(logits, topk, 128)
    x = O.make_activation(T, K, seed=seed + 1)
    xs = torch.zeros(token_of_row.numel(), K, dtype=torch.bfloat16)
    valid = token_of_row >= 0
    xs[valid] = x[token_of_row[valid]]
    qx, sx = ops.groupwise_activation_quant(xs.to(dev))
    return qx, sx, m_indices.to(dev), valid.to(dev)


def test_walking_grouped_kernels_repeatable_and_equal_to_sliced_calls(dev):
    """The grouped kernel in which a workgroup walks several tiles, plain and with the SwiGLU + requantisation
    epilogue: five runs give the same bits, and those bits equal what the same problem gives when it is cut along N
    into calls small enough to take the one-tile-per-workgroup kernels (same arithmetic, other schedule)."""
    E, topk = 7, 2
    for K, I, T in ((1536, 1024, 3300), (2048, 768, 4500), (896, 1024, 3300)):
        qx, sx, mi, valid = _grouped_problem(dev, T, E, K, topk, seed=K)
        rows = qx.shape[0]
        qg, sg = ops.per_block_cast_to_fp8(O.make_weight((E, I, K), seed=6, std=0.05).to(dev))
        qu, su = ops.per_block_cast_to_fp8(O.make_weight((E, I, K), seed=7, std=0.05).to(dev))
        qw, sw = torch.cat([qg, qu], 1).contiguous(), torch.cat([sg, su], 1).contiguous()
        N = 2 * I
        assert (rows // 128) * (N // 256) > 384, "shape must take the walking form"
        runs = []
        for _ in range(5):
            o = torch.full((rows, N), 7.0, dtype=torch.bfloat16, device=dev)
            ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qw, sw), o, mi)
            runs.append(o)
        assert all(torch.equal(runs[0], r) for r in runs[1:]), f"grouped K={K}: runs differ"
        # the same product from calls of N / 4 columns (fewer than 384 tiles each: the generic kernel)
        parts = []
        for c in range(4):
            n0, n1 = c * N // 4, (c + 1) * N // 4
            o = torch.full((rows, n1 - n0), 7.0, dtype=torch.bfloat16, device=dev)
            ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qw[:, n0:n1].contiguous(), sw[:, n0 // 128:n1 // 128].contiguous()), o, mi)
            parts.append(o)
        assert torch.equal(torch.cat(parts, 1), runs[0]), f"grouped K={K}: walking form differs from the sliced calls"
        # SwiGLU epilogue
        qi, si = ops.interleave_gate_up((qg, sg), (qu, su))
        outs = [ops.grouped_gemm_swiglu_quant((qx, sx), (qi, si), mi) for _ in range(5)]
        for q, sc in outs[1:]:
            assert torch.equal(q.view(torch.uint8)[valid], outs[0][0].view(torch.uint8)[valid]) and torch.equal(sc[valid], outs[0][1][valid]), \
                f"grouped SwiGLU K={K}: runs differ"
        q0, s0 = ops.swiglu_quant(runs[0][:, :I], runs[0][:, I:])
        assert torch.equal(outs[0][0].view(torch.uint8)[valid], q0.view(torch.uint8)[valid]) and torch.equal(outs[0][1][valid], s0[valid])


def test_grouped_short_k_kernel_equal_to_sliced_calls(dev):
    """5 or 6 K steps (an expert's down projection): the kernel that keeps a tile row's activation fragments in
    registers and walks the row's tiles.  Against the same problem cut along N into calls of 256 columns (the
    one-tile-per-workgroup kernels: same arithmetic, other schedule): same bits, bf16 and fp32, with an expert without
    tokens, fewer tile rows than CUs (every row cut into pieces) and more (whole rows first, then pieces); the rows of
    padding keep what the output held; five runs agree."""
    from cosmos_rl_amd import _lib
    E = 7
    for K, N, T, topk in ((768, 4096, 4700, 2), (640, 4096, 4700, 2), (768, 2048, 8300, 4)):
        qx, sx, mi, valid = _grouped_problem(dev, T, E, K, topk, seed=K + T)
        rows = qx.shape[0]
        qw, sw = ops.per_block_cast_to_fp8(O.make_weight((E, N, K), seed=8, std=0.05).to(dev))
        for dt, code in ((torch.bfloat16, _lib.OUT_BF16), (torch.float32, _lib.OUT_F32)):
            assert "gemm_grouped_xres" in _lib.gemm_dispatch_info(_lib.DISPATCH_GROUPED, rows, N, K, out_dtype=code), (rows, N, K)
            assert "gemm_grouped_xres" not in _lib.gemm_dispatch_info(_lib.DISPATCH_GROUPED, rows, 256, K, out_dtype=code)
            runs = []
            for _ in range(5):
                o = torch.full((rows, N), 7.0, dtype=dt, device=dev)
                ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qw, sw), o, mi)
                runs.append(o)
            assert all(torch.equal(runs[0], r) for r in runs[1:]), f"K={K} N={N} {dt}: runs differ"
            parts = []
            for n0 in range(0, N, 256):
                o = torch.full((rows, 256), 7.0, dtype=dt, device=dev)
                ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qw[:, n0:n0 + 256].contiguous(), sw[:, n0 // 128:n0 // 128 + 2].contiguous()), o, mi)
                parts.append(o)
            assert torch.equal(torch.cat(parts, 1), runs[0]), f"K={K} N={N} {dt}: differs from the sliced calls"
            assert bool((runs[0][~valid] == 7.0).all()) and not bool((runs[0][valid] == 7.0).all(1).any())
        # an output with a row pitch, through the C entry point: the columns beyond N keep their contents
        wide = torch.full((rows, N + 64), 3.0, dtype=torch.bfloat16, device=dev)
        lib = _lib.load()
        _lib.check(lib.cfp8_gemm_grouped_block128(qx.data_ptr(), K, sx.data_ptr(), qw.data_ptr(), sw.data_ptr(), mi.data_ptr(), wide.data_ptr(), N + 64,
                                                  _lib.OUT_BF16, rows, N, K, E, torch.cuda.current_stream().cuda_stream))
        ref = torch.full((rows, N), 3.0, dtype=torch.bfloat16, device=dev)
        ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qw, sw), ref, mi)
        assert torch.equal(wide[:, :N], ref) and bool((wide[:, N:] == 3.0).all())


def test_walking_kernels_equal_to_sliced_calls(dev):
    """Rowwise and block-scaled: a problem with more tiles than CUs (the walking kernels) against the same problem cut
    along N into calls that fit one round of workgroups (one tile per workgroup, or the generic kernel): same bits."""
    g = torch.Generator(device=dev).manual_seed(9)
    # (the third to fifth: a last round of 16, 96 and 40 tiles, which the walking kernel's workgroups take as quarter tiles)
    for mode, (M, N, K), cuts in (("row", (2304, 11520, 512), 3), ("row", (8192, 7680, 896), 6), ("row", (2048, 8704, 512), 2),
                                  ("row", (2048, 11264, 640), 2), ("row", (1024, 18944, 3584), 2), ("blk", (1024, 12288, 1536), 2),
                                  ("blk", (2048, 6400, 640), 2)):
        qx = torch.randint(0, 256, (M, K), generator=g, device=dev, dtype=torch.uint8)
        qw = torch.randint(0, 256, (N, K), generator=g, device=dev, dtype=torch.uint8)
        qx[(qx & 0x7F) == 0x7F] = 0x30
        qw[(qw & 0x7F) == 0x7F] = 0x30
        a, b = qx.view(torch.float8_e4m3fn), qw.view(torch.float8_e4m3fn)
        for dt in (torch.float32, torch.bfloat16):
            if mode == "row":
                sx = torch.rand(M, 1, generator=g, device=dev) + 0.5
                sw = torch.rand(N, 1, generator=g, device=dev) + 0.5
                whole = ops.scaled_mm(a, b.t(), sx, sw.t(), out_dtype=dt)
                parts = [ops.scaled_mm(a, b[c * N // cuts:(c + 1) * N // cuts].t(), sx, sw[c * N // cuts:(c + 1) * N // cuts].t(), out_dtype=dt)
                         for c in range(cuts)]
            else:
                sx = torch.rand(M, K // 128, generator=g, device=dev) + 0.5
                sw = torch.rand(N // 128, K // 128, generator=g, device=dev) + 0.5
                whole = torch.empty(M, N, dtype=dt, device=dev)
                ops.gemm_fp8_fp8_bf16_nt((a, sx), (b, sw), whole)
                parts = []
                for c in range(cuts):
                    n0, n1 = c * N // cuts, (c + 1) * N // cuts
                    o = torch.empty(M, n1 - n0, dtype=dt, device=dev)
                    ops.gemm_fp8_fp8_bf16_nt((a, sx), (b[n0:n1], sw[n0 // 128:n1 // 128].clone()), o)
                    parts.append(o)
            assert torch.equal(torch.cat(parts, 1), whole), f"{mode} {M}x{N}x{K} {dt}: walking form differs from the sliced calls"


def test_random_shapes_all_dispatch_paths(dev):
    """Seeded sweep over row counts on both sides of every dispatch threshold (16, 32, 64, 128, 256, 512, multiples of
    256 and not), N a multiple of 16 or 256, K 1..9 steps: rowwise mm, fused linear and block-scaled mm."""
    import random
    rnd = random.Random(2024)
    Ms = [1, 5, 16, 17, 33, 64, 65, 127, 129, 255, 257, 300, 511, 513, 600, 768, 1000, 1030, 1279]
    for it in range(24):
        M = rnd.choice(Ms)
        N = 256 * rnd.randint(1, 4) if rnd.random() < 0.4 else 16 * rnd.randint(1, 60)
        K = 128 * rnd.randint(1, 9)
        mode = rnd.choice(["row", "lin", "blk"])
        g = torch.Generator().manual_seed(it)
        x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
        if mode == "blk":
            qx, sx = O.quant_group128(x)
            qw, sw = O.quant_block128(w)
            ref = O.scaled_mm_block128(qx, sx, qw, sw, accum=torch.float64)
            out = torch.empty(M, N, dtype=torch.float32, device=dev)
            ops.gemm_fp8_fp8_bf16_nt((f8(qx, dev), sx.to(dev)), (f8(qw, dev), sw.to(dev)), out)
        else:
            qw, sw = O.quant_rowwise(w)
            ref = O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)
            if mode == "lin":
                out = ops.fp8_linear(x.to(dev), f8(qw, dev).t(), sw.to(dev), out_dtype=torch.float32)
            else:
                qx, sx = O.quant_rowwise(x)
                out = ops.scaled_mm(f8(qx, dev), f8(qw, dev).t(), sx.to(dev), sw.to(dev).t(), out_dtype=torch.float32)
        err = O.rel_frobenius(out.cpu(), ref)
        assert err <= TIGHT, f"{mode} M={M} N={N} K={K}: {err:.3e}"


def test_gemm_errors(dev):
    a = torch.zeros(16, 100, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    b = torch.zeros(32, 100, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    with pytest.raises(ValueError):  # K % 128
        ops.scaled_mm(a, b.t(), torch.ones(16, 1, device=dev), torch.ones(1, 32, device=dev))
    a = torch.zeros(16, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    b = torch.zeros(128, 32, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)  # row-major [K, N]
    with pytest.raises(ValueError):
        ops.scaled_mm(a, b, torch.ones(16, 1, device=dev), torch.ones(1, 32, device=dev))
    out = ops.scaled_mm(torch.zeros(0, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
                        torch.zeros(32, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn).t(),
                        torch.ones(0, 1, device=dev), torch.ones(1, 32, device=dev))
    assert tuple(out.shape) == (0, 32)
