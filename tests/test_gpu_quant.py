"""Parity of the HIP quantizers with the CPU oracle: fp8 bytes and fp32 scales bit-exact.
Every call goes through the C ABI (cosmos_rl_amd.ops -> ctypes -> libcosmosfp8.so)."""
import pytest
import torch

from oracle import fp8_oracle as O
from cosmos_rl_amd import ops, _lib

pytestmark = pytest.mark.gpu


def u8(t):
    return t.contiguous().view(torch.uint8).cpu()


def bits(t):
    return t.contiguous().view(torch.int32).cpu()


def assert_bytes(got, want, what):
    got, want = u8(got), want
    if not torch.equal(got, want):
        bad = (got != want).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(f"{what}: {bad.shape[0]} byte mismatches, first at {i}: got {int(got[i]):#x} want {int(want[i]):#x}")


def assert_scales(got, want, what):
    g, w = bits(got).reshape(-1), want.contiguous().view(torch.int32).reshape(-1)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.shape[0]} scale mismatches, first at {i}: got {int(g[i]):#x} want {int(w[i]):#x}")


def all_bf16_patterns():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


# ---------------------------------------------------------------------------- rowwise
def test_rowwise_cfg1(dev):
    """benchmark config 1: [4864, 896], N(0, 0.02) with 0.1% x20 outliers, seed 1235."""
    w = O.make_weight((4864, 896), seed=1235, outlier_frac=1e-3, outlier_mul=20.0)
    q, s = ops.scaled_fp8_quant(w.to(dev), scale=None, use_per_token_if_dynamic=True)
    assert q.dtype == torch.float8_e4m3fn and tuple(s.shape) == (4864, 1)
    qo, so = O.quant_rowwise(w)
    assert_scales(s, so, "cfg1 scales")
    assert_bytes(q, qo, "cfg1 bytes")


@pytest.mark.parametrize("cols", [8, 64, 136, 512, 896, 1024, 2048, 3584, 4096, 4104, 8192, 10248, 12288, 12296, 16384,
                                  18944, 20480, 20488, 24576, 24584, 32768, 32776, 40000])
def test_rowwise_widths(dev, cols):
    """Every kernel variant: wave-per-row (V=1,2,4,8), block-per-row (V=4,5,6,8,10,12,16) on both sides of each
    limit, streaming."""
    rows = 37 if cols < 20000 else 5
    g = torch.Generator().manual_seed(cols)
    w = (torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * 3)).to(torch.bfloat16)
    q, s = ops.quant_rowwise(w.to(dev))
    qo, so = O.quant_rowwise(w)
    assert_scales(s, so, f"cols={cols} scales")
    assert_bytes(q, qo, f"cols={cols} bytes")


def test_rowwise_exhaustive_patterns(dev):
    """All 65536 bf16 patterns as data under 256 different row scales.  For one planted amax
    `a`, the patterns whose magnitude does not exceed `a` (others become 0) are spread over 16
    rows of 4096 columns; element 0 of each row is overwritten with `a` so that every row has
    exactly that amax, and a 17th row carries the 16 overwritten patterns."""
    pats = all_bf16_patterns()
    pf = pats.float()
    g = torch.Generator().manual_seed(7)
    finite_pos = pats[torch.isfinite(pf) & (pf > 0)]
    amaxes = torch.cat([torch.exp(torch.rand(200, generator=g) * 60 - 40).to(torch.bfloat16),
                        torch.tensor([448.0, 1.0, 2.0 ** -20, 3.0e38]).to(torch.bfloat16),
                        finite_pos[torch.randint(0, finite_pos.numel(), (52,), generator=g)]])
    blocks = []
    for a in amaxes:
        keep = torch.isfinite(pf) & (pf.abs() <= a.float())
        body = torch.where(keep, pats, torch.zeros_like(pats)).view(16, 4096).clone()
        extra = torch.zeros(1, 4096, dtype=torch.bfloat16)
        extra[0, 1:17] = body[:, 0]
        extra[0, 0] = a
        body[:, 0] = a
        blocks += [body, extra]
    w = torch.cat(blocks)
    q, s = ops.quant_rowwise(w.to(dev))
    qo, so = O.quant_rowwise(w)
    assert_scales(s, so, "exhaustive scales")
    assert_bytes(q, qo, "exhaustive bytes")


def test_rowwise_edge_rows(dev):
    """zero row (scale 0x2720D7C5, bytes 0x00/0x80), NaN row, Inf row, subnormals, ragged stride."""
    cols = 256
    w = torch.zeros(6, cols, dtype=torch.bfloat16)
    w[0, 3] = -0.0
    w[1, 5] = float("nan"); w[1, 6] = 1.0
    w[2, 7] = float("inf"); w[2, 8] = -2.0; w[2, 9] = float("-inf")
    w[3] = torch.linspace(-1e-38, 1e-38, cols).to(torch.bfloat16)
    w[4] = torch.linspace(-3, 3, cols).to(torch.bfloat16)
    w[5, 0] = 1e-13
    q, s = ops.quant_rowwise(w.to(dev))
    qo, so = O.quant_rowwise(w)
    assert int(bits(s)[0]) == 0x2720D7C5
    assert set(u8(q)[0].tolist()) <= {0x00, 0x80} and int(u8(q)[0, 3]) == 0x80
    assert_scales(s, so, "edge scales")
    assert_bytes(q, qo, "edge bytes")
    # non-contiguous rows (a column slice keeps stride(1) == 1)
    big = O.make_weight((64, 1024), seed=3)
    view = big.to(dev)[:, 128:640]
    q2, s2 = ops.quant_rowwise(view)
    qo2, so2 = O.quant_rowwise(big[:, 128:640].contiguous())
    assert_scales(s2, so2, "strided scales")
    assert_bytes(q2, qo2, "strided bytes")


def test_rowwise_empty_and_errors(dev):
    q, s = ops.quant_rowwise(torch.empty(0, 128, dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 128) and s.shape == (0, 1)
    with pytest.raises(ValueError):
        ops.quant_rowwise(torch.zeros(4, 12, dtype=torch.bfloat16, device=dev))  # cols % 8
    with pytest.raises(ValueError):
        ops.quant_rowwise(torch.zeros(4, 16, dtype=torch.float32, device=dev))
    with pytest.raises(RuntimeError):
        ops.quant_rowwise(torch.zeros(4, 16, dtype=torch.bfloat16))  # CPU tensor: no fallback


def test_rowwise_properties_full_size(dev):
    """Qwen2.5-7B gate_up [37888, 3584] on the GPU only: every non-zero row holds a +-448 byte,
    re-quantising the dequantised tensor is idempotent, and row permutation commutes."""
    g = torch.Generator(device=dev).manual_seed(11)
    w = (torch.randn(37888, 3584, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    q, s = ops.quant_rowwise(w)
    qb = q.view(torch.uint8)
    assert bool((((qb & 0x7F) == 0x7E).any(dim=1)).all())
    deq = (q.float() * s).to(torch.bfloat16)
    q2, s2 = ops.quant_rowwise(deq)
    # dequantised values are bf16-rounded, so compare through one more round trip
    q3, s3 = ops.quant_rowwise((q2.float() * s2).to(torch.bfloat16))
    assert torch.equal(q2.view(torch.uint8), q3.view(torch.uint8))
    perm = torch.randperm(37888, generator=g, device=dev)
    qp, sp = ops.quant_rowwise(w[perm])
    assert torch.equal(qp.view(torch.uint8), qb[perm]) and torch.equal(sp, s[perm])


def _recv(rows, cols, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * 3)
    if dtype == torch.float16:
        w = w.clamp(-6e4, 6e4)
    w = w.to(dtype)
    if rows > 4:
        w[0] = 0
        w[1, 3] = float("nan")
        w[2, 5] = float("inf")
        if dtype == torch.float32:
            w[3, :8] = torch.tensor([0x3F808000, 0x3F818000, 0x7F7FFFFF, 0x00008000, 0x00018000, 0x80008000, 0x3F807FFF,
                                     0x3FFF8000], dtype=torch.int64).to(torch.int32).view(torch.float32)
            w[4] = 3.3e38
        if dtype == torch.float16:
            w[3, :4] = torch.tensor([0x0001, 0x03FF, 0x8001, 0x7BFF], dtype=torch.int32).to(torch.int16).view(torch.float16)
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cols", [8, 136, 896, 3584, 4104, 18944, 40000])
def test_rowwise_from_transfer_dtype(dev, dtype, cols):
    """cfp8_quant_rowwise_from: quant_rowwise(recv.to(bf16)) for every source dtype and kernel variant,
    bytes and scales bit-exact, written straight into caller storage."""
    rows = 21 if cols < 20000 else 5
    w = _recv(rows, cols, dtype, seed=cols + 1)
    q = torch.empty(rows, cols, dtype=torch.float8_e4m3fn, device=dev)
    s = torch.empty(rows, 1, dtype=torch.float32, device=dev)
    ops.quant_rowwise_into(w.to(dev), q, s)
    qo, so = O.quant_rowwise_from(w)
    assert_scales(s, so, f"{dtype} cols={cols} scales")
    assert_bytes(q, qo, f"{dtype} cols={cols} bytes")


def test_rowwise_from_into_engine_parameter(dev):
    """Destination = a row range of the engine's transposed fp8 parameter (strides (1, in_dim)) and of its
    [out, 1] scale parameter; rows outside the range stay untouched."""
    out_dim, in_dim, a, b = 96, 264, 16, 80
    w = _recv(b - a, in_dim, torch.float32, seed=3)
    buf = torch.full((out_dim, in_dim), 0x55, dtype=torch.uint8, device=dev)
    param = buf.view(torch.float8_e4m3fn).t()                  # [in_dim, out_dim], strides (1, in_dim)
    scale = torch.full((out_dim, 1), -1.0, dtype=torch.float32, device=dev)
    ops.quant_rowwise_into(w.to(dev), param[:, a:b], scale[a:b])
    qo, so = O.quant_rowwise_from(w)
    assert_bytes(buf[a:b], qo, "rows in range")
    assert_scales(scale[a:b], so, "scales in range")
    assert (buf[:a] == 0x55).all() and (buf[b:] == 0x55).all()
    assert (scale[:a] == -1).all() and (scale[b:] == -1).all()
    with pytest.raises(ValueError):
        ops.quant_rowwise_into(w.to(dev), param[:, a:b + 1], scale[a:b])
    with pytest.raises(ValueError):
        ops.quant_rowwise_into(w.to(dev).to(torch.float64), param[:, a:b], scale[a:b])


def test_rowwise_multi_matches_single_calls_and_oracle(dev):
    """cfp8_quant_rowwise_multi: a batch that mixes every kernel variant (row lengths 8 .. 40000), the three source
    dtypes, empty tensors and more tensors of one class than a launch table holds - bytes and scales equal the
    oracle's and those of one call per tensor."""
    spec = [(37, 8, torch.bfloat16), (21, 136, torch.float32), (64, 896, torch.bfloat16), (33, 3584, torch.bfloat16),
            (5, 3584, torch.float16), (12, 4104, torch.bfloat16), (9, 18944, torch.bfloat16), (3, 40000, torch.bfloat16),
            (0, 64, torch.bfloat16), (7, 18944, torch.float32), (16, 1288, torch.bfloat16), (4, 2056, torch.bfloat16),
            (6, 2568, torch.bfloat16), (2, 3080, torch.bfloat16)]
    spec += [(4 + i % 7, 3584, torch.bfloat16) for i in range(45)]        # one class, more than one table
    ws = [_recv(r, c, dt, seed=1000 + i) for i, (r, c, dt) in enumerate(spec)]
    gs = [w.to(dev) for w in ws]
    qs = [torch.full(w.shape, 0x55, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn) for w in ws]
    ss = [torch.full((w.shape[0], 1), -1.0, dtype=torch.float32, device=dev) for w in ws]
    ops.quant_rowwise_multi_into(gs, qs, ss)
    for i, w in enumerate(ws):
        if w.shape[0] == 0:
            continue
        qo, so = O.quant_rowwise_from(w)
        assert_scales(ss[i], so, f"tensor {i} {tuple(w.shape)} {w.dtype} scales")
        assert_bytes(qs[i], qo, f"tensor {i} {tuple(w.shape)} {w.dtype} bytes")
        q1 = torch.empty_like(qs[i]); s1 = torch.empty_like(ss[i])
        ops.quant_rowwise_into(gs[i], q1, s1)
        assert torch.equal(q1.view(torch.uint8), qs[i].view(torch.uint8)) and torch.equal(bits(s1), bits(ss[i]))
    q2, s2 = ops.quant_rowwise_multi(gs[:4])
    assert all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(q2, qs[:4]))
    assert tuple(s2[0].shape) == (37, 1)


def test_rowwise_multi_into_engine_parameters(dev):
    """Destinations are the engine's transposed fp8 parameters (strides (1, in_dim)), one of them a row range."""
    shapes = [(96, 264), (64, 264), (48, 1024)]
    ws = [_recv(r, c, torch.bfloat16, seed=50 + i) for i, (r, c) in enumerate(shapes)]
    bufs = [torch.full((r + 8, c), 0x55, dtype=torch.uint8, device=dev) for r, c in shapes]
    params = [b.view(torch.float8_e4m3fn).t()[:, 4:4 + r] for b, (r, c) in zip(bufs, shapes)]
    scales = [torch.empty(r, 1, dtype=torch.float32, device=dev) for r, _ in shapes]
    ops.quant_rowwise_multi_into([w.to(dev) for w in ws], params, scales)
    for w, b, sc in zip(ws, bufs, scales):
        qo, so = O.quant_rowwise(w)
        assert_bytes(b[4:4 + w.shape[0]], qo, "rows in range")
        assert_scales(sc, so, "scales")
        assert (b[:4] == 0x55).all() and (b[4 + w.shape[0]:] == 0x55).all()
    with pytest.raises(ValueError):
        ops.quant_rowwise_multi_into([ws[0].to(dev)], params[:1], [scales[0][:5]])
    with pytest.raises(ValueError):
        ops.quant_rowwise_multi_into([ws[0].to(dev)], params[:1], scales[:2])


# ---------------------------------------------------------------------------- tensorwise
def test_tensorwise_multi(dev):
    """A Qwen2.5-7B-shaped layer set at reduced width plus ragged extras, in one call."""
    shapes = [(3584, 512), (512, 512), (512, 512), (3584, 512), (1184, 512), (1184, 512), (512, 1184),
              (8, 8), (1, 8), (300, 72), (2048 * 8 + 8,), (0, 16)]
    ws = [O.make_weight(sh, seed=100 + i, std=0.02 * (i + 1)) for i, sh in enumerate(shapes)]
    qs, scales = ops.quant_tensorwise_multi([w.to(dev) for w in ws])
    for i, w in enumerate(ws):
        qo, so = O.quant_tensorwise(w)
        assert_scales(scales[i:i + 1], so, f"tensor {i} scale")
        assert_bytes(qs[i], qo, f"tensor {i} bytes")
        assert qs[i].shape == w.shape


def test_tensorwise_many_tensors_and_batches(dev, monkeypatch):
    """More tensors than one descriptor table holds (48), so several batches are launched."""
    ws = [O.make_weight((16 + 8 * (i % 5), 64), seed=500 + i, std=0.01 * (1 + i % 7)) for i in range(131)]
    qs, scales = ops.quant_tensorwise_multi([w.to(dev) for w in ws])
    for i, w in enumerate(ws):
        qo, so = O.quant_tensorwise(w)
        assert_scales(scales[i:i + 1], so, f"tensor {i} scale")
        assert_bytes(qs[i], qo, f"tensor {i} bytes")


def test_tensorwise_edges(dev):
    w = torch.zeros(64, 64, dtype=torch.bfloat16)
    q, s = ops.quant_tensorwise(w.to(dev))
    assert int(bits(s)[0]) == 0x2720D7C5 and int(u8(q).max()) == 0
    w[5, 5] = float("nan")
    q, s = ops.quant_tensorwise(w.to(dev))
    qo, so = O.quant_tensorwise(w)
    assert_scales(s, so, "nan scale"); assert_bytes(q, qo, "nan bytes")
    w[5, 5] = float("inf"); w[6, 6] = 3.0
    q, s = ops.quant_tensorwise(w.to(dev))
    qo, so = O.quant_tensorwise(w)
    assert_scales(s, so, "inf scale"); assert_bytes(q, qo, "inf bytes")
    # scaled_fp8_quant without per-token = tensorwise
    w = O.make_weight((96, 160), seed=9)
    q, s = ops.scaled_fp8_quant(w.to(dev))
    qo, so = O.quant_tensorwise(w)
    assert tuple(s.shape) == (1,)
    assert_scales(s, so, "per-tensor scale"); assert_bytes(q, qo, "per-tensor bytes")


def _two_pass(tensors, dev):
    """The split-phase entry points in sequence: always the two separate launches."""
    n = len(tensors)
    qs = [torch.empty(t.shape, dtype=torch.float8_e4m3fn, device=dev) for t in tensors]
    sc = torch.empty(n, dtype=torch.float32, device=dev)
    ws = torch.empty(n * _lib.TENSORWISE_AMAX_SLOTS, dtype=torch.float32, device=dev)
    d = (_lib.TensorDesc * n)()
    for i, (t, q) in enumerate(zip(tensors, qs)):
        d[i].x, d[i].q, d[i].scale, d[i].numel = t.data_ptr(), q.data_ptr(), sc.data_ptr() + 4 * i, t.numel()
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(_lib.load().cfp8_tensorwise_amax_multi(d, n, ws.data_ptr(), st))
    _lib.check(_lib.load().cfp8_tensorwise_cast_multi(d, n, ws.data_ptr(), st))
    return qs, sc


def test_tensorwise_read_once_launch(dev):
    """Tensors large enough for the launch that keeps them on the chip between the passes (106-141 MB), mixed
    with smaller ones in one call: against the oracle, against the two separate passes, twice in a row, with a
    NaN and an infinity (the scale is then not finite and the bytes take the integer path), through the entry
    point that allocates nothing, and with the launch switched off."""
    lib = _lib.load()
    assert lib.cfp8_tensorwise_resident(-1) == 0          # opt-in: off until a caller says the GPU is its own
    lib.cfp8_tensorwise_resident(1)
    g = torch.Generator(device=dev).manual_seed(77)
    shapes = [(18944, 3584), (512, 3584), (14336, 4096), (3584, 3584), (3584, 18944), (13568, 4096), (17280, 4096)]
    ws = [(torch.randn(sh, generator=g, device=dev) * (0.01 * (i + 1))).to(torch.bfloat16) for i, sh in enumerate(shapes)]
    # amax = 0.00799560546875: fp32(amax / fp32(amax / 448)) is 448.0000305, the value next to 448 - the resident
    # kernel's cast has no clamp and relies on the conversion to round that to 448
    ws[0].clamp_(-0.0079, 0.0079)
    ws[0][0, 0], ws[0][18943, 3583], ws[0][9000, 77] = 0.00799560546875, -0.00799560546875, 0.00799560546875
    ws[0][5, 5], ws[0][5, 6] = -0.0, 0.0     # signed zeros keep their sign (bytes 0x80 and 0x00)
    ws[2][7000, 123] = float("inf")          # non-finite scale in a tensor that is kept on the chip
    ws[4][11, 18000] = float("nan")
    ws[5].zero_()                             # amax 0: the scale floor
    ws[6][17279, 4095] = 300.0               # exactly the capacity of 256 CUs; the maximum in the last element of the last chunk
    qs, scales, given_up = ops.quant_tensorwise_multi(ws, return_status=True)
    assert int(given_up) == 0                             # every meeting of the read-once launch completed
    q2, s2 = _two_pass(ws, dev)
    for i in range(len(ws)):
        assert torch.equal(u8(qs[i]), u8(q2[i])), f"tensor {i}: bytes differ from the two separate passes"
    assert torch.equal(bits(scales), bits(s2))
    for i in (0, 2, 4, 5, 6):                 # the oracle on the CPU: a second or two per tensor of this size
        qo, so = O.quant_tensorwise(ws[i].cpu())
        assert_scales(scales[i:i + 1], so, f"tensor {i} scale")
        assert_bytes(qs[i], qo, f"tensor {i} bytes")
    assert int(bits(scales)[5]) == 0x2720D7C5 and int(u8(qs[5]).max()) == 0
    assert [int(u8(qs[0])[i, j]) for i, j in ((0, 0), (18943, 3583), (9000, 77))] == [0x7E, 0xFE, 0x7E]
    assert float(ws[0][0, 0].float().cpu() / scales[0].cpu()) > 448.0
    assert int(u8(qs[0])[5, 5]) == 0x80 and int(u8(qs[0])[5, 6]) == 0x00
    # the meeting words are cleared in front of every launch: a second call starts from zero again
    qs_b, scales_b = ops.quant_tensorwise_multi(ws)
    assert all(torch.equal(u8(a), u8(b)) for a, b in zip(qs, qs_b)) and torch.equal(bits(scales), bits(scales_b))
    # the library's own slots
    outs = [torch.empty(w.shape, dtype=torch.float8_e4m3fn, device=dev) for w in ws]
    sc = torch.empty(len(ws), dtype=torch.float32, device=dev)
    ops.quant_tensorwise_multi_static(ws, outs, sc)
    assert all(torch.equal(u8(a), u8(b)) for a, b in zip(qs, outs)) and torch.equal(bits(scales), bits(sc))
    # switched off: every tensor takes the two separate passes; same results
    assert lib.cfp8_tensorwise_resident(0) == 1
    qs_c, scales_c = ops.quant_tensorwise_multi(ws)
    assert all(torch.equal(u8(a), u8(b)) for a, b in zip(qs, qs_c)) and torch.equal(bits(scales), bits(scales_c))
    with ops.gpu_is_mine():
        assert lib.cfp8_tensorwise_resident(-1) == 1
    assert lib.cfp8_tensorwise_resident(-1) == 0


def test_tensorwise_read_once_launch_gives_up_and_is_repaired(dev):
    """The read-once launch when its workgroups cannot meet.  Forced from the host: every meeting expects one arrival
    more than the grid has workgroups and waits 1 ms, so no meeting completes, every workgroup gives the first
    tensor up and leaves its kernel normally; the repair kernels behind the launch redo the given-up tensors as two
    ordinary passes.  Results must be the bits of the two-pass path, the status count must name the large tensors,
    and with the real arrival count restored the same call reports none."""
    lib = _lib.load()
    g = torch.Generator(device=dev).manual_seed(78)
    shapes = [(18944, 3584), (512, 3584), (3584, 18944), (64, 64), (13568, 4096)]
    ws = [(torch.randn(sh, generator=g, device=dev) * (0.01 * (i + 1))).to(torch.bfloat16) for i, sh in enumerate(shapes)]
    ws[2][5, 5] = float("nan")
    want_q, want_s = _two_pass(ws, dev)
    prev = lib.cfp8_tensorwise_resident(1)
    try:
        _lib.check(lib.cfp8_tensorwise_resident_tuning(1000, 1))
        torch.cuda.synchronize()
        qs, scales, given_up = ops.quant_tensorwise_multi(ws, return_status=True)
        torch.cuda.synchronize()
        assert int(given_up) == 3, f"{int(given_up)} tensors reported as given up, 3 took the read-once launch"
        assert torch.equal(bits(scales), bits(want_s)), "scales after repair differ from the two passes"
        for i in range(len(ws)):
            assert torch.equal(u8(qs[i]), u8(want_q[i])), f"tensor {i}: bytes after repair differ from the two passes"
        # the library's own slots: same path, status read with a null workspace
        outs = [torch.empty(w.shape, dtype=torch.float8_e4m3fn, device=dev) for w in ws]
        sc = torch.empty(len(ws), dtype=torch.float32, device=dev)
        ops.quant_tensorwise_multi_static(ws, outs, sc)
        cnt = torch.zeros((), dtype=torch.int32, device=dev)
        _lib.check(lib.cfp8_tensorwise_status(None, len(ws), cnt.data_ptr(), torch.cuda.current_stream().cuda_stream))
        assert int(cnt) == 3
        assert all(torch.equal(u8(a), u8(b)) for a, b in zip(outs, want_q)) and torch.equal(bits(sc), bits(want_s))
    finally:
        _lib.check(lib.cfp8_tensorwise_resident_tuning(20000, 0))
    try:
        qs, scales, given_up = ops.quant_tensorwise_multi(ws, return_status=True)
        assert int(given_up) == 0
        assert torch.equal(bits(scales), bits(want_s)) and all(torch.equal(u8(a), u8(b)) for a, b in zip(qs, want_q))
    finally:
        lib.cfp8_tensorwise_resident(prev)


def test_tensorwise_read_once_several_tensors_at_a_time(dev):
    """Tensors of a half to an eighth of the chip's capacity are held several at a time, each by a group of CUs that
    meets within itself.  Every group count the library uses (8, 5, 3, 2 and 1 on 256 CUs), more tensors than groups so
    that a second round runs with some groups idle, sizes that differ within a class, a NaN, an infinity and an
    all-zero tensor among them: the bits of the two separate passes, and again after every meeting has been made to
    give up from the host (all 26 tensors reported, all repaired)."""
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    if cus != 256:
        pytest.skip("the shapes below are sized for the group capacities of 256 CUs")
    g = torch.Generator(device=dev).manual_seed(81)
    rows = [2048] * 6 + [2304] * 5 + [3584] * 4 + [3840] * 3 + [6000] * 2 + [6400] * 2 + [8192, 9000, 9728] + [18944]
    ws = [(torch.randn(r, 3584, generator=g, device=dev) * (0.01 * (i % 7 + 1))).to(torch.bfloat16) for i, r in enumerate(rows)]
    ws[3][2047, 3583] = float("nan")       # group count 8, first round
    ws[9][0, 0] = float("inf")             # group count 8, second round
    ws[12].zero_()                          # group count 5: the scale floor
    ws[16][3839, 3583] = 250.0             # the maximum in the tensor's last element
    ws[20][5999, 0] = -300.0
    want_q, want_s = _two_pass(ws, dev)
    prev = lib.cfp8_tensorwise_resident(1)
    try:
        for _ in range(2):
            qs, scales, given_up = ops.quant_tensorwise_multi(ws, return_status=True)
            assert int(given_up) == 0
            assert torch.equal(bits(scales), bits(want_s)), "scales differ from the two passes"
            for i in range(len(ws)):
                assert torch.equal(u8(qs[i]), u8(want_q[i])), f"tensor {i} ({rows[i]} rows): bytes differ from the two passes"
        assert int(bits(scales)[12]) == 0x2720D7C5 and int(u8(qs[12]).max()) == 0
        _lib.check(lib.cfp8_tensorwise_resident_tuning(1000, 1))
        try:
            torch.cuda.synchronize()
            qs, scales, given_up = ops.quant_tensorwise_multi(ws, return_status=True)
            torch.cuda.synchronize()
            assert int(given_up) == len(ws), f"{int(given_up)} tensors reported as given up, {len(ws)} took the read-once launch"
            assert torch.equal(bits(scales), bits(want_s)), "scales after repair differ from the two passes"
            for i in range(len(ws)):
                assert torch.equal(u8(qs[i]), u8(want_q[i])), f"tensor {i}: bytes after repair differ from the two passes"
        finally:
            _lib.check(lib.cfp8_tensorwise_resident_tuning(20000, 0))
    finally:
        lib.cfp8_tensorwise_resident(prev)


def test_tensorwise_read_once_launches_on_two_streams(dev):
    """Two read-once calls at the same time on two streams of one process - what the entry point's contract rules out.
    Each launch needs every CU, so they cannot both be resident, and they share the array through which workgroups
    meet; the launch number in every meeting tag keeps either from taking the other's words for arrivals.  Whatever
    the hardware makes of the overlap (one launch after the other, or meetings that run into the bound of the wait
    and are repaired), both calls must return the bits of the two-pass path."""
    lib = _lib.load()
    g = torch.Generator(device=dev).manual_seed(80)
    sets = [[(torch.randn(18944, 3584, generator=g, device=dev) * (0.01 * (i + 1 + 3 * k))).to(torch.bfloat16) for i in range(3)] for k in range(2)]
    wants = [_two_pass(ws, dev) for ws in sets]
    prev = lib.cfp8_tensorwise_resident(1)
    try:
        _lib.check(lib.cfp8_tensorwise_resident_tuning(3000, 0))
        streams = [torch.cuda.Stream(device=dev) for _ in range(2)]
        torch.cuda.synchronize()
        got = [None, None]
        for _ in range(3):
            for k in range(2):
                with torch.cuda.stream(streams[k]):
                    got[k] = ops.quant_tensorwise_multi(sets[k])
            torch.cuda.synchronize()
            for k in range(2):
                qs, scales = got[k]
                assert torch.equal(bits(scales), bits(wants[k][1])), f"stream {k}: scales differ from the two passes"
                assert all(torch.equal(u8(a), u8(b)) for a, b in zip(qs, wants[k][0])), f"stream {k}: bytes differ from the two passes"
    finally:
        _lib.check(lib.cfp8_tensorwise_resident_tuning(20000, 0))
        lib.cfp8_tensorwise_resident(prev)


def test_tensorwise_split_phase_cast_saturates(dev):
    """The split-phase cast with slots that hold LESS than the tensor's own maximum (another rank's data, a stale
    workspace): quotients beyond 448 saturate to +-448 like the reference's clamp, infinities too, NaN stays NaN."""
    g = torch.Generator().manual_seed(79)
    x = (torch.randn(300, 1024, generator=g) * 0.02).to(torch.bfloat16)
    x[0, 0], x[0, 1], x[0, 2], x[0, 3], x[0, 4] = 5.0, -7.0, float("inf"), float("-inf"), float("nan")
    x[1, 0], x[1, 1] = 3.0e38, -3.0e38
    xd = x.to(dev)
    n = 1
    q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=dev)
    sc = torch.empty(n, dtype=torch.float32, device=dev)
    ws = torch.zeros(n * _lib.TENSORWISE_AMAX_SLOTS, dtype=torch.float32, device=dev)
    amax = torch.tensor(0.05, dtype=torch.float32)           # smaller than the data's maximum
    ws[3] = amax
    d = (_lib.TensorDesc * n)()
    d[0].x, d[0].q, d[0].scale, d[0].numel = xd.data_ptr(), q.data_ptr(), sc.data_ptr(), xd.numel()
    _lib.check(_lib.load().cfp8_tensorwise_cast_multi(d, n, ws.data_ptr(), torch.cuda.current_stream().cuda_stream))
    scale = amax / 448.0
    assert torch.equal(bits(sc), scale.view(torch.int32).reshape(1))
    want = O._cast_with_scale(x.float(), scale)
    assert_bytes(q, want, "saturating split-phase cast")
    assert [int(v) for v in u8(q)[0, :5]] == [0x7E, 0xFE, 0x7E, 0xFE, 0x7F] and [int(v) for v in u8(q)[1, :2]] == [0x7E, 0xFE]


def test_tensorwise_qwen25_7b_full_pass(dev):
    """The benchmark's headline call itself: all 197 linear weights of a Qwen2.5-7B-shaped decoder (7.07e9 elements) in
    one cfp8_quant_tensorwise_multi call with the read-once launch allowed, i.e. two resident launches of 48 + 36
    tensors and the two passes over the other 113.  Every scale against the closed form of torch's amax, and for
    every tensor four sampled rows of bytes against the oracle's cast with that scale; then the same through the
    entry point that allocates nothing."""
    lib = _lib.load()
    shapes = [((3584, 3584), 28), ((3584, 3584), 28), ((512, 3584), 28), ((512, 3584), 28), ((18944, 3584), 28),
              ((18944, 3584), 28), ((3584, 18944), 28), ((152064, 3584), 1)]
    g = torch.Generator(device=dev).manual_seed(1236)
    tensors = []
    for k, (sh, mult) in enumerate(shapes):
        for j in range(mult):
            t = torch.empty(sh, dtype=torch.bfloat16, device=dev)
            t.normal_(0.0, 0.02 * (1 + (k + j) % 3), generator=g)   # neighbouring tensors differ in scale
            tensors.append(t)
    n = len(tensors)
    assert n == 197 and sum(t.numel() for t in tensors) == 7_070_285_824
    amax = torch.stack([t.abs().amax().float() for t in tensors]).cpu()
    want_scales = O.scale_from_amax(amax)

    def check(outs, scales, what):
        assert_scales(scales, want_scales, f"{what}: scales")
        for i, (t, q) in enumerate(zip(tensors, outs)):
            rows = torch.tensor([0, t.shape[0] // 3, (2 * t.shape[0]) // 3 + 1, t.shape[0] - 1])
            want = O._cast_with_scale(t[rows.to(dev)].cpu(), want_scales[i])
            assert_bytes(q.view(torch.uint8)[rows.to(dev)], want, f"{what}: tensor {i} {tuple(t.shape)} rows {rows.tolist()}")

    prev = lib.cfp8_tensorwise_resident(1)
    try:
        outs, scales, given_up = ops.quant_tensorwise_multi(tensors, return_status=True)
        assert int(given_up) == 0
        check(outs, scales, "workspace entry")
        for q in outs:
            q.view(torch.uint8).fill_(0x55)
        sc = torch.full((n,), -1.0, dtype=torch.float32, device=dev)
        ops.quant_tensorwise_multi_static(tensors, outs, sc)
        check(outs, sc, "no-allocation entry")
    finally:
        lib.cfp8_tensorwise_resident(prev)


def test_tensorwise_full_size_properties(dev):
    """lm_head-sized tensor [152064, 3584] on the GPU only: scale equals the closed form of the
    torch amax, the set holds +-448, and the bytes equal a rowwise-kernel-free recomputation on a
    slice checked against the oracle."""
    g = torch.Generator(device=dev).manual_seed(5)
    w = (torch.randn(152064, 3584, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    q, s = ops.quant_tensorwise(w)
    amax = w.abs().amax().float().cpu()  # CPU: torch's GPU division by a scalar is a reciprocal multiply
    want = torch.clamp(amax, min=1e-12) / 448.0
    assert torch.equal(s.cpu().view(torch.int32), want.reshape(1).view(torch.int32))
    assert bool(((q.view(torch.uint8) & 0x7F) == 0x7E).any())
    rows = torch.tensor([0, 1, 77777, 152063])
    sl = w[rows.to(dev)].cpu()
    want_bytes = O._cast_with_scale(sl, s.cpu())
    assert_bytes(q[rows.to(dev)], want_bytes, "lm_head slice")


# ---------------------------------------------------------------------------- block 128x128
@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (200, 136), (1, 8), (130, 1032), (3, 256, 384), (2, 200, 136)])
def test_block128(dev, shape):
    w = O.make_weight(shape, seed=sum(shape), std=0.02)
    # per-block dynamic range
    w = (w.float() * torch.exp(torch.randn(*shape, generator=torch.Generator().manual_seed(1)) * 0.5)).to(torch.bfloat16)
    q, s = ops.per_block_cast_to_fp8(w.to(dev))
    qo, so = O.quant_block128(w)
    assert s.shape == so.shape
    assert_scales(s, so, f"block {shape} scales")
    assert_bytes(q, qo, f"block {shape} bytes")


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (208, 136), (2, 144, 264)])
def test_block128_transposed(dev, shape):
    w = O.make_weight(shape, seed=sum(shape) + 1, std=0.05)
    q, s = ops.per_block_cast_to_fp8(w.to(dev), transpose_out=True)
    qo, so = O.quant_block128(w)
    assert_scales(s, so, f"blockT {shape} scales")
    assert_bytes(q, qo.transpose(-1, -2).contiguous(), f"blockT {shape} bytes")


def test_block128_cfg4_and_dequant_roundtrip(dev):
    """benchmark config 4 weight [7168, 18432] -> scales [56, 144]; a 512x512 corner against the
    oracle, the whole tensor through weight_dequant (the in-tree inverse pins the layout)."""
    w = O.make_weight((7168, 18432), seed=1238)
    wd = w.to(dev)
    q, s = ops.prepare_fp8_weight(wd)
    assert tuple(s.shape) == (56, 144)
    qo, so = O.quant_block128(w[:512, 17920:])
    assert_scales(s[:4, 140:], so, "cfg4 corner scales")
    assert_bytes(q[:512, 17920:], qo, "cfg4 corner bytes")
    y = ops.weight_dequant(q, s, out_dtype=torch.float32)
    blocks_amax = wd.float().abs().view(56, 128, 144, 128).amax(dim=(1, 3))
    err = (y - wd.float()).abs().view(56, 128, 144, 128).amax(dim=(1, 3))
    # half an e4m3 ulp at the top binade is 16/448 of amax; values are far below that bound mostly
    assert bool((err <= blocks_amax * (16.0 / 448.0) * 1.001 + 1e-30).all())
    yo = O.weight_dequant(u8(q[:256, :256]), s[:2, :2].cpu())
    assert torch.equal(y[:256, :256].cpu(), yo)
    yb = ops.weight_dequant(q[:256, :256].contiguous(), s[:2, :2].contiguous(), out_dtype=torch.bfloat16)
    assert torch.equal(yb.cpu(), yo.to(torch.bfloat16))


@pytest.mark.parametrize("shape", [(1, 8), (5, 24), (130, 520), (131, 1032), (257, 2056), (1048700, 8)])
def test_weight_dequant_shapes(dev, shape):
    """Ragged rows and columns at each block width of the dequantiser (64, 128, 256 vectors), and a matrix with
    more row quads than the grid's y extent holds (the kernel then strides): bit-equal to the oracle, both dtypes."""
    M, N = shape
    g = torch.Generator().manual_seed(M * 31 + N)
    q = torch.randint(0, 256, (M, N), generator=g, dtype=torch.uint8)
    q[q == 0x7F] = 0x7E
    q[q == 0xFF] = 0xFE
    s = torch.rand((M + 127) // 128, (N + 127) // 128, generator=g) * 3e-3 + 1e-5
    yo = O.weight_dequant(q, s)
    qd = q.to(dev).view(torch.float8_e4m3fn)
    y = ops.weight_dequant(qd, s.to(dev), out_dtype=torch.float32)
    assert torch.equal(y.cpu(), yo)
    yb = ops.weight_dequant(qd, s.to(dev), out_dtype=torch.bfloat16)
    assert torch.equal(yb.cpu(), yo.to(torch.bfloat16))


# ---------------------------------------------------------------------------- 1x128 groups
@pytest.mark.parametrize("shape", [(4, 128), (33, 896), (7, 200), (1, 8), (129, 2048), (64, 7168)])
def test_group128(dev, shape):
    x = O.make_activation(*shape, seed=shape[0] * 31 + shape[1], chan_outlier_frac=0.01, outlier_mul=30.0)
    q, s = ops.groupwise_activation_quant(x.to(dev))
    qo, so = O.quant_group128(x)
    assert_scales(s, so, f"group {shape} scales")
    assert_bytes(q, qo, f"group {shape} bytes")


@pytest.mark.parametrize("shape", [(4, 128), (33, 896), (7, 200), (129, 2048)])
def test_group128_deepep_formula(dev, shape):
    """per_token_cast_to_fp8 exactly as the reference's tests/test_deepep.py states it."""
    x = O.make_activation(*shape, seed=shape[0] * 17 + shape[1])
    x[0, :8] = 0
    if shape[1] >= 256:
        x[1, 128:256] = 1e-6  # below the 1e-4 amax floor
    q, s = ops.per_token_cast_to_fp8(x.to(dev))
    qo, so = O.group128_cast_deepep(x)
    assert_scales(s, so, f"deepep {shape} scales")
    assert_bytes(q, qo, f"deepep {shape} bytes")


@pytest.mark.parametrize("shape", [(4, 128), (33, 896), (7, 200), (1, 8), (129, 2048), (4096, 7168), (1048700, 8)])
def test_per_token_cast_back(dev, shape):
    """per_token_cast_back (tests/test_deepep.py:86-108) with float scales: bit-equal to the oracle in bf16 (NaN
    bytes compare as NaN), the round trip through the quantiser stays within half an e4m3 step, fp32 output too."""
    m, n = shape
    g = torch.Generator().manual_seed(m * 13 + n)
    q = torch.randint(0, 256, (m, n), generator=g, dtype=torch.uint8)
    s = torch.rand(m, (n + 127) // 128, generator=g) * 3e-3 + 1e-6
    want = O.per_token_cast_back(q, s)
    got = ops.per_token_cast_back(q.to(dev).view(torch.float8_e4m3fn), s.to(dev)).cpu()
    nan = want.isnan()
    assert torch.equal(got.isnan(), nan) and torch.equal(got[~nan].view(torch.int16), want[~nan].view(torch.int16))
    got32 = ops.per_token_cast_back(q.to(dev).view(torch.float8_e4m3fn), s.to(dev), out_dtype=torch.float32).cpu()
    want32 = O.group128_dequant(q, s)
    assert torch.equal(got32[~nan], want32[~nan])
    if m <= 4096:
        x = O.make_activation(m, n, seed=m + n)
        qx, sx = ops.per_token_cast_to_fp8(x.to(dev))
        back = ops.per_token_cast_back(qx, sx).float().cpu()
        step = sx.cpu().repeat_interleave(128, 1)[:, :n] * 16.0          # half an e4m3 step at the top binade
        assert bool(((back - x.float()).abs() <= step * 1.01 + x.float().abs() * 2 ** -8).all())


def test_per_token_cast_back_packed_e8m0_scales(dev):
    """The reference's `x_scales.dtype == torch.int` branch: four exponent bytes per int32, lowest byte first."""
    g = torch.Generator().manual_seed(5)
    m, n = 37, 1000                                        # eight groups (two int32 per row), the last one 104 columns
    q = torch.randint(0, 256, (m, n), generator=g, dtype=torch.uint8)
    e = torch.randint(100, 140, (m, 8), generator=g, dtype=torch.uint8)
    e[0, 0], e[1, 1], e[2, 2] = 0, 255, 1                    # zero, infinity, the smallest normal scale
    packed = e.view(torch.int32)
    want = O.per_token_cast_back(q, packed)
    got = ops.per_token_cast_back(q.to(dev).view(torch.float8_e4m3fn), packed.to(dev)).cpu()
    nan = want.isnan()
    assert torch.equal(got.isnan(), nan) and torch.equal(got[~nan].view(torch.int16), want[~nan].view(torch.int16))
    assert ops.per_token_cast_back(torch.empty(0, 16, dtype=torch.float8_e4m3fn, device=dev), torch.empty(0, 1, device=dev)).shape == (0, 16)


def test_group128_edges(dev):
    x = torch.zeros(5, 384, dtype=torch.bfloat16)
    x[1, 130] = float("nan")
    x[2, 10] = float("inf"); x[2, 11] = 1.0
    x[3, 300] = -0.0
    q, s = ops.prepare_fp8_input(x.to(dev))
    qo, so = O.quant_group128(x)
    assert_scales(s, so, "group edge scales")
    assert_bytes(q, qo, "group edge bytes")
    q, s = ops.prepare_fp8_input(torch.empty(0, 256, dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 256) and s.shape == (0, 2)


# ---------------------------------------------------------------------------- SwiGLU + 1x128 requantisation
def _np16(t):
    import numpy as np
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("M,I", [(1, 128), (37, 200), (300, 768), (129, 1536), (64, 8)])
def test_swiglu_quant_bit_exact(dev, M, I):
    """cfp8_swiglu_quant_group128 against the C restatement of the same fp32 operation sequence: bytes and
    scales bit-exact, including NaN / Inf groups, ragged tail groups and saturating products."""
    import numpy as np
    from oracle import c_oracle as C
    g = torch.Generator().manual_seed(M * 7 + I)
    gate = (torch.randn(M, I, generator=g) * 4).to(torch.bfloat16)
    up = (torch.randn(M, I, generator=g) * torch.exp(torch.randn(M, 1, generator=g) * 2)).to(torch.bfloat16)
    if I >= 8:
        gate[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 80.0, -80.0, 1e-3, -1e-3]).to(torch.bfloat16)
    if M > 4:
        gate[1, 3] = float("nan")
        up[2, 5] = float("inf")
        gate[3] = 0
        up[4] = 0
    q, s = ops.swiglu_quant(gate.to(dev), up.to(dev))
    qo, so = C.swiglu_quant_group128(_np16(gate), _np16(up))
    qo, so = torch.from_numpy(qo), torch.from_numpy(so)
    nan = torch.isnan(so)
    assert_scales(s.cpu()[~nan], so[~nan], f"swiglu {M}x{I} scales")
    assert bool(torch.isnan(s.cpu()[nan]).all())
    # NaN groups: canonical 0x7F bytes on both sides
    assert_bytes(q, qo, f"swiglu {M}x{I} bytes")


def test_swiglu_every_gate_pattern(dev):
    """All 65536 bf16 gate patterns, one 1x128 group each (the whole group holds the pattern, up = 1 except one
    element of 0.5): the group's scale is |bf16(silu(g))| / 448, which is injective in that bf16 value, and the
    bytes carry its sign - so equal scales and bytes mean the kernel's SiLU equals the defining fp32 sequence
    of the C restatement after rounding to bf16 for every input, including those that take the hardware
    exponential / reciprocal path."""
    import numpy as np
    from oracle import c_oracle as C
    gate = all_bf16_patterns().reshape(65536, 1).expand(65536, 128).contiguous()
    up = torch.ones(65536, 128, dtype=torch.bfloat16)
    up[:, 5] = 0.5
    q, s = ops.swiglu_quant(gate.to(dev), up.to(dev))
    qo, so = C.swiglu_quant_group128(_np16(gate), _np16(up))
    qo, so = torch.from_numpy(qo), torch.from_numpy(so)
    nan = torch.isnan(so).reshape(-1)
    assert int(nan.sum()) < 600                                         # NaN patterns and -inf
    assert_scales(s.cpu().reshape(-1)[~nan], so.reshape(-1)[~nan], "silu of every bf16 pattern: scales")
    assert bool(torch.isnan(s.cpu().reshape(-1)[nan]).all())
    assert_bytes(q, qo, "silu of every bf16 pattern: bytes")


def test_swiglu_quant_fused_gate_up_layout_and_torch_semantics(dev):
    """gate and up as the two column halves of one [M, 2I] GEMM output (row pitch 2I), and the result
    against torch's own silu(g) * u followed by the 1x128 quantiser: dequantised values within fp8
    resolution everywhere, hidden-state flips of one bf16 ulp allowed on at most 0.1 % of the groups."""
    M, I = 257, 768
    g = torch.Generator().manual_seed(5)
    gu = (torch.randn(M, 2 * I, generator=g) * 3).to(torch.bfloat16)
    gud = gu.to(dev)
    q, s = ops.swiglu_quant(gud[:, :I], gud[:, I:])
    q2, s2 = ops.swiglu_quant(gud[:, :I].contiguous(), gud[:, I:].contiguous())
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
    qo, so = O.swiglu_quant_group128(gu[:, :I], gu[:, I:])
    same_scale = (s.cpu().view(torch.int32) == so.view(torch.int32))
    assert float((~same_scale).float().mean()) <= 1e-3
    got = O.group128_dequant(u8(q), s.cpu())
    want = O.group128_dequant(qo, so)
    assert O.rel_frobenius(got, want) <= 1e-3
