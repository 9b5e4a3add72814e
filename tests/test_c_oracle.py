"""The scalar C restatement (oracle/fp8_ref.c) against the torch oracle, and the CPU proof of the
division shortcut the kernels use."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import fp8_oracle as O


@pytest.fixture(scope="module", autouse=True)
def _built():
    C.build()


def u16(x):
    return x.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_encoder_exhaustive_bf16_and_random_fp32():
    lib = C.load()
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    want = O.e4m3_bytes(pats).numpy()
    got = np.array([lib.fp8ref_e4m3_from_f32(float(v)) for v in pats.numpy()], dtype=np.uint8)
    assert (got == want).all()
    g = torch.Generator().manual_seed(0)
    v = torch.cat([(torch.rand(50000, generator=g) * 2 - 1) * 500, (torch.rand(50000, generator=g) * 2 - 1) * 0.05])
    want = O.e4m3_bytes(v).numpy()
    got = np.array([lib.fp8ref_e4m3_from_f32(float(x)) for x in v.numpy()], dtype=np.uint8)
    assert (got == want).all()
    back = np.array([lib.fp8ref_e4m3_to_f32(b) for b in range(256)], dtype=np.float32)
    tb = O.e4m3_to_f32(torch.arange(256, dtype=torch.uint8)).numpy()
    assert ((back == tb) | (np.isnan(back) & np.isnan(tb))).all()


def _weights(shape, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(*shape, generator=g) * torch.exp(torch.randn(shape[0], 1, generator=g) * 3)
    w = w.to(torch.bfloat16)
    w[0] = 0
    if shape[0] > 3:
        w[1, 0] = float("nan")
        w[2, 1] = float("inf")
    return w


def test_rowwise_and_tensorwise_agree():
    w = _weights((64, 200), 1)
    q, s = C.quant_rowwise(u16(w))
    qo, so = O.quant_rowwise(w)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()
    w = O.make_weight((40, 72), seed=2)
    q, s = C.quant_tensorwise(u16(w))
    qo, so = O.quant_tensorwise(w)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()


def _special_f32():
    """fp32 patterns that exercise the bf16 rounding: ties both ways, carries into the exponent,
    overflow to infinity, subnormals, signed zeros, infinities, NaNs, plus random bit patterns."""
    pats = [0x3F800000, 0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x3FFF8000, 0x7F7F7FFF, 0x7F7F8000,
            0x7F7FFFFF, 0x7F800000, 0x7FC00000, 0x7F800001, 0x00000000, 0x00000001, 0x00008000, 0x00018000,
            0x007F8000, 0x007FFFFF, 0x00800000]
    pats = pats + [p | 0x80000000 for p in pats]
    g = torch.Generator().manual_seed(7)
    rnd = torch.randint(-2**31, 2**31 - 1, (200000,), generator=g, dtype=torch.int64).to(torch.int32)
    return torch.cat([torch.tensor(pats, dtype=torch.int64).to(torch.int32), rnd]).view(torch.float32)


def test_bf16_rounding_matches_torch():
    """The transfer-dtype cast: the C search over the two neighbouring bf16 values agrees with torch's
    own fp32 -> bf16 conversion on every special pattern and 200k random bit patterns (NaNs compare as NaN)."""
    lib = C.load()
    v = _special_f32()
    want = v.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([lib.fp8ref_bf16_from_f32(float(x)) for x in v.numpy()], dtype=np.uint16)
    nan = np.isnan(v.numpy())
    assert (got[~nan] == want[~nan]).all()
    assert ((got[nan] & 0x7FFF) > 0x7F80).all() and ((want[nan] & 0x7FFF) > 0x7F80).all()
    # closed forms: a tie goes to the even mantissa, the largest fp32 rounds to infinity
    assert lib.fp8ref_bf16_from_f32(float(np.uint32(0x3F808000).view(np.float32))) == 0x3F80
    assert lib.fp8ref_bf16_from_f32(float(np.uint32(0x3F818000).view(np.float32))) == 0x3F82
    assert lib.fp8ref_bf16_from_f32(float(np.uint32(0x7F7FFFFF).view(np.float32))) == 0x7F80


def test_rowwise_from_fp32_agrees():
    g = torch.Generator().manual_seed(5)
    w = torch.randn(48, 264, generator=g) * torch.exp(torch.randn(48, 1, generator=g) * 4)
    w[0] = 0
    w[1, 3] = float("nan")
    w[2, 5] = float("inf")
    w[3] = _special_f32()[:264]
    w[4] = 3.3e38  # rounds to bf16 infinity
    q, s = C.quant_rowwise_f32(w.numpy())
    qo, so = O.quant_rowwise_from(w)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()
    # bf16 input: the transfer-dtype form is the plain rowwise quantiser
    wb = w.to(torch.bfloat16)
    qa, sa = O.quant_rowwise_from(wb)
    qb, sb = O.quant_rowwise(wb)
    assert torch.equal(qa, qb) and torch.equal(sa.view(torch.int32), sb.view(torch.int32))


def test_block_and_group_agree():
    w = _weights((200, 264), 3)
    q, s = C.quant_block128(u16(w))
    qo, so = O.quant_block128(w)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()
    x = _weights((33, 328), 4)
    q, s = C.quant_group128(u16(x), 0)
    qo, so = O.quant_group128(x)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()
    x = O.make_activation(33, 328, seed=5)
    x[3] = 0
    q, s = C.quant_group128(u16(x), 1)
    qo, so = O.group128_cast_deepep(x)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()


def test_division_shortcut_is_exact():
    """r = 1/s; q0 = x*r; e = fma(q0, s, -x); q1 = fma(-e, r, q0) equals the IEEE quotient x/s bit for bit wherever
    |x/s| >= 2^-11, and its e4m3 byte - converted without a clamp - is the byte of the clamped IEEE quotient, signed
    zeros included, for all bf16 x with |x/s| <= 448 (1 + 2^-22) (a scale is the amax / 448 of a set x belongs to) and
    1500 scales spanning the fp32 range; among them amax values whose own quotient is the fp32 value above 448."""
    g = torch.Generator().manual_seed(0)
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    pos = pats[(pats > 0) & torch.isfinite(pats)]
    amax = torch.cat([torch.rand(500, generator=g) * 2, torch.exp(torch.rand(500, generator=g) * 170 - 85).clamp(max=3e38),
                      pos[::66], torch.tensor([0.0, 1e-12, 1e-13, 3.3895e38, 448.0, 0.00799560546875, 0.0084228515625])])
    scales = O.scale_from_amax(amax).numpy()
    bad, soft = C.check_fast_div(scales)
    assert bad == 0 and soft == 0


def _swiglu_inputs(M, I, seed):
    g = torch.Generator().manual_seed(seed)
    gate = (torch.randn(M, I, generator=g) * 3).to(torch.bfloat16)
    up = (torch.randn(M, I, generator=g) * 2).to(torch.bfloat16)
    gate[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 80.0, -80.0, 1e-3, -1e-3]).to(torch.bfloat16)
    return gate, up


def test_exp32_accuracy_and_silu_closed_forms():
    """The fixed fp32 exp sequence stays within 2 ulp of the fp64 exponential over its whole range, and
    silu has its closed-form values at 0 and at both ends."""
    lib = C.load()
    worst = 0.0
    for x in np.linspace(-87.0, 88.0, 60001).astype(np.float32):
        want = np.exp(np.float64(x))
        worst = max(worst, abs(np.float64(lib.fp8ref_exp32(float(x))) - want) / np.float64(np.spacing(np.float32(want))))
    assert worst < 2.0
    assert lib.fp8ref_exp32(0.0) == 1.0
    assert lib.fp8ref_silu32(0.0) == 0.0 and lib.fp8ref_silu32(40.0) == 40.0
    assert lib.fp8ref_silu32(-120.0) == 0.0 and np.signbit(np.float32(lib.fp8ref_silu32(-120.0)))
    assert np.isnan(lib.fp8ref_silu32(float("nan")))
    assert abs(lib.fp8ref_silu32(1.0) - 1.0 / (1.0 + np.exp(-1.0))) < 1e-7


def test_swiglu_restatement_against_torch_ops():
    """bf16(bf16(silu(g)) * u) of the C restatement against torch's silu(g) * u on bf16 tensors: equal except
    where torch's exp differs in the last fp32 bit and flips a bf16 rounding - at most 0.1 % of the elements,
    each by one bf16 ulp - and the quantised result is the 1x128 quantiser applied to that hidden state."""
    gate, up = _swiglu_inputs(96, 768, 21)
    h = torch.from_numpy(C.swiglu(u16(gate), u16(up)).view(np.int16)).view(torch.bfloat16)
    want = O.swiglu_hidden(gate, up)
    diff = (h.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert int(diff.max()) <= 1
    assert float((diff != 0).float().mean()) <= 1e-3
    q, s = C.swiglu_quant_group128(u16(gate), u16(up))
    qo, so = O.quant_group128(h)
    assert (q == qo.numpy()).all() and (s.view(np.int32) == so.numpy().view(np.int32)).all()
