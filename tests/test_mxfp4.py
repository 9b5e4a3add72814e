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
