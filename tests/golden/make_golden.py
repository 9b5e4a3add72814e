#!/usr/bin/env python3
"""Writes tests/golden/fp8_golden.npz: small seeded inputs and the outputs of the CPU oracle.

The reference holds no FP8 golden vector of its own (its FP8 test only checks module classes,
tests/test_fp8.py:55-118 upstream), and its arithmetic lives in wheels that are not installed
here, so these vectors freeze the oracle: a later change to the oracle, to torch's CPU e4m3 cast
or to the C restatement shows up as a diff against data committed before the change.  Each vector
is cross-checked against the scalar C restatement before it is written.

Run from the repository root:  python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import c_oracle as C  # noqa: E402
from oracle import fp8_oracle as O  # noqa: E402


def u16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    out = {}
    # config 1, first 8 rows and rows holding the planted outliers' maxima
    w = O.make_weight((4864, 896), seed=1235, outlier_frac=1e-3, outlier_mul=20.0)
    rows = torch.cat([torch.arange(8), w.float().abs().amax(1).topk(4).indices])
    sub = w[rows].contiguous()
    q, s = O.quant_rowwise(sub)
    qc, sc = C.quant_rowwise(u16(sub))
    assert (qc == q.numpy()).all() and (sc.view(np.int32) == s.numpy().view(np.int32)).all()
    out.update(rowwise_rows=rows.numpy(), rowwise_x=u16(sub), rowwise_q=q.numpy(), rowwise_s=s.numpy())
    # tensorwise
    t = O.make_weight((24, 64), seed=2)
    q, s = O.quant_tensorwise(t)
    qc, sc = C.quant_tensorwise(u16(t))
    assert (qc == q.numpy()).all() and (sc.view(np.int32) == s.numpy().view(np.int32)).all()
    out.update(tensor_x=u16(t), tensor_q=q.numpy(), tensor_s=s.numpy())
    # block 128x128 with ragged edges
    b = O.make_weight((130, 136), seed=3, std=0.05)
    q, s = O.quant_block128(b)
    qc, sc = C.quant_block128(u16(b))
    assert (qc == q.numpy()).all() and (sc.view(np.int32) == s.numpy().view(np.int32)).all()
    out.update(block_x=u16(b), block_q=q.numpy(), block_s=s.numpy())
    # 1x128 groups, both formulas
    g = O.make_activation(5, 200, seed=4, chan_outlier_frac=0.02, outlier_mul=30.0)
    q, s = O.quant_group128(g)
    qc, sc = C.quant_group128(u16(g), 0)
    assert (qc == q.numpy()).all() and (sc.view(np.int32) == s.numpy().view(np.int32)).all()
    q1, s1 = O.group128_cast_deepep(g)
    qc, sc = C.quant_group128(u16(g), 1)
    assert (qc == q1.numpy()).all() and (sc.view(np.int32) == s1.numpy().view(np.int32)).all()
    out.update(group_x=u16(g), group_q=q.numpy(), group_s=s.numpy(), deepep_q=q1.numpy(), deepep_s=s1.numpy())
    # GEMMs on quantised operands (fp64 accumulation, stored as fp32)
    x = O.make_activation(16, 256, seed=5, chan_outlier_frac=0.01, outlier_mul=30.0)
    wt = O.make_weight((32, 256), seed=6)
    qx, sx = O.quant_rowwise(x)
    qw, sw = O.quant_rowwise(wt)
    out.update(mm_qa=qx.numpy(), mm_sa=sx.numpy(), mm_qb=qw.numpy(), mm_sb=sw.numpy(),
               mm_out=O.scaled_mm_rowwise(qx, sx, qw, sw, accum=torch.float64).numpy())
    qxg, sxg = O.quant_group128(x)
    qwb, swb = O.quant_block128(wt)
    out.update(bmm_qa=qxg.numpy(), bmm_sa=sxg.numpy(), bmm_qb=qwb.numpy(), bmm_sb=swb.numpy(),
               bmm_out=O.scaled_mm_block128(qxg, sxg, qwb, swb, accum=torch.float64).numpy())
    path = Path(__file__).resolve().parent / "fp8_golden.npz"
    np.savez_compressed(path, **out)
    print(f"wrote {path} ({path.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
