"""Committed fixtures (tests/golden/fp8_golden.npz, written by tests/golden/make_golden.py):
the torch oracle and the C restatement must reproduce them on the CPU, the HIP kernels on the GPU."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import fp8_oracle as O

G = np.load(Path(__file__).resolve().parent / "golden" / "fp8_golden.npz")


def bf16(u16):
    return torch.from_numpy(u16.view(np.int16).copy()).view(torch.bfloat16)


def same(q, s, qname, sname):
    assert (np.asarray(q) == G[qname]).all(), qname
    assert (np.asarray(s).view(np.int32) == G[sname].view(np.int32)).all(), sname


def test_fixture_inputs_are_the_seeded_ones():
    w = O.make_weight((4864, 896), seed=1235, outlier_frac=1e-3, outlier_mul=20.0)
    assert torch.equal(w[torch.from_numpy(G["rowwise_rows"])], bf16(G["rowwise_x"]))


def test_oracle_reproduces_fixtures():
    q, s = O.quant_rowwise(bf16(G["rowwise_x"])); same(q.numpy(), s.numpy(), "rowwise_q", "rowwise_s")
    q, s = O.quant_tensorwise(bf16(G["tensor_x"])); same(q.numpy(), s.numpy(), "tensor_q", "tensor_s")
    q, s = O.quant_block128(bf16(G["block_x"])); same(q.numpy(), s.numpy(), "block_q", "block_s")
    q, s = O.quant_group128(bf16(G["group_x"])); same(q.numpy(), s.numpy(), "group_q", "group_s")
    q, s = O.group128_cast_deepep(bf16(G["group_x"])); same(q.numpy(), s.numpy(), "deepep_q", "deepep_s")
    t = lambda k: torch.from_numpy(G[k])
    out = O.scaled_mm_rowwise(t("mm_qa"), t("mm_sa"), t("mm_qb"), t("mm_sb"), accum=torch.float64)
    assert np.array_equal(out.numpy(), G["mm_out"])
    out = O.scaled_mm_block128(t("bmm_qa"), t("bmm_sa"), t("bmm_qb"), t("bmm_sb"), accum=torch.float64)
    assert np.array_equal(out.numpy(), G["bmm_out"])


def test_c_restatement_reproduces_fixtures():
    C.build()
    same(*C.quant_rowwise(G["rowwise_x"]), "rowwise_q", "rowwise_s")
    same(*C.quant_tensorwise(G["tensor_x"]), "tensor_q", "tensor_s")
    same(*C.quant_block128(G["block_x"]), "block_q", "block_s")
    same(*C.quant_group128(G["group_x"], 0), "group_q", "group_s")
    same(*C.quant_group128(G["group_x"], 1), "deepep_q", "deepep_s")


@pytest.mark.gpu
def test_kernels_reproduce_fixtures(dev):
    from cosmos_rl_amd import ops

    def run(fn, xname):
        q, s = fn(bf16(G[xname]).to(dev))
        return q.view(torch.uint8).cpu().numpy(), s.cpu().numpy()

    same(*run(ops.quant_rowwise, "rowwise_x"), "rowwise_q", "rowwise_s")
    same(*run(ops.quant_tensorwise, "tensor_x"), "tensor_q", "tensor_s")
    same(*run(ops.per_block_cast_to_fp8, "block_x"), "block_q", "block_s")
    same(*run(ops.groupwise_activation_quant, "group_x"), "group_q", "group_s")
    same(*run(ops.per_token_cast_to_fp8, "group_x"), "deepep_q", "deepep_s")
    f8 = lambda k: torch.from_numpy(G[k]).to(dev).view(torch.float8_e4m3fn)
    t = lambda k: torch.from_numpy(G[k]).to(dev)
    out = ops.scaled_mm(f8("mm_qa"), f8("mm_qb").t(), t("mm_sa"), t("mm_sb").t(), out_dtype=torch.float32)
    assert O.rel_frobenius(out.cpu(), torch.from_numpy(G["mm_out"])) <= 1e-4
    outb = torch.empty(16, 32, dtype=torch.float32, device=dev)
    ops.gemm_fp8_fp8_bf16_nt((f8("bmm_qa"), t("bmm_sa")), (f8("bmm_qb"), t("bmm_sb")), outb)
    assert O.rel_frobenius(outb.cpu(), torch.from_numpy(G["bmm_out"])) <= 1e-4
