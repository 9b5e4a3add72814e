"""The walking GEMM kernels count their vector-memory operations by hand (``s_waitcnt vmcnt(N)`` in front of a
barrier); this test fails when the compiler's listing of those kernels stops matching what was counted."""
import json
import re
import shutil
from pathlib import Path

import pytest

import isa_counts

FIXTURE = Path(__file__).resolve().parent / "golden" / "walking_kernels_isa_counts.json"

pytestmark = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(), reason="needs hipcc")


@pytest.fixture(scope="module")
def census():
    return isa_counts.census(isa_counts.assembly())


def test_census_matches_fixture(census):
    want = json.loads(FIXTURE.read_text())["kernels"]
    assert sorted(census) == sorted(want), "a walking kernel was added or removed: regenerate the fixture after the GPU parity tests"
    for name, rec in census.items():
        assert rec == want[name], (
            f"{name}: the compiler now emits different memory operations or barriers than the hand-written wait counts "
            f"were derived from ({rec} != {want[name]}). Re-derive the counts in gemm_fp8.hip, run the walking kernels' "
            "bit-equality tests on a GPU, then regenerate with tests/golden/make_isa_counts.py")


def test_no_scratch_and_counts_add_up(census):
    for name, rec in census.items():
        ops = rec["vector_memory"]
        assert not any(k.startswith("scratch_") or k.startswith("flat_") for k in ops), f"{name} spills or uses flat addressing: {ops}"
        stores = sum(n for k, n in ops.items() if "_store_" in k)
        pairs = rec["hand_written_vmcnt_before_barrier"]
        m = re.match(r"(\w+)<(.*)>", name)
        args = [int(a) for a in m.group(2).split(",")]
        if m.group(1) == "gemm_block_w8p_kernel":
            bm, bn = args[0], args[1]
            a_it, b_it = bm // 64, bn // 64
            # every barrier of the K loop lets the b_it newest weight loads pass; the one of a tile's first step also the
            # stores of the previous tile's epilogue, all of which are issued unconditionally
            assert b_it in pairs and b_it + stores in pairs, (name, pairs, stores)
            # direct-to-LDS operand loads: prologue (2 activation + 3 weight stages), the peeled first step, the loop body
            assert ops["buffer_load_dwordx4 lds"] == 2 * a_it + 3 * b_it + 2 * (a_it + b_it), (name, ops)
        else:
            assert pairs, name
