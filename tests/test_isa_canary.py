"""The walking GEMM kernels and the 256 x 256 MXFP4 kernel count their vector-memory operations by hand (``s_waitcnt vmcnt(N)`` in front of a
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
        assert rec["scratch_between_mfmas"] == 0, f"{name} spills inside its K loop: {ops}"
        assert not any(k.startswith("flat_") for k in ops), f"{name} uses flat addressing: {ops}"
        m = re.match(r"(\w+)<(.*)>", name)
        args = [int(a) for a in m.group(2).split(",")]
        mx4 = {"gemm_mxfp4_256_kernel": (8, 4, 1, 64), "gemm_mxfp4_128_kernel": (4, 4, 1, 32), "gemm_mxfp4_128x512_kernel": (4, 8, 2, 64)}
        if m.group(1) in mx4:
            # per wave and K step x activation + w weight loads of 16 bytes and s scale loads of 4 bytes (and so many
            # MFMAs); the prologue requests 2 activation and 3 weight / scale stages.  The barrier of a step lets the
            # w + s newest pass, the prologue's barrier everything behind its first 1 + x + w + s loads (the row scales
            # for the epilogue, which come first, are a global_load ... lds).  A few values that only the epilogue needs
            # may be spilled across the loop, never inside it.  The compiler may emit the K loop more than once.
            x, w, sc, mfma_per_step = mx4[m.group(1)]
            pairs = [n for n in rec["hand_written_vmcnt_before_barrier"] if n]
            copies = pairs.count(w + sc)
            assert copies >= 1 and pairs == [w + sc] * copies + [x + 2 * (w + sc)], (name, rec)
            assert ops["buffer_load_dwordx4 lds"] == (2 * x + 3 * w) + copies * (x + w), (name, ops)
            assert ops["buffer_load_dword lds"] == 3 * sc + copies * sc and ops["global_load_lds_dword"] == 1, (name, ops)
            assert rec["mfma"] == copies * mfma_per_step, (name, rec)
            continue
        if m.group(1) == "gemm_grouped_xres_kernel":
            # <K steps, fp32 output>: one barrier in the middle of every K step; the weight loads of a step (8 per wave) are
            # requested three steps ahead, the prologue requests three steps.  bf16: a tile leaves as 16 stores spread over
            # steps 1 .. 4 of the next tile (4 each, in the half in front of the barrier), so a barrier may leave the 8
            # loads of the step in between and the stores of that step and of its own in flight; fp32: 32 stores in front
            # of the first barrier of the next tile.  The last tile's stores are issued once more behind the loop.
            kt, f32 = args
            stores_per_tile = 32 if f32 else 16
            assert ops["buffer_load_dwordx4 lds"] == 3 * 8 + kt * 8, (name, ops)
            assert ops["buffer_store_dwordx4"] == 2 * stores_per_tile, (name, ops)
            stores_at = lambda k: 4 if 1 <= k % kt <= 4 else 0   # (python's % wraps a negative step into the tile before)
            want = [40, 40] + [8] * (kt - 2) if f32 else [8 + stores_at(k - 1) + stores_at(k) for k in range(kt)]
            assert rec["hand_written_vmcnt_before_barrier"] == sorted(want), (name, rec)
            # a unit's activation fragments (two 16-byte loads each) and scales, at the kernel's start and at a unit switch
            assert ops["buffer_load_dwordx4"] == 2 * kt * 4 * 2 and ops["buffer_load_dword"] == 2 * kt * 4, (name, ops)
            assert rec["mfma"] == kt * 32, (name, rec)
            assert not any(k.startswith("scratch_") for k in ops), f"{name} spills: {ops}"
            continue
        if m.group(1) in ("gemm_rowwise_strip_kernel", "gemm_mxfp4_strip_kernel"):
            # a ring of S stages: the prologue requests S - 1 tiles, every step one more; the barrier of a step lets the
            # loads of the S - 2 tiles behind the one it needs pass
            bm = args[0]
            if m.group(1) == "gemm_rowwise_strip_kernel":
                x4, w4, s1, stages = bm // 32, (args[1] * 16 + 31) // 32, 0, 8 if bm == 64 else 5
            else:
                x4, w4, s1, stages = bm // 32, 2, 1, 9 if bm == 64 else 6
            per_step = x4 + w4 + s1
            pairs = [n for n in rec["hand_written_vmcnt_before_barrier"] if n]
            assert pairs and set(pairs) == {(stages - 2) * per_step}, (name, rec)
            assert ops["buffer_load_dwordx4 lds"] == (stages - 1 + len(pairs)) * (x4 + w4), (name, ops)
            assert ops.get("buffer_load_dword lds", 0) == (stages - 1 + len(pairs)) * s1, (name, ops)
            assert not any(k.startswith("scratch_") for k in ops), f"{name} spills: {ops}"
            continue
        assert not any(k.startswith("scratch_") for k in ops), f"{name} spills: {ops}"
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


def test_resident_tensorwise_kernel_merged_phase():
    """The resident tensorwise kernel stores a slot and requests it anew with the next tensor's chunk.  That only
    overlaps stores and loads while (a) no kept vector is spilled, (b) nothing waits for a vector-memory operation
    between the first direct-to-LDS load and the last load of the phase, and (c) every LDS slot is read (by an
    instruction the source writes out) before the direct-to-LDS load that overwrites it is issued."""
    import subprocess
    import tempfile

    from cosmos_rl_amd import _build

    with tempfile.TemporaryDirectory() as tmp:
        out = Path(tmp) / "quant_tensorwise.s"
        cmd = [_build.hipcc(), *_build.HIPCC_FLAGS, f"-I{_build.INCLUDE_DIR}", f"-I{_build.CSRC_DIR}", "--cuda-device-only", "-S",
               str(_build.CSRC_DIR / "quant_tensorwise.hip"), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr
        lines = out.read_text().splitlines()
    start = next(i for i, line in enumerate(lines) if re.match(r"^_ZN4cfp8\d+tensorwise_resident_kernel\w*:", line))
    end = next(i for i in range(start, len(lines)) if lines[i].startswith(".Lfunc_end"))
    body = lines[start:end]
    assert not any(re.match(r"^\s+scratch_", line) for line in body), "the resident kernel spills"
    dma = [i for i, line in enumerate(body) if re.match(r"^\s+buffer_load_dwordx4 .*\blds\b", line)]
    assert len(dma) == 13, f"{len(dma)} direct-to-LDS loads, one per LDS slot expected"
    # the register slots' loads follow the last direct-to-LDS load: the next 32 plain 16-byte buffer loads
    plain = [i for i, line in enumerate(body) if i > dma[-1] and re.match(r"^\s+buffer_load_dwordx4 (?!.*\blds\b)", line)][:32]
    assert len(plain) == 32
    phase = body[dma[0]:plain[-1] + 1]
    assert not any("s_waitcnt vmcnt" in line for line in phase), "a wait for vector memory inside the merged phase"
    # one written-out LDS read in front of every direct-to-LDS load (slot l is read, then requested anew)
    reads = [i for i, line in enumerate(body) if re.match(r"^\s+ds_read_b128 ", line) and i < dma[-1]]
    for k, d in enumerate(dma):
        lo = dma[k - 1] if k else 0
        assert any(lo < r < d for r in reads), f"no LDS read between direct-to-LDS loads {k - 1} and {k}"
