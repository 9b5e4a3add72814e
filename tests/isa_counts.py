"""Instruction census of the GEMM kernels with hand-counted waits, from hipcc's own assembly listing of
csrc/gemm_fp8.hip, csrc/gemm_grouped_xres.hip and csrc/gemm_mxfp4.hip.

gemm_rowwise_256p_kernel, gemm_block_w8p_kernel, gemm_grouped_xres_kernel, the strip kernels and the direct-to-LDS kernels of gemm_mxfp4.hip order their
LDS traffic with hand-written
``s_waitcnt vmcnt(N)`` + ``s_barrier`` pairs: N is the number of vector-memory operations the author
counted between the loads a barrier needs and the barrier.  That is right only while the compiler
emits exactly those operations, so the census (vector-memory instructions by kind, barriers, the N of
every hand-written pair, no scratch accesses) is kept as a fixture: a toolchain or source change that
adds, drops or converts one memory operation in these kernels changes it, and the test that compares
against the fixture then asks for the bit-equality tests of the walking kernels to be run again on a
GPU before the fixture is regenerated.  Needs hipcc, no GPU.
"""
from __future__ import annotations

import re
import subprocess
import sys
import tempfile
from collections import Counter
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "cosmos-rl_amd"))
from cosmos_rl_amd import _build  # noqa: E402

WALKING = ("gemm_rowwise_256p_kernel", "gemm_block_w8p_kernel", "gemm_mxfp4_256_kernel", "gemm_mxfp4_128_kernel",
           "gemm_mxfp4_128x512_kernel", "gemm_rowwise_strip_kernel", "gemm_mxfp4_strip_kernel", "gemm_block_256_kernel",
           "gemm_grouped_xres_kernel")
SOURCES = ("gemm_fp8.hip", "gemm_grouped_xres.hip", "gemm_mxfp4.hip")
_VMEM = re.compile(r"^\s+((?:buffer|global|flat|scratch)_(?:load|store|atomic)\w*)\b(.*)")
_PAIR = re.compile(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)")


def assembly() -> list[str]:
    """hipcc -S of the GEMM sources for gfx950 with the library's own flags (about 20 s)."""
    lines: list[str] = []
    with tempfile.TemporaryDirectory() as tmp:
        for src in SOURCES:
            out = Path(tmp) / (src + ".s")
            cmd = [_build.hipcc(), *_build.HIPCC_FLAGS, *_build.EXTRA_FLAGS.get(src, []), f"-I{_build.INCLUDE_DIR}", f"-I{_build.CSRC_DIR}",
                   "--cuda-device-only", "-S", str(_build.CSRC_DIR / src), "-o", str(out)]
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError(f"hipcc -S failed:\n{res.stderr}")
            lines += out.read_text().splitlines()
    return lines


def demangled_key(symbol: str) -> str:
    """_ZN4cfp821gemm_block_w8p_kernelILi128ELi256ELi2ELb0ELb1EEEvNS_8GemmArgsE -> gemm_block_w8p_kernel<128,256,2,0,1>"""
    m = re.match(r"_ZN4cfp8\d+([a-z0-9_]+?)I(.*)EEvNS_\d+\w+ArgsE$", symbol)
    if not m:
        return symbol
    args = re.findall(r"L[ib](\d+)E", m.group(2))
    return f"{m.group(1)}<{','.join(args)}>"


def census(lines: list[str]) -> dict[str, dict]:
    out: dict[str, dict] = {}
    i = 0
    while i < len(lines):
        m = re.match(r"^(_ZN4cfp8\w+):", lines[i])
        if not m or not any(w in m.group(1) for w in WALKING):
            i += 1
            continue
        j = i + 1
        while not lines[j].startswith(".Lfunc_end"):
            j += 1
        body = lines[i:j]
        ops: Counter[str] = Counter()
        pairs: list[int] = []
        barriers = 0
        mfmas = [k for k, line in enumerate(body) if re.match(r"^\s+v_mfma", line)]
        spills_between_mfmas = 0  # scratch accesses inside the K loop (anything between the first and the last MFMA)
        for k, line in enumerate(body):
            v = _VMEM.match(line)
            if v:
                ops[v.group(1) + (" lds" if re.search(r"\blds\b", v.group(2)) else "")] += 1
                if v.group(1).startswith("scratch_") and mfmas and mfmas[0] < k < mfmas[-1]:
                    spills_between_mfmas += 1
            if "s_barrier" in line:
                barriers += 1
                p = _PAIR.search(body[k - 1])
                if p:
                    pairs.append(int(p.group(1)))
        out[demangled_key(m.group(1))] = {"vector_memory": dict(sorted(ops.items())), "barriers": barriers,
                                         "hand_written_vmcnt_before_barrier": sorted(pairs), "mfma": len(mfmas),
                                         "scratch_between_mfmas": spills_between_mfmas}
        i = j
    return out
