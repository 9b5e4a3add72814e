"""Writes tests/golden/walking_kernels_isa_counts.json from the current source and toolchain.

Run it only after the bit-equality tests of the walking kernels have passed on a GPU with the library built from
the same source (tests/test_gpu_gemm.py: test_walking_kernels_equal_to_sliced_calls,
test_walking_grouped_kernels_repeatable_and_equal_to_sliced_calls, test_grouped_swiglu_epilogue_matches_unfused).

    python tests/golden/make_isa_counts.py
"""
import json
import subprocess
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
import isa_counts  # noqa: E402

if __name__ == "__main__":
    version = subprocess.run([isa_counts._build.hipcc(), "--version"], capture_output=True, text=True).stdout.splitlines()
    record = {"hipcc": [l for l in version if "HIP version" in l or "clang version" in l], "kernels": isa_counts.census(isa_counts.assembly())}
    path = Path(__file__).resolve().parent / "walking_kernels_isa_counts.json"
    path.write_text(json.dumps(record, indent=1, sort_keys=True) + "\n")
    print(f"wrote {path}: {len(record['kernels'])} kernels")
