"""Build libviola_hip.so for gfx950 with hipcc, in-tree next to the sources.

python -m viola_amd.csrc.build        (or called by __graft_entry__.build())
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIBRARY = HERE / "libviola_hip.so"
ARCH = "gfx950"
# -ffp-contract=off: the quantize / optimizer / codec kernels follow the reference's un-fused
# fp32 operation order so FP8 codes and scales come out bit-exact. The GEMM files apply their
# scale with an explicit fmaf.
COMMON = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
SOURCES = ["quantize.hip", "gemm.hip", "gemm_fast.hip", "gemm_fast_tensor.hip", "gemm_fast_mx.hip", "ns.hip", "ns_fast.hip", "optim.hip", "misc.hip", "tensor.hip"]


def hipcc():
    for candidate in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if candidate and (os.path.isabs(candidate) and os.path.exists(candidate) or not os.path.isabs(candidate)):
            return candidate
    raise RuntimeError("hipcc not found")


def _filter(text):
    return "\n".join(line for line in text.splitlines() if "is not a recognized feature for this target" not in line)


def build(verbose=True, incremental=False):
    """Compile every source and link. incremental=True (a development convenience) reuses objects that
    are newer than their source and every header."""
    compiler = hipcc()
    objects = []
    newest_header = max(h.stat().st_mtime for h in HERE.glob("*.hpp"))

    def compile_one(name):
        obj = HERE / (name.rsplit(".", 1)[0] + ".o")
        if incremental and obj.exists() and obj.stat().st_mtime > newest_header and obj.stat().st_mtime > (HERE / name).stat().st_mtime:
            return obj
        cmd = [compiler, *COMMON, "-c", str(HERE / name), "-o", str(obj)]
        result = subprocess.run(cmd, capture_output=True, text=True)
        message = _filter(result.stdout + result.stderr)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed for {name}:\n{message}")
        if verbose and message.strip():
            print(message, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    link = [compiler, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objects), "-o", str(LIBRARY)]
    result = subprocess.run(link, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError("link failed:\n" + _filter(result.stdout + result.stderr))
    return LIBRARY


if __name__ == "__main__":
    print(build(incremental="--incremental" in sys.argv))
