"""Builds libbhi_hip.so for gfx950 next to the package (python -m bf16_huffman_infer_amd.csrc.build)."""
import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
SOURCES = ["bhi_api.hip", "bhi_huffman.hip", "bhi_ans.hip", "bhi_nibble.hip", "bhi_reference.hip", "bhi_attention.hip"]
LIB = os.path.join(PKG, "libbhi_hip.so")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first five dwords of every kernel's arguments arrive in registers (the fused GEMV
    # picks its group member from them before its first memory access)
    "-mllvm", "-amdgpu-kernarg-preload-count=5",
    "-Wall", "-Wno-unused-variable",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")


def build(verbose: bool = True, defines=(), lib: str = LIB) -> str:
    """Compiles every source to an object of its own (in parallel) and links them."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory(prefix="bhi_build_") as tmp:
        objs = [os.path.join(tmp, s.replace(".hip", ".o")) for s in SOURCES]
        cmds = [[hipcc, *FLAGS, *[f"-D{d}" for d in defines], "-c", os.path.join(HERE, s), "-o", o]
                for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=min(len(cmds), os.cpu_count() or 1)) as pool:
            list(pool.map(lambda c: _run(c, verbose), cmds))
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib], verbose)
    return lib


if __name__ == "__main__":
    build()
    sys.exit(0)
