"""Builds liblyra_hip.so (the gfx950 decode kernels + C ABI) in-tree with hipcc."""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys
import tempfile

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "liblyra_hip.so")
# (object name, source, extra flags).  decode_gemm.hip is compiled in four passes that run in parallel: the K-split kernels
# with the option that keeps matrix-core accumulators in ordinary vector registers (fewer instructions there), the rest
# without it (the expert kernel would spill registers with it); the kernels for e5m2 weights in passes of their own.
_VGPR_FORM = ("-mllvm", "-amdgpu-mfma-vgpr-form")
UNITS = (
    ("abi", "abi.hip", ()),
    ("decode_attention", "decode_attention.hip", ()),
    ("decode_gemm", "decode_gemm.hip", ("-DLYRA_GEMM_PART=1",)),
    ("decode_gemm_splitk", "decode_gemm.hip", ("-DLYRA_GEMM_PART=2", *_VGPR_FORM)),
    ("decode_gemm_e5m2", "decode_gemm.hip", ("-DLYRA_GEMM_PART=3",)),
    ("decode_gemm_splitk_e5m2", "decode_gemm.hip", ("-DLYRA_GEMM_PART=4", *_VGPR_FORM)),
    ("decode_fused", "decode_fused.hip", ()),
)
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep the compiler from forming packed-FP32 VALU instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)
_NOISE = "is not a recognized feature for this target"  # host pass does not know the device feature


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(line for line in proc.stderr.splitlines() if _NOISE not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{err}")
    return err


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory(prefix="lyra_build_") as tmp:
        jobs = []
        for name, src, extra in UNITS:
            obj = os.path.join(tmp, name + ".o")
            jobs.append((obj, [hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]))
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
            errs = list(pool.map(_run, [cmd for _, cmd in jobs]))
        errs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *(obj for obj, _ in jobs), "-o", LIB_PATH]))
    if verbose:
        for err in errs:
            if err.strip():
                print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
