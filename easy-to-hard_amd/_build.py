"""Builds libe2h_quant.so (the C-ABI library declared in include/e2h_quant.h) with hipcc for gfx950.

The library is built in-tree, next to this file, so that it travels with the source tree; nothing is
installed into site-packages and no JIT cache is involved.
"""

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "libe2h_quant.so"
LIB_PATH = PKG_DIR / LIB_NAME

SOURCES = ["e2h_abi.hip", "e2h_quantize.hip", "e2h_int4_mm.hip", "e2h_int4_staged.hip", "e2h_int4_rows64.hip", "e2h_int8_mm.hip", "e2h_int8_stream.hip", "e2h_int4_gemm.hip", "e2h_int4_gemm128.hip", "e2h_int8_gemm.hip", "e2h_attention.hip", "e2h_sample.hip", "e2h_probe.hip"]

# -ffp-contract=off: the quantizers are bit-exact restatements of separate torch ops; an FMA formed
# across two of them would change codes.  packed-fp32-ops is switched off because some packed float32
# forms have produced wrong results on the target machines.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Per-source additions.  The 32x32-tile matmul mixes MFMA accumulators with float32 FMAs on the same values; with
# the accumulators in the accumulation register file every FMA needs copies in and out (3 extra instructions per FMA),
# so that file is compiled with MFMA results kept in ordinary vector registers.
EXTRA_FLAGS = {"e2h_int4_gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "e2h_int4_staged.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
               "e2h_int4_rows64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}  # (the int8 kernel of the same shape has no such FMAs)


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; the e2h kernels cannot be built")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(map(str, cmd)), proc.stdout))
    return proc.stdout


def build_library(verbose=False):
    """Compile every HIP source for gfx950 and link libe2h_quant.so.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    sources = [s for s in SOURCES if (CSRC / s).exists()]

    def compile_one(src):
        obj = obj_dir / (Path(src).stem + ".o")
        out = _run([hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", str(CSRC / src), "-o", str(obj)])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(sources), 6)) as pool:
        objs = list(pool.map(compile_one, sources))
    tmp = PKG_DIR / (LIB_NAME + ".tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
