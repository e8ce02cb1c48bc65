"""Build libparoatten_hip.so (device code for gfx950 only) with hipcc, and the PyTorch-ROCm C++
extension paroatten_amd/_ext.so (host code only, binds the library's C ABI) with g++, both in-tree.

    python paroatten_amd/build.py

(run as a script, not with -m: importing the package loads the library, which fails while the
library is missing or older than the header)

No hipify, no torch headers: the library is plain HIP behind a C ABI (include/paroatten.h).
IEEE fp32 arithmetic is part of the quantisation / RoPE specification, so fast-math stays off and
fp contraction is disabled; packed-FP32 instruction selection is disabled for every source.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIBDIR = PKG / "lib"
LIB = LIBDIR / "libparoatten_hip.so"
SOURCES = ["paro_common.hip", "quant_int8.hip", "v_fp8.hip", "v_channel.hip", "rope_permute.hip", "fused_prep.hip", "mask_bits.hip", "attn_sparse.hip", "attn_sparse_w64.hip", "attn_sparse_pv16.hip"]
ARCH = "gfx950"
# measurement aids behind bench.py --mfma-ceiling / --proxy-ceiling: a library of their own (include/paroatten_diag.h),
# outside the drop-in boundary
DIAG_LIB = LIBDIR / "libparoatten_diag.so"
DIAG_SOURCES = ["diag.hip"]

FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results straight into VGPRs: no accvgpr moves around the softmax
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str, verbose: bool) -> Path:
    obj = LIBDIR / (Path(src).stem + ".o")
    cmd = [hipcc(), *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    if verbose and r.stderr.strip():
        # the host pass warns that it does not know the packed-fp32 feature: harmless
        lines = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if lines:
            print("\n".join(lines), file=sys.stderr)
    return obj


EXT = PKG / "_ext.so"


def build_ext(verbose: bool = False) -> Path:
    """Compile csrc/torch_binding.cpp (pybind11 + torch headers, no device code) into
    paroatten_amd/_ext.so, linked against libparoatten_hip.so ($ORIGIN/lib) and torch's libraries."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    tlib = Path(torch.__file__).resolve().parent / "lib"
    inc = [*ce.include_paths("cuda"), sysconfig.get_paths()["include"], str(PKG.parent / "include")]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_ext",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-Wno-deprecated-declarations",
           *[f"-I{i}" for i in inc], str(CSRC / "torch_binding.cpp"), "-o", str(EXT),
           f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
           f"-L{LIBDIR}", "-lparoatten_hip", "-Wl,-rpath,$ORIGIN/lib", f"-Wl,-rpath,{tlib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"g++ failed on torch_binding.cpp:\n{r.stdout}\n{r.stderr}")
    if verbose and r.stderr.strip():
        print(r.stderr, file=sys.stderr)
    return EXT


def build(force: bool = True, verbose: bool = False) -> Path:
    """Compile every HIP source and link the shared library.  Always compiles when force."""
    LIBDIR.mkdir(exist_ok=True)
    if not force and LIB.exists():
        newest = max(p.stat().st_mtime for p in list(CSRC.iterdir()) + [PKG.parent / "include" / "paroatten.h"])
        if LIB.stat().st_mtime >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + len(DIAG_SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES + DIAG_SOURCES))
    for lib, members in ((LIB, objs[:len(SOURCES)]), (DIAG_LIB, objs[len(SOURCES):])):
        cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, members), "-o", str(lib)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    path = build(force="--force" in sys.argv or True, verbose=True)
    print(path)
    if "--no-ext" not in sys.argv:
        print(build_ext(verbose=True))
