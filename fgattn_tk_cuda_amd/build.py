"""In-tree build of the gfx950 library and of the PyTorch operator extension.

``python -m fgattn_tk_cuda_amd.build``            builds both
``python -m fgattn_tk_cuda_amd.build --lib-only`` builds libspattn_hip.so only

hipcc cross-compiles for gfx950 without a GPU.  Outputs stay inside the package
directory so that they travel with the source tree.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "_obj"
LIB = PKG / "libspattn_hip.so"
EXT_DIR = PKG / "spattn"

HIP_SOURCES = [
    "attn_inst_tokens.hip",
    "attn_inst_blocks.hip",
    "attn_inst_dense.hip",
    "mask_kernels.hip",
    "bitmask_kernels.hip", "blocklist_kernels.hip", "topk_kernels.hip", "order_kernels.hip",
    "capi.hip",
]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-command-line-argument",
    # no packed-fp32 VALU forms in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd: list[str]) -> None:
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


POISON_LIB = PKG / "libspattn_hip_poison.so"


def build_lib(verbose: bool = True, poison: bool = False) -> Path:
    """Compile every HIP translation unit and link libspattn_hip.so.

    poison=True builds libspattn_hip_poison.so instead: the same library with -DSPATTN_POISON_RING,
    whose attention kernels fill every ring slot with NaNs between the barrier that frees it and the
    copy that refills it (a debug build for the copy pipeline; tests compare it bit for bit with
    the product library)."""
    objdir = CSRC / ("_obj_poison" if poison else "_obj")
    objdir.mkdir(exist_ok=True)
    hipcc = _hipcc()
    flags = HIPCC_FLAGS + (["-DSPATTN_POISON_RING"] if poison else [])
    jobs = []
    for src in HIP_SOURCES:
        obj = objdir / (src.replace(".hip", ".o"))
        jobs.append([hipcc, *flags, "-c", str(CSRC / src), "-o", str(obj)])
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(_run, jobs))
    objs = [str(objdir / s.replace(".hip", ".o")) for s in HIP_SOURCES]
    out = POISON_LIB if poison else LIB
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *objs])
    if verbose:
        print("built", out)
    return out


def ext_path() -> Path:
    import sysconfig

    return EXT_DIR / ("cuda_attn" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_torch_ext(verbose: bool = True) -> Path:
    """Compile the torch.ops.cuda_attn binding (host C++ only) and link it to the library."""
    import torch
    from torch.utils import cpp_extension as ce

    out = ext_path()
    inc = []
    for p in ce.include_paths(device_type="cuda") if "device_type" in ce.include_paths.__code__.co_varnames else ce.include_paths():
        inc += ["-I", p]
    import sysconfig

    inc += ["-I", sysconfig.get_paths()["include"], "-I", "/opt/rocm/include", "-I", str(PKG.parent / "include")]
    torch_lib = str(Path(torch.__file__).resolve().parent / "lib")
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=cuda_attn",
        "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
        *inc, str(CSRC / "torch_ext.cpp"), "-o", str(out),
        "-L", torch_lib, "-L", str(PKG), "-L", "/opt/rocm/lib",
        "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10_hip", "-ltorch_hip", "-lamdhip64", "-lspattn_hip",
        "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + torch_lib, "-Wl,-rpath,/opt/rocm/lib",
    ]
    _run(cmd)
    if verbose:
        print("built", out)
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib-only", action="store_true")
    args = ap.parse_args(argv)
    build_lib()
    if not args.lib_only:
        build_torch_ext()
        build_lib(poison=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
