"""In-tree build of the gpustack_amd HIP extension for gfx950 (MI355X).

Drives hipcc directly (no hipify, no CUDA compat layer): the .hip sources
are native HIP/CDNA4 and the binding file links against torch-ROCm's native
c10/hip API. The resulting _hip_ops.so lives inside the package so it
travels with repo snapshots (and stays out of git via .gitignore).
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
SO_PATH = PKG_DIR / "_hip_ops.so"
ARCH = os.environ.get("GPUSTACK_AMD_ARCH", "gfx950")

HIP_SOURCES = ["pointwise.hip", "attn_decode.hip", "attn_prefill.hip", "skinny_gemm.hip", "gemm8.hip", "gemm8_lab.hip", "moe_gemm.hip", "w4_gemm.hip", "mla_decode.hip"]
CPP_SOURCES = ["bindings.cpp"]
# the fp32-residual op family lives in its own small library: a checkout
# that serves only such a model compiles these few files and nothing else
LATENT_SO_PATH = PKG_DIR / "_hip_latent.so"
LATENT_SOURCES = ["resid32.hip", "latent_attn.hip", "grouped_ff.hip",
                  "latent_bindings.cpp"]


# pre/post-norm fp32-stream row kernels + paged rotary attention (argmax
# comes with resid32.hip): again a library of its own
PAGED_SO_PATH = PKG_DIR / "_hip_paged.so"
PAGED_SOURCES = ["rowmix32.hip", "roperows32.hip", "ragged_attn.hip",
                 "resid32.hip", "paged_bindings.cpp"]

# layer-norm fp32-stream row kernels, head-norm cache write, scored routing
# and the recurrent mixers (page-wise value stores come with rowmix32.hip)
STATE_SO_PATH = PKG_DIR / "_hip_state.so"
STATE_SOURCES = ["lnrows32.hip", "state_scan.hip", "delta_scan.hip",
                 "rowmix32.hip", "state_bindings.cpp"]


def _torch_paths():
    import torch

    troot = Path(torch.__file__).resolve().parent
    includes = [
        str(troot / "include"),
        str(troot / "include" / "torch" / "csrc" / "api" / "include"),
        sysconfig.get_paths()["include"],
        str(CSRC),
    ]
    libdir = str(troot / "lib")
    abi = "1" if torch._C._GLIBCXX_USE_CXX11_ABI else "0"
    return includes, libdir, abi


def _common_flags(abi: str, ext_name: str = "_hip_ops"):
    return [
        "-O3",
        # no packed-fp32 VALU forms (v_pk_*_f32) from ordinary float code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-std=c++17",
        "-fPIC",
        f"--offload-arch={ARCH}",
        f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        "-DUSE_ROCM=1",
        "-D__HIP_PLATFORM_AMD__=1",
        "-DHIPBLAS_V2",
        "-DHIP_ENABLE_WARP_SYNC_BUILTINS=1",
        f"-DTORCH_EXTENSION_NAME={ext_name}",
        "-Wno-unused-result",
        "-fvisibility=hidden",
    ]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(
            f"build command failed ({' '.join(cmd[:3])} ...):\n{proc.stderr[-8000:]}"
        )


def build(verbose: bool = False, force: bool = False) -> Path:
    includes, libdir, abi = _torch_paths()
    inc_flags = [f"-I{p}" for p in includes]
    flags = _common_flags(abi)

    objs = []
    newest_src = 0.0
    for src in HIP_SOURCES + CPP_SOURCES + ["common.h"]:
        p = CSRC / src
        if p.exists():
            newest_src = max(newest_src, p.stat().st_mtime)
    if SO_PATH.exists() and not force and SO_PATH.stat().st_mtime >= newest_src:
        return SO_PATH

    build_dir = CSRC / ".build"
    build_dir.mkdir(exist_ok=True)
    for src in HIP_SOURCES + CPP_SOURCES:
        obj = build_dir / (Path(src).stem + ".o")
        srcp = CSRC / src
        if (
            not force
            and obj.exists()
            and obj.stat().st_mtime >= srcp.stat().st_mtime
            and obj.stat().st_mtime >= (CSRC / "common.h").stat().st_mtime
        ):
            objs.append(str(obj))
            continue
        cmd = ["hipcc", *flags, *inc_flags, "-c", str(srcp), "-o", str(obj)]
        if src.endswith(".cpp"):
            cmd.insert(1, "-x")
            cmd.insert(2, "hip")  # binding file still needs hip runtime types
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        _run(cmd)
        objs.append(str(obj))

    link = [
        "hipcc",
        "-shared",
        f"--offload-arch={ARCH}",
        *objs,
        f"-L{libdir}",
        "-ltorch",
        "-ltorch_hip",
        "-ltorch_cpu",
        "-lc10",
        "-lc10_hip",
        "-ltorch_python",
        "-L/opt/rocm/lib",
        "-lamdhip64",
        f"-Wl,-rpath,{libdir}",
        "-o",
        str(SO_PATH),
    ]
    if verbose:
        print(" ".join(link), file=sys.stderr)
    _run(link)
    return SO_PATH


def build_latent(verbose: bool = False, force: bool = True) -> Path:
    """Compile the fp32-residual op family into `_hip_latent.so`."""
    return _build_small("_hip_latent", LATENT_SOURCES, LATENT_SO_PATH,
                        verbose, force)


def build_paged(verbose: bool = False, force: bool = True) -> Path:
    """Compile the paged rotary attention family into `_hip_paged.so`."""
    return _build_small("_hip_paged", PAGED_SOURCES, PAGED_SO_PATH,
                        verbose, force)


def build_state(verbose: bool = False, force: bool = True) -> Path:
    """Compile the layer-norm stream / recurrent mixer family into
    `_hip_state.so`."""
    return _build_small("_hip_state", STATE_SOURCES, STATE_SO_PATH,
                        verbose, force)


def _build_small(ext_name: str, sources: list[str], so_path: Path,
                 verbose: bool, force: bool) -> Path:
    """Compile one small extension, its files in parallel. Objects are
    built under a private name and the library is moved into place at the
    end, so a concurrent reader never sees a half-written file."""
    includes, libdir, abi = _torch_paths()
    inc_flags = [f"-I{p}" for p in includes]
    flags = _common_flags(abi, ext_name)
    build_dir = CSRC / f".build{ext_name}"
    build_dir.mkdir(exist_ok=True)
    newest = max((CSRC / s).stat().st_mtime
                 for s in sources + ["common.h"])
    if (so_path.exists() and not force
            and so_path.stat().st_mtime >= newest):
        return so_path
    cmds, objs = [], []
    for src in sources:
        obj = build_dir / (Path(src).stem + ".o")
        cmd = ["hipcc", *flags, *inc_flags, "-c", str(CSRC / src), "-o", str(obj)]
        if src.endswith(".cpp"):
            cmd[1:1] = ["-x", "hip"]
        cmds.append(cmd)
        objs.append(str(obj))
    if verbose:
        for c in cmds:
            print(" ".join(c), file=sys.stderr)
    procs = [subprocess.Popen(c, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                              text=True) for c in cmds]
    for c, pr in zip(cmds, procs):
        _out, err = pr.communicate()
        if pr.returncode != 0:
            raise RuntimeError(f"build command failed ({' '.join(c[:3])} ...):"
                               f"\n{err[-8000:]}")
    tmp = build_dir / f"{ext_name}.{os.getpid()}.so"
    _run(["hipcc", "-shared", f"--offload-arch={ARCH}", *objs, f"-L{libdir}",
          "-ltorch", "-ltorch_hip", "-ltorch_cpu", "-lc10", "-lc10_hip",
          "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64",
          f"-Wl,-rpath,{libdir}", "-o", str(tmp)])
    os.replace(tmp, so_path)
    return so_path


if __name__ == "__main__":
    if "--latent" in sys.argv:
        build_latent(verbose=True)
        print(f"built {LATENT_SO_PATH}")
    elif "--paged" in sys.argv:
        build_paged(verbose=True)
        print(f"built {PAGED_SO_PATH}")
    elif "--state" in sys.argv:
        build_state(verbose=True)
        print(f"built {STATE_SO_PATH}")
    else:
        build(verbose=True, force="--force" in sys.argv)
        build_latent(verbose=True)
        build_paged(verbose=True)
        build_state(verbose=True)
        print(f"built {SO_PATH} {LATENT_SO_PATH} {PAGED_SO_PATH} "
              f"{STATE_SO_PATH}")
