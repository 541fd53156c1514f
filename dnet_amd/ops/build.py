"""In-tree build of the dnet_amd HIP extension for gfx950.

Drives hipcc directly (no hipify, no JIT cache outside the repo): the
resulting ``_C.so`` lives next to this file so it travels with the repo
snapshot to GPU boxes. hipcc cross-compiles gfx950 on machines with no GPU.

Every source under ``csrc/`` is compiled to its own object (in parallel,
cached by mtime under ``csrc/.obj``) and the objects are linked once: a
one-file edit recompiles one translation unit, and a cold build costs the
slowest file instead of the sum of all files.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

OPS_DIR = Path(__file__).resolve().parent
CSRC = OPS_DIR / "csrc"
OBJ_DIR = CSRC / ".obj"
SO_PATH = OPS_DIR / "_C.so"
ARCH = os.environ.get("PYTORCH_ROCM_ARCH", "gfx950")


def _sources() -> list[Path]:
    return sorted(CSRC.glob("*.cpp"))


def _headers() -> list[Path]:
    return sorted(CSRC.glob("*.h"))


def _newest_mtime(paths) -> float:
    return max(p.stat().st_mtime for p in paths)


def needs_build() -> bool:
    if not SO_PATH.exists():
        return True
    return _newest_mtime(_sources() + _headers()) > SO_PATH.stat().st_mtime


def _jobs() -> int:
    n = os.environ.get("MAX_JOBS")
    if n:
        return max(1, min(16, int(n)))
    return max(1, min(16, os.cpu_count() or 4))


def build(verbose: bool = True, force: bool = False) -> Path:
    if not force and not needs_build():
        return SO_PATH
    from torch.utils import cpp_extension as ce

    includes = ce.include_paths() + [sysconfig.get_paths()["include"]]
    lib_dirs = ce.library_paths()
    hipcc = os.environ.get("HIPCC", "hipcc")
    flags = [
        "-O3",
        "-std=c++17",
        f"--offload-arch={ARCH}",
        "-fPIC",
        "-fno-gpu-rdc",
        # packed-fp32 VALU forms are kept out of every kernel in this
        # extension (device-side feature flag; the host pass ignores it)
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-DTORCH_EXTENSION_NAME=_C",
        "-DUSE_ROCM=1",
        "-D__HIP_PLATFORM_AMD__=1",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        # match the wheel's ABI
        "-D_GLIBCXX_USE_CXX11_ABI=1",
    ]
    for inc in includes:
        flags += ["-I", inc]
    OBJ_DIR.mkdir(exist_ok=True)
    hdr_mtime = _newest_mtime(_headers()) if _headers() else 0.0

    def compile_one(src: Path) -> Path:
        obj = OBJ_DIR / (src.name + ".o")
        if (not force and obj.exists()
                and obj.stat().st_mtime >= max(src.stat().st_mtime,
                                               hdr_mtime)):
            return obj
        cmd = [hipcc, *flags, "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[dnet_amd.ops.build] hipcc -c", src.name, file=sys.stderr,
                  flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with ThreadPoolExecutor(_jobs()) as pool:
        objs = list(pool.map(compile_one, _sources()))
    link = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}",
            "-fno-gpu-rdc", *[str(o) for o in objs]]
    for d in lib_dirs:
        link += ["-L", d, f"-Wl,-rpath,{d}"]
    link += ["-ltorch", "-ltorch_python", "-lc10", "-ltorch_hip",
             "-lc10_hip", "-lamdhip64", "-o", str(SO_PATH)]
    if verbose:
        print("[dnet_amd.ops.build] link", SO_PATH.name, file=sys.stderr,
              flush=True)
    subprocess.run(link, check=True)
    return SO_PATH


if __name__ == "__main__":
    build(force="--force" in sys.argv)
