"""Build recipe for the native parts (run here on CPU; hipcc cross-compiles gfx950).

  libffa_hip.so        C ABI + gfx950 kernels            hipcc  (csrc/*.hip, csrc/*.cpp)
  ff_attention*.so     pybind11 torch extension          g++    (csrc/torch_ffa_api.cpp)

Counterpart of the reference's setup.py:4-16 (CUDAExtension) and compile.sh:6-9
(libffa.so).  Both artefacts are written next to this file so that they travel with the
source tree; nothing is installed into site-packages.

    python -m fastforwardattention_amd._build            # build everything
    python -m fastforwardattention_amd._build --lib      # C-ABI library only
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libffa_hip.so"
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
EXT_PATH = PKG_DIR / f"ff_attention{EXT_SUFFIX}"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

HIP_ARCH = "gfx950"
# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32.
HIPCC_FLAGS = [
    f"--offload-arch={HIP_ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # Leading scalar kernel arguments arrive in SGPRs with the wave (the split kernels take what
    # their first loads need that way); kernels whose only argument is a struct are unaffected.
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function",
]


LIB_HASH = PKG_DIR / "libffa_hip.srchash"
EXT_HASH = PKG_DIR / "ff_attention.srchash"
EXT_SRC = CSRC / "torch_ffa_api.cpp"


def _digest(files, salt) -> str:
    import hashlib
    h = hashlib.sha256(salt.encode())
    for f in sorted(files):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    return h.hexdigest()


def lib_source_hash() -> str:
    """Digest of what libffa_hip.so is compiled from (sources, headers, flags)."""
    files = [f for pat in ("*.hip", "*.cpp", "*.h", "*.inc") for f in CSRC.glob(pat) if f != EXT_SRC]
    return _digest(files + list(INCLUDE.glob("*.h")), " ".join(HIPCC_FLAGS))


def ext_source_hash() -> str:
    """Digest of what the torch extension is compiled from."""
    return _digest([EXT_SRC, *INCLUDE.glob("*.h")], "ext")


def _run(cmd):
    print("+", " ".join(str(c) for c in cmd), flush=True)
    subprocess.run([str(c) for c in cmd], check=True)


def build_lib() -> Path:
    """The device code is seven translation units (the decode kernels once per element type and
    transform switch, the rest), compiled side by side into objects under build/, then linked
    with the host sources."""
    hipcc = ROCM / "bin" / "hipcc"
    units = ["ffa_decode_f16.hip", "ffa_decode_bf16.hip", "ffa_decode_f32.hip", "ffa_decode_f16_xform.hip",
             "ffa_decode_bf16_xform.hip", "ffa_decode_f32_xform.hip", "ffa_kernels.hip"]
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    procs = []
    for u in units:
        cmd = [str(hipcc), *flags, "-c", f"-I{INCLUDE}", f"-I{CSRC}", str(CSRC / u), "-o", str(obj_dir / (u + ".o"))]
        print("+", " ".join(cmd), flush=True)
        procs.append((u, subprocess.Popen(cmd)))
    failed = [u for u, p in procs if p.wait() != 0]
    if failed:
        raise RuntimeError(f"hipcc failed on {failed}")
    objs = [obj_dir / (u + ".o") for u in units]
    _run([hipcc, *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", *objs, CSRC / "ffa_api.cpp", CSRC / "ffa_plan.cpp",
          "-o", LIB_PATH])
    LIB_HASH.write_text(lib_source_hash())
    return LIB_PATH


def build_ext() -> Path:
    import torch
    from torch.utils import cpp_extension as ce

    inc = [f"-I{p}" for p in ce.include_paths()] + [
        f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}", f"-I{ROCM / 'include'}"]
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
           "-DTORCH_EXTENSION_NAME=ff_attention", "-DTORCH_API_INCLUDE_EXTENSION_H",
           *inc, CSRC / "torch_ffa_api.cpp", "-o", EXT_PATH,
           f"-L{torch_lib}", f"-L{PKG_DIR}", f"-L{ROCM / 'lib'}",
           "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
           "-lffa_hip", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", f"-Wl,-rpath,{ROCM / 'lib'}"]
    _run(cmd)
    EXT_HASH.write_text(ext_source_hash())
    return EXT_PATH


def build_all() -> None:
    build_lib()
    build_ext()


def _current(artefact, hash_file, digest) -> bool:
    try:
        return artefact.exists() and hash_file.read_text().strip() == digest()
    except OSError:
        return False


def ensure_built() -> None:
    """Tests, the smoke run and the benchmark load what is built.  An artefact is rebuilt when
    it is missing or when a file it is compiled from has changed since its build (a digest of
    the sources is kept next to each artefact), so a green run speaks for the tree as it is."""
    if not _current(LIB_PATH, LIB_HASH, lib_source_hash):
        build_lib()
    if not _current(EXT_PATH, EXT_HASH, ext_source_hash):
        build_ext()


if __name__ == "__main__":
    if "--lib" in sys.argv:
        build_lib()
    elif "--ext" in sys.argv:
        build_ext()
    else:
        build_all()
