"""C++ host-side checks that need no GPU:

* a translation unit written against the reference's c_ffa_api.h (c_ffa_api.h:5-20:
  call_attention<T>, do_attention<T>) compiles against include/ffa_reference_shim.h with
  -Wall -Wextra -Werror and links against the built libffa_hip.so;
* ffa_api.cpp + ffa_plan.cpp (argument validation, planning, workspace carving) are built with
  AddressSanitizer and UndefinedBehaviorSanitizer, the launchers replaced by checking stubs, and
  driven by a randomized sequence of C-ABI calls (tests/host_cpp/host_fuzz.cpp)."""
import os
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
INCLUDE = ROOT / "include"
CSRC = ROOT / "fastforwardattention_amd" / "csrc"
PKG = ROOT / "fastforwardattention_amd"
CPP = ROOT / "tests" / "host_cpp"

pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not available")


def _run(cmd, **kw):
    res = subprocess.run([str(c) for c in cmd], capture_output=True, text=True, **kw)
    assert res.returncode == 0, f"{' '.join(str(c) for c in cmd)}\n{res.stdout}\n{res.stderr}"
    return res


def test_reference_shim_compiles_with_the_reference_call_sites():
    _run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", f"-I{INCLUDE}", CPP / "shim_user.cpp"])
    # The header is also plain C++11 (the reference builds with nvcc's default dialect).
    _run(["g++", "-std=c++11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", f"-I{INCLUDE}", CPP / "shim_user.cpp"])


def test_reference_shim_links_against_the_library(tmp_path):
    lib = PKG / "libffa_hip.so"
    if not lib.exists():
        pytest.skip("libffa_hip.so not built")
    rocm_lib = Path(os.environ.get("ROCM_PATH", "/opt/rocm")) / "lib"
    exe = tmp_path / "shim_user"
    _run(["g++", "-std=c++17", f"-I{INCLUDE}", CPP / "shim_user.cpp", "-o", exe, f"-L{PKG}", "-lffa_hip",
          f"-Wl,-rpath-link,{rocm_lib}", f"-Wl,-rpath,{PKG}"])
    assert exe.exists()


def test_host_logic_under_sanitizers(tmp_path):
    exe = tmp_path / "host_fuzz"
    _run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
          f"-I{INCLUDE}", f"-I{CSRC}", CPP / "host_fuzz.cpp", CSRC / "ffa_api.cpp", CSRC / "ffa_plan.cpp", "-o", exe])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)  # a preloaded library ahead of the ASan runtime stops the program at start-up
    for seed in (1, 2, 3):
        res = _run([exe, "200000", str(seed)], env=env)
        assert "host fuzz: 200000 calls" in res.stdout
