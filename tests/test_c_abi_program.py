"""A plain C99 program (tests/c_abi/roundtrip.c) against include/cortex_hip.h:
what a JNA / JavaCPP binding relies on.  The header must compile as C with no
C++ or HIP headers, every symbol the program uses must link from the shared
library, and on a GPU the program's own checks must pass."""
import pathlib
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
SRC = ROOT / "tests" / "c_abi" / "roundtrip.c"
LIBDIR = ROOT / "cortex_amd"


def build(out: pathlib.Path, src: pathlib.Path = SRC) -> None:
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-O1", f"-I{ROOT / 'include'}", str(src),
           "-o", str(out), f"-L{LIBDIR}", "-lcortex_hip", "-lm", f"-Wl,-rpath,{LIBDIR}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_c99_caller_compiles_and_links(tmp_path):
    assert (LIBDIR / "libcortex_hip.so").exists(), "build the library first: python -m cortex_amd.build"
    build(tmp_path / "roundtrip")
    build(tmp_path / "callrate", ROOT / "tests" / "c_abi" / "callrate.c")


@pytest.mark.gpu
def test_c99_caller_runs(tmp_path):
    exe = tmp_path / "roundtrip"
    build(exe)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert res.stdout.strip() == "ok"
