"""The library driven from plain C, without Python in between (tests/c_abi_caller.c)."""
import os
import shutil
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="gcc not found")
def test_c_program_links_and_runs(tmp_path):
    libdir = os.path.join(ROOT, "cltorch_amd")
    assert os.path.exists(os.path.join(libdir, "libthcl_hip.so")), "library not built"
    exe = str(tmp_path / "c_abi_caller")
    cmd = ["gcc", "-std=c99", "-Wall", "-O1", "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "c_abi_caller.c"),
           "-L", libdir, "-lthcl_hip", "-lm", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout + r.stderr)[-3000:]
