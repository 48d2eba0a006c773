import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def cl():
    """The HIP library through its ctypes mirror; fails loudly if it is not built."""
    import cltorch_amd
    cltorch_amd.state()
    return cltorch_amd


@pytest.fixture(scope="session")
def hooks_lib():
    """Test-only entry points over the library's internal host logic: tests/test_hooks.cpp linked with
    the library's own object files into tests/_build/libthcl_test_hooks.so (nothing of it ships)."""
    import ctypes as C
    import subprocess
    from cltorch_amd import build as b
    objs = [os.path.join(b.OBJ, s + ".o") for s in b.SOURCES]
    if not all(os.path.exists(o) for o in objs):
        b.build()
    out_dir = os.path.join(ROOT, "tests", "_build")
    os.makedirs(out_dir, exist_ok=True)
    so = os.path.join(out_dir, "libthcl_test_hooks.so")
    src = os.path.join(ROOT, "tests", "test_hooks.cpp")
    newest = max(os.path.getmtime(p) for p in objs + [src])
    if not os.path.exists(so) or os.path.getmtime(so) < newest:
        obj = os.path.join(out_dir, "test_hooks.o")
        flags = [f for f in b.COMMON if f != "-fvisibility=hidden"]
        subprocess.check_call([b.hipcc()] + b.HOST_ONLY + flags + ["-DTHCL_HOOKS_PLANNERS", "-c", src, "-o", obj])
        # -Bsymbolic: calls between the entry points stay inside this library even when the shipped one is loaded too
        subprocess.check_call([b.hipcc(), "-shared", "-fPIC", "-Wl,-Bsymbolic", f"--offload-arch={b.ARCH}", "-o", so, obj] + objs + ["-lhiprtc", "-pthread"])
    return C.CDLL(so)
