"""Run by tests/test_gpu_scan_norm.py in a process of its own with THCL_SCAN_CHAIN_SPINS=0 and THCL_SCAN_CHAIN_MUTE=0:
block 0 of the single-pass scan publishes nothing and no wait polls a second time, so every block that needs block 0's
totals gives up at once.  The kernel must still end normally, the next wait for the stream must report the scan as
failed (once), and the library must go on working.  Prints `scan give-up ok`."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import cltorch_amd as cl  # noqa: E402

assert os.environ.get("THCL_SCAN_CHAIN_SPINS") == "0" and os.environ.get("THCL_SCAN_CHAIN_MUTE") == "0"
n = 1 << 24
x = cl.ClTensor(n).fill(1.0)
y = x.cumsum(1)                      # queued; the kernel's waits run out
try:
    cl.synchronize()
except cl.ClError as e:
    assert "did not run at the same time" in str(e), str(e)
else:
    raise SystemExit("the failed scan was not reported")
cl.synchronize()                     # reported once
small = cl.ClTensor(np.arange(1, 1001, dtype=np.float32))
assert small.cumsum(1).float()[-1] == 500500.0      # short rows take other kernels
assert float(small.sum()) == 500500.0
print("scan give-up ok")
