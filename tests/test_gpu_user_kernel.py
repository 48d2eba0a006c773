"""torch.ClKernel: user kernels compiled at run time (src/UserKernel.cpp).
Golden output of the reference's own example: README.md:135-220 adds 3 to
{3, 5, 2} and prints {6, 8, 5}."""
import numpy as np
import pytest

import oracle
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32

README_SRC = """
   int linearId = get_global_id(0);
   if(linearId < nElements) {
     output_data[linearId] = input_data[linearId] + 3.0f;
   }
"""


def test_readme_example(cl):
    k = cl.ClKernel({"input": {"nElements": "int", "input": "torch.ClTensor"}, "output": {"output": "torch.ClTensor"},
                     "src": README_SRC})
    x = cl.ClTensor(np.array([3, 5, 2], dtype=F))
    y = cl.ClTensor(np.array([6, 4, 2], dtype=F))
    k.run({"nElements": 3, "input": x, "output": y})
    assert y.float().tolist() == [6.0, 8.0, 5.0]
    assert x.float().tolist() == [3.0, 5.0, 2.0]
    k.run({"nElements": 3, "input": y, "output": x}, {"numWorkgroups": 10, "workgroupSize": 32})   # README.md:223-225
    assert x.float().tolist() == [9.0, 11.0, 8.0]
    src = k.getRenderedKernel()
    assert "user_kernel" in src and "input_data" in src and "struct THClTensorInfoCl" in src


def test_strided_views_helpers_local_memory_and_scalars(cl):
    rows, cols = 96, 64
    x = oracle.uniform(91, rows * cols).reshape(rows, cols)
    px = Pair.dense(cl, x).transpose(0, 1)                 # 64 x 96 view, strides (1, 64)
    out = cl.ClTensor(cols, rows)
    out.zero()
    k = cl.ClKernel({
        "input": {"src": "ClTensor", "scale": "float", "n": "int"},
        "inout": {"dst": "ClTensor"},
        "name": "scaled_gather",
        "funcs": """
          int view_offset(global struct THClTensorInfoCl *info, int linear) {
            int off = info->offset;
            for (int d = info->dims - 1; d >= 0; d--) {
              off += (linear % (int)info->sizes[d]) * (int)info->strides[d];
              linear /= (int)info->sizes[d];
            }
            return off;
          }""",
        "src": """
          local float stage[64];
          int i = get_global_id(0);
          int l = get_local_id(0);
          stage[l] = (i < n) ? src_data[view_offset(src_info, i)] : 0.0f;
          barrier(CLK_LOCAL_MEM_FENCE);
          // neighbour exchange inside the work-group: dst[i] = scale * src[i ^ 1]
          if (i < n) dst_data[view_offset(dst_info, i)] += scale * stage[l ^ 1];
        """})
    n = rows * cols
    k.run({"src": px.dev, "scale": 2.5, "n": n, "dst": out})
    flat = px.view.gather().reshape(-1)
    want = (F(2.5) * flat.reshape(-1, 2)[:, ::-1].reshape(-1)).astype(F).reshape(cols, rows)
    assert_bit_equal(out.float(), want, "gather through descriptors + LDS exchange")
    assert_bit_equal(px.device_storage(), x.reshape(-1), "input untouched")
    # a narrowed destination: the descriptor's offset must be honoured
    big = cl.ClTensor(2 * n)
    big.zero()
    win = big.narrow(1, n // 2 + 1, n)
    k.run({"src": px.dev, "scale": 1.0, "n": n, "dst": win})
    got = big.float()
    assert np.all(got[:n // 2] == 0) and np.all(got[n // 2 + n:] == 0)
    assert_bit_equal(got[n // 2:n // 2 + n], flat.reshape(-1, 2)[:, ::-1].reshape(-1), "offset view")


def test_errors(cl):
    with pytest.raises(cl.ClError):
        cl.ClKernel({"input": {"a": "ClTensor"}, "src": ""})
    with pytest.raises(cl.ClError):
        cl.ClKernel({"output": {"n": "int"}, "src": "int i = 0;"})              # scalars are inputs only
    with pytest.raises(cl.ClError):
        cl.ClKernel({"input": {"a": "double"}, "src": "int i = 0;"})
    with pytest.raises(cl.ClError):
        cl.ClKernel({"input": {"a": "ClTensor"}, "src": "int i = 0;", "bogus": 1})
    k = cl.ClKernel({"input": {"a": "ClTensor"}, "src": "int i = get_global_id(0); (void)i;"})
    with pytest.raises(cl.ClError, match="at least one output"):
        k.run({"a": cl.ClTensor(4)})
    bad = cl.ClKernel({"output": {"a": "ClTensor"}, "src": "this is not C"})
    with pytest.raises(cl.ClError, match="error"):
        bad.run({"a": cl.ClTensor(4)})
    ok = cl.ClKernel({"output": {"a": "ClTensor"}, "src": "a_data[get_global_id(0)] = 1.0f;"})
    with pytest.raises(cl.ClError):
        ok.run({})
    with pytest.raises(cl.ClError):
        ok.run({"a": cl.ClTensor()})                                              # no storage
    t = cl.ClTensor(64)
    ok.run({"a": t})
    assert t.float().tolist() == [1.0] * 64


def test_reference_script(cl, capsys):
    """src/test/test_userkernel.lua: more work-items than elements, the bound test in the body, print()."""
    src = """
   int linearId = get_global_id(0);
   if(linearId < nElements) {
     output_data[linearId] = input_data[linearId] + 3.0f;
   }
"""
    k = cl.ClKernel({"input": {"nElements": "int", "input": "torch.ClTensor"}, "output": {"output": "torch.ClTensor"}, "src": src})
    text = k.print()
    assert capsys.readouterr().out == text
    assert text.startswith("Original source\n===============\n" + src) and "Generated source\n================\n" in text
    assert k.getRawKernel() == src and "input_data" in k.getRenderedKernel()
    x, y = cl.ClTensor([3, 5, 2]), cl.ClTensor([6, 4, 2])
    k.run({"nElements": 3, "input": x, "output": y}, {"numWorkgroups": 10, "workgroupSize": 32})
    assert y.float().tolist() == [6, 8, 5] and x.float().tolist() == [3, 5, 2]
