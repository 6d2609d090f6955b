"""llc_hip_matmul_static, the entry point that allocates nothing: same bits as llc_hip_matmul on products whose
reduction is split (partial sums in scratch memory: the library's static device array here, a grown buffer
there), two calls in a row, the second on a smaller input that reuses the array with the first call's contents
still in it.  Called through the C-ABI (ctypes), like every GPU test."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")


def _operands(m, n, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    a = (torch.rand(m, k, generator=g) * 2 - 1).to(dtype).cuda()
    w = (torch.rand(n, k, generator=g) * 2 - 1).to(dtype).cuda()  # a Linear weight, consumed as its transposed view
    bias = (torch.rand(n, generator=g) * 2 - 1).to(dtype).cuda()
    return a, w.t(), bias


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_entry_equals_matmul_on_two_calls_in_a_row(dtype):
    from llcompiler_amd import ops
    # reductions long enough, and outputs small enough, that both products split k (and keep partial sums)
    first = _operands(1024, 768, 3072, dtype, 1)
    second = _operands(512, 384, 2048, dtype, 2)
    outs = []
    for a, b, bias in (first, second):
        out = torch.full((a.shape[0], b.shape[1]), float("nan"), dtype=dtype, device="cuda")
        ops.matmul_static(a, b, out, ops.Epilogue(bias=bias, act="relu"))
        outs.append(out)
    torch.cuda.synchronize()
    for (a, b, bias), got in zip((first, second), outs):
        want = ops.matmul(a, b, ops.Epilogue(bias=bias, act="relu"))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(got.float().cpu().numpy(), want.float().cpu().numpy())
        assert not torch.isnan(got).any()


def test_static_entry_takes_no_device_memory():
    """hipMemGetInfo reads the same before and after (outputs allocated beforehand)."""
    from llcompiler_amd import ops
    a, b, bias = _operands(1024, 768, 3072, torch.float32, 3)
    out = torch.empty((1024, 768), dtype=torch.float32, device="cuda")
    ops.matmul_static(a, b, out)  # first call on the device: looks the array's address up
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        ops.matmul_static(a, b, out, ops.Epilogue(bias=bias))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0


def test_static_entry_without_a_split_reduction_and_errors():
    from llcompiler_amd import ops
    from llcompiler_amd._capi import LlcHipError
    a, b, _ = _operands(300, 200, 128, torch.float32, 4)
    out = torch.empty((300, 200), dtype=torch.float32, device="cuda")
    ops.matmul_static(a, b, out)
    want = ops.matmul(a, b)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), want.cpu().numpy())
    with pytest.raises(LlcHipError):
        ops.matmul_static(a, b, torch.empty((300, 201), dtype=torch.float32, device="cuda"))
