"""The compiled torch extension over the C ABI (tests/integration/torch_binding.cpp): the
binding a maintainer of the reference would swap in for pytorch_binding/binding.cpp.  It is
built by tests/integration/build_binding.py (or __graft_entry__.build()); these tests skip
when it has not been built."""
import importlib
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

HERE = Path(__file__).resolve().parent


@pytest.fixture(scope="module")
def binding():
    sys.path.insert(0, str(HERE / "integration"))
    try:
        return importlib.import_module("mg_torch_binding")
    except ImportError as exc:
        pytest.skip(f"mg_torch_binding is not built ({exc}); run python tests/integration/build_binding.py")
    finally:
        sys.path.pop(0)


def test_module_surface_and_host_side_checks(binding):
    """Function names and the error text for host tensors follow binding.cpp:9-11,136-139."""
    assert callable(binding.rmsnorm_forward) and callable(binding.rmsnorm_backward)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        binding.rmsnorm_forward(torch.ones(2, 8), torch.ones(8), 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_binding_matches_oracle_and_ctypes_path(binding, dtype):
    import gpu_util as U
    from mgrrmsnorm_amd import ops

    rows, cols, eps = 300, 4096, 1e-6
    x, dy, w = U.rmsnorm_inputs(rows, cols, dtype, seed=5)
    y_ref, s_ref, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, eps, dtype)
    xd, dyd, wd = x.cuda(), dy.cuda(), w.cuda()
    y, s = binding.rmsnorm_forward(xd, wd, eps)
    dx, dw = binding.rmsnorm_backward(dyd, xd, wd, s)
    U.assert_matches(y, y_ref, dtype, "y")
    np.testing.assert_allclose(s.cpu().numpy(), s_ref, rtol=1e-6)
    U.assert_matches(dx, dx_ref, dtype, "dx", floor=floor)
    assert dw.dtype == wd.dtype   # binding.cpp:90
    # same library underneath: bit-identical to the ctypes path
    y2, s2 = ops.rmsnorm_forward(xd, wd, eps)
    dx2, dw2 = ops.rmsnorm_backward(dyd, xd, wd, s2)
    assert torch.equal(y, y2) and torch.equal(s, s2) and torch.equal(dx, dx2) and torch.equal(dw, dw2)


@pytest.mark.gpu
def test_binding_checks_shapes_on_the_gpu(binding):
    x = torch.ones((4, 64), device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError, match="Weight size must match hidden size"):
        binding.rmsnorm_forward(x, torch.ones(32, device="cuda", dtype=torch.float16), 1e-6)
    with pytest.raises(RuntimeError, match="Input must be 2D"):
        binding.rmsnorm_forward(x.view(2, 2, 64), torch.ones(64, device="cuda", dtype=torch.float16), 1e-6)
    with pytest.raises(RuntimeError, match="Unsupported dtype"):
        binding.rmsnorm_forward(x.double(), torch.ones(64, device="cuda", dtype=torch.float64), 1e-6)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        binding.rmsnorm_forward(x.t(), torch.ones(4, device="cuda", dtype=torch.float16), 1e-6)
