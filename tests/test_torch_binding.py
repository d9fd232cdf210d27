"""The compiled torch extension over the C ABI (mgrrmsnorm_amd/csrc/torch_binding.cpp, built
by mgrrmsnorm_amd._build into mgrrmsnorm_amd/_binding*.so): what replaces the reference's
pytorch_binding/binding.cpp.  It must agree bit for bit with the ctypes binding of the same
library, and its C++ autograd nodes with the Python autograd.Functions."""
import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def binding():
    try:
        from mgrrmsnorm_amd import _binding
    except ImportError as exc:
        pytest.fail(f"mgrrmsnorm_amd._binding is not built ({exc}); run python -m mgrrmsnorm_amd._build")
    return _binding


def test_module_surface_and_host_side_checks(binding):
    """Function names and the error text for host tensors follow binding.cpp:9-11,136-139."""
    from mgrrmsnorm_amd import _lib, ops

    for name in ("rmsnorm_forward", "rmsnorm_backward", "rmsnorm_backward_f32", "swiglu_forward", "swiglu_backward",
                 "rmsnorm", "swiglu"):
        assert callable(getattr(binding, name)), name
    assert binding.abi_version() == _lib.ABI_VERSION          # the library it loaded
    assert binding.built_abi_version() == _lib.ABI_VERSION    # the header it was compiled against
    assert ops.backend() == "extension"      # the package uses it as soon as it is built
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        binding.rmsnorm_forward(torch.ones(2, 8), torch.ones(8), 1e-6)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        binding.swiglu_forward(torch.ones(2, 8), 4)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        binding.rmsnorm(torch.ones(2, 8), torch.ones(8), 1e-6)


def test_stale_extension_is_refused():
    """An extension compiled against another version of the header, or one without the
    compile-time constant at all (built before it existed), must not be used."""
    import types

    from mgrrmsnorm_amd import _lib, ops

    v = _lib.ABI_VERSION
    ok = types.SimpleNamespace(__file__="x.so", abi_version=lambda: v, built_abi_version=lambda: v)
    ops._check_extension_abi(ok)
    old_header = types.SimpleNamespace(__file__="x.so", abi_version=lambda: v, built_abi_version=lambda: v - 1)
    with pytest.raises(RuntimeError, match=f"compiled against ABI {v - 1}"):
        ops._check_extension_abi(old_header)
    no_constant = types.SimpleNamespace(__file__="x.so", abi_version=lambda: v)
    with pytest.raises(RuntimeError, match="compiled against ABI None"):
        ops._check_extension_abi(no_constant)
    old_library = types.SimpleNamespace(__file__="x.so", abi_version=lambda: v + 1, built_abi_version=lambda: v)
    with pytest.raises(RuntimeError, match=f"loaded a libmegagemm_hip.so of ABI {v + 1}"):
        ops._check_extension_abi(old_library)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_binding_matches_oracle_and_ctypes_path(binding, dtype):
    import gpu_util as U
    from mgrrmsnorm_amd import ops_ctypes

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
    dx3, dw32, dwc = binding.rmsnorm_backward_f32(dyd, xd, wd, s)
    U.assert_dw(dw32, dw_ref)
    assert torch.equal(dx3, dx) and torch.equal(dwc, dw)
    dx4, none1, none2 = binding.rmsnorm_backward_f32(dyd, xd, wd, s, need_weight_grad=False)
    assert none1 is None and none2 is None and torch.equal(dx4, dx)
    # same library underneath: bit-identical to the ctypes binding
    y2, s2 = ops_ctypes.rmsnorm_forward(xd, wd, eps)
    dx2, dw2 = ops_ctypes.rmsnorm_backward(dyd, xd, wd, s2)
    assert torch.equal(y, y2) and torch.equal(s, s2) and torch.equal(dx, dx2) and torch.equal(dw, dw2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_swiglu_binding_matches_oracle_and_ctypes_path(binding, dtype):
    import gpu_util as U
    from mgrrmsnorm_amd import ops_ctypes

    M, H = 130, 1376
    gu = U.cpu_randn((M, 2 * H), 3).to(U.DTYPES[dtype])
    dh = U.cpu_randn((M, H), 4).to(U.DTYPES[dtype])
    h_ref, d_ref, floor = U.swiglu_reference(gu, dh, dtype)
    gud, dhd = gu.cuda(), dh.cuda()
    h = binding.swiglu_forward(gud, H)
    d = binding.swiglu_backward(dhd, gud, H)
    U.assert_matches(h, h_ref, dtype, "h")
    U.assert_matches(d, d_ref, dtype, "dgu", floor=floor)
    assert torch.equal(h, ops_ctypes.swiglu_forward(gud, H)) and torch.equal(d, ops_ctypes.swiglu_backward(dhd, gud, H))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cpp_autograd_nodes_match_python_functions(binding, dtype):
    """binding.rmsnorm / binding.swiglu (autograd nodes in C++) against RMSNormFunction /
    MegaGemmFunction (Python autograd.Functions over the same kernels): identical bits."""
    from mgrrmsnorm_amd import MegaGemmFunction, RMSNormFunction

    g = torch.Generator().manual_seed(9)
    x = torch.randn((3, 50, 768), generator=g).to(dtype).cuda()
    w = (1 + 0.02 * torch.randn(768, generator=g)).to(dtype).cuda()
    dy = torch.randn((3, 50, 768), generator=g).to(dtype).cuda()
    outs = []
    for fn in (lambda a, b: binding.rmsnorm(a, b, 1e-6), lambda a, b: RMSNormFunction.apply(a, b, 1e-6)):
        xa, wa = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        y = fn(xa, wa)
        assert y.shape == x.shape and y.requires_grad
        y.backward(dy)
        outs.append((y.detach(), xa.grad, wa.grad))
    for a, b in zip(*outs):
        assert a.dtype == b.dtype and torch.equal(a, b)
    # only the input needs a gradient: no dW is produced
    xa = x.clone().requires_grad_(True)
    binding.rmsnorm(xa, w, 1e-6).backward(dy)
    assert torch.equal(xa.grad, outs[0][1]) and w.grad is None
    # nothing needs a gradient: plain forward, no node
    assert binding.rmsnorm(x, w, 1e-6).grad_fn is None
    with torch.no_grad():
        assert torch.equal(binding.rmsnorm(x.clone().requires_grad_(True), w, 1e-6), outs[0][0])

    H = 344
    gu = torch.randn((4, 33, 2 * H), generator=g).to(dtype).cuda()
    dh = torch.randn((4, 33, H), generator=g).to(dtype).cuda()
    outs = []
    for fn in (binding.swiglu, MegaGemmFunction.apply):
        ga = gu.clone().requires_grad_(True)
        h = fn(ga, H)
        assert h.shape == (4, 33, H)
        h.backward(dh)
        outs.append((h.detach(), ga.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert binding.swiglu(gu, H).grad_fn is None
    with pytest.raises(RuntimeError, match="2\\*hidden_dim"):
        binding.swiglu(gu, H + 1)


@pytest.mark.gpu
def test_cpp_autograd_nodes_refuse_a_second_derivative(binding):
    x = torch.randn((4, 64), device="cuda", requires_grad=True)
    w = torch.ones(64, device="cuda", requires_grad=True)
    y = binding.rmsnorm(x, w, 1e-5)
    (gx,) = torch.autograd.grad(y.sum(), x, create_graph=False)
    assert not gx.requires_grad
    y = binding.rmsnorm(x, w, 1e-5)
    dy = torch.ones_like(y, requires_grad=True)
    with pytest.raises(RuntimeError, match="differentiate twice"):
        torch.autograd.grad(y, x, grad_outputs=dy, create_graph=True)


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
    with pytest.raises(RuntimeError, match="weight dtype"):
        binding.rmsnorm(x, torch.ones(64, device="cuda", dtype=torch.float32), 1e-6)


@pytest.mark.gpu
def test_modules_give_the_same_bits_through_either_binding(binding, monkeypatch):
    """megagemm.RMSNorm / MegaGemmTriton through the compiled extension (C++ autograd nodes)
    and through the ctypes binding (Python autograd.Functions): same outputs and gradients."""
    import megagemm
    from mgrrmsnorm_amd import ops

    torch.manual_seed(3)
    norm = megagemm.RMSNorm(1024, 1e-6).cuda().to(torch.bfloat16)
    mlp = megagemm.MegaGemmTriton(1024).cuda().to(torch.bfloat16)
    x = torch.randn(4, 40, 1024, device="cuda", dtype=torch.bfloat16)
    g = torch.randn(4, 40, 1024, device="cuda", dtype=torch.bfloat16)

    def run():
        for p in list(norm.parameters()) + list(mlp.parameters()):
            p.grad = None
        xa = x.clone().requires_grad_(True)
        y = mlp(norm(xa))
        y.backward(g)
        return [y.detach(), xa.grad, norm.weight.grad, mlp.w12.weight.grad, mlp.w3.weight.grad]

    assert ops.backend() == "extension"
    via_extension = run()
    monkeypatch.setattr(ops, "_binding", None)
    monkeypatch.setattr(ops, "_resolved", True)
    assert ops.backend() == "ctypes"
    via_ctypes = run()
    for a, b in zip(via_extension, via_ctypes):
        assert torch.equal(a, b)
