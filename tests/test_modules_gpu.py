"""The nn.Module / autograd surface on the GPU: the reference's own test flow
(test_rmsnorm.py:31-130: seed 42, [32*128, 4096] fp32, w ~ randn, eps 1e-5, loss = out.sum(),
abs tolerances 1e-4 / 1e-3, gradcheck with its settings), the benchmark script's block
check (benchmark_swiglu.py:40-58,85-89,121-129), and the drop-in module names."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import gpu_util as U

pytestmark = pytest.mark.gpu


def _formula(x, w, eps):
    # test_rmsnorm.py:55-56
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def test_reference_manual_check_flow():
    from megagemm import RMSNorm

    torch.manual_seed(42)
    hidden = 4096
    inp = torch.randn(32 * 128, hidden, device="cuda", requires_grad=True)
    weight = torch.randn(hidden, device="cuda", requires_grad=True)
    inp_ref = inp.detach().clone().requires_grad_(True)
    w_ref = weight.detach().clone().requires_grad_(True)
    out_ref = _formula(inp_ref, w_ref, 1e-5)
    out_ref.sum().backward()

    model = RMSNorm(hidden).to("cuda")
    model.weight = torch.nn.Parameter(weight.detach().clone())
    out = model(inp)
    out.sum().backward()

    assert (out - out_ref.detach()).abs().max() < 1e-4            # asserted by the reference
    assert (inp.grad - inp_ref.grad).abs().max() < 1e-3           # only printed by the reference
    # dW entries are sums of 4096 terms of size ~1: compare on the scale of the data
    assert (model.weight.grad - w_ref.grad).abs().max() < 1e-3 * w_ref.grad.abs().max()


def test_reference_gradcheck_settings():
    from megagemm import RMSNormFunction

    torch.manual_seed(0)
    x = torch.randn(8, 128, device="cuda", dtype=torch.float32, requires_grad=True)
    w = torch.randn(128, device="cuda", dtype=torch.float32, requires_grad=True)
    assert torch.autograd.gradcheck(RMSNormFunction.apply, (x, w, 1e-5), eps=1e-3, atol=1e-2, rtol=1e-3,
                                    nondet_tol=0.0)


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_module_on_3d_input_matches_oracle(dtype):
    from mgrrmsnorm_amd import RMSNorm

    td = U.DTYPES[dtype]
    B, S, C = 4, 37, 1024
    x, dy, w = U.rmsnorm_inputs(B * S, C, dtype, seed=8)
    y_ref, _, dx_ref, dw_ref, floor = U.rmsnorm_reference(x, dy, w, 1e-6, dtype)
    norm = RMSNorm(C, 1e-6).cuda().to(td)
    with torch.no_grad():
        norm.weight.copy_(w.cuda())
    xin = x.cuda().view(B, S, C).requires_grad_(True)
    y = norm(xin)
    assert y.shape == (B, S, C) and y.dtype == td
    y.backward(dy.cuda().view(B, S, C))
    U.assert_matches(y.view(-1, C), y_ref, dtype, "y")
    U.assert_matches(xin.grad.view(-1, C), dx_ref, dtype, "dx", floor=floor)
    assert norm.weight.grad.dtype == td and norm.weight.grad.shape == (C,)
    # grad_weight is the fp32 column sum rounded once to the weight type
    U.assert_matches(norm.weight.grad, dw_ref, dtype, "dW (weight dtype)",
                     floor=np.full(C, np.abs(dw_ref).max() * 64))


def test_non_contiguous_inputs_and_grads():
    from mgrrmsnorm_amd import RMSNorm

    norm = RMSNorm(256, 1e-6).cuda()
    base = torch.randn(16, 512, device="cuda")
    x = base[:, ::2]                       # non-contiguous view
    assert not x.is_contiguous()
    xr = x.detach().clone().requires_grad_(True)
    xin = x.detach().requires_grad_(True)
    y = norm(xin)
    yr = _formula(xr, norm.weight.detach(), 1e-6)
    torch.testing.assert_close(y, yr, rtol=1e-5, atol=1e-6)
    g = torch.randn(512, 16, device="cuda").t()[:, ::2]   # non-contiguous upstream gradient
    y.backward(g)
    yr.backward(g)
    torch.testing.assert_close(xin.grad, xr.grad, rtol=1e-4, atol=1e-5)


def test_weight_dtype_must_match_input():
    from mgrrmsnorm_amd import RMSNorm

    norm = RMSNorm(64).cuda()              # fp32 weight
    with pytest.raises(RuntimeError, match="weight dtype"):
        norm(torch.randn(4, 64, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="Unsupported dtype"):
        norm.double()(torch.randn(4, 64, device="cuda", dtype=torch.float64))


def test_extension_module_shim_returns():
    import rmsnorm_cuda_ops

    x = torch.randn(64, 512, device="cuda", dtype=torch.float16)
    w = torch.randn(512, device="cuda", dtype=torch.float16)
    out, inv_rms = rmsnorm_cuda_ops.rmsnorm_forward(x, w, 1e-5)
    assert out.shape == x.shape and out.dtype == x.dtype
    assert inv_rms.shape == (64,) and inv_rms.dtype == torch.float32
    gi, gw = rmsnorm_cuda_ops.rmsnorm_backward(torch.ones_like(x), x, w, inv_rms)
    assert gi.shape == x.shape and gi.dtype == x.dtype
    assert gw.shape == w.shape and gw.dtype == w.dtype          # weight dtype, as binding.cpp:90
    with pytest.raises(RuntimeError, match="must be contiguous"):
        rmsnorm_cuda_ops.rmsnorm_forward(x.t(), w, 1e-5)
    with pytest.raises(RuntimeError, match="Input must be 2D"):
        rmsnorm_cuda_ops.rmsnorm_forward(x.view(4, 16, 512), w, 1e-5)
    with pytest.raises(RuntimeError, match="Weight size must match hidden size"):
        rmsnorm_cuda_ops.rmsnorm_forward(x, w[:100].contiguous(), 1e-5)


class _UnfusedSwiGLU(torch.nn.Module):
    """Separate gate / up / down projections with F.silu, the baseline the reference's
    benchmark compares against (benchmark_swiglu.py:40-58)."""

    def __init__(self, d_model, hidden):
        super().__init__()
        self.w1 = torch.nn.Linear(d_model, hidden, bias=False)
        self.w2 = torch.nn.Linear(d_model, hidden, bias=False)
        self.w3 = torch.nn.Linear(hidden, d_model, bias=False)

    def forward(self, x):
        return self.w3(F.silu(self.w1(x)) * self.w2(x))


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-2), (torch.bfloat16, 6e-2), (torch.float32, 1e-4)])
def test_swiglu_block_against_unfused_baseline(dtype, tol):
    from megagemm import MegaGemmTriton

    torch.manual_seed(1)
    d_model = 1024
    block = MegaGemmTriton(d_model).cuda().to(dtype)
    base = _UnfusedSwiGLU(d_model, block.hidden).cuda().to(dtype)
    with torch.no_grad():                                         # benchmark_swiglu.py:85-89
        block.w12.weight[: block.hidden] = base.w1.weight
        block.w12.weight[block.hidden:] = base.w2.weight
        block.w3.weight.copy_(base.w3.weight)
    x = torch.randn(8, 128, d_model, device="cuda", dtype=dtype)
    xa = x.clone().requires_grad_(True)
    xb = x.clone().requires_grad_(True)
    ya, yb = block(xa), base(xb)
    assert ya.shape == (8, 128, d_model)
    assert (ya - yb).abs().max().item() < tol                     # the reference's check: < 1e-2 in fp16
    g = torch.randn_like(ya)
    ya.backward(g)
    yb.backward(g)
    scale = xb.grad.abs().max().item()
    assert (xa.grad - xb.grad).abs().max().item() < 2e-2 * scale
    gw = torch.cat([base.w1.weight.grad, base.w2.weight.grad])
    assert (block.w12.weight.grad - gw).abs().max().item() < 2e-2 * gw.abs().max().item()


def test_swiglu_block_at_the_benchmark_size():
    """The SwiGLU block configuration of the benchmark at its own size: d_model 4096,
    hidden 11008 (hidden_multiple = 2.6875), x [8, 1024, 4096] bf16, weights N(0, 0.02), against
    the unfused PyTorch block with the same weights (benchmark_swiglu.py:40-58,85-89).  The two
    sides differ by the rounding of bf16 intermediates and by the order in which two matmuls
    of different shape add up their terms, hence tolerances rather than ulps; the activation
    itself is held to 1 ulp against the oracle in test_swiglu_gpu.py."""
    from megagemm import MegaGemmTriton

    torch.manual_seed(42)
    d_model, dtype = 4096, torch.bfloat16
    block = MegaGemmTriton(d_model, hidden_multiple=2.6875).cuda().to(dtype)
    assert block.hidden == 11008 and block.w12.weight.shape == (22016, 4096) and block.w3.weight.shape == (4096, 11008)
    base = _UnfusedSwiGLU(d_model, block.hidden).cuda().to(dtype)
    with torch.no_grad():
        for p in base.parameters():
            p.normal_(0.0, 0.02)
        block.w12.weight[: block.hidden] = base.w1.weight
        block.w12.weight[block.hidden:] = base.w2.weight
        block.w3.weight.copy_(base.w3.weight)
    x = torch.randn(8, 1024, d_model, device="cuda", dtype=dtype)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = block(xa), base(xb)
    assert ya.shape == (8, 1024, d_model)
    diff = (ya.float() - yb.float())
    scale = yb.float().abs().max().item()
    assert diff.abs().max().item() < 2e-2 * scale
    assert (diff.norm() / yb.float().norm()).item() < 1e-2
    g = torch.randn_like(ya)
    ya.backward(g)
    yb.backward(g)
    for got, ref in ((xa.grad, xb.grad), (block.w3.weight.grad, base.w3.weight.grad),
                     (block.w12.weight.grad, torch.cat([base.w1.weight.grad, base.w2.weight.grad]))):
        err = (got.float() - ref.float())
        assert err.abs().max().item() < 3e-2 * ref.float().abs().max().item()
        assert (err.norm() / ref.float().norm()).item() < 1e-2


def test_activation_function_gradient_layout():
    """MegaGemmFunction.backward returns [d_gate | d_up] for the fused input and None for
    hidden_dim (megagemm/swiglu.py:131)."""
    from megagemm import MegaGemmFunction

    H = 96
    t = torch.randn(3, 5, 2 * H, device="cuda", requires_grad=True)
    out = MegaGemmFunction.apply(t, H)
    assert out.shape == (3, 5, H)
    r = t.detach().clone().requires_grad_(True)
    ref = F.silu(r[..., :H]) * r[..., H:]
    g = torch.randn_like(out)
    out.backward(g)
    ref.backward(g)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(t.grad, r.grad, rtol=1e-4, atol=1e-5)


def test_state_dict_round_trip_between_module_names():
    import megagemm
    import mgrrmsnorm_amd

    a = megagemm.MegaGemmTriton(256).cuda()
    b = mgrrmsnorm_amd.MegaGemmTriton(256).cuda()
    b.load_state_dict(a.state_dict())
    x = torch.randn(4, 256, device="cuda")
    assert torch.equal(a(x), b(x))
    n1, n2 = megagemm.RMSNorm(256).cuda(), mgrrmsnorm_amd.RMSNorm(256).cuda()
    n2.load_state_dict(n1.state_dict())
    assert torch.equal(n1(x), n2(x))


def test_module_forward_backward_under_graph_capture():
    """The nn.Module path (allocation through torch's caching allocator, launches through the
    C ABI) captured into one HIP graph: replays, separated by eager work, reproduce the eager
    gradients.  This is the way to run small shapes without paying the Python round trip."""
    from mgrrmsnorm_amd import MegaGemmFunction, RMSNorm

    torch.manual_seed(3)
    C, H = 2048, 1024
    norm = RMSNorm(C, 1e-6).cuda().to(torch.bfloat16)
    x = torch.randn(256, C, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    proj = torch.randn(C, 2 * H, device="cuda", dtype=torch.bfloat16) * 0.05
    g = torch.randn(256, H, device="cuda", dtype=torch.bfloat16)

    def step():
        x.grad = None
        norm.weight.grad = None
        out = MegaGemmFunction.apply(norm(x) @ proj, H)
        out.backward(g)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                     # warm-up off the default stream, as capture requires
        for _ in range(3):
            want_out = step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = (want_out.clone(), x.grad.clone(), norm.weight.grad.clone())

    graph = torch.cuda.CUDAGraph()
    x.grad = None
    norm.weight.grad = None
    with torch.cuda.graph(graph):
        out = step()
    for i in range(3):
        torch.zeros(1024, device="cuda").add_(1)       # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want[0]), f"replay {i}: output"
        assert torch.equal(x.grad, want[1]), f"replay {i}: dx"
        assert torch.equal(norm.weight.grad, want[2]), f"replay {i}: dW"


def test_concurrent_calls_from_several_threads():
    """The library is re-entrant: four threads, each on its own stream, run forward+backward
    at the same time and each gets the answer a lone call gives."""
    import threading

    from mgrrmsnorm_amd import ops

    torch.manual_seed(11)
    C = 2048
    w = (1 + 0.02 * torch.randn(C, device="cuda")).to(torch.bfloat16)
    xs = [torch.randn(300 + 17 * i, C, device="cuda").to(torch.bfloat16) for i in range(4)]
    gs = [torch.randn_like(x) for x in xs]
    want = []
    for x, g in zip(xs, gs):
        y, s = ops.rmsnorm_forward(x, w, 1e-6)
        dx, dw32, _ = ops.rmsnorm_backward_f32(g, x, w, s)
        want.append((y, dx, dw32))
    torch.cuda.synchronize()
    got, errors = [None] * 4, []

    def work(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    y, s = ops.rmsnorm_forward(xs[i], w, 1e-6)
                    dx, dw32, _ = ops.rmsnorm_backward_f32(gs[i], xs[i], w, s)
            stream.synchronize()
            got[i] = (y, dx, dw32)
        except Exception as exc:  # surfaced below, in the main thread
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(4):
        for a, b in zip(got[i], want[i]):
            assert torch.equal(a, b), f"thread {i}"


def test_double_backward_is_refused_cleanly():
    """The backward pass is not itself differentiable (as in the reference, whose backward
    calls an opaque extension): asking for a second derivative raises instead of returning
    something wrong."""
    from mgrrmsnorm_amd import RMSNorm

    norm = RMSNorm(128).cuda()
    x = torch.randn(4, 128, device="cuda", requires_grad=True)
    (gx,) = torch.autograd.grad(norm(x).sum(), x, create_graph=True)
    with pytest.raises(RuntimeError):
        gx.sum().backward()


def test_inference_path_equals_autograd_path():
    """Under torch.no_grad() the modules skip the autograd node; outputs are bit-identical."""
    from mgrrmsnorm_amd import MegaGemmTriton, RMSNorm

    torch.manual_seed(4)
    norm = RMSNorm(1024, 1e-6).cuda().to(torch.bfloat16)
    mlp = MegaGemmTriton(1024).cuda().to(torch.bfloat16)
    x = torch.randn(3, 50, 1024, device="cuda", dtype=torch.bfloat16)
    y_grad = mlp(norm(x))
    assert y_grad.requires_grad
    with torch.no_grad():
        y_inf = mlp(norm(x))
    assert not y_inf.requires_grad and torch.equal(y_grad.detach(), y_inf)
    for p in list(norm.parameters()) + list(mlp.parameters()):
        p.requires_grad_(False)
    assert torch.equal(mlp(norm(x)), y_inf)          # frozen weights, input without grad
    xg = x.clone().requires_grad_(True)              # frozen weights, input with grad: autograd path
    mlp(norm(xg)).sum().backward()
    assert xg.grad is not None


def test_frozen_weight_skips_the_dw_reduction():
    from mgrrmsnorm_amd import RMSNorm

    norm = RMSNorm(512, 1e-6).cuda()
    x = torch.randn(40, 512, device="cuda", requires_grad=True)
    norm(x).sum().backward()
    want = x.grad.clone()
    assert norm.weight.grad is not None
    norm.weight.requires_grad_(False)
    norm.weight.grad = None
    x.grad = None
    norm(x).sum().backward()
    assert norm.weight.grad is None and torch.equal(x.grad, want)


def test_backward_on_the_calling_thread_gives_the_same_bits():
    """torch.autograd.set_multithreading_enabled(False) makes the engine run the backward pass
    on the calling thread instead of its device worker; the nodes must not care."""
    from mgrrmsnorm_amd import MegaGemmTriton, RMSNorm

    torch.manual_seed(11)
    norm = RMSNorm(2048, 1e-6).cuda().to(torch.bfloat16)
    mlp = MegaGemmTriton(2048).cuda().to(torch.bfloat16)
    x = torch.randn(5, 33, 2048, device="cuda", dtype=torch.bfloat16)
    dy = torch.randn_like(x)

    def grads():
        xg = x.clone().requires_grad_(True)
        for p in list(norm.parameters()) + list(mlp.parameters()):
            p.grad = None
        mlp(norm(xg)).backward(dy)
        return [xg.grad.clone()] + [p.grad.clone() for p in list(norm.parameters()) + list(mlp.parameters())]

    want = grads()
    with torch.autograd.set_multithreading_enabled(False):
        got = grads()
    assert all(torch.equal(a, b) for a, b in zip(want, got))
