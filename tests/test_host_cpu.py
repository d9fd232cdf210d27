"""Host-side mirror of the reference's Python surface, checked without a GPU: names,
signatures, defaults, parameter names and shapes, repr text, hidden-size rounding, lazy
exports, and the error behaviour for tensors the kernels cannot take."""
import importlib
import inspect

import pytest
import torch


def test_lazy_exports_and_unknown_attribute():
    import mgrrmsnorm_amd as m

    assert m.__version__ == "0.1.0"
    # the reference's four names and version; the one addition is the autograd-threading helper
    assert set(m.__all__) == {"RMSNorm", "RMSNormFunction", "MegaGemmTriton", "MegaGemmFunction", "__version__",
                              "backward_on_calling_thread"}
    for name in ("RMSNorm", "RMSNormFunction", "MegaGemmTriton", "MegaGemmFunction"):
        assert getattr(m, name).__name__ == name
    with pytest.raises(AttributeError, match="has no attribute 'Nope'"):
        m.Nope


def test_backward_on_calling_thread_wraps_torchs_switch():
    import threading

    import megagemm

    seen = []

    class Probe(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            return x * 2

        @staticmethod
        def backward(ctx, g):
            seen.append(threading.get_ident())
            return g * 2

    assert torch.autograd.is_multithreading_enabled()
    with megagemm.backward_on_calling_thread():
        assert not torch.autograd.is_multithreading_enabled()
        x = torch.ones(4, requires_grad=True)
        Probe.apply(x).sum().backward()
    assert torch.autograd.is_multithreading_enabled()
    assert seen == [threading.get_ident()] and torch.equal(x.grad, torch.full((4,), 2.0))


def test_megagemm_alias_package():
    import megagemm
    import mgrrmsnorm_amd

    assert megagemm.RMSNorm is mgrrmsnorm_amd.RMSNorm
    assert megagemm.MegaGemmTriton is mgrrmsnorm_amd.MegaGemmTriton
    assert megagemm.__version__ == mgrrmsnorm_amd.__version__
    with pytest.raises(AttributeError, match="module 'megagemm' has no attribute"):
        megagemm.missing_name
    from megagemm import MegaGemmFunction, RMSNormFunction  # noqa: F401


def test_extension_module_alias():
    ops = importlib.import_module("rmsnorm_cuda_ops")
    assert list(inspect.signature(ops.rmsnorm_forward).parameters) == ["input", "weight", "epsilon"]
    assert list(inspect.signature(ops.rmsnorm_backward).parameters) == ["grad_output", "input", "weight", "inv_rms"]


def test_rmsnorm_module_surface():
    from mgrrmsnorm_amd import RMSNorm, RMSNormFunction

    sig = inspect.signature(RMSNorm.__init__)
    assert list(sig.parameters)[:3] == ["self", "hidden_size", "epsilon"]
    assert sig.parameters["epsilon"].default == 1e-5
    fsig = inspect.signature(RMSNormFunction.forward)
    assert list(fsig.parameters) == ["ctx", "input", "weight", "epsilon"]
    assert fsig.parameters["epsilon"].default == 1e-5

    n = RMSNorm(4096)
    assert n.hidden_size == 4096 and n.epsilon == 1e-5
    assert list(n.state_dict()) == ["weight"]
    assert n.weight.shape == (4096,) and n.weight.dtype == torch.float32 and bool((n.weight == 1).all())
    assert repr(n) == "RMSNorm(hidden_size=4096, eps=1e-05)"
    assert RMSNorm(8, 1e-6).epsilon == 1e-6           # positional, as BASELINE writes RMSNorm(hidden, eps)
    assert RMSNorm(8, eps=1e-6).epsilon == 1e-6       # torch.nn.RMSNorm spelling
    assert n.half().weight.dtype == torch.float16


@pytest.mark.parametrize("d_model,kwargs,hidden", [
    (4096, {}, 6912), (2048, {}, 3584), (4096, {"hidden_multiple": 2.6875}, 11008),
    (1024, {"multiple_of": 64}, 1728), (512, {"multiple_of": 1, "hidden_multiple": 4}, 2048),
])
def test_swiglu_module_surface(d_model, kwargs, hidden):
    from mgrrmsnorm_amd import MegaGemmTriton

    m = MegaGemmTriton(d_model, **kwargs)
    assert m.hidden == hidden
    assert list(m.state_dict()) == ["w12.weight", "w3.weight"]
    assert m.w12.weight.shape == (2 * hidden, d_model) and m.w3.weight.shape == (d_model, hidden)
    assert m.w12.bias is None and m.w3.bias is None
    assert m.extra_repr() == f"d_model={d_model}, hidden={hidden} (Triton Accelerated)"


def test_swiglu_signature_defaults():
    from mgrrmsnorm_amd import MegaGemmFunction, MegaGemmTriton

    sig = inspect.signature(MegaGemmTriton.__init__)
    assert list(sig.parameters) == ["self", "d_model", "multiple_of", "hidden_multiple"]
    assert sig.parameters["multiple_of"].default == 256
    assert sig.parameters["hidden_multiple"].default == 5 / 3
    assert list(inspect.signature(MegaGemmFunction.forward).parameters) == ["ctx", "w12_out", "hidden_dim"]


def test_cpu_tensors_are_refused_not_silently_computed():
    """There is no CPU fallback: a host tensor is an error, as in the reference
    (binding.cpp:9 CHECK_CUDA)."""
    from mgrrmsnorm_amd import MegaGemmFunction, RMSNorm, ops

    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        RMSNorm(16)(torch.randn(2, 16))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        MegaGemmFunction.apply(torch.randn(2, 32), 16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ops.rmsnorm_backward(torch.randn(2, 16), torch.randn(2, 16), torch.ones(16), torch.ones(2))


def test_swiglu_rejects_wrong_width():
    from mgrrmsnorm_amd import MegaGemmFunction

    with pytest.raises(RuntimeError, match="2\\*hidden_dim"):
        MegaGemmFunction.apply(torch.randn(2, 30), 16)


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    from mgrrmsnorm_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libmegagemm_hip.so")
    with pytest.raises(RuntimeError, match="HIP library not built"):
        _lib.load()


def test_unsupported_dtype_message():
    from mgrrmsnorm_amd import _lib

    with pytest.raises(RuntimeError, match="Unsupported dtype"):
        _lib.dtype_code(torch.float64)
    assert [_lib.dtype_code(d) for d in (torch.float32, torch.float16, torch.bfloat16)] == [0, 1, 2]


def test_binding_choice_can_be_forced_to_ctypes():
    """mgrrmsnorm_amd.ops uses the compiled extension when it is built and the ctypes binding
    when MGRRMSNORM_BINDING=ctypes is set before the first call; both reject host tensors
    with the reference's message (binding.cpp:9)."""
    import os
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    code = ("import torch\nfrom mgrrmsnorm_amd import ops\nprint(ops.backend())\n"
            "try:\n    ops.rmsnorm_forward(torch.ones(2, 8), torch.ones(8), 1e-6)\n"
            "except RuntimeError as e:\n    print('error:', e)\n")
    outs = {}
    for choice in ("", "ctypes"):
        env = dict(os.environ, MGRRMSNORM_BINDING=choice, PYTHONPATH=str(root))
        proc = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, stdout=subprocess.PIPE,
                              stderr=subprocess.STDOUT, text=True, timeout=300)
        assert proc.returncode == 0, proc.stdout
        outs[choice] = proc.stdout
    assert outs["ctypes"].splitlines()[0] == "ctypes"
    assert outs[""].splitlines()[0] in ("extension", "ctypes")      # extension once it is built
    for text in outs.values():
        assert "must be a CUDA tensor" in text
