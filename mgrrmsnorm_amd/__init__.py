"""mgrrmsnorm_amd: RMSNorm and the SwiGLU activation as hand-written HIP kernels for
MI355X (gfx950), behind the Python surface of MadrasLe/MGRrmsnorm's `megagemm` package.

    from mgrrmsnorm_amd import RMSNorm, MegaGemmTriton      # or: from megagemm import ...
    norm = RMSNorm(4096).cuda().to(torch.bfloat16)
    mlp = MegaGemmTriton(4096).cuda().to(torch.bfloat16)

The four public names are resolved on first access, so importing the package needs neither
a GPU nor the built library (reference: megagemm/__init__.py:31-44); the first operator
call on a machine without the library raises RuntimeError.
"""
__version__ = "0.1.0"

_EXPORTS = {
    "RMSNorm": "rmsnorm",
    "RMSNormFunction": "rmsnorm",
    "MegaGemmTriton": "swiglu",
    "MegaGemmFunction": "swiglu",
}

__all__ = [*_EXPORTS, "backward_on_calling_thread", "__version__"]


def backward_on_calling_thread():
    """Context manager: run autograd's backward passes on the thread that calls `.backward()`.

        with mgrrmsnorm_amd.backward_on_calling_thread():
            for batch in loader:
                loss(model(batch)).backward()

    By default torch's autograd engine hands every backward pass on a GPU to a worker thread of
    its own.  For operators as short as these (RMSNorm forward + backward at 4096 x 4096 bf16 is
    35 us of GPU time) waking that thread on another core costs more than the kernels: measured
    through `megagemm.RMSNorm`, 38-62 us per forward+backward call with the default (which core
    the worker sits on is the scheduler's choice) against 35 us -- the kernels' own time -- on the
    calling thread.  This wraps torch's own switch, `torch.autograd.set_multithreading_enabled(False)`;
    it has no counterpart in the reference and changes no result, only where the backward pass
    is enqueued from."""
    import torch

    return torch.autograd.set_multithreading_enabled(False)


def __getattr__(name):
    sub = _EXPORTS.get(name)
    if sub is None:
        raise AttributeError(f"module '{__name__}' has no attribute '{name}'")
    import importlib

    value = getattr(importlib.import_module(f"{__name__}.{sub}"), name)
    globals()[name] = value
    return value


def __dir__():
    return sorted(list(globals()) + list(_EXPORTS))
