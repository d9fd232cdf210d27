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

__all__ = [*_EXPORTS, "__version__"]


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
