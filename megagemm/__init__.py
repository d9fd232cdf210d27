"""Drop-in alias: `import megagemm` resolves to the MI355X implementation in
mgrrmsnorm_amd, so code written against MadrasLe/MGRrmsnorm's package name
(megagemm/__init__.py:27-52) runs unchanged."""
from mgrrmsnorm_amd import __all__, __version__  # noqa: F401


def __getattr__(name):
    import mgrrmsnorm_amd

    try:
        return getattr(mgrrmsnorm_amd, name)
    except AttributeError:
        raise AttributeError(f"module 'megagemm' has no attribute '{name}'") from None
