"""Drop-in for the reference's compiled extension module `rmsnorm_cuda_ops`
(pytorch_binding/binding.cpp:136-139): scripts that `import rmsnorm_cuda_ops` and call
rmsnorm_forward / rmsnorm_backward (test_rmsnorm.py:2-20) get the MI355X kernels."""
from mgrrmsnorm_amd.ops import rmsnorm_backward, rmsnorm_forward  # noqa: F401

__all__ = ["rmsnorm_forward", "rmsnorm_backward"]
