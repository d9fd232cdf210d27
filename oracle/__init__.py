"""CPU oracle for the RMSNorm / SwiGLU path: test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package.  The product (mgrrmsnorm_amd) never does.
"""
from .oracle import (  # noqa: F401
    build,
    rmsnorm_fwd_f32,
    rmsnorm_fwd_f64,
    rmsnorm_bwd_f32,
    rmsnorm_bwd_f64,
    swiglu_fwd_f32,
    swiglu_fwd_f64,
    swiglu_bwd_f32,
    swiglu_bwd_f64,
    to_f32,
    round_to,
    ordered_bits,
    ulp_distance,
)
