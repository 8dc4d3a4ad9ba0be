"""CPU oracle for the NAtS-L hybrid attention forward path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it is the checker the HIP kernels are compared against (tests, the
smoke check and the benchmark's CPU-baseline leg), never the thing measured or
shipped.  Every function cites the reference file:line it restates; the
reference itself is Triton-only and cannot run on a CPU.
"""
from . import routing, softmax_branch, linear_branch, mixed, norm_gate, layer, decode, cache  # noqa: F401
