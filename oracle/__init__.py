"""CPU checker for the row-wise reduce-then-normalize operators.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the bench's
CPU-baseline leg.  The shipped library and its Python loader never import it.
"""
from .rownorm_oracle import *  # noqa: F401,F403
