"""CPU oracle for the FlashSinkhorn hot path (TEST INFRASTRUCTURE ONLY).

This package is a dense / row-chunked numpy restatement of the reference's own
PyTorch implementation of the streaming Sinkhorn path.  It exists to check the
HIP kernels; nothing in the shipped package imports it.  Only the tests, the
smoke entry and the CPU-baseline leg of the benchmark may call it.

Every function cites the reference file:line it restates.  Pin status per
function is listed in ``oracle/sinkhorn_ref.py``'s header.
"""

from oracle.sinkhorn_ref import *  # noqa: F401,F403
from oracle.hvp_ref import *  # noqa: F401,F403
