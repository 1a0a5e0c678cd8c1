"""CPU oracle of the small-batch GEMM / GEMV path.  Test infrastructure only: imported by
tests/, by the smoke check and by the bench's cpu_baseline leg, never by fastgate_amd."""
from .oracle import *  # noqa: F401,F403
