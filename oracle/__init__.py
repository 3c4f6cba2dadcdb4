"""CPU oracle for the MFMA GEMM hot path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package. The shipped library (composable_kernel_amd) never does.

Two layers:

* ``lit``  -- ctypes binding of ``libck_oracle.so`` (oracle/ck_oracle.cpp), the
  literal restatement of the reference's host ReferenceGemm / ReferenceConvFwd /
  ReferenceBatchedGemm (file:line citations in that source).
* ``fast`` -- numpy forms used for full-size checks: int8 GEMMs run as fp32 BLAS
  GEMMs (every partial sum is an integer below 2**24, hence exact and
  order-independent), followed by the same fp32 epilogue arithmetic.
* ``ref``  -- ctypes binding of ``oracle/_ref/libck_ref.so`` (the reference's own
  host operators compiled in place) when that file exists; ``None`` otherwise.
"""
from . import lit, fast  # noqa: F401
from .lit import EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND  # noqa: F401
from .refshim import load_ref  # noqa: F401
