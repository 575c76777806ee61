"""cutlass-kernels_amd -- MI355X (gfx950) fused multi-head-attention forward behind a C-ABI.

The product is ``libcfk_fmha.so`` (hand-written HIP, see ``csrc/``) and its C header ``include/cfk_fmha.h``.
This package is the thin Python host side used by the tests and the benchmark: ctypes bindings over the
C-ABI (``fmha``), and the seeded input generators of the reference driver (``testbed``).  There is no CPU
fallback: every call fails loudly if the HIP library has not been built.

The directory name is not a Python identifier; load it with ``__graft_entry__.load_package()`` or put the
repository root on ``sys.path`` and use ``importlib`` as that helper does.
"""
from . import fmha, testbed  # noqa: F401
from .fmha import (CFK_FP16, CFK_FP32, CFK_FP8_E4M3, CfkError, build, fmha_forward, fmha_forward_kernel, fmha_forward_mfma,  # noqa: F401
                   fmha_forward_plan, gemm, gemm_f16, last_error, lib, lib_path, version)
