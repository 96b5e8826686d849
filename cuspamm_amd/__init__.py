"""cuspamm_amd -- gfx950 (MI355X) SpAMM engine behind a C ABI.

The compute lives in ``libspamm_gfx950.so`` (hand-written HIP kernels, see
``csrc/``); this package is the thin host-side mirror of the C ABI declared in
``include/spamm.h``.  There is no CPU fallback: loading fails loudly when the
library has not been built (``python -m cuspamm_amd.build``).
"""
from .api import (  # noqa: F401
    ROLE_A,
    ROLE_B,
    FLAG_TIMING,
    FLAG_A_EQ_B,
    FLAG_REUSE_A,
    FLAG_REUSE_B,
    FLAG_PRUNE,
    NOALLOC_WORKSPACE_BYTES,
    OPT_NUM_XCD,
    OPT_GATE_CHUNK_WORDS,
    OPT_GEMM_RING,
    OPT_GEMM_SHAPE,
    SpammContext,
    SpammError,
    SpammParams,
    SpammStats,
    load_library,
    load_csv,
    load_mtx,
    library_path,
)
