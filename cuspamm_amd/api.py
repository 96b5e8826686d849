"""ctypes mirror of include/spamm.h.

Matrices are torch CUDA tensors (torch is only the device allocator and stream
provider); every call goes through the C ABI with raw device pointers.
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libspamm_gfx950.so"

ROLE_A = 0
ROLE_B = 1
FLAG_A_EQ_B = 1
FLAG_TIMING = 2
FLAG_REUSE_A = 4
FLAG_REUSE_B = 8
FLAG_PRUNE = 16

OPT_NUM_XCD, OPT_GATE_CHUNK_WORDS, OPT_GEMM_RING, OPT_GEMM_SHAPE = 1, 2, 3, 4

OK, EINVAL, ENOMEM, EHIP, ESTATE, ENODEV, ELIMIT = 0, -1, -2, -3, -4, -5, -6
NOALLOC_WORKSPACE_BYTES = 40 << 20


class SpammParams(ctypes.Structure):
    """spamm_params: run-time form of para.h / main.h constants (M,K,N,LoNum,Norm)."""
    _fields_ = [("M", ctypes.c_int64), ("K", ctypes.c_int64), ("N", ctypes.c_int64),
                ("tile", ctypes.c_int32), ("tau", ctypes.c_float),
                ("flags", ctypes.c_uint32), ("reserved", ctypes.c_uint32)]


class SpammStats(ctypes.Structure):
    _fields_ = [("total_products", ctypes.c_int64), ("kept_products", ctypes.c_int64),
                ("ms_normmap_a", ctypes.c_float), ("ms_normmap_b", ctypes.c_float),
                ("ms_gate", ctypes.c_float), ("ms_gemm", ctypes.c_float),
                ("ms_total", ctypes.c_float), ("timing_valid", ctypes.c_int32)]


class SpammError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s failed: %s (code %d)" % (what, _strerror(code), code))


_lib = None


def library_path():
    # SPAMM_LIBRARY_PATH lets a developer load an alternative build of the same ABI
    return os.environ.get("SPAMM_LIBRARY_PATH") or os.path.join(HERE, _LIB_NAME)


def load_library():
    """Loads libspamm_gfx950.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python -m cuspamm_amd.build` "
            "(the SpAMM engine has no CPU or PyTorch fallback)" % path)
    # torch ships its own HIP runtime; import it first so that both share one copy.
    import torch  # noqa: F401
    L = ctypes.CDLL(path)
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_float
    L.spamm_create.argtypes = [ctypes.POINTER(vp), ctypes.c_int]
    L.spamm_destroy.argtypes = [vp]
    L.spamm_set_stream.argtypes = [vp, vp]
    L.spamm_multiply.argtypes = [vp, ctypes.POINTER(SpammParams), vp, vp, vp]
    L.spamm_multiply_noalloc.argtypes = [vp, ctypes.POINTER(SpammParams), vp, vp, vp]
    L.spamm_normmap_f32.argtypes = [vp, ctypes.c_int, vp, i64, i64, i32]
    L.spamm_normmap_f16.argtypes = [vp, ctypes.c_int, vp, i64, i64, i32]
    L.spamm_multiply_f16.argtypes = [vp, ctypes.POINTER(SpammParams), vp, vp, vp]
    L.spamm_error_vs_dense_f64.argtypes = [vp, vp, i64, i64, ctypes.POINTER(ctypes.c_double)]
    L.spamm_dropped_bound.argtypes = [vp, f32, ctypes.POINTER(ctypes.c_double)]
    L.spamm_dropped_bound_tiles.argtypes = [vp, f32, vp]
    L.spamm_set_option.argtypes = [vp, ctypes.c_int, ctypes.c_int]
    L.spamm_load_csv_f32.argtypes = [ctypes.c_char_p, i64, i64, i64, vp]
    L.spamm_load_mtx_f32.argtypes = [ctypes.c_char_p, i64, i64, i64, vp]
    L.spamm_gate.argtypes = [vp, f32]
    L.spamm_gemm_gated.argtypes = [vp, vp]
    L.spamm_set_normmaps.argtypes = [vp, vp, vp, i64, i64, i64, i32]
    L.spamm_tau_for_ratio.argtypes = [vp, ctypes.c_double, ctypes.POINTER(ctypes.c_float),
                                      ctypes.POINTER(ctypes.c_double)]
    L.spamm_tune_bisect.argtypes = [vp, ctypes.c_double, ctypes.c_double, ctypes.c_int,
                                    ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    L.spamm_count_kept.argtypes = [vp, ctypes.c_double, ctypes.POINTER(ctypes.c_int64),
                                   ctypes.POINTER(ctypes.c_double)]
    L.spamm_get_normmap.argtypes = [vp, ctypes.c_int, vp]
    L.spamm_get_counts.argtypes = [vp, vp]
    L.spamm_get_klist.argtypes = [vp, vp]
    L.spamm_get_mask.argtypes = [vp, vp]
    L.spamm_get_fp16.argtypes = [vp, ctypes.c_int, vp]
    L.spamm_get_macro_counts.argtypes = [vp, vp, vp]
    L.spamm_get_stats.argtypes = [vp, ctypes.POINTER(SpammStats)]
    L.spamm_fill_decay_f32.argtypes = [vp, vp, i64, i64, vp, ctypes.c_uint64, ctypes.c_int]
    L.spamm_synchronize.argtypes = [vp]
    L.spamm_strerror.argtypes = [ctypes.c_int]
    L.spamm_strerror.restype = ctypes.c_char_p
    L.spamm_last_hip_error.argtypes = [vp]
    L.spamm_version.restype = ctypes.c_int
    _lib = L
    return L


def _strerror(code):
    try:
        return load_library().spamm_strerror(code).decode()
    except Exception:  # pragma: no cover
        return "?"


def _check(code, what):
    if code != OK:
        raise SpammError(code, what)


def _devptr(t, dtype_name):
    import torch
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("expected a CUDA tensor")
    if str(t.dtype) != "torch." + dtype_name:
        raise TypeError("expected dtype %s, got %s" % (dtype_name, t.dtype))
    if not t.is_contiguous():
        raise ValueError("expected a contiguous (row-major) tensor")
    return ctypes.c_void_p(t.data_ptr())


def _check_out(A, B, C, M, N):
    """The GEMM writes M x N floats through C's pointer: refuse anything smaller or elsewhere before
    a kernel is launched (an out-of-bounds store is a device fault, not an error code)."""
    if getattr(C, "dim", lambda: 0)() != 2 or tuple(C.shape) != (M, N):
        raise ValueError("C must have shape (%d, %d), got %s" % (M, N, tuple(getattr(C, "shape", ()))))
    if B.device != A.device or C.device != A.device:
        raise ValueError("A, B and C must be on the same device")


class SpammContext:
    """One device + one stream + reusable workspaces (spamm_ctx)."""

    def __init__(self, device=0, use_torch_stream=True):
        self._lib = load_library()
        self._h = ctypes.c_void_p()
        _check(self._lib.spamm_create(ctypes.byref(self._h), int(device)), "spamm_create")
        self.device = int(device)
        self._shape = None
        if use_torch_stream:
            import torch
            self.set_stream(torch.cuda.current_stream(self.device).cuda_stream)

    def close(self):
        if self._h:
            self._lib.spamm_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- plumbing
    def set_stream(self, raw_stream):
        _check(self._lib.spamm_set_stream(self._h, ctypes.c_void_p(raw_stream or 0)),
               "spamm_set_stream")

    def set_option(self, option, value):
        _check(self._lib.spamm_set_option(self._h, int(option), int(value)), "spamm_set_option")

    def synchronize(self):
        _check(self._lib.spamm_synchronize(self._h), "spamm_synchronize")

    def last_hip_error(self):
        return int(self._lib.spamm_last_hip_error(self._h))

    # -- the multiply call
    def multiply(self, A, B, tile, tau, C=None, timing=False, reuse_a=False, reuse_b=False, a_eq_b=False,
                 prune=False):
        """C = SpAMM(A, B).  fp32 or fp16 inputs (both the same dtype).  With reuse_a / reuse_b the
        operand's fp16 copy and norm map from the previous call are kept (pass the same tensor, it
        only supplies the shape).  prune: tau-aware conversion passes (same C, mask and counts; the
        fp16 copies are then incomplete, see SPAMM_FLAG_PRUNE)."""
        import torch
        if A.dim() != 2 or B.dim() != 2:
            raise ValueError("A and B must be matrices")
        M, K = A.shape
        K2, N = B.shape
        if K != K2:
            raise ValueError("inner dimensions differ")
        if A.dtype != B.dtype:
            raise TypeError("A and B must have the same dtype")
        if C is None:
            C = torch.empty((M, N), dtype=torch.float32, device=A.device)
        _check_out(A, B, C, M, N)
        flags = ((FLAG_TIMING if timing else 0) | (FLAG_REUSE_A if reuse_a else 0) |
                 (FLAG_REUSE_B if reuse_b else 0) | (FLAG_A_EQ_B if a_eq_b else 0) |
                 (FLAG_PRUNE if prune else 0))
        p = SpammParams(M, K, N, int(tile), float(tau), flags, 0)
        if A.dtype == torch.float16:
            _check(self._lib.spamm_multiply_f16(self._h, ctypes.byref(p), _devptr(A, "float16"),
                                                _devptr(B, "float16"), _devptr(C, "float32")),
                   "spamm_multiply_f16")
        else:
            _check(self._lib.spamm_multiply(self._h, ctypes.byref(p), _devptr(A, "float32"),
                                            _devptr(B, "float32"), _devptr(C, "float32")),
                   "spamm_multiply")
        self._shape = (M // tile, K // tile, N // tile, int(tile), M, K, N)
        return C

    def multiply_noalloc(self, A, B, tile, tau, C, timing=False, a_eq_b=False, prune=False):
        """spamm_multiply_noalloc: the same multiply in the library's fixed device workspace (fp32 inputs,
        caller-provided C, no device allocation inside the call; SpammError ELIMIT beyond the workspace)."""
        if getattr(A, "dim", lambda: 0)() != 2 or getattr(B, "dim", lambda: 0)() != 2:
            raise ValueError("A and B must be matrices")
        M, K = A.shape
        K2, N = B.shape
        if K != K2:
            raise ValueError("inner dimensions differ")
        _check_out(A, B, C, M, N)
        flags = (FLAG_TIMING if timing else 0) | (FLAG_A_EQ_B if a_eq_b else 0) | (FLAG_PRUNE if prune else 0)
        p = SpammParams(M, K, N, int(tile), float(tau), flags, 0)
        _check(self._lib.spamm_multiply_noalloc(self._h, ctypes.byref(p), _devptr(A, "float32"),
                                                _devptr(B, "float32"), _devptr(C, "float32")),
               "spamm_multiply_noalloc")
        self._shape = (M // tile, K // tile, N // tile, int(tile), M, K, N)
        return C

    def multiply_raw(self, params, dA, dB, dC):
        """Pointer-level call (ints are raw device addresses); returns the error code."""
        return int(self._lib.spamm_multiply(self._h, ctypes.byref(params), ctypes.c_void_p(dA),
                                            ctypes.c_void_p(dB), ctypes.c_void_p(dC)))

    # -- stages
    def normmap_f32(self, role, X, tile):
        rows, cols = X.shape
        _check(self._lib.spamm_normmap_f32(self._h, int(role), _devptr(X, "float32"), rows, cols,
                                           int(tile)), "spamm_normmap_f32")
        s = list(self._shape) if self._shape and self._shape[3] == tile else [0, 0, 0, tile, 0, 0, 0]
        if role == ROLE_A:
            s[0], s[1], s[4], s[5] = rows // tile, cols // tile, rows, cols
        else:
            s[1], s[2], s[5], s[6] = rows // tile, cols // tile, rows, cols
        self._shape = tuple(s)

    def normmap_f16(self, role, X, tile):
        rows, cols = X.shape
        _check(self._lib.spamm_normmap_f16(self._h, int(role), _devptr(X, "float16"), rows, cols,
                                           int(tile)), "spamm_normmap_f16")
        s = list(self._shape) if self._shape and self._shape[3] == tile else [0, 0, 0, tile, 0, 0, 0]
        if role == ROLE_A:
            s[0], s[1], s[4], s[5] = rows // tile, cols // tile, rows, cols
        else:
            s[1], s[2], s[5], s[6] = rows // tile, cols // tile, rows, cols
        self._shape = tuple(s)

    def error_vs_dense(self, C, row0=0, row1=None):
        """(||C - D||_F, ||D||_F, ||C||_F) over rows [row0, row1), D = exact fp64 product of the
        resident fp16 operands."""
        if row1 is None:
            row1 = C.shape[0]
        out = (ctypes.c_double * 3)()
        _check(self._lib.spamm_error_vs_dense_f64(self._h, _devptr(C, "float32"), int(row0), int(row1), out),
               "spamm_error_vs_dense_f64")
        return out[0], out[1], out[2]

    def dropped_bound_tiles(self, tau):
        """Per output tile: sum over dropped k of nA[i,k]*nB[k,j] (float64 [nbM, nbN])."""
        nbM, nbK, nbN = self._shape[:3]
        out = np.empty((nbM, nbN), dtype=np.float64)
        _check(self._lib.spamm_dropped_bound_tiles(self._h, float(tau), out.ctypes.data), "spamm_dropped_bound_tiles")
        return out

    def dropped_bound(self, tau):
        out = ctypes.c_double(0)
        _check(self._lib.spamm_dropped_bound(self._h, float(tau), ctypes.byref(out)), "spamm_dropped_bound")
        return float(out.value)

    def set_normmaps(self, nA, nB, tile):
        nA = np.ascontiguousarray(nA, dtype=np.float32)
        nB = np.ascontiguousarray(nB, dtype=np.float32)
        nbM, nbK = nA.shape
        nbK2, nbN = nB.shape
        if nbK != nbK2:
            raise ValueError("norm map shapes differ")
        _check(self._lib.spamm_set_normmaps(self._h, nA.ctypes.data, nB.ctypes.data, nbM, nbK, nbN,
                                            int(tile)), "spamm_set_normmaps")
        self._shape = (nbM, nbK, nbN, int(tile), nbM * tile, nbK * tile, nbN * tile)

    def gate(self, tau):
        _check(self._lib.spamm_gate(self._h, float(tau)), "spamm_gate")

    # -- tau selection (norm maps must be present)
    def tau_for_ratio(self, ratio):
        tau, ach = ctypes.c_float(0), ctypes.c_double(0)
        _check(self._lib.spamm_tau_for_ratio(self._h, float(ratio), ctypes.byref(tau), ctypes.byref(ach)),
               "spamm_tau_for_ratio")
        return float(tau.value), float(ach.value)

    def tune_bisect(self, expected=0.75, tol=0.01, max_rounds=20):
        tau, ach = ctypes.c_float(0), ctypes.c_double(0)
        _check(self._lib.spamm_tune_bisect(self._h, float(expected), float(tol), int(max_rounds),
                                           ctypes.byref(tau), ctypes.byref(ach)), "spamm_tune_bisect")
        return float(tau.value), float(ach.value)

    def count_kept(self, threshold):
        cnt, sm = ctypes.c_int64(0), ctypes.c_double(0)
        _check(self._lib.spamm_count_kept(self._h, float(threshold), ctypes.byref(cnt), ctypes.byref(sm)),
               "spamm_count_kept")
        return int(cnt.value), float(sm.value)

    def gemm_gated(self, C):
        _check(self._lib.spamm_gemm_gated(self._h, _devptr(C, "float32")), "spamm_gemm_gated")
        return C

    # -- read-back
    def get_normmap(self, role):
        nbM, nbK, nbN = self._shape[:3]
        shp = (nbM, nbK) if role == ROLE_A else (nbK, nbN)
        out = np.empty(shp, dtype=np.float32)
        _check(self._lib.spamm_get_normmap(self._h, int(role), out.ctypes.data), "spamm_get_normmap")
        return out

    def get_counts(self):
        nbM, nbK, nbN = self._shape[:3]
        out = np.empty((nbM, nbN), dtype=np.int32)
        _check(self._lib.spamm_get_counts(self._h, out.ctypes.data), "spamm_get_counts")
        return out

    def get_klist(self):
        nbM, nbK, nbN = self._shape[:3]
        out = np.empty((nbM, nbN, nbK), dtype=np.uint16)
        _check(self._lib.spamm_get_klist(self._h, out.ctypes.data), "spamm_get_klist")
        return out

    def get_mask(self):
        nbM, nbK, nbN = self._shape[:3]
        out = np.empty((nbM, nbN, (nbK + 63) // 64), dtype=np.uint64)
        _check(self._lib.spamm_get_mask(self._h, out.ctypes.data), "spamm_get_mask")
        return out

    def get_macro_counts(self):
        """(counts [macro rows, macro columns, 2] = list length / kept-by-all entries per 256 x 256 macro
        tile of C, sched [16] = per XCD macro tiles with work, then all macro tiles)."""
        M, N = self._shape[4], self._shape[6]
        counts = np.empty(((M + 255) // 256, (N + 255) // 256, 2), dtype=np.int32)
        sched = np.empty(16, dtype=np.int32)
        _check(self._lib.spamm_get_macro_counts(self._h, counts.ctypes.data, sched.ctypes.data), "spamm_get_macro_counts")
        return counts, sched

    def get_fp16(self, role):
        M, K, N = self._shape[4:7]
        shp = (M, K) if role == ROLE_A else (K, N)
        out = np.empty(shp, dtype=np.uint16)
        _check(self._lib.spamm_get_fp16(self._h, int(role), out.ctypes.data), "spamm_get_fp16")
        return out

    def get_stats(self):
        st = SpammStats()
        _check(self._lib.spamm_get_stats(self._h, ctypes.byref(st)), "spamm_get_stats")
        return st

    # -- synthetic inputs
    def fill_decay(self, X, table, seed, random=True):
        rows, cols = X.shape
        table = np.ascontiguousarray(table, dtype=np.float32)
        if table.size < max(rows, cols):
            raise ValueError("decay table shorter than max(rows, cols)")
        _check(self._lib.spamm_fill_decay_f32(self._h, _devptr(X, "float32"), rows, cols,
                                              table.ctypes.data, int(seed), 1 if random else 0),
               "spamm_fill_decay_f32")
        return X


def load_csv(path, rows, cols, ld=None):
    """Dense CSV, one matrix row per line, into a zero-filled (rows, ld) fp32 array (host)."""
    ld = cols if ld is None else ld
    out = np.empty((rows, ld), dtype=np.float32)
    _check(load_library().spamm_load_csv_f32(os.fsencode(path), rows, cols, ld, out.ctypes.data), "spamm_load_csv_f32")
    return out


def load_mtx(path, rows, cols, ld=None):
    """'row col val' triples (1-based, first line skipped) into a zero-filled (rows, ld) fp32 array (host)."""
    ld = cols if ld is None else ld
    out = np.empty((rows, ld), dtype=np.float32)
    _check(load_library().spamm_load_mtx_f32(os.fsencode(path), rows, cols, ld, out.ctypes.data), "spamm_load_mtx_f32")
    return out
