"""ctypes binding of oracle/liboracle.so -- TEST INFRASTRUCTURE ONLY.

The host checker restates the cuSpAMM algorithm in plain C (see
spamm_oracle.c for the reference lines each function follows).  Only tests,
the smoke check and the bench's cpu_baseline leg import this module; the
product package never does.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_u64p = np.ctypeslib.ndpointer(dtype=np.uint64, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_i64 = ctypes.c_int64

_lib = None


def build():
    """Compiles liboracle.so with gcc (always rebuilds)."""
    subprocess.run(["make", "-C", HERE, "-B", "liboracle.so"], check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    L = ctypes.CDLL(LIB_PATH)
    L.orc_num_threads.restype = ctypes.c_int
    L.orc_set_num_threads.argtypes = [ctypes.c_int]
    L.orc_f32_to_f16.argtypes = [_f32p, _i64, _u16p]
    L.orc_f16_to_f32.argtypes = [_u16p, _i64, _f32p]
    L.orc_fill_decay.argtypes = [_f32p, _i64, _i64, _f32p, ctypes.c_uint64, ctypes.c_int]
    L.orc_normmap.argtypes = [_u16p, _i64, _i64, ctypes.c_int, ctypes.c_int, _f32p]
    L.orc_normmap.restype = ctypes.c_int
    L.orc_normmap_ref16_model.argtypes = [_u16p, _i64, _i64, _f32p]
    L.orc_normmap_ref16_model.restype = ctypes.c_int
    L.orc_gate.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_float,
                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    L.orc_gate.restype = _i64
    L.orc_gemm_gated.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_int, _i32p, _u16p,
                                 _f32p, _i64, _i64]
    L.orc_gemm_gated.restype = ctypes.c_int
    L.orc_gemm_dense_f64.argtypes = [_f32p, _f32p, _i64, _i64, _i64, _i64, _f64p]
    L.orc_frob_diff.argtypes = [_f32p, _f64p, _i64, _f64p]
    L.orc_frob_diff_f32.argtypes = [_f32p, _f32p, _i64, _f64p]
    L.orc_dropped_bound.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_float, _i64, _i64]
    L.orc_dropped_bound.restype = ctypes.c_double
    L.orc_dropped_bound_tiles.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_float, _f64p]
    L.orc_dropped_bound_tiles.restype = None
    L.orc_tau_for_ratio.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_double,
                                    ctypes.POINTER(ctypes.c_double)]
    L.orc_tau_for_ratio.restype = ctypes.c_float
    L.orc_tune_bisect.argtypes = [_f32p, _f32p, _i64, _i64, _i64, ctypes.c_double,
                                  ctypes.c_double, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    L.orc_tune_bisect.restype = ctypes.c_float
    _lib = L
    return L


def num_threads():
    return int(lib().orc_num_threads())


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    h = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16(x.reshape(-1), x.size, h.reshape(-1))
    return h


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    x = np.empty(h.shape, dtype=np.float32)
    lib().orc_f16_to_f32(h.reshape(-1), h.size, x.reshape(-1))
    return x


def decay_table(kind, n, lam=0.0, c=1.0, v=1.0):
    """fp32 table of decay(d), d = 0..n-1, evaluated in fp64 then rounded once.

    kind: 'exp'  -> exp(-lam*d)            (seeded-uniform family)
          'alg'  -> 1/(1+d)^2
          'none' -> 1
          'ref_exp' -> c * v^d             (tool.cu:409-422)
          'ref_alg' -> c / (d^v + 1)       (tool.cu:426-436)
    """
    d = np.arange(n, dtype=np.float64)
    if kind == "exp":
        t = np.exp(-lam * d)
    elif kind == "alg":
        t = 1.0 / (1.0 + d) ** 2
    elif kind == "none":
        t = np.ones(n)
    elif kind == "ref_exp":
        t = np.float32(c) * np.power(np.float64(np.float32(v)), d).astype(np.float32)
    elif kind == "ref_alg":
        t = np.float32(c) / (np.power(d, np.float64(np.float32(v))).astype(np.float32) + np.float32(1))
    else:
        raise ValueError(kind)
    return np.ascontiguousarray(t, dtype=np.float32)


def fill_decay(rows, cols, table, seed, random=True):
    X = np.empty((rows, cols), dtype=np.float32)
    table = np.ascontiguousarray(table, dtype=np.float32)
    assert table.size >= max(rows, cols)
    lib().orc_fill_decay(X.reshape(-1), rows, cols, table, seed, 1 if random else 0)
    return X


def normmap(hbits, tile, role):
    hbits = np.ascontiguousarray(hbits, dtype=np.uint16)
    rows, cols = hbits.shape
    nm = np.empty((rows // tile, cols // tile), dtype=np.float32)
    rc = lib().orc_normmap(hbits.reshape(-1), rows, cols, tile, role, nm.reshape(-1))
    if rc != 0:
        raise ValueError("orc_normmap: bad tile or dimensions")
    return nm


def normmap_ref16_model(hbits):
    """Model of the reference's fp16 norm kernel (tile 32; fp16-rounded squares, fp16 column sums).
    Parity unpinned by construction -- only for counting how many gate decisions could differ."""
    hbits = np.ascontiguousarray(hbits, dtype=np.uint16)
    rows, cols = hbits.shape
    nm = np.empty((rows // 32, cols // 32), dtype=np.float32)
    rc = lib().orc_normmap_ref16_model(hbits.reshape(-1), rows, cols, nm.reshape(-1))
    if rc != 0:
        raise ValueError("orc_normmap_ref16_model: dimensions must be multiples of 32")
    return nm


def gate(nA, nB, tau, want_klist=True, want_mask=True):
    """Returns (kept_total, counts[nbM,nbN], klist[nbM,nbN,nbK] u16, mask[nbM,nbN,words] u64)."""
    nA = np.ascontiguousarray(nA, dtype=np.float32)
    nB = np.ascontiguousarray(nB, dtype=np.float32)
    nbM, nbK = nA.shape
    nbK2, nbN = nB.shape
    assert nbK == nbK2
    words = (nbK + 63) // 64
    counts = np.zeros((nbM, nbN), dtype=np.int32)
    klist = np.zeros((nbM, nbN, nbK), dtype=np.uint16) if want_klist else None
    mask = np.zeros((nbM, nbN, words), dtype=np.uint64) if want_mask else None
    total = lib().orc_gate(nA.reshape(-1), nB.reshape(-1), nbM, nbK, nbN, np.float32(tau),
                           counts.ctypes.data,
                           klist.ctypes.data if want_klist else None,
                           mask.ctypes.data if want_mask else None)
    return int(total), counts, klist, mask


def gemm_gated(Af, Bf, tile, counts, klist, ti0=0, ti1=None, out=None):
    """Af, Bf: fp32 arrays of fp16-representable values. Returns C (rows outside
    [ti0*tile, ti1*tile) untouched / zero)."""
    Af = np.ascontiguousarray(Af, dtype=np.float32)
    Bf = np.ascontiguousarray(Bf, dtype=np.float32)
    M, K = Af.shape
    K2, N = Bf.shape
    assert K == K2
    if ti1 is None:
        ti1 = M // tile
    C = out if out is not None else np.zeros((M, N), dtype=np.float32)
    rc = lib().orc_gemm_gated(Af.reshape(-1), Bf.reshape(-1), M, K, N, tile,
                              np.ascontiguousarray(counts, dtype=np.int32).reshape(-1),
                              np.ascontiguousarray(klist, dtype=np.uint16).reshape(-1),
                              C.reshape(-1), ti0, ti1)
    if rc != 0:
        raise ValueError("orc_gemm_gated: bad dimensions")
    return C


def gemm_dense_f64(Af, Bf, r0=0, r1=None):
    Af = np.ascontiguousarray(Af, dtype=np.float32)
    Bf = np.ascontiguousarray(Bf, dtype=np.float32)
    M, K = Af.shape
    _, N = Bf.shape
    if r1 is None:
        r1 = M
    Cd = np.empty((r1 - r0, N), dtype=np.float64)
    lib().orc_gemm_dense_f64(Af.reshape(-1), Bf.reshape(-1), K, N, r0, r1, Cd.reshape(-1))
    return Cd


def frob_diff(X, Y):
    """(||X-Y||_F, ||Y||_F, ||X||_F) with fp64 accumulation; Y fp64 or fp32."""
    X = np.ascontiguousarray(X, dtype=np.float32)
    out = np.zeros(3, dtype=np.float64)
    if Y.dtype == np.float64:
        Y = np.ascontiguousarray(Y)
        lib().orc_frob_diff(X.reshape(-1), Y.reshape(-1), X.size, out)
    else:
        Y = np.ascontiguousarray(Y, dtype=np.float32)
        lib().orc_frob_diff_f32(X.reshape(-1), Y.reshape(-1), X.size, out)
    return tuple(out.tolist())


def dropped_bound(nA, nB, tau, ti0=0, ti1=None):
    nA = np.ascontiguousarray(nA, dtype=np.float32)
    nB = np.ascontiguousarray(nB, dtype=np.float32)
    nbM, nbK = nA.shape
    _, nbN = nB.shape
    if ti1 is None:
        ti1 = nbM
    return float(lib().orc_dropped_bound(nA.reshape(-1), nB.reshape(-1), nbM, nbK, nbN,
                                         np.float32(tau), ti0, ti1))


def dropped_bound_tiles(nA, nB, tau):
    nA = np.ascontiguousarray(nA, dtype=np.float32)
    nB = np.ascontiguousarray(nB, dtype=np.float32)
    nbM, nbK = nA.shape
    _, nbN = nB.shape
    out = np.zeros(nbM * nbN, dtype=np.float64)
    lib().orc_dropped_bound_tiles(nA.reshape(-1), nB.reshape(-1), nbM, nbK, nbN, np.float32(tau), out)
    return out.reshape(nbM, nbN)


def tau_for_ratio(nA, nB, ratio):
    nA = np.ascontiguousarray(nA, dtype=np.float32)
    nB = np.ascontiguousarray(nB, dtype=np.float32)
    nbM, nbK = nA.shape
    _, nbN = nB.shape
    ach = ctypes.c_double(0)
    tau = lib().orc_tau_for_ratio(nA.reshape(-1), nB.reshape(-1), nbM, nbK, nbN, ratio,
                                  ctypes.byref(ach))
    return float(tau), float(ach.value)


def tune_bisect(nA, nB, expected=0.75, tol=0.01, max_rounds=20):
    nA = np.ascontiguousarray(nA, dtype=np.float32)
    nB = np.ascontiguousarray(nB, dtype=np.float32)
    nbM, nbK = nA.shape
    _, nbN = nB.shape
    ach = ctypes.c_double(0)
    tau = lib().orc_tune_bisect(nA.reshape(-1), nB.reshape(-1), nbM, nbK, nbN, expected, tol,
                                max_rounds, ctypes.byref(ach))
    return float(tau), float(ach.value)


def spamm(A, B, tile, tau):
    """Whole pipeline on fp32 inputs. Returns dict with everything the GPU path exposes."""
    hA = f32_to_f16_bits(A)
    hB = f32_to_f16_bits(B)
    nA = normmap(hA, tile, 0)
    nB = normmap(hB, tile, 1)
    total, counts, klist, mask = gate(nA, nB, tau)
    Af = f16_bits_to_f32(hA)
    Bf = f16_bits_to_f32(hB)
    C = gemm_gated(Af, Bf, tile, counts, klist)
    return dict(hA=hA, hB=hB, nA=nA, nB=nB, kept=total, counts=counts, klist=klist, mask=mask,
                Af=Af, Bf=Bf, C=C)
