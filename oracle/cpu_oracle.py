"""TEST INFRASTRUCTURE: Python face of the CPU oracle.

Two independent restatements of the reference's CPU (llvm-target) result for the
GEMM / batched GEMM / conv computes:

* ``te_literal_*``  -- ctypes calls into ``libamos_oracle.so`` (``te_literal.c``):
  the loop nests with TVM's exact dtype semantics (multiply in the input dtype,
  cast, sequential accumulate; reference: src/te/operation/compute_op.cc:293-329,
  src/target/llvm/codegen_llvm.cc:593-625,899-924), in ``mode="te_literal"`` or
  ``mode="exact"``.
* ``lib_*`` -- numpy library forms: up-cast inputs, fp32 (or fp64 / int64)
  ``matmul`` and a window-view convolution.  This is the "fp32-accumulated CPU
  result" tolerances are quoted against, and what the scipy goldens of the
  reference's tutorials compute (reference:
  python/tvm/topi/testing/conv2d_nchw_python.py:48-73, conv3d_ncdhw_python.py:24-61,
  batch_matmul.py:22-44).

Only tests, ``__graft_entry__.smoke()`` and the benchmark's CPU-baseline leg may
import this module.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

DTYPE_CODE = {"float16": 0, "bfloat16": 1, "int8": 2}
MODE_CODE = {"te_literal": 0, "exact": 1}


def load():
    """Load libamos_oracle.so (built by ``make -C oracle``)."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.path.join(_HERE, "libamos_oracle.so")
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: run `make -C oracle` (or __graft_entry__.build())" % path)
    lib = ctypes.CDLL(path)
    i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    lib.oracle_gemm.argtypes = [i32, i32, i64, i64, i64, i32, i32, vp, i64, vp, i64, vp, i64, i64, i64, i32]
    lib.oracle_gemm.restype = i32
    lib.oracle_bgemm.argtypes = [i32, i32, i64, i64, i64, i64, i32, i32, vp, i64, i64, vp, i64, i64,
                                 vp, i64, i64, i64, i64, i32]
    lib.oracle_bgemm.restype = i32
    lib.oracle_conv.argtypes = [i32, i32] + [i64] * 18 + [vp, vp, vp, i64, i64, i32]
    lib.oracle_conv.restype = i32
    lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
    lib.oracle_half_to_float.restype = ctypes.c_float
    lib.oracle_float_to_half.argtypes = [ctypes.c_float]
    lib.oracle_float_to_half.restype = ctypes.c_uint16
    lib.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
    lib.oracle_bf16_to_float.restype = ctypes.c_float
    lib.oracle_float_to_bf16.argtypes = [ctypes.c_float]
    lib.oracle_float_to_bf16.restype = ctypes.c_uint16
    lib.oracle_max_threads.restype = i32
    _LIB = lib
    return lib


# ---- bf16 helpers (numpy has no bfloat16): bf16 tensors travel as uint16 bit patterns ----
def float_to_bf16_bits(x):
    """fp32 array -> uint16 bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def bf16_bits_to_float(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _raw(x, dtype):
    """array -> (contiguous array whose buffer holds the element bit patterns, dtype code)."""
    x = np.ascontiguousarray(x)
    if dtype == "float16":
        assert x.dtype == np.float16
    elif dtype == "bfloat16":
        assert x.dtype == np.uint16, "bf16 operands are passed as uint16 bit patterns"
    elif dtype == "int8":
        assert x.dtype == np.int8
    else:
        raise ValueError("unsupported dtype %r" % (dtype,))
    return x, DTYPE_CODE[dtype]


def _out_dtype(dtype):
    return np.int32 if dtype == "int8" else np.float32


def upcast(x, dtype):
    """operand array -> float64 values"""
    if dtype == "bfloat16":
        return bf16_bits_to_float(x).astype(np.float64)
    return np.asarray(x).astype(np.float64)


# ---- te_literal loop nests (C) -------------------------------------------------------------
def te_literal_gemm(a, b, dtype, trans_a=False, trans_b=False, mode="te_literal", rows=None, threads=1):
    """C[M,N] = sum_k A(m,k) B(k,n).  a is [M,K] ([K,M] if trans_a), b is [K,N] ([N,K] if trans_b).
    rows=(m0, m1) computes only that slab (the rest of C stays 0)."""
    lib = load()
    a, code = _raw(a, dtype)
    b, _ = _raw(b, dtype)
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == K
    c = np.zeros((M, N), dtype=_out_dtype(dtype))
    m0, m1 = rows if rows is not None else (0, M)
    rc = lib.oracle_gemm(code, MODE_CODE[mode], M, N, K, int(trans_a), int(trans_b), a.ctypes.data,
                         a.shape[1], b.ctypes.data, b.shape[1], c.ctypes.data, N, m0, m1, threads)
    if rc:
        raise RuntimeError("oracle_gemm failed: %d" % rc)
    return c


def te_literal_bgemm(a, b, dtype, trans_a=False, trans_b=False, mode="te_literal", batches=None, threads=1):
    """batched form; a is [B,M,K] (or [B,K,M]), b is [B,K,N] (or [B,N,K])."""
    lib = load()
    a, code = _raw(a, dtype)
    b, _ = _raw(b, dtype)
    B = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if trans_a else a.shape[1:]
    N = b.shape[1] if trans_b else b.shape[2]
    c = np.zeros((B, M, N), dtype=_out_dtype(dtype))
    b0, b1 = batches if batches is not None else (0, B)
    rc = lib.oracle_bgemm(code, MODE_CODE[mode], B, M, N, K, int(trans_a), int(trans_b), a.ctypes.data,
                          a.shape[2], a.shape[1] * a.shape[2], b.ctypes.data, b.shape[2],
                          b.shape[1] * b.shape[2], c.ctypes.data, N, M * N, b0, b1, threads)
    if rc:
        raise RuntimeError("oracle_bgemm failed: %d" % rc)
    return c


def _triple(v):
    if isinstance(v, (tuple, list)):
        assert len(v) == 3
        return tuple(int(t) for t in v)
    return (int(v),) * 3


def conv_out_shape(x_shape, w_shape, stride, pad, dil):
    N, C, D, H, W = x_shape
    K, _, T, R, S = w_shape
    st, pd, dl = _triple(stride), _triple(pad), _triple(dil)
    out = []
    for ext, k, s, p, d in zip((D, H, W), (T, R, S), st, pd, dl):
        eff = (k - 1) * d + 1
        out.append((ext + 2 * p - eff) // s + 1)
    return (N, K) + tuple(out)


def te_literal_conv3d(x, w, dtype, stride=1, pad=0, dil=1, mode="te_literal", images=None, threads=1):
    """x NCDHW, w KCTRS -> y NKDPQ"""
    lib = load()
    x, code = _raw(x, dtype)
    w, _ = _raw(w, dtype)
    N, C, D, H, W = x.shape
    K, C2, T, R, S = w.shape
    assert C == C2
    st, pd, dl = _triple(stride), _triple(pad), _triple(dil)
    y = np.zeros(conv_out_shape(x.shape, w.shape, st, pd, dl), dtype=_out_dtype(dtype))
    n0, n1 = images if images is not None else (0, N)
    rc = lib.oracle_conv(code, MODE_CODE[mode], N, C, D, H, W, K, T, R, S, *st, *pd, *dl,
                         x.ctypes.data, w.ctypes.data, y.ctypes.data, n0, n1, threads)
    if rc:
        raise RuntimeError("oracle_conv failed: %d" % rc)
    return y


def te_literal_conv2d(x, w, dtype, stride=1, pad=0, dil=1, mode="te_literal", images=None, threads=1):
    """x NCHW, w KCRS -> y NKPQ (the D = T = 1 case of conv3d)"""
    def lift(v, unit):
        if isinstance(v, (tuple, list)):
            return (unit, int(v[0]), int(v[1]))
        return (unit, int(v), int(v))
    x5 = np.ascontiguousarray(x)[:, :, None]
    w5 = np.ascontiguousarray(w)[:, :, None]
    y = te_literal_conv3d(x5, w5, dtype, lift(stride, 1), lift(pad, 0), lift(dil, 1), mode, images, threads)
    return y[:, :, 0]


# ---- numpy library forms ----------------------------------------------------------------------
def lib_gemm(a, b, dtype, trans_a=False, trans_b=False, acc="float32"):
    """up-cast matmul; acc in {"float32", "float64"}.  int8 runs in float64, which is exact:
    every partial sum is an integer below K * 2^14 < 2^53."""
    if dtype == "int8":
        A = np.asarray(a).astype(np.float64)
        B = np.asarray(b).astype(np.float64)
    else:
        A = upcast(a, dtype).astype(acc)
        B = upcast(b, dtype).astype(acc)
    if trans_a:
        A = np.swapaxes(A, -1, -2)
    if trans_b:
        B = np.swapaxes(B, -1, -2)
    C = np.matmul(A, B)
    return np.rint(C).astype(np.int32) if dtype == "int8" else C


def lib_conv3d(x, w, dtype, stride=1, pad=0, dil=1, acc="float32"):
    """window-view convolution: y[n,k,o...] = sum_{c,t,r,s} xpad[n,c,o*s+t*d...] w[k,c,t,r,s]"""
    st, pd, dl = _triple(stride), _triple(pad), _triple(dil)
    if dtype == "int8":  # float64 is exact for int8 data (see lib_gemm)
        X = np.asarray(x).astype(np.float64)
        Wt = np.asarray(w).astype(np.float64)
    else:
        X = upcast(x, dtype).astype(acc)
        Wt = upcast(w, dtype).astype(acc)
    N, C, D, H, W = X.shape
    K, _, T, R, S = Wt.shape
    Xp = np.pad(X, ((0, 0), (0, 0), (pd[0],) * 2, (pd[1],) * 2, (pd[2],) * 2))
    _, _, OD, OP, OQ = conv_out_shape(x.shape, w.shape, st, pd, dl)
    Y = np.zeros((N, K, OD, OP, OQ), dtype=Xp.dtype)
    for t in range(T):
        for r in range(R):
            for s in range(S):
                win = Xp[:, :,
                         t * dl[0]: t * dl[0] + (OD - 1) * st[0] + 1: st[0],
                         r * dl[1]: r * dl[1] + (OP - 1) * st[1] + 1: st[1],
                         s * dl[2]: s * dl[2] + (OQ - 1) * st[2] + 1: st[2]]
                # [N,C,OD,OP,OQ] x [K,C] -> [N,K,OD,OP,OQ]
                Y += np.einsum("ncdpq,kc->nkdpq", win, Wt[:, :, t, r, s], optimize=True)
    return np.rint(Y).astype(np.int32) if dtype == "int8" else Y


def lib_conv2d(x, w, dtype, stride=1, pad=0, dil=1, acc="float32"):
    def lift(v, unit):
        if isinstance(v, (tuple, list)):
            return (unit, int(v[0]), int(v[1]))
        return (unit, int(v), int(v))
    y = lib_conv3d(np.asarray(x)[:, :, None], np.asarray(w)[:, :, None], dtype, lift(stride, 1),
                   lift(pad, 0), lift(dil, 1), acc)
    return y[:, :, 0]


# ---- error measures used by every fp16 / bf16 parity test ---------------------------------------
def rel_errors(got, ref):
    """(max_rel, mean_rel) with the denominator floored at 1e-2 * rms(ref):
    |got - ref| / max(|ref|, 1e-2 * rms(ref)).  The floor keeps outputs that cross zero from
    dominating; it is stated here once and used by every floating-point parity test."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    floor = max(1e-2 * rms, 1e-30)
    err = np.abs(got - ref) / np.maximum(np.abs(ref), floor)
    return float(err.max()) if err.size else 0.0, float(err.mean()) if err.size else 0.0
