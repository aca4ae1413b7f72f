"""ctypes/numpy front end of the CPU oracle (oracle/tcec_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  Nothing under wmma_extension_amd/ imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "_build", "liboracle.so")

SPLIT_F16, SPLIT_BF16X2, SPLIT_BF16X3 = 0, 1, 2
USE_A, USE_B, USE_ACC = 0, 1, 2


def build():
    res = subprocess.run(["make", "-C", _DIR, "-B"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + res.stdout)
    return LIB_PATH


_LIB = None
_c = ctypes
_fp = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_dp = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_ll = _c.c_longlong
_i = _c.c_int


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            build()
        h = ctypes.CDLL(LIB_PATH)
        h.orc_f32_to_f16.restype = _c.c_uint16
        h.orc_f32_to_f16.argtypes = [_c.c_float]
        h.orc_f16_to_f32.restype = _c.c_float
        h.orc_f16_to_f32.argtypes = [_c.c_uint16]
        h.orc_f32_to_bf16.restype = _c.c_uint16
        h.orc_f32_to_bf16.argtypes = [_c.c_float]
        h.orc_bf16_to_f32.restype = _c.c_float
        h.orc_bf16_to_f32.argtypes = [_c.c_uint16]
        h.orc_split_array.restype = None
        h.orc_split_array.argtypes = [_i, _fp, _ll, _u16p, _c.c_void_p, _c.c_void_p]
        h.orc_frag_num_elements.restype = _i
        h.orc_frag_num_elements.argtypes = [_i] * 4
        h.orc_frag_rows.restype = _i
        h.orc_frag_rows.argtypes = [_i] * 4
        h.orc_frag_cols.restype = _i
        h.orc_frag_cols.argtypes = [_i] * 4
        h.orc_frag_ij.restype = None
        h.orc_frag_ij.argtypes = [_i] * 6 + [_c.POINTER(_i)] * 2
        h.orc_frag_map.restype = None
        h.orc_frag_map.argtypes = [_i] * 6 + [_c.POINTER(_i)] * 2
        h.orc_foreach_mem_index.restype = _i
        h.orc_foreach_mem_index.argtypes = [_i] * 7
        h.orc_foreach_v_index.restype = _i
        h.orc_foreach_v_index.argtypes = [_i] * 7
        h.orc_tcec_matmul.restype = None
        h.orc_tcec_matmul.argtypes = [_i, _i, _i, _i, _fp, _ll, _ll, _fp, _ll, _ll,
                                      _c.c_void_p, _fp, _ll, _ll, _i, _i, _i]
        h.orc_tcec_matmul_model.restype = None
        h.orc_tcec_matmul_model.argtypes = [_i, _i, _i, _i, _fp, _ll, _ll, _fp, _ll, _ll,
                                            _c.c_void_p, _fp, _ll, _ll, _i, _i, _i, _i]
        h.orc_mfma_dot.restype = _c.c_float
        h.orc_mfma_dot.argtypes = [_fp, _fp, _i, _i, _c.c_float]
        h.orc_mfma_tile.restype = None
        h.orc_mfma_tile.argtypes = [_i, _i, _i, _i, np.ctypeslib.ndpointer(np.uint16, flags="C"),
                                    np.ctypeslib.ndpointer(np.uint16, flags="C"), _c.c_void_p, _fp]
        h.orc_to_tf32.restype = _c.c_float
        h.orc_to_tf32.argtypes = [_c.c_float]
        h.orc_gemm_f64.restype = None
        h.orc_gemm_f64.argtypes = [_i, _i, _i, _fp, _ll, _ll, _fp, _ll, _ll, _dp, _ll, _ll]
        h.orc_gemm_f32.restype = None
        h.orc_gemm_f32.argtypes = [_i, _i, _i, _fp, _ll, _ll, _fp, _ll, _ll, _fp, _ll, _ll]
        h.orc_epilogue.restype = None
        h.orc_epilogue.argtypes = [_ll, _fp, _c.c_float, _c.c_float, _fp, _fp, _i]
        h.orc_fp32_policy_matmul.restype = None
        h.orc_fp32_policy_matmul.argtypes = [_i, _i, _i, _fp, _ll, _ll, _fp, _ll, _ll, _c.c_void_p, _fp, _i]
        h.orc_gemm_f32_tn.restype = None
        h.orc_gemm_f32_tn.argtypes = [_i, _i, _i, _fp, _i, _fp, _i, _fp, _i]
        for name in ("orc_max_rel_err", "orc_max_abs_err", "orc_frobenius_residual"):
            fn = getattr(h, name)
            fn.restype = _c.c_double
            fn.argtypes = [_fp, _dp, _ll]
        h.orc_num_threads.restype = _i
        h.orc_num_threads.argtypes = []
        h.orc_split_terms.restype = _i
        h.orc_split_terms.argtypes = [_i]
        h.orc_split_scale.restype = _c.c_float
        h.orc_split_scale.argtypes = [_i]
        _LIB = h
    return _LIB


# ------------------------------------------------------------ conversions
def f32_to_f16_bits(v):
    return lib().orc_f32_to_f16(float(np.float32(v)))


def f32_to_bf16_bits(v):
    return lib().orc_f32_to_bf16(float(np.float32(v)))


def split(kind, v):
    """v: float32 array -> list of uint16 arrays (one per term)."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    n_terms = lib().orc_split_terms(kind)
    outs = [np.zeros(v.shape, dtype=np.uint16) for _ in range(3)]
    lib().orc_split_array(kind, v.reshape(-1), v.size, outs[0].reshape(-1),
                          outs[1].ctypes.data_as(_c.c_void_p),
                          outs[2].ctypes.data_as(_c.c_void_p))
    return outs[:n_terms]


def f16_bits_to_f32(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def terms_to_f32(kind, bits):
    return f16_bits_to_f32(bits) if kind == SPLIT_F16 else bf16_bits_to_f32(bits)


def split_scale(kind):
    return float(lib().orc_split_scale(kind))


# ------------------------------------------------------------ layout model
def frag_shape(use, M, N, K):
    h = lib()
    return h.orc_frag_rows(use, M, N, K), h.orc_frag_cols(use, M, N, K), \
        h.orc_frag_num_elements(use, M, N, K)


def frag_ij_table(use, M, N, K):
    """(64, R, 2) int32: (i,j) of every (lane, register)."""
    _, _, R = frag_shape(use, M, N, K)
    out = np.zeros((64, R, 2), dtype=np.int32)
    i, j = _i(), _i()
    for lane in range(64):
        for reg in range(R):
            lib().orc_frag_ij(use, M, N, K, lane, reg, ctypes.byref(i), ctypes.byref(j))
            out[lane, reg] = (i.value, j.value)
    return out


def frag_map_table(use, M, N, K):
    """two (rows, cols) int32 arrays: lane and register of every (i,j)."""
    rows, cols, _ = frag_shape(use, M, N, K)
    tid = np.zeros((rows, cols), dtype=np.int32)
    fid = np.zeros((rows, cols), dtype=np.int32)
    t, f = _i(), _i()
    for i in range(rows):
        for j in range(cols):
            lib().orc_frag_map(use, M, N, K, i, j, ctypes.byref(t), ctypes.byref(f))
            tid[i, j], fid[i, j] = t.value, f.value
    return tid, fid


def foreach_tables(use, M, N, K, col):
    """(64,R) mem_index of foreach and (64,R) vector index of foreach_v (-1 = skipped)."""
    _, _, R = frag_shape(use, M, N, K)
    mem = np.zeros((64, R), dtype=np.int32)
    vidx = np.zeros((64, R), dtype=np.int32)
    for lane in range(64):
        for reg in range(R):
            mem[lane, reg] = lib().orc_foreach_mem_index(use, M, N, K, int(col), lane, reg)
            vidx[lane, reg] = lib().orc_foreach_v_index(use, M, N, K, int(col), lane, reg)
    return mem, vidx


# ------------------------------------------------------------------ GEMMs
def _strides(x):
    assert x.dtype in (np.float32, np.float64)
    return x.strides[0] // x.itemsize, x.strides[1] // x.itemsize


def _base(x):
    """A C-contiguous array that owns the memory x is a (possibly transposed) view of."""
    b = x
    while b.base is not None and isinstance(b.base, np.ndarray):
        b = b.base
    return b


def _as_strided_arg(x):
    """Return (flat contiguous buffer, row stride, col stride) for a 2-D array
    that is either C- or F-contiguous."""
    if x.flags["C_CONTIGUOUS"]:
        return x.reshape(-1), x.shape[1], 1
    if x.flags["F_CONTIGUOUS"]:
        return x.T.reshape(-1), 1, x.shape[0]
    x = np.ascontiguousarray(x)
    return x.reshape(-1), x.shape[1], 1


def gemm_f64(A, B):
    """A (m,k), B (k,n) float32 -> (m,n) float64 with FP64 accumulation."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2
    a, ar, ac = _as_strided_arg(A)
    b, br, bc = _as_strided_arg(B)
    D = np.zeros((m, n), dtype=np.float64)
    lib().orc_gemm_f64(m, n, k, a, ar, ac, b, br, bc, D.reshape(-1), n, 1)
    return D


def gemm_f32(A, B):
    """Plain fp32 loop (float accumulator, k ascending, no FMA)."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2
    a, ar, ac = _as_strided_arg(A)
    b, br, bc = _as_strided_arg(B)
    D = np.zeros((m, n), dtype=np.float32)
    lib().orc_gemm_f32(m, n, k, a, ar, ac, b, br, bc, D.reshape(-1), n, 1)
    return D


def epilogue(t, alpha, beta, C=None, api_form=False):
    """alpha * t + beta * C as the driver's kernels round it: t * alpha, then one fused
    multiply-add of beta * C (beta == 0: C is not read).  api_form: as the GEMM written on the
    public API rounds it (beta * C first, then one fused multiply-add of alpha * t)."""
    t = np.ascontiguousarray(t, dtype=np.float32)
    c = np.ascontiguousarray(C if C is not None else np.zeros_like(t), dtype=np.float32)
    assert c.shape == t.shape
    out = np.empty_like(t)
    lib().orc_epilogue(t.size, t.reshape(-1), float(alpha), float(beta), c.reshape(-1), out.reshape(-1), int(api_form))
    return out


def fp32_policy_matmul(A, B, C=None, main_outside=False):
    """D = A*B (+C) as the fp32 policy runs on the gfx950 matrix core: fused multiply-adds in the
    order k = x + 4g (x = 0..3, g = 0..3) within every 16 of k, starting from C (main_outside:
    every 16 of k from zero, added with an fp32 add - mma_rn_sync)."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2 and k % 16 == 0
    a, ar, ac = _as_strided_arg(A)
    b, br, bc = _as_strided_arg(B)
    D = np.zeros((m, n), dtype=np.float32)
    cptr = None
    if C is not None:
        C = np.ascontiguousarray(C, dtype=np.float32)
        assert C.shape == (m, n)
        cptr = C.ctypes.data_as(_c.c_void_p)
    lib().orc_fp32_policy_matmul(m, n, k, a, ar, ac, b, br, bc, cptr, D.reshape(-1), int(main_outside))
    return D


def gemm_f32_tn(A, Bt):
    """Timing variant: A (m,k) and Bt (n,k) both C-contiguous; returns C^T (n,m)."""
    m, k = A.shape
    n, _ = Bt.shape
    D = np.zeros((n, m), dtype=np.float32)
    lib().orc_gemm_f32_tn(m, n, k, A.reshape(-1), k, Bt.reshape(-1), k, D.reshape(-1), m)
    return D


def to_tf32(v):
    """fp32 -> tf32 with ties away from zero (the reference's cvt.rna)."""
    return np.float32(lib().orc_to_tf32(float(np.float32(v))))


def mfma_dot(a, b, c=0.0, bf16=False):
    """One output element of a raw MFMA in the gfx950 accumulate model: a, b hold values that are
    exactly representable in the 16-bit type."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    assert a.shape == b.shape and a.ndim == 1
    return np.float32(lib().orc_mfma_dot(a, b, a.size, int(bf16), float(np.float32(c))))


def mfma_tile(type_, a_bits, b_bits, c=None):
    """D = A*B + C of one raw MFMA in the gfx950 accumulate model; a_bits (M,K) and b_bits (K,N) are
    uint16 bit patterns (type_ 0 half, 1 bfloat16), c (M,N) fp32 or None."""
    a_bits = np.ascontiguousarray(a_bits).view(np.uint16)
    b_bits = np.ascontiguousarray(b_bits).view(np.uint16)
    M, K = a_bits.shape
    K2, N = b_bits.shape
    assert K == K2 and K <= 64
    d = np.zeros((M, N), dtype=np.float32)
    cptr = None
    if c is not None:
        c = np.ascontiguousarray(c, dtype=np.float32)
        cptr = c.ctypes.data_as(_c.c_void_p)
    lib().orc_mfma_tile(type_, M, N, K, a_bits, b_bits, cptr, d.reshape(-1))
    return d


def tcec_matmul(A, B, C=None, kind=SPLIT_F16, ec=True, fk=32, main_outside=True, hw_model=False):
    """TCEC emulation of D = A*B (+C) with k blocks of fk.  hw_model: every matrix instruction in
    the measured accumulate arithmetic of the gfx950 matrix core instead of an exact sum rounded
    once."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2
    a, ar, ac = _as_strided_arg(A)
    b, br, bc = _as_strided_arg(B)
    D = np.zeros((m, n), dtype=np.float32)
    cptr = None
    if C is not None:
        C = np.ascontiguousarray(C, dtype=np.float32)
        cptr = C.ctypes.data_as(_c.c_void_p)
    lib().orc_tcec_matmul_model(m, n, k, fk, a, ar, ac, b, br, bc, cptr, D.reshape(-1), n, 1,
                                kind, int(ec), int(main_outside), int(hw_model))
    return D


def max_rel_err(x, ref):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ref = np.ascontiguousarray(ref, dtype=np.float64).reshape(-1)
    return lib().orc_max_rel_err(x, ref, x.size)


def max_abs_err(x, ref):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ref = np.ascontiguousarray(ref, dtype=np.float64).reshape(-1)
    return lib().orc_max_abs_err(x, ref, x.size)


def frobenius_residual(x, ref):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ref = np.ascontiguousarray(ref, dtype=np.float64).reshape(-1)
    return lib().orc_frobenius_residual(x, ref, x.size)


def num_threads():
    return lib().orc_num_threads()
