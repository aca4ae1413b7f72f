"""Host-side calls into the gfx950 TCEC library, on torch CUDA tensors.

torch is used for device memory and streams only; all arithmetic happens in
the HIP kernels behind the C-ABI (include/wmmae_tcec.h).  The functions keep
the argument meaning of the reference's GEMM harness
(test/tcec/batch_gemm.cu:433-443: m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
batch) and of its one-warp test kernels.
"""
import ctypes
import enum

import torch

from . import _lib


class Policy(enum.IntEnum):
    """Arithmetic policies (reference: tcec/detail/policy.hpp:50-99)."""
    F16_EC = 0      # half, with_ec
    F16_NOEC = 1    # half, without_ec
    BF16X3_EC = 2   # tf32 policy carried by a three-term bf16 split
    BF16X2_EC = 3   # bfloat16, with_ec (two terms)
    BF16_NOEC = 4   # bfloat16, without_ec


FLAG_RN_MAIN = 1
FLAG_PATH_PACKED = 2    # take this path instead of the estimated one
FLAG_PATH_FUSED = 4
FLAG_PATH_DIRECT = 8

TYPE_HALF, TYPE_BF16, TYPE_TF32 = 0, 1, 2
USE_A, USE_B, USE_ACC = 0, 1, 2


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _f(v):
    return ctypes.byref(ctypes.c_float(float(v)))


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("device tensors required")


def _room(t):
    """Bytes from t's first element to the end of its storage."""
    return t.untyped_storage().nbytes() - t.storage_offset() * t.element_size()


def _check_matrix(name, t, rows, cols, ld, batch=1, stride=0, device=None):
    """A column-major rows x cols fp32 matrix (leading dimension ld, `batch` of them `stride`
    apart) must lie inside the tensor's storage: the kernels take raw pointers, so a wrong dtype
    or a short tensor would read or write out of bounds on the GPU."""
    if t is None:
        return
    if t.dtype != torch.float32:
        raise ValueError(f"{name}: float32 tensor required, got {t.dtype}")
    if device is not None and t.device != device:
        raise ValueError(f"{name}: on {t.device}, expected {device}")
    if rows <= 0 or cols <= 0 or batch <= 0:
        return
    if stride < 0:
        raise ValueError(f"{name}: negative batch stride")
    need = ((batch - 1) * stride + (cols - 1) * ld + rows) * 4
    if ld >= rows and _room(t) < need:
        raise ValueError(f"{name}: needs {need} bytes from its first element, tensor has {_room(t)}")


def _check_gemm_operands(transa, transb, m, n, k, A, lda, B, ldb, C, ldc, batch=1,
                         stride_a=0, stride_b=0, stride_c=0):
    dev = C.device if C is not None else None
    ta, tb = transa in "Nn", transb in "Nn"
    _check_matrix("A", A, m if ta else k, k if ta else m, lda, batch, stride_a, dev)
    _check_matrix("B", B, k if tb else n, n if tb else k, ldb, batch, stride_b, dev)
    _check_matrix("C", C, m, n, ldc, batch, stride_c, dev)


def _check_bytes(name, t, need, device=None):
    if t is None:
        return
    if device is not None and t.device != device:
        raise ValueError(f"{name}: on {t.device}, expected {device}")
    if _room(t) < need:
        raise ValueError(f"{name}: needs {need} bytes, tensor has {_room(t)}")


def query(what):
    out = ctypes.c_longlong(0)
    _lib.check(_lib.lib().wmmae_query(int(what), ctypes.byref(out)), "wmmae_query")
    return out.value


def workspace_bytes(m, n, k, batch=1, policy=Policy.F16_EC):
    out = ctypes.c_size_t(0)
    _lib.check(_lib.lib().wmmae_tcec_sgemm_workspace_bytes(m, n, k, batch, int(policy),
                                                           ctypes.byref(out)),
               "wmmae_tcec_sgemm_workspace_bytes")
    return out.value


PATH_FUSED, PATH_PACKED, PATH_PACKED_SPLIT_K, PATH_DIRECT, PATH_DIRECT_SPLIT_K = 0, 1, 2, 3, 4


def sgemm_path(m, n, k, batch=1, policy=Policy.F16_EC, flags=0):
    """Which path the GEMM entry points take for this shape (PATH_* above)."""
    out = ctypes.c_int(-1)
    _lib.check(_lib.lib().wmmae_tcec_sgemm_path(m, n, k, batch, int(policy), flags,
                                                ctypes.byref(out)), "wmmae_tcec_sgemm_path")
    return out.value


def sgemm_k_slices(m, n, k, batch=1, policy=Policy.F16_EC, flags=0):
    """How many K slices the GEMM entry points cut this product into on the path `flags`
    select (1: none)."""
    out = ctypes.c_int(-1)
    _lib.check(_lib.lib().wmmae_tcec_sgemm_k_slices(m, n, k, batch, int(policy), flags,
                                                    ctypes.byref(out)), "wmmae_tcec_sgemm_k_slices")
    return out.value


def path_estimates(m, n, k, batch=1, policy=Policy.F16_EC):
    """(fused, packed, direct) time estimates in seconds the driver chooses its path with
    (inf: the path cannot take the product)."""
    out = (ctypes.c_double * 3)()
    _lib.check(_lib.lib().wmmae_tcec_path_estimates(m, n, k, batch, int(policy), out),
               "wmmae_tcec_path_estimates")
    return tuple(out)


class timed_gemm_kernel:
    """Within the block, this thread's packed- and direct-path calls record `begin` / `end`
    (torch.cuda.Event with timing) right before and after their MFMA GEMM kernel:
    begin.elapsed_time(end) after a synchronisation is that kernel's time inside the whole call."""

    def __init__(self, begin, end):
        self.begin, self.end = begin, end

    def __enter__(self):
        # (a torch event gets its handle at its first record)
        for e in (self.begin, self.end):
            if not e.cuda_event:
                e.record()
        _lib.check(_lib.lib().wmmae_tcec_time_gemm_kernel(ctypes.c_void_p(self.begin.cuda_event),
                                                          ctypes.c_void_p(self.end.cuda_event)),
                   "wmmae_tcec_time_gemm_kernel")
        return self

    def __exit__(self, *exc):
        _lib.lib().wmmae_tcec_time_gemm_kernel(None, None)
        return False


class forced_k_slices:
    """Test aid: within the block, this thread's GEMM calls cut K into `slices` slices."""

    def __init__(self, slices):
        self.slices = slices

    def __enter__(self):
        _lib.check(_lib.lib().wmmae_tcec_force_k_slices(self.slices), "wmmae_tcec_force_k_slices")
        return self

    def __exit__(self, *exc):
        _lib.lib().wmmae_tcec_force_k_slices(0)
        return False


def pack_bytes(rows, k, batch=1, policy=Policy.F16_EC):
    out = ctypes.c_size_t(0)
    _lib.check(_lib.lib().wmmae_tcec_pack_bytes(rows, k, batch, int(policy), ctypes.byref(out)),
               "wmmae_tcec_pack_bytes")
    return out.value


def sgemm(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
          policy=Policy.F16_EC, flags=0, workspace=None):
    """C = alpha*op(A)*op(B) + beta*C, column-major BLAS convention."""
    _need_cuda(A, B, C, workspace)
    _check_gemm_operands(transa, transb, m, n, k, A, lda, B, ldb, C, ldc)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = _lib.lib().wmmae_tcec_sgemm(transa.encode(), transb.encode(), m, n, k, _f(alpha),
                                     _ptr(A), lda, _ptr(B), ldb, _f(beta), _ptr(C), ldc,
                                     int(policy), flags, _ptr(workspace), ws_bytes, _stream())
    _lib.check(st, "wmmae_tcec_sgemm")


STATIC_SCRATCH_BYTES = 64 << 20


def sgemm_static(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                 policy=Policy.F16_EC, flags=0):
    """sgemm on the library's own fixed workspace: allocates nothing."""
    _need_cuda(A, B, C)
    _check_gemm_operands(transa, transb, m, n, k, A, lda, B, ldb, C, ldc)
    st = _lib.lib().wmmae_tcec_sgemm_static(transa.encode(), transb.encode(), m, n, k, _f(alpha),
                                            _ptr(A), lda, _ptr(B), ldb, _f(beta), _ptr(C), ldc,
                                            int(policy), flags, _stream())
    _lib.check(st, "wmmae_tcec_sgemm_static")


def sgemm_strided_batched(transa, transb, m, n, k, alpha, A, lda, stride_a, B, ldb, stride_b,
                          beta, C, ldc, stride_c, batch, policy=Policy.F16_EC, flags=0,
                          workspace=None):
    _need_cuda(A, B, C, workspace)
    _check_gemm_operands(transa, transb, m, n, k, A, lda, B, ldb, C, ldc, batch,
                         stride_a, stride_b, stride_c)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = _lib.lib().wmmae_tcec_sgemm_strided_batched(
        transa.encode(), transb.encode(), m, n, k, _f(alpha), _ptr(A), lda, stride_a,
        _ptr(B), ldb, stride_b, _f(beta), _ptr(C), ldc, stride_c, batch, int(policy), flags,
        _ptr(workspace), ws_bytes, _stream())
    _lib.check(st, "wmmae_tcec_sgemm_strided_batched")


def sgemm_batched(transa, transb, m, n, k, alpha, A_array, lda, B_array, ldb, beta, C_array, ldc,
                  batch, policy=Policy.F16_EC, flags=0, workspace=None):
    """A_array / B_array / C_array: int64 device tensors holding `batch` device pointers
    (the launch_bgemm / cublasSgemmBatched convention)."""
    _need_cuda(A_array, B_array, C_array, workspace)
    for name, arr in (("A_array", A_array), ("B_array", B_array), ("C_array", C_array)):
        if arr is not None and (arr.dtype != torch.int64 or arr.numel() < batch):
            raise ValueError(f"{name}: int64 tensor of at least {batch} device pointers required")
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = _lib.lib().wmmae_tcec_sgemm_batched(
        transa.encode(), transb.encode(), m, n, k, _f(alpha), _ptr(A_array), lda, _ptr(B_array), ldb,
        _f(beta), _ptr(C_array), ldc, batch, int(policy), flags, _ptr(workspace), ws_bytes, _stream())
    _lib.check(st, "wmmae_tcec_sgemm_batched")


def pack(policy, rows, k, X, row_stride, k_stride, packed, batch=1, batch_stride=0):
    _need_cuda(X, packed)
    if X is not None and X.dtype != torch.float32:
        raise ValueError(f"X: float32 tensor required, got {X.dtype}")
    if X is not None and rows > 0 and k > 0 and batch > 0 and min(row_stride, k_stride, batch_stride) >= 0:
        _check_bytes("X", X, 4 * ((batch - 1) * batch_stride + (rows - 1) * row_stride
                                  + (k - 1) * k_stride + 1), packed.device)
    st = _lib.lib().wmmae_tcec_pack(int(policy), rows, k, _ptr(X), row_stride, k_stride,
                                    batch_stride, batch, _ptr(packed),
                                    packed.numel() * packed.element_size(), _stream())
    _lib.check(st, "wmmae_tcec_pack")


def gemm_packed_workspace_bytes(policy, m, n, k, batch=1):
    out = ctypes.c_size_t(0)
    _lib.check(_lib.lib().wmmae_tcec_gemm_packed_workspace_bytes(int(policy), m, n, k, batch,
                                                                 ctypes.byref(out)),
               "wmmae_tcec_gemm_packed_workspace_bytes")
    return out.value


def gemm_packed(policy, m, n, k, alpha, packed_a, packed_b, beta, C, ldc, batch=1,
                stride_c=0, flags=0, workspace=None):
    _need_cuda(packed_a, packed_b, C, workspace)
    _check_matrix("C", C, m, n, ldc, batch, stride_c)
    if k > 0 and m > 0 and n > 0 and batch > 0:
        _check_bytes("packed_a", packed_a, pack_bytes(m, k, batch, policy), C.device)
        _check_bytes("packed_b", packed_b, pack_bytes(n, k, batch, policy), C.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = _lib.lib().wmmae_tcec_gemm_packed(int(policy), m, n, k, _f(alpha), _ptr(packed_a),
                                           _ptr(packed_b), _f(beta), _ptr(C), ldc, stride_c,
                                           batch, flags, _ptr(workspace), ws_bytes, _stream())
    _lib.check(st, "wmmae_tcec_gemm_packed")


def matmul_tn(A, B, policy=Policy.F16_EC, flags=0, workspace=None, out=None):
    """The reference harness layout: A is (m,k) row-major, B is given as (n,k)
    row-major (= k x n column-major), result (n,m) row-major (= m x n column-major,
    ldc = m).  Returns the tensor holding C column-major, i.e. C^T as a torch view."""
    m, k = A.shape
    n, k2 = B.shape
    assert k == k2 and A.is_contiguous() and B.is_contiguous()
    if out is None:
        out = torch.empty((n, m), dtype=torch.float32, device=A.device)
    elif tuple(out.shape) != (n, m) or not out.is_contiguous():
        raise ValueError(f"out: contiguous ({n}, {m}) tensor required, got {tuple(out.shape)}")
    sgemm("T", "N", m, n, k, 1.0, A, k, B, k, 0.0, out, m, policy, flags, workspace)
    return out


# --------------------------------------------------------------- harness
def primitive_tiles(tiles):
    """tiles: (T,256) fp32.  Returns dict of the per-tile outputs."""
    _need_cuda(tiles)
    T = tiles.shape[0]
    dev = tiles.device
    out = {
        "a_row": torch.empty((T, 64, 4), dtype=torch.float16, device=dev),
        "a_col": torch.empty((T, 64, 4), dtype=torch.float16, device=dev),
        "b_row": torch.empty((T, 64, 4), dtype=torch.float16, device=dev),
        "b_col": torch.empty((T, 64, 4), dtype=torch.float16, device=dev),
        "acc": torch.empty((T, 256), dtype=torch.float32, device=dev),
        "vec": torch.empty((T, 32), dtype=torch.float32, device=dev),
    }
    st = _lib.lib().wmmae_primitive_tiles(_ptr(tiles), T, _ptr(out["a_row"]), _ptr(out["a_col"]),
                                          _ptr(out["b_row"]), _ptr(out["b_col"]),
                                          _ptr(out["acc"]), _ptr(out["vec"]), _stream())
    _lib.check(st, "wmmae_primitive_tiles")
    return out


def layout_dump(use, m, n, k, col, device="cuda"):
    rows = k if use == USE_B else m
    cols = k if use == USE_A else n
    R = rows * cols // 64
    ij = torch.full((64, R, 2), -7, dtype=torch.int32, device=device)
    mem = torch.full((64, R), -7, dtype=torch.int32, device=device)
    vidx = torch.full((64, R), -7, dtype=torch.int32, device=device)
    tid = torch.full((rows, cols), -7, dtype=torch.int32, device=device)
    fid = torch.full((rows, cols), -7, dtype=torch.int32, device=device)
    st = _lib.lib().wmmae_layout_dump(use, m, n, k, int(col), _ptr(ij), _ptr(mem), _ptr(vidx),
                                      _ptr(tid), _ptr(fid), _stream())
    _lib.check(st, "wmmae_layout_dump")
    return ij, mem, vidx, tid, fid


def mma_tile(shape, type_, ec, inst, a, b, c, a_col, b_col, c_col, d_col, rounding, d):
    _need_cuda(a, b, c, d)
    st = _lib.lib().wmmae_tcec_mma_tile(shape, type_, int(ec), inst, _ptr(d), _ptr(a), _ptr(b),
                                        _ptr(c), int(a_col), int(b_col), int(c_col), int(d_col),
                                        rounding, _stream())
    _lib.check(st, "wmmae_tcec_mma_tile")
    return d


def mma_tile_native(type_, ec, a_frag_col, b_frag_col, a, b, d_col, d):
    _need_cuda(a, b, d)
    st = _lib.lib().wmmae_tcec_mma_tile_native(type_, int(ec), int(a_frag_col), int(b_frag_col),
                                               _ptr(d), _ptr(a), _ptr(b), int(d_col), _stream())
    _lib.check(st, "wmmae_tcec_mma_tile_native")
    return d


def matvec(type_, ec, a, x, a_col, left_vector):
    _need_cuda(a, x)
    y = torch.empty(32, dtype=torch.float32, device=a.device)
    st = _lib.lib().wmmae_tcec_matvec(type_, int(ec), _ptr(y), _ptr(a), _ptr(x), int(a_col),
                                      int(left_vector), _stream())
    _lib.check(st, "wmmae_tcec_matvec")
    return y


def frag_dump(use, type_, ec, frag_col, src, from_vector, mem_col):
    _need_cuda(src)
    terms = 1 if not ec else (3 if type_ == TYPE_TF32 else 2)
    E = 32 * 32 // 64
    out = torch.zeros((terms, E, 64), dtype=torch.int16, device=src.device)
    st = _lib.lib().wmmae_tcec_frag_dump(use, type_, int(ec), int(frag_col), _ptr(out), _ptr(src),
                                         int(from_vector), int(mem_col), _stream())
    _lib.check(st, "wmmae_tcec_frag_dump")
    return out


def elementwise(type_, ec, inst, base, do_neg, do_integrate, device="cuda"):
    out = torch.zeros(32 * 32 + 64, dtype=torch.float32, device=device)
    st = _lib.lib().wmmae_tcec_elementwise(type_, int(ec), inst, _ptr(out), float(base), int(do_neg),
                                           int(do_integrate), _stream())
    _lib.check(st, "wmmae_tcec_elementwise")
    return out


def api_gemm(type_, ec, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, rounding=0):
    """Tiled GEMM written against the public device API only (rounding: 0 tcec::mma_sync,
    1 mma_rn_sync, 2 mma_rz_sync)."""
    _need_cuda(A, B, C)
    _check_gemm_operands("T", "N", m, n, k, A, lda, B, ldb, C, ldc)
    if rounding == 0:
        st = _lib.lib().wmmae_tcec_api_gemm(type_, int(ec), m, n, k, _f(alpha), _ptr(A), lda, _ptr(B), ldb,
                                            _f(beta), _ptr(C), ldc, _stream())
        _lib.check(st, "wmmae_tcec_api_gemm")
        return
    st = _lib.lib().wmmae_tcec_api_gemm_rounding(type_, int(ec), int(rounding), m, n, k, _f(alpha), _ptr(A), lda,
                                                 _ptr(B), ldb, _f(beta), _ptr(C), ldc, _stream())
    _lib.check(st, "wmmae_tcec_api_gemm_rounding")


def api_gemm_batched(type_, ec, m, n, k, alpha, A_array, lda, B_array, ldb, beta, C_array, ldc, batch):
    """api_gemm on int64 device tensors of `batch` matrix pointers (launch_bgemm's convention)."""
    _need_cuda(A_array, B_array, C_array)
    for name, arr in (("A_array", A_array), ("B_array", B_array), ("C_array", C_array)):
        if arr.dtype != torch.int64 or arr.numel() < batch:
            raise ValueError(f"{name}: int64 tensor of at least {batch} device pointers required")
    st = _lib.lib().wmmae_tcec_api_gemm_batched(type_, int(ec), m, n, k, _f(alpha), _ptr(A_array), lda,
                                                _ptr(B_array), ldb, _f(beta), _ptr(C_array), ldc, batch,
                                                _stream())
    _lib.check(st, "wmmae_tcec_api_gemm_batched")


def mfma_probe(type_, m, n, k, a_bits, b_bits, c):
    """a_bits (m,k) / b_bits (k,n): int16 tensors of raw 16-bit patterns; c (m,n) fp32."""
    _need_cuda(a_bits, b_bits, c)
    d = torch.empty((m, n), dtype=torch.float32, device=c.device)
    st = _lib.lib().wmmae_mfma_probe(type_, m, n, k, _ptr(d), _ptr(a_bits), _ptr(b_bits), _ptr(c),
                                     _stream())
    _lib.check(st, "wmmae_mfma_probe")
    return d


def mfma_source_hazard_probe(producer, gap, device):
    """256 accumulator values of the hazard probe (40: the MFMA saw the register just written,
    32: it saw the old contents); see include/wmmae_tcec_aux.h."""
    d = torch.empty(256, dtype=torch.float32, device=device)
    st = _lib.lib().wmmae_mfma_source_hazard_probe(producer, gap, _ptr(d), _stream())
    _lib.check(st, "wmmae_mfma_source_hazard_probe")
    return d


def utils_cp_async(size, mode, src):
    """src: 256 elements of `size` bytes (any dtype, CUDA); returns the copy made through LDS."""
    _need_cuda(src)
    dst = torch.full_like(src, -1)
    st = _lib.lib().wmmae_utils_cp_async(size, mode, _ptr(dst), _ptr(src), _stream())
    _lib.check(st, "wmmae_utils_cp_async")
    return dst


def utils_cp_async_pipeline(size, copies, groups, src):
    """src: groups * copies * 64 elements of `size` bytes (CUDA).  Returns (the copy made by a
    three-stage cp_async / commit / wait_group<2> pipeline of one wave, the wave's outstanding
    vector-memory instructions at start, after every wait_group and at the end)."""
    _need_cuda(src)
    dst = torch.full_like(src, -1)
    pending = torch.full((groups + 2,), -1, dtype=torch.int32, device=src.device)
    st = _lib.lib().wmmae_utils_cp_async_pipeline(size, copies, groups, _ptr(dst), _ptr(src),
                                                  _ptr(pending), _stream())
    _lib.check(st, "wmmae_utils_cp_async_pipeline")
    return dst, pending


def print_fragment(type_, ec, src, base):
    """Device printf of a primitive and a TCEC fragment (one wave) to the process's stdout."""
    _need_cuda(src)
    if src.dtype != torch.float32 or src.numel() < 256:
        raise ValueError("src: 256 float32 values required")
    st = _lib.lib().wmmae_print_fragment(type_, int(ec), _ptr(src), float(base), _stream())
    _lib.check(st, "wmmae_print_fragment")


def utils_cast(dst_type, x):
    """x: fp32 CUDA tensor -> int16 bit patterns (dst_type 0 half, 1 bfloat16) or fp32 (2 tf32, 3 float)."""
    _need_cuda(x)
    out = torch.empty(x.shape, dtype=torch.int16 if dst_type in (0, 1) else torch.float32, device=x.device)
    st = _lib.lib().wmmae_utils_cast(dst_type, _ptr(x), _ptr(out), x.numel(), _stream())
    _lib.check(st, "wmmae_utils_cast")
    return out


def mma_complex(type_, ec, a, b, c, a_col, b_col, c_col, d_col, rounding=0, mul=1.0):
    """a, b, c: (32*32*2,) fp32 CUDA tensors of interleaved (re, im) pairs; returns d likewise."""
    _need_cuda(a, b, c)
    d = torch.full_like(a, float("nan"))
    st = _lib.lib().wmmae_tcec_mma_complex(type_, ec, _ptr(d), _ptr(a), _ptr(b), _ptr(c), a_col, b_col,
                                           c_col, d_col, rounding, float(mul), _stream())
    _lib.check(st, "wmmae_tcec_mma_complex")
    return d


def fragment_ops(op, use, elem, alpha, a, b):
    """a, b: (16,16) fp32 CUDA tensors (row-major tiles); returns the (16,16) result."""
    _need_cuda(a, b)
    out = torch.full((16, 16), float("nan"), dtype=torch.float32, device=a.device)
    st = _lib.lib().wmmae_fragment_ops(op, use, elem, float(alpha), _ptr(a), _ptr(b), _ptr(out), _stream())
    _lib.check(st, "wmmae_fragment_ops")
    return out


def fragment_eye(shape, identity, alpha, device):
    n = 16 if shape == 0 else 32
    out = torch.full((n, n), float("nan"), dtype=torch.float32, device=device)
    st = _lib.lib().wmmae_fragment_eye(shape, identity, float(alpha), _ptr(out), _stream())
    _lib.check(st, "wmmae_fragment_eye")
    return out


def direct_product(elem, terms, from_float, u, v):
    """u, v: (16,) fp32 CUDA tensors; returns h (16,16) with h[i, j] = u[i] v[j]."""
    _need_cuda(u, v)
    h = torch.full((16, 16), float("nan"), dtype=torch.float32, device=u.device)
    st = _lib.lib().wmmae_direct_product(elem, terms, from_float, _ptr(u), _ptr(v), _ptr(h), _stream())
    _lib.check(st, "wmmae_direct_product")
    return h.t()            # stored column-major


def clock_samples(nsamples, period_ticks, stream=None, device="cuda:0"):
    """Start the shader-clock sampler on `stream` (a torch.cuda.Stream; default: current).
    Returns the (nsamples, 2) int64 CUDA tensor it fills: [:, 0] 100 MHz counter, [:, 1] shader cycles."""
    out = torch.zeros((nsamples, 2), dtype=torch.int64, device=device)
    s = ctypes.c_void_p(stream.cuda_stream) if stream is not None else _stream()
    st = _lib.lib().wmmae_clock_samples(_ptr(out), nsamples, int(period_ticks), s)
    _lib.check(st, "wmmae_clock_samples")
    return out


PRIMITIVE_SHAPES = {0: (16, 16, 16), 1: (16, 16, 32), 2: (32, 32, 8), 3: (32, 32, 16)}


def primitive_mma(elem, shape, a, b, c, a_col, b_col, c_col, d_col, d=None, wrappers=False):
    """a, b, c: flat fp32 CUDA images of the operands in the given layouts; returns flat d
    (written into `d` when the caller passes one, e.g. a view at an odd offset).
    wrappers=True runs the same MMA through the tcec::detail function objects."""
    _need_cuda(a, b, c, d)
    m, n, _ = PRIMITIVE_SHAPES[shape]
    if wrappers:
        shape += 8
    if d is None:
        d = torch.full((m * n,), float("nan"), dtype=torch.float32, device=a.device)
    assert d.numel() == m * n and d.is_contiguous()
    st = _lib.lib().wmmae_primitive_mma(elem, shape, _ptr(d), _ptr(a), _ptr(b), _ptr(c), a_col, b_col,
                                        c_col, d_col, _stream())
    _lib.check(st, "wmmae_primitive_mma")
    return d


def foreach_ec(a, b):
    _need_cuda(a, b)
    d = torch.full((256,), float("nan"), dtype=torch.float32, device=a.device)
    _lib.check(_lib.lib().wmmae_foreach_ec(_ptr(d), _ptr(a), _ptr(b), _stream()), "wmmae_foreach_ec")
    return d


def gevm(x, e):
    _need_cuda(x, e)
    y = torch.full((16,), float("nan"), dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().wmmae_gevm(_ptr(y), _ptr(x), _ptr(e), _stream()), "wmmae_gevm")
    return y
