"""Host-side checks of the C-ABI that need no GPU: the library loads, exports
every declared symbol, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest

from wmma_extension_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def h():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.lib()


def test_header_and_library_agree(h):
    text = open(os.path.join(ROOT, "include", "wmmae_tcec.h")).read()
    aux = open(os.path.join(ROOT, "include", "wmmae_tcec_aux.h")).read()
    declared = set(re.findall(r"\b(wmmae_[a-z0-9_]+)\s*\(", text))
    declared_aux = set(re.findall(r"\b(wmmae_[a-z0-9_]+)\s*\(", aux))
    # the measurement aids live in their own header, outside the product ABI
    assert declared_aux == {"wmmae_clock_samples", "wmmae_mfma_probe", "wmmae_direct_read_first",
                            "wmmae_tcec_sgemm_k_slices", "wmmae_tcec_force_k_slices", "wmmae_tcec_time_gemm_kernel",
                            "wmmae_tcec_path_estimates", "wmmae_mfma_source_hazard_probe"} and not (declared & declared_aux)
    declared |= declared_aux
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert getattr(h, name) is not None


def test_status_strings(h):
    assert h.wmmae_status_string(0) == b"success"
    for code in range(-7, 0):
        assert h.wmmae_status_string(code) not in (b"success", b"unknown status")
    assert h.wmmae_status_string(-99) == b"unknown status"


def test_sizes_are_host_only(h):
    out = ctypes.c_size_t(0)
    assert h.wmmae_tcec_pack_bytes(16, 32, 1, 0, ctypes.byref(out)) == 0
    assert out.value == 2 * 1024                # one chunk, two terms
    assert h.wmmae_tcec_pack_bytes(4096, 4096, 1, 0, ctypes.byref(out)) == 0
    assert out.value == 4096 * 4096 * 4          # hi + lo = 4 bytes per element
    assert h.wmmae_tcec_pack_bytes(4096, 4096, 1, 2, ctypes.byref(out)) == 0
    assert out.value == 4096 * 4096 * 6
    assert h.wmmae_tcec_pack_bytes(17, 33, 3, 1, ctypes.byref(out)) == 0
    assert out.value == 3 * 2 * 2 * 1024         # batch 3, 2 row blocks x 2 k tiles, one term
    assert h.wmmae_tcec_sgemm_workspace_bytes(4096, 4096, 4096, 1, 0, ctypes.byref(out)) == 0
    assert out.value == 2 * 4096 * 4096 * 4
    # split-K room: none for square problems, slices of C for the K-heavy shape
    assert h.wmmae_tcec_gemm_packed_workspace_bytes(0, 4096, 4096, 4096, 1, ctypes.byref(out)) == 0
    assert out.value == 0
    assert h.wmmae_tcec_gemm_packed_workspace_bytes(0, 1024, 1024, 262144, 1, ctypes.byref(out)) == 0
    assert out.value > 0 and out.value % (1024 * 1024 * 4) == 0
    assert h.wmmae_tcec_pack_bytes(16, 32, 1, 9, ctypes.byref(out)) == -1
    assert h.wmmae_tcec_pack_bytes(-1, 32, 1, 0, ctypes.byref(out)) == -1
    assert h.wmmae_tcec_pack_bytes(16, 32, 1, 0, None) == -2


def _sgemm(h, ta=b"T", tb=b"N", m=64, n=64, k=64, alpha=True, A=1, lda=64, B=1, ldb=64,
           beta=True, C=1, ldc=64, policy=0, flags=0):
    one = ctypes.c_float(1.0)
    return h.wmmae_tcec_sgemm(ta, tb, m, n, k, ctypes.byref(one) if alpha else None,
                              ctypes.c_void_p(A), lda, ctypes.c_void_p(B), ldb,
                              ctypes.byref(one) if beta else None, ctypes.c_void_p(C), ldc,
                              policy, flags, None, 0, None)


def test_sgemm_argument_validation(h):
    # all of these return before any device access (the pointers are fake)
    assert _sgemm(h, ta=b"X") == -1
    assert _sgemm(h, tb=b"?") == -1
    assert _sgemm(h, m=-1) == -1
    assert _sgemm(h, k=-5) == -1
    assert _sgemm(h, policy=7) == -1
    assert _sgemm(h, flags=16) == -1
    assert _sgemm(h, flags=2 | 8) == -1         # at most one path flag
    assert _sgemm(h, flags=8, k=3, lda=3, ldb=3) == -4    # direct path: k >= 4
    assert _sgemm(h, flags=8, ta=b"N") == -4               # ... and k contiguous
    assert _sgemm(h, flags=8 | 1) == -4                      # ... and no RN_MAIN
    assert _sgemm(h, flags=8, policy=2) == -4                # ... and at most two terms
    assert _sgemm(h, alpha=False) == -2
    assert _sgemm(h, beta=False) == -2
    assert _sgemm(h, A=0) == -2
    assert _sgemm(h, B=0) == -2
    assert _sgemm(h, C=0) == -2
    assert _sgemm(h, lda=63) == -3              # 'T': lda >= k
    assert _sgemm(h, ldb=10) == -3
    assert _sgemm(h, ldc=63) == -3
    assert _sgemm(h, ta=b"N", m=128, lda=64) == -3   # 'N': lda >= m
    # empty problems succeed without touching anything
    assert _sgemm(h, m=0, A=0, B=0, C=0) == 0
    assert _sgemm(h, n=0, A=0, B=0, C=0) == 0


def test_other_entry_points_validate(h):
    one = ctypes.c_float(1.0)
    p = ctypes.c_void_p
    assert h.wmmae_tcec_pack(0, 16, 32, p(0), 32, 1, 0, 1, p(16), 4096, None) == -2
    assert h.wmmae_tcec_pack(0, 16, 32, p(16), 32, 2, 0, 1, p(16), 4096, None) == -3
    assert h.wmmae_tcec_pack(0, 16, 32, p(16), 32, 1, 0, 1, p(24), 4096, None) == -7
    assert h.wmmae_tcec_pack(0, 16, 32, p(16), 32, 1, 0, 1, p(32), 100, None) == -5
    assert h.wmmae_tcec_gemm_packed(0, 16, 16, 32, ctypes.byref(one), p(16), p(16),
                                    ctypes.byref(one), p(0), 16, 0, 1, 0, None, 0, None) == -2
    assert h.wmmae_tcec_gemm_packed(0, 16, 16, 32, ctypes.byref(one), p(16), p(16),
                                    ctypes.byref(one), p(16), 8, 0, 1, 0, None, 0, None) == -3
    assert h.wmmae_tcec_gemm_packed(0, 16, 16, 32, ctypes.byref(one), p(8), p(16),
                                    ctypes.byref(one), p(16), 16, 0, 1, 0, None, 0, None) == -7
    assert h.wmmae_primitive_tiles(p(0), 4, p(0), p(0), p(0), p(0), p(0), p(0), None) == -2
    assert h.wmmae_primitive_tiles(p(0), -1, p(0), p(0), p(0), p(0), p(0), p(0), None) == -1
    assert h.wmmae_layout_dump(0, 16, 16, 16, 0, p(0), p(0), p(0), p(0), p(0), None) == -2
    assert h.wmmae_layout_dump(0, 8, 8, 4, 0, p(8), p(8), p(8), p(8), p(8), None) == -4
    assert h.wmmae_tcec_mma_tile(0, 0, 1, 0, p(0), p(8), p(8), p(0), 0, 0, 0, 0, 0, None) == -2
    assert h.wmmae_tcec_mma_tile(3, 0, 1, 0, p(8), p(8), p(8), p(0), 0, 0, 0, 0, 0, None) == -1
    assert h.wmmae_tcec_mma_tile(0, 5, 1, 0, p(8), p(8), p(8), p(0), 0, 0, 0, 0, 0, None) == -1
    assert h.wmmae_mfma_probe(0, 8, 8, 8, p(8), p(8), p(8), p(8), None) == -4
    assert h.wmmae_mfma_probe(2, 16, 16, 16, p(8), p(8), p(8), p(8), None) == -1
    out = ctypes.c_longlong(0)
    assert h.wmmae_query(0, ctypes.byref(out)) == 0 and out.value == 100
    assert h.wmmae_query(3, ctypes.byref(out)) == 0 and out.value == 5
    assert h.wmmae_query(0, None) == -2
    assert h.wmmae_query(42, ctypes.byref(out)) == -1


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libwmmae_tcec.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()


def test_harness_entries_reject_bad_arguments_on_the_host(h):
    """The newer harness entry points return their status before any launch when
    an argument is wrong (fake non-null pointers are never dereferenced)."""
    p = ctypes.c_void_p(64)
    f = ctypes.c_float
    # complex one-wave product
    assert h.wmmae_tcec_mma_complex(0, 1, None, p, p, p, 0, 0, 0, 0, 0, f(1.0), None) == -2
    assert h.wmmae_tcec_mma_complex(0, 1, p, p, p, p, 0, 0, 0, 0, 5, f(1.0), None) == -1
    assert h.wmmae_tcec_mma_complex(0, 1, p, p, p, p, 0, 0, 0, 0, 0, f(0.0), None) == -1
    assert h.wmmae_tcec_mma_complex(3, 1, p, p, p, p, 0, 0, 0, 0, 0, f(1.0), None) == -4   # fp32 has no EC
    assert h.wmmae_tcec_mma_complex(9, 0, p, p, p, p, 0, 0, 0, 0, 0, f(1.0), None) == -1
    # fp32 policy on the real entry points
    assert h.wmmae_tcec_mma_tile(0, 3, 1, 1, p, p, p, p, 0, 0, 0, 0, 0, None) == -4
    assert h.wmmae_tcec_matvec(3, 1, p, p, p, 0, 0, None) == -4
    assert h.wmmae_tcec_frag_dump(0, 3, 0, 0, p, p, 0, 0, None) == -4
    assert h.wmmae_tcec_frag_dump(0, 0, 1, 0, p, p, 0, 3, None) == -1
    assert h.wmmae_tcec_frag_dump(0, 0, 1, 0, p, ctypes.c_void_p(72), 0, 2, None) == -7
    # fragment operators, eye, direct product
    assert h.wmmae_fragment_ops(6, 0, 0, f(1.0), p, p, p, None) == -1
    assert h.wmmae_fragment_ops(0, 3, 0, f(1.0), p, p, p, None) == -1
    assert h.wmmae_fragment_ops(0, 2, 0, f(1.0), p, p, p, None) == -4    # half accumulators do not exist
    assert h.wmmae_fragment_ops(0, 0, 0, f(1.0), None, p, p, None) == -2
    assert h.wmmae_fragment_eye(2, 0, f(1.0), p, None) == -1
    assert h.wmmae_fragment_eye(0, 0, f(1.0), None, None) == -2
    assert h.wmmae_direct_product(2, 2, 0, p, p, p, None) == -1
    assert h.wmmae_direct_product(0, 4, 0, p, p, p, None) == -1
    assert h.wmmae_direct_product(0, 2, 0, p, None, p, None) == -2
    # utils
    assert h.wmmae_utils_cp_async(12, 0, p, p, None) == -1
    assert h.wmmae_utils_cp_async(4, 7, p, p, None) == -1
    assert h.wmmae_utils_cp_async(16, 0, p, ctypes.c_void_p(72), None) == -7
    assert h.wmmae_utils_cp_async_pipeline(4, 2, 3, None, p, p, None) == -2
    assert h.wmmae_utils_cp_async_pipeline(4, 2, 3, p, p, None, None) == -2
    assert h.wmmae_utils_cp_async_pipeline(12, 2, 3, p, p, p, None) == -1
    assert h.wmmae_utils_cp_async_pipeline(4, 5, 3, p, p, p, None) == -1
    assert h.wmmae_utils_cp_async_pipeline(4, 2, 0, p, p, p, None) == -1
    assert h.wmmae_utils_cp_async_pipeline(16, 2, 3, p, ctypes.c_void_p(72), p, None) == -7
    assert h.wmmae_utils_cast(0, None, p, 4, None) == -2
    assert h.wmmae_utils_cast(0, p, p, -1, None) == -1
    assert h.wmmae_utils_cast(0, p, p, 0, None) == 0                       # nothing to do
    # clock sampler: bounded by construction
    assert h.wmmae_clock_samples(None, 10, 100, None) == -2
    assert h.wmmae_clock_samples(p, 0, 100, None) == -1
    assert h.wmmae_clock_samples(p, 100000, 100000, None) == -1            # would run for 100 s


def test_primitive_entries_reject_bad_arguments_on_the_host(h):
    p = ctypes.c_void_p(64)
    assert h.wmmae_primitive_mma(3, 0, p, p, p, p, 0, 0, 0, 0, None) == -1
    assert h.wmmae_primitive_mma(0, 4, p, p, p, p, 0, 0, 0, 0, None) == -1
    assert h.wmmae_primitive_mma(0, 12, p, p, p, p, 0, 0, 0, 0, None) == -1    # 8 + shape: wrappers
    assert h.wmmae_primitive_mma(2, 9, p, p, p, p, 0, 0, 0, 0, None) == -4
    assert h.wmmae_primitive_mma(2, 1, p, p, p, p, 0, 0, 0, 0, None) == -4     # fp32 has no 16x16x32
    assert h.wmmae_primitive_mma(0, 0, None, p, p, p, 0, 0, 0, 0, None) == -2
    assert h.wmmae_foreach_ec(p, None, p, None) == -2
    assert h.wmmae_gevm(None, p, p, None) == -2


def test_sgemm_path_query_on_the_baseline_workloads():
    """wmmae_tcec_sgemm_path needs no GPU: the batched 256^3 products and the K-heavy
    product (with K slices) take the GEMM kernel that splits the fp32 operands itself,
    4096^3 and 16384^3 packed operands, small batched products and the round-to-nearest
    variant the single kernel; bad arguments are turned down."""
    import ctypes
    from wmma_extension_amd import _lib
    h = _lib.lib()
    out = ctypes.c_int(-1)
    for args, want in (((256, 256, 256, 1024, 0, 0), 3), ((4096, 4096, 4096, 1, 0, 0), 1),
                       ((16384, 16384, 16384, 1, 2, 0), 1), ((1024, 1024, 262144, 1, 0, 0), 4),
                       ((1024, 1024, 262144, 1, 2, 0), 2), ((128, 128, 128, 1024, 0, 0), 0),
                       ((512, 512, 1024, 256, 0, 1), 0), ((512, 512, 1024, 256, 1, 1), 1)):
        assert h.wmmae_tcec_sgemm_path(*args, ctypes.byref(out)) == 0
        assert out.value == want, args
    assert h.wmmae_tcec_sgemm_path(16, 16, 16, 1, 0, 0, None) == -2
    assert h.wmmae_tcec_sgemm_path(-1, 16, 16, 1, 0, 0, ctypes.byref(out)) == -1
    assert h.wmmae_tcec_sgemm_path(16, 16, 16, 1, 9, 0, ctypes.byref(out)) == -1
    assert h.wmmae_tcec_sgemm_path(16, 16, 16, 1, 0, 2, ctypes.byref(out)) == -1


def test_slice_counts_the_estimates_choose():
    """The number of K slices is what the workspace query sizes its planes for (planes of
    m*n*batch floats).  Pinned on the shapes the estimate was checked against on MI355X
    (with no GPU the library plans for 256 compute units): the K-heavy baseline product is
    cut into one slice per XCD, outputs from 1792^2 up are not cut at k = 4096 with two
    terms, small outputs with a short loop are."""
    import ctypes
    from wmma_extension_amd import _lib
    h = _lib.lib()
    h.wmmae_tcec_gemm_packed_workspace_bytes.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_size_t)]
    def planes(policy, m, n, k, batch=1):
        out = ctypes.c_size_t(0)
        assert h.wmmae_tcec_gemm_packed_workspace_bytes(policy, m, n, k, batch, ctypes.byref(out)) == 0
        assert out.value % (m * n * batch * 4) == 0
        return out.value // (m * n * batch * 4)
    assert planes(0, 1024, 1024, 262144) == 8
    assert planes(2, 1024, 1024, 262144) == 8    # three terms: 256x128 tiles too, one slice per XCD
    # room for the larger of the two kernels' plans: four slices of 128x128 tiles on packed
    # operands, eight for the kernel that splits the fp32 operands itself (32 tiles of 256x128)
    assert planes(0, 1024, 1024, 4096) == 8
    assert planes(2, 1024, 1024, 4096) == 4      # three terms: packed operands only
    assert planes(0, 1280, 1280, 4096) == 5      # 250 tiles of 256x128: one round
    assert planes(0, 512, 512, 1024) == 5
    assert planes(0, 1000, 900, 50000, 2) == 4
    out = ctypes.c_int(-1)
    for shape in ((1792, 1792, 4096), (2048, 2048, 2048)):
        assert h.wmmae_tcec_sgemm_path(*shape, 1, 0, 0, ctypes.byref(out)) == 0 and out.value == 1, shape


def test_k_slice_query_and_hook(h):
    """The slice count per path, and the hook that fixes it for the calling thread: the forced
    count is canonical (no empty slices), at most 32, at least six stages a slice, shows in the
    workspace query, and 0 hands the choice back to the estimates."""
    out = ctypes.c_int(-1)
    ws = ctypes.c_size_t(0)
    def slices(m, n, k, batch, policy, flags):
        assert h.wmmae_tcec_sgemm_k_slices(m, n, k, batch, policy, flags, ctypes.byref(out)) == 0
        return out.value
    PACKED, FUSED, DIRECT = 2, 4, 8
    assert slices(1024, 1024, 4096, 1, 0, PACKED) == 4 and slices(1024, 1024, 4096, 1, 0, DIRECT) == 8
    assert slices(1024, 1024, 4096, 1, 0, FUSED) == 1
    assert slices(1024, 1024, 262144, 1, 0, 0) == 8 and slices(4096, 4096, 4096, 1, 0, 0) == 1
    assert slices(0, 16, 16, 1, 0, 0) == 1
    assert h.wmmae_tcec_sgemm_k_slices(64, 64, 64, 1, 2, DIRECT, ctypes.byref(out)) == -4   # three terms
    assert h.wmmae_tcec_sgemm_k_slices(64, 64, 64, 1, 0, 16, ctypes.byref(out)) == -1
    assert h.wmmae_tcec_sgemm_k_slices(64, 64, 64, 1, 0, 0, None) == -2
    try:
        assert h.wmmae_tcec_force_k_slices(5) == 0
        assert slices(4096, 4096, 4096, 1, 0, PACKED) == 5 and slices(4096, 4096, 4096, 1, 0, DIRECT) == 5
        h.wmmae_tcec_gemm_packed_workspace_bytes.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_size_t)]
        assert h.wmmae_tcec_gemm_packed_workspace_bytes(0, 512, 512, 4096, 1, ctypes.byref(ws)) == 0
        assert ws.value == 5 * 512 * 512 * 4
        assert slices(512, 512, 32 * 33, 1, 0, PACKED) == 5       # 33 stages: 7 7 7 7 5
        assert slices(512, 512, 32 * 35, 1, 0, PACKED) == 5
        assert slices(512, 512, 32 * 29, 1, 0, PACKED) == 4       # at least six stages a slice
        assert slices(512, 512, 64, 1, 0, PACKED) == 1
        assert h.wmmae_tcec_force_k_slices(7) == 0
        assert slices(512, 512, 32 * 48, 1, 0, PACKED) == 7       # 7 7 7 7 7 7 6
        assert slices(512, 512, 32 * 45, 1, 0, PACKED) == 7
        assert h.wmmae_tcec_force_k_slices(24) == 0
        assert slices(512, 512, 32 * 150, 1, 0, PACKED) == 22     # 7 stages a slice: 22 slices, no empty one
        assert h.wmmae_tcec_force_k_slices(100) == 0
        assert slices(512, 512, 1 << 20, 1, 0, DIRECT) == 32
        assert h.wmmae_tcec_force_k_slices(-1) == -1
    finally:
        assert h.wmmae_tcec_force_k_slices(0) == 0
    assert slices(4096, 4096, 4096, 1, 0, PACKED) == 1
    # the hook belongs to the thread that set it
    import threading
    seen = []
    assert h.wmmae_tcec_force_k_slices(3) == 0
    t = threading.Thread(target=lambda: seen.append(slices(4096, 4096, 4096, 1, 0, PACKED)))
    t.start(); t.join()
    assert seen == [1] and slices(4096, 4096, 4096, 1, 0, PACKED) == 3
    assert h.wmmae_tcec_force_k_slices(0) == 0


def test_path_query_is_the_smallest_estimate(h):
    """wmmae_tcec_path_estimates exposes what the driver chooses with: the path reported by
    wmmae_tcec_sgemm_path is the one with the smallest estimate (each estimate no smaller than
    the time the host needs to issue that path's launches: 11, 14.3 and 11.5 us); a path the
    product cannot take has infinity; estimates grow with the work."""
    import math
    import random
    est = (ctypes.c_double * 3)()
    out = ctypes.c_int(-1)
    rnd = random.Random(7)
    floors = (11.0e-6, 14.3e-6, 11.5e-6)
    seen = set()
    for _ in range(400):
        m, n = int(2 ** rnd.uniform(3, 12.5)), int(2 ** rnd.uniform(3, 12.5))
        k, batch, policy = int(2 ** rnd.uniform(2, 15)), rnd.choice([1, 1, 2, 8, 64, 256]), rnd.randrange(5)
        assert h.wmmae_tcec_path_estimates(m, n, k, batch, policy, est) == 0
        e = [max(x, f) for x, f in zip(est, floors)]
        assert all(x > 0 for x in est)
        terms = {0: 2, 1: 1, 2: 3, 3: 2, 4: 1}[policy]
        assert math.isinf(est[2]) == (terms == 3 or k < 4)           # the direct kernel: at most two terms, k >= 4
        assert math.isinf(est[0]) == (k % 4 != 0 and k > 96)          # the single kernel wants 16-byte requests
        assert not math.isinf(est[1])
        assert h.wmmae_tcec_sgemm_path(m, n, k, batch, policy, 0, ctypes.byref(out)) == 0
        best = min(range(3), key=lambda i: (e[i], (1, 0, 2)[i]))      # ties go to packed, then fused
        assert {0: 0, 1: 1, 2: 1, 3: 2, 4: 2}[out.value] == best, (m, n, k, batch, policy, list(est), out.value)
        seen.add(best)
        # four times the entries: the two GEMM-kernel paths do not get faster (the single kernel's
        # estimate has a step where the products stop being cut into K slices)
        more = (ctypes.c_double * 3)()
        assert h.wmmae_tcec_path_estimates(m, n, k, 4 * batch, policy, more) == 0
        assert all(b >= a * 0.999 or math.isinf(a) for a, b in list(zip(est, more))[1:]), (m, n, k, batch, policy)
    assert seen == {0, 1, 2}
    assert h.wmmae_tcec_path_estimates(0, 16, 16, 1, 0, est) == -1
    assert h.wmmae_tcec_path_estimates(16, 16, 16, 1, 7, est) == -1
    assert h.wmmae_tcec_path_estimates(16, 16, 16, 1, 0, None) == -2


def test_direct_kernel_reads_stay_inside_their_rows(h):
    """The GEMM kernel that loads the fp32 operands itself reads 16 bytes per lane and stage.  For
    every k from 4 on, every stage and every lane, the four floats lie inside the row of k floats
    (address arithmetic evaluated on the host from the kernel's own functions): rows may end at
    an allocation's last float."""
    first = ctypes.c_longlong(0)
    for k in list(range(4, 200)) + [999, 1000, 1001, 4100, 16387, 100003]:
        stages = (k + 31) // 32
        for tail in ((1,) if k % 32 else (0, 1)):
            for stage in sorted({0, 1, stages // 2, stages - 2, stages - 1} & set(range(stages))):
                seen = set()
                for lane in range(64):
                    assert h.wmmae_direct_read_first(tail, k, stage, lane, ctypes.byref(first)) == 0
                    f = first.value
                    assert 0 <= f and f + 4 <= k, (k, tail, stage, lane, f)
                    seen.update(range(f, f + 4))
                # together the lanes of a row cover the stage's part of the row
                assert seen >= set(range(32 * stage, min(k, 32 * stage + 32))), (k, tail, stage)
    assert h.wmmae_direct_read_first(1, 3, 0, 0, ctypes.byref(first)) == -1
    assert h.wmmae_direct_read_first(0, 33, 0, 0, ctypes.byref(first)) == -1
    assert h.wmmae_direct_read_first(1, 33, 2, 0, ctypes.byref(first)) == -1
    assert h.wmmae_direct_read_first(1, 33, 0, 64, ctypes.byref(first)) == -1
    assert h.wmmae_direct_read_first(1, 33, 0, 0, None) == -2
