"""Pins the oracle's TCEC emulator and reference GEMM loops (CPU only)."""
import os

import numpy as np
import pytest

KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "primitive_kat.npz"))
KINDS = [0, 1, 2]


def _uniform(rng, *shape):
    return rng.uniform(-1, 1, shape).astype(np.float32)


def test_reference_loops_match_numpy(orc):
    rng = np.random.default_rng(0)
    A, B = _uniform(rng, 37, 53), _uniform(rng, 53, 29)
    assert np.array_equal(orc.gemm_f64(A, B), A.astype(np.float64) @ B.astype(np.float64)) or \
        np.abs(orc.gemm_f64(A, B) - A.astype(np.float64) @ B.astype(np.float64)).max() < 1e-13
    # fp32 loop: k ascending, product and sum rounded separately
    ref = np.zeros((37, 29), dtype=np.float32)
    for l in range(53):
        ref = (ref + (A[:, l:l + 1] * B[l:l + 1, :]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(orc.gemm_f32(A, B), ref)
    # column-major inputs give the same numbers
    assert np.array_equal(orc.gemm_f32(np.asfortranarray(A), np.asfortranarray(B)), ref)
    assert np.array_equal(orc.gemm_f32_tn(A, np.ascontiguousarray(B.T)).T, ref) or \
        orc.max_rel_err(orc.gemm_f32_tn(A, np.ascontiguousarray(B.T)).T, ref.astype(np.float64)) < 1e-6


def test_error_metrics(orc):
    ref = np.array([1.0, -4.0, 2.0])
    x = np.array([1.5, -4.0, 2.0], dtype=np.float32)
    assert orc.max_abs_err(x, ref) == 0.5
    assert orc.max_rel_err(x, ref) == 0.5 / 4.0
    assert abs(orc.frobenius_residual(x, ref) - 0.5 / np.sqrt(21.0)) < 1e-15


@pytest.mark.parametrize("kind", KINDS)
def test_identity_b_returns_the_split_sum(orc, kind):
    """B = I: every output is hi + lo/scale of the matching A element, exactly."""
    rng = np.random.default_rng(1)
    A = _uniform(rng, 32, 32)
    D = orc.tcec_matmul(A, np.eye(32, dtype=np.float32), kind=kind, ec=True)
    terms = [orc.terms_to_f32(kind, t) for t in orc.split(kind, A)]
    if kind == 0:
        expect = (terms[0] + terms[1] / np.float32(2048)).astype(np.float32)
    else:
        # error part accumulates smallest term first: (lo + mid) then + hi
        err = terms[1] if len(terms) == 2 else (terms[2] + terms[1]).astype(np.float32)
        expect = (terms[0] + err).astype(np.float32)
    assert np.array_equal(D, expect)
    D0 = orc.tcec_matmul(A, np.eye(32, dtype=np.float32), kind=kind, ec=False)
    assert np.array_equal(D0, terms[0])


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("main_outside", [True, False])
def test_exactly_representable_inputs_are_exact(orc, kind, main_outside):
    """Small integers times powers of two: every partial sum is exact, so the
    emulator must equal the exact product whatever the accumulation order."""
    rng = np.random.default_rng(2)
    A = (rng.integers(-8, 9, (32, 64)) * 0.25).astype(np.float32)
    B = (rng.integers(-8, 9, (64, 16)) * 0.5).astype(np.float32)
    C = rng.integers(-100, 100, (32, 16)).astype(np.float32)
    exact = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float32)
    for ec in (True, False):
        D = orc.tcec_matmul(A, B, C, kind=kind, ec=ec, main_outside=main_outside)
        assert np.array_equal(D, exact)


def test_without_ec_equals_gemm_of_rounded_inputs(orc):
    rng = np.random.default_rng(3)
    A, B = _uniform(rng, 32, 32), _uniform(rng, 32, 32)
    A16 = A.astype(np.float16).astype(np.float32)
    B16 = B.astype(np.float16).astype(np.float32)
    D = orc.tcec_matmul(A, B, kind=0, ec=False, fk=32)
    exact = A16.astype(np.float64) @ B16.astype(np.float64)
    assert np.array_equal(D, exact.astype(np.float32))   # one k block: a single rounding


def test_reference_accuracy_gates(orc):
    """N = 32, uniform[-1,1]: with_ec < 1e-5, without_ec < 1e-2 in max abs error
    (test/tcec/mma.cu:5-21), and with_ec no worse than 2x plain fp32."""
    rng = np.random.default_rng(4)
    worst = {True: 0.0, False: 0.0}
    for _ in range(20):
        A, B, C = _uniform(rng, 32, 32), _uniform(rng, 32, 32), _uniform(rng, 32, 32)
        ref = orc.gemm_f64(A, B) + C
        for ec in (True, False):
            for kind in (0, 2):
                D = orc.tcec_matmul(A, B, C, kind=kind, ec=ec)
                e = orc.max_abs_err(D, ref)
                if not (kind == 2 and not ec):
                    worst[ec] = max(worst[ec], e)
        e32 = orc.max_abs_err((orc.gemm_f32(A, B) + C).astype(np.float32), ref)
        assert orc.max_abs_err(orc.tcec_matmul(A, B, C, kind=0, ec=True), ref) <= 2 * e32
    assert worst[True] < float(KAT["threshold_with_ec"])
    assert 1e-5 < worst[False] < float(KAT["threshold_without_ec"])


def test_dropped_term_would_be_caught(orc):
    """The gates above are sharp enough: a split with the correction left out,
    or with the scale forgotten, is far outside them."""
    rng = np.random.default_rng(5)
    A, B = _uniform(rng, 32, 32), _uniform(rng, 32, 32)
    ref = orc.gemm_f64(A, B)
    hi_a, lo_a = [orc.terms_to_f32(0, t).astype(np.float64) for t in orc.split(0, A)]
    hi_b, lo_b = [orc.terms_to_f32(0, t).astype(np.float64) for t in orc.split(0, B)]
    one_sided = hi_a @ hi_b + (lo_a @ hi_b) / 2048            # a0*b1 dropped
    unscaled = hi_a @ hi_b + (lo_a @ hi_b + hi_a @ lo_b)       # /2048 forgotten
    assert np.abs(one_sided - ref).max() > 1e-5
    assert np.abs(unscaled - ref).max() > 1e-2
    full = hi_a @ hi_b + (lo_a @ hi_b + hi_a @ lo_b) / 2048
    assert np.abs(full - ref).max() < 1e-6


def test_batch_gemm_ramp_fixture(orc):
    """The deterministic ramps of the reference's GEMM harness
    (test/tcec/batch_gemm.cu:507-513) against its FP64 loop."""
    m = n = k = 64
    A = KAT["bgemm_a"].reshape(m, k)          # row-major m x k
    Bt = KAT["bgemm_b"].reshape(n, k)         # column-major k x n
    ref = KAT["bgemm_c64"]
    assert np.allclose(orc.gemm_f64(A, Bt.T), ref, rtol=1e-15)
    D = orc.tcec_matmul(A, Bt.T, kind=2, ec=True)
    assert orc.frobenius_residual(D, ref) < 2e-7
    # the ramps reach 64: fine for fp16 (max 65504) too
    D = orc.tcec_matmul(A, Bt.T, kind=0, ec=True)
    assert orc.frobenius_residual(D, ref) < 2e-7
