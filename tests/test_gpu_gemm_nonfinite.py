"""NaN, infinities and values outside the 16-bit terms' range through the GEMM driver.

The split is the reference's (tcec/tcec.hpp:219-223 with tcec/detail/scale.hpp:8-20): the
leading term is the operand rounded to fp16 / bf16, so an operand the 16-bit type cannot hold
becomes an infinity there and its residual term an infinity of the other sign or a NaN - the
reference has the same limit (it casts with the same rounding and no range check).  What a
caller sees, for every policy and every path of the driver:

  * C(i, :) is non-finite for every row i of op(A) that holds a NaN, an infinity or a value
    that overflows the policy's 16-bit type, C(:, j) likewise for the columns of op(B);
  * every other element of C is what the same product gives without those values
    (one row / column never leaks into another);
  * beta == 0 never reads C, so NaNs already in C do not survive.

Overflow thresholds: fp16 terms round |v| >= 65520 to infinity; bf16 terms |v| >= 3.3962e38
(the fp32 values above bf16's largest finite number plus half a step).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8
F16_POLICIES = (0, 1)


def _planted(rng, m, n, k):
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    rows = {"nan": 3, "inf": m // 2, "over_f16": m - 2, "over_bf16": 17}
    cols = {"ninf": 5, "over_f16": n - 1}
    A[rows["nan"], 7 % k] = np.nan
    A[rows["inf"], k - 1] = np.inf
    A[rows["over_f16"], k // 3] = 70000.0
    A[rows["over_bf16"], 0] = 3.4e38
    B[k // 2, cols["ninf"]] = -np.inf
    B[1 % k, cols["over_f16"]] = -1.0e5
    return A, B, rows, cols


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(200, 136, 328), (300, 260, 96), (1100, 520, 1000)])
def test_nonfinite_operands_stay_in_their_rows_and_columns(tc, orc, dev, policy, shape):
    from wmma_extension_amd._lib import WmmaeError
    m, n, k = shape
    rng = np.random.default_rng(1234 + policy)
    A, B, rows, cols = _planted(rng, m, n, k)
    f16 = policy in F16_POLICIES
    bad_rows = [rows["nan"], rows["inf"], rows["over_bf16"]] + ([rows["over_f16"]] if f16 else [])
    bad_cols = [cols["ninf"]] + ([cols["over_f16"]] if f16 else [])
    good_r = np.setdiff1d(np.arange(m), bad_rows)
    good_c = np.setdiff1d(np.arange(n), bad_cols)
    ref = orc.gemm_f64(A[good_r], B[:, good_c])
    e32 = orc.max_rel_err(orc.gemm_f32(A[good_r], B[:, good_c]), ref)
    tol = {0: 2 * e32 + 2.0**-21, 2: 2 * e32 + 2.0**-21, 3: 2.0**-14, 1: 2.0**-9, 4: 2.0**-6}[policy]

    dA = torch.from_numpy(A).to(dev)                       # op(A) = 'T': m rows of k floats
    dB = torch.from_numpy(np.ascontiguousarray(B.T)).to(dev)
    ran = []
    for flags in (0, PACKED, FUSED, DIRECT):
        dC = torch.full((n, m), float("nan"), dtype=torch.float32, device=dev)   # beta = 0
        ws = torch.empty(tc.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
        try:
            tc.sgemm("T", "N", m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m, policy, flags, ws)
        except WmmaeError as e:
            assert e.status == -4 and flags == DIRECT      # three terms: no direct kernel
            continue
        torch.cuda.synchronize()
        D = dC.cpu().numpy().T
        ran.append(flags)
        for i in bad_rows:
            assert not np.isfinite(D[i, :]).any(), (flags, "row", i)
        for j in bad_cols:
            assert not np.isfinite(D[:, j]).any(), (flags, "col", j)
        clean = D[np.ix_(good_r, good_c)]
        assert np.isfinite(clean).all(), flags
        assert orc.max_rel_err(clean, ref) <= tol, (flags, orc.max_rel_err(clean, ref), tol)
        if flags != 0 and (m, n, k) != (1100, 520, 1000):
            # the oracle's model of the matrix core takes infinities and NaNs as the hardware does:
            # element by element the same class, and the same bits where finite
            kind, ec = {0: (0, True), 1: (0, False), 2: (2, True), 3: (1, True), 4: (1, False)}[policy]
            emu = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
            assert np.array_equal(np.isnan(D), np.isnan(emu)) and np.array_equal(np.isinf(D), np.isinf(emu)), flags
            fin = np.isfinite(emu)
            assert np.array_equal(D[fin].view(np.uint32), emu[fin].view(np.uint32)), flags
    assert 0 in ran and PACKED in ran and FUSED in ran


def test_values_inside_the_range_of_the_terms_are_finite(tc, orc, dev):
    """The largest operands each policy carries: 65504 for the fp16 split, bf16's largest
    finite value for the bf16 splits (products kept inside fp32's range by a small B)."""
    m, n, k = 64, 64, 64
    rng = np.random.default_rng(9)
    for policy, big in ((0, 65504.0), (1, 65504.0), (2, 3.3895e38), (3, 3.3895e38), (4, 3.3895e38)):
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = (rng.uniform(-1, 1, (k, n)) * (1.0 if policy < 2 else 2.0**-20)).astype(np.float32)
        A[5, 9] = big
        A[6, 1] = -big
        dA = torch.from_numpy(A).to(dev)
        dB = torch.from_numpy(np.ascontiguousarray(B.T)).to(dev)
        dC = torch.empty((n, m), dtype=torch.float32, device=dev)
        tc.sgemm("T", "N", m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m, policy)
        torch.cuda.synchronize()
        D = dC.cpu().numpy().T
        assert np.isfinite(D).all(), policy
        ref = orc.gemm_f64(A, B)
        assert orc.max_rel_err(D, ref) <= (2.0**-18 if policy in (0, 2) else 2.0**-6), policy
