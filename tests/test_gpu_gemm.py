"""The TCEC SGEMM driver (C-ABI) against the CPU oracle: FP64 loop, TCEC
emulator, plain fp32 comparator, and size-independent properties."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

POL_KIND = {0: (0, True), 1: (0, False), 2: (2, True), 3: (1, True), 4: (1, False)}


def _gemm(tc, dev, A, B, policy, alpha=1.0, beta=0.0, C=None, ta="T", tb="N", flags=0,
          workspace=None, ld_pad=0):
    """A (m,k), B (k,n) numpy -> C (m,n) numpy, through wmmae_tcec_sgemm.
    ta/tb choose how the operands are laid out in device memory (BLAS, column major)."""
    m, k = A.shape
    n = B.shape[1]
    # column-major storage of op(A): 'N' -> m x k col-major (= A.T C-order), 'T' -> k x m col-major (= A C-order)
    a_store = A.T if ta == "N" else A
    b_store = B.T if tb == "N" else B
    lda = max(1, a_store.shape[1]) + ld_pad
    ldb = max(1, b_store.shape[1]) + ld_pad
    ldc = m + ld_pad

    def dev_padded(x, ld):
        buf = torch.zeros((x.shape[0], ld), dtype=torch.float32, device=dev)
        buf[:, :x.shape[1]] = torch.from_numpy(np.ascontiguousarray(x)).to(dev)
        return buf
    dA, dB = dev_padded(a_store, lda), dev_padded(b_store, ldb)
    dC = torch.full((n, ldc), 777.0, dtype=torch.float32, device=dev)
    if C is not None:
        dC[:, :m] = torch.from_numpy(np.ascontiguousarray(C.T)).to(dev)
    tc.sgemm(ta, tb, m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc, policy, flags, workspace)
    torch.cuda.synchronize()
    out = dC.cpu().numpy()
    if ld_pad:
        assert (out[:, m:] == 777.0).all()          # padding untouched
    return out[:, :m].T.copy()


def _check(orc, D, A, B, policy, ref=None, C=None, alpha=1.0, beta=0.0):
    kind, ec = POL_KIND[policy]
    ref = (alpha * orc.gemm_f64(A, B) + (beta * C if C is not None else 0)) if ref is None else ref
    err = orc.max_rel_err(D, ref)
    e32 = orc.max_rel_err((alpha * orc.gemm_f32(A, B) + (beta * C if C is not None else 0))
                          .astype(np.float32), ref)
    k = A.shape[1]
    if ec and kind != 1:
        # gate: no worse than 2x plain fp32 SGEMM on the same inputs.  For short
        # sums fp32 itself is nearly exact and the split's own resolution
        # (2^-22 per product) is what is left, so that floor is allowed there.
        assert err <= 2 * e32 + (0.0 if k >= 256 else 2.0**-21), (err, e32)
    elif ec:
        assert err <= 2.0**-14
    else:
        assert err <= (2.0**-9 if kind == 0 else 2.0**-6)
    return err, e32


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("mnk", [(128, 128, 128), (256, 128, 64), (64, 64, 32), (512, 256, 160),
                                 (1024, 640, 96)])
def test_sgemm_aligned_shapes(tc, orc, dev, policy, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(m + n + k + policy)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    D = _gemm(tc, dev, A, B, policy)
    _check(orc, D, A, B, policy)
    kind, ec = POL_KIND[policy]
    # the driver's instruction sequence per output element (32 of k per step, error products
    # before the leading one, everything chained through the matrix core) in the oracle's
    # model of that core: same bits
    emu = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
    assert np.array_equal(D.view(np.uint32), emu.view(np.uint32)), np.abs(D - emu).max()


def _random_patterns(rng, shape, emin, emax, zeros=0.02):
    """fp32 values with uniformly drawn sign, exponent (emin .. emax) and mantissa bits."""
    e = rng.integers(emin, emax + 1, shape)
    bits = ((rng.integers(0, 2, shape).astype(np.uint32) << 31) | ((e + 127).astype(np.uint32) << 23)
            | rng.integers(0, 1 << 23, shape).astype(np.uint32))
    v = bits.view(np.float32).copy()
    v[rng.random(shape) < zeros] = 0.0
    return v


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("regime", ["wide", "tiny_a", "subnormal_a", "huge"])
def test_sgemm_wide_exponent_range_same_bits_as_the_model(tc, orc, dev, policy, regime):
    """Operands far from [-1, 1]: exponents over the whole range a policy's 16-bit type holds
    (and past it: fp16 terms of values above 65504 are infinities), operands whose terms are
    subnormal in that type, and fp32 subnormals - where residual terms underflow and sums end
    below 2^-126 - and bf16 operands of 2^56 .. 2^63, whose sums leave fp32's range.  The packed,
    the single-kernel and the direct path give the bits of the oracle's model of the matrix core
    there too, infinities and NaNs in the same places."""
    from wmma_extension_amd._lib import WmmaeError
    kind, ec = POL_KIND[policy]
    f16 = kind == 0
    if regime == "huge" and f16:
        pytest.skip("fp16 terms of such operands are infinities: tests/test_gpu_gemm_nonfinite.py")
    for (m, n, k) in ((200, 136, 328), (64, 64, 32)):
        rng = np.random.default_rng(1000 + 10 * policy + m + len(regime))
        if regime == "huge":
            # products up to 2^127 and sums beyond fp32's range: infinities and NaNs where the
            # model has them
            A, B = _random_patterns(rng, (m, k), 56, 63), _random_patterns(rng, (k, n), 56, 63)
        elif regime == "wide":
            lo, hi = (-40, 15) if f16 else (-60, 60)
            A, B = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (k, n), lo, hi)
        elif regime == "tiny_a":
            lo, hi = (-30, -10) if f16 else (-126, -100)
            A, B = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (k, n), -3, 3)
        else:
            A = (rng.integers(0, 1 << 24, (m, k)).astype(np.uint32)
                 | (rng.integers(0, 2, (m, k)).astype(np.uint32) << 31)).view(np.float32)
            B = _random_patterns(rng, (k, n), -3, 3)
        emu = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
        ran = 0
        for flag in (2, 4, 8):
            try:
                D = _gemm(tc, dev, A, B, policy, flags=flag)
            except WmmaeError as e:
                assert flag == 8 and e.status == -4 and policy == 2, (flag, e)   # direct: one or two terms
                continue
            ran += 1
            fin = np.isfinite(emu)
            assert np.array_equal(np.isnan(D), np.isnan(emu)) and np.array_equal(np.isinf(D), np.isinf(emu))
            assert np.array_equal(np.signbit(D[~np.isnan(emu)]), np.signbit(emu[~np.isnan(emu)]))
            assert np.array_equal(D[fin].view(np.uint32), emu[fin].view(np.uint32)), \
                (policy, regime, (m, n, k), flag, int((D[fin].view(np.uint32) != emu[fin].view(np.uint32)).sum()))
        assert ran >= 2
        if regime == "subnormal_a" and not f16:
            assert (np.abs(emu) < 2.0 ** -110).all() and (emu != 0).mean() > 0.9   # sums around 2^-126 and below


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("mnk", [(200, 136, 328), (512, 256, 160), (520, 392, 1000), (64, 64, 32)])
def test_sgemm_rn_main_flag_same_bits_as_the_model(tc, orc, dev, policy, mnk):
    """WMMAE_FLAG_RN_MAIN: the leading product of every 32 of k starts from zero on the matrix
    core and is added with an fp32 add outside it (the reference's mma_rn_sync,
    tcec/tcec.hpp:673-694); the error products stay chained.  The oracle's model in that order
    gives the bits, on the packed path, the single kernel and the library's choice, with alpha
    and beta too."""
    m, n, k = mnk
    kind, ec = POL_KIND[policy]
    rng = np.random.default_rng(m + 3 * n + k + policy)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    emu = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=True, hw_model=True)
    chained = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
    if k > 32:
        assert not np.array_equal(emu, chained)                  # the flag does change the bits
    for path_flag in (0, 2, 4):
        if tc.sgemm_k_slices(m, n, k, 1, policy, 1 | path_flag) > 1:
            continue
        D = _gemm(tc, dev, A, B, policy, flags=1 | path_flag)
        assert np.array_equal(D.view(np.uint32), emu.view(np.uint32)), (path_flag, int((D != emu).sum()))
        D = _gemm(tc, dev, A, B, policy, alpha=-0.75, beta=1.5, C=C, flags=1 | path_flag)
        assert np.array_equal(D.view(np.uint32), orc.epilogue(emu, -0.75, 1.5, C).view(np.uint32)), path_flag


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (17, 5, 3), (100, 37, 77), (129, 255, 33), (300, 200, 100),
                                 (16, 16, 1000), (1000, 3, 8), (700, 37, 77), (130, 1031, 45)])
def test_sgemm_ragged_shapes(tc, orc, dev, policy, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(m * 7 + n * 3 + k + policy)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    for ld_pad in (0, 3):
        D = _gemm(tc, dev, A, B, policy, ld_pad=ld_pad)
        _check(orc, D, A, B, policy)


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("trans", ["NN", "NT", "TN", "TT"])
def test_sgemm_transposes_alpha_beta(tc, orc, dev, policy, trans):
    m, n, k = 96, 80, 72
    rng = np.random.default_rng(ord(trans[0]) + 2 * ord(trans[1]) + policy)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    base = _gemm(tc, dev, A, B, policy, ta="T", tb="N")
    D = _gemm(tc, dev, A, B, policy, ta=trans[0], tb=trans[1])
    assert np.array_equal(D, base)               # the layout of the inputs does not change a bit
    D = _gemm(tc, dev, A, B, policy, alpha=-1.5, beta=0.75, C=C, ta=trans[0], tb=trans[1], ld_pad=4)
    expect = (np.float32(-1.5) * base + np.float32(0.75) * C).astype(np.float32)
    assert np.abs(D - expect).max() <= 2.0**-22 * np.abs(expect).max()
    # beta == 0 must not read C (NaN in C stays out)
    D = _gemm(tc, dev, A, B, policy, alpha=1.0, beta=0.0, C=np.full((m, n), np.nan, np.float32),
              ta=trans[0], tb=trans[1])
    assert np.array_equal(D, base)


def test_sgemm_k_zero_and_workspace(tc, orc, dev):
    m, n = 20, 12
    C = np.arange(m * n, dtype=np.float32).reshape(m, n)
    D = _gemm(tc, dev, np.zeros((m, 0), np.float32), np.zeros((0, n), np.float32), 0,
              alpha=1.0, beta=2.0, C=C)
    assert np.array_equal(D, 2 * C)
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, (64, 64)).astype(np.float32)
    B = rng.uniform(-1, 1, (64, 64)).astype(np.float32)
    ws = torch.empty(tc.workspace_bytes(64, 64, 64), dtype=torch.uint8, device=dev)
    assert np.array_equal(_gemm(tc, dev, A, B, 0, workspace=ws), _gemm(tc, dev, A, B, 0))
    # products that go through packed operands (a K-heavy one with K slices, a large one
    # without) need room for them
    from wmma_extension_amd._lib import WmmaeError
    small = torch.empty(16, dtype=torch.uint8, device=dev)
    for (m, n, k), path in (((128, 128, 8192), tc.PATH_PACKED_SPLIT_K), ((3072, 3072, 3072), tc.PATH_PACKED)):
        assert tc.sgemm_path(m, n, k) == path
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        ws = torch.empty(tc.workspace_bytes(m, n, k), dtype=torch.uint8, device=dev)
        assert np.array_equal(_gemm(tc, dev, A, B, 0, workspace=ws), _gemm(tc, dev, A, B, 0))
        with pytest.raises(WmmaeError) as e:
            _gemm(tc, dev, A, B, 0, workspace=small)
        assert e.value.status == -5


@pytest.mark.parametrize("policy", [0, 2])
def test_sgemm_exact_inputs_bit_exact(tc, orc, dev, policy):
    """Small dyadic inputs: all partial sums exact -> result equals the exact product
    whatever the tiling, for every tile configuration the dispatcher can choose."""
    rng = np.random.default_rng(8)
    for m, n, k in ((64, 64, 64), (256, 256, 96), (2048, 4096, 64)):
        A = (rng.integers(-8, 9, (m, k)) * 0.25).astype(np.float32)
        B = (rng.integers(-8, 9, (k, n)) * 0.5).astype(np.float32)
        D = _gemm(tc, dev, A, B, policy)
        assert np.array_equal(D, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


@pytest.mark.parametrize("policy", [0, 2])
def test_sgemm_identity_and_scaling_properties(tc, orc, dev, policy):
    """B = I reproduces A to the split's resolution; scaling an operand by a power
    of two scales the result exactly (size independent properties)."""
    rng = np.random.default_rng(12)
    n = 512
    A = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    I = np.eye(n, dtype=np.float32)
    D = _gemm(tc, dev, A, I, policy)
    kind, _ = POL_KIND[policy]
    assert np.array_equal(D, orc.tcec_matmul(A, I, kind=kind, ec=True))
    assert np.abs(D - A).max() <= 2.0**-21
    # magnitudes in [2^-4, 1): scaling by 4 and 0.5 keeps every fp16 term normal,
    # so the split commutes with the scaling and the result scales exactly
    A = (rng.uniform(2.0**-4, 1, (n, n)) * rng.choice([-1, 1], (n, n))).astype(np.float32)
    B = (rng.uniform(2.0**-4, 1, (n, n)) * rng.choice([-1, 1], (n, n))).astype(np.float32)
    D1 = _gemm(tc, dev, A, B, policy)
    D2 = _gemm(tc, dev, (A * np.float32(4)).astype(np.float32), (B * np.float32(0.5)).astype(np.float32), policy)
    assert np.array_equal(D2, D1 * np.float32(2))


def test_strided_batched(tc, orc, dev):
    """Independent 64^3 products, N(0,1) entries, reference layout (T,N)."""
    batch, m, n, k = 5, 64, 48, 80
    rng = np.random.default_rng(33)
    A = rng.standard_normal((batch, m, k)).astype(np.float32)
    Bt = rng.standard_normal((batch, n, k)).astype(np.float32)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(Bt).to(dev)
    dC = torch.zeros((batch, n, m), dtype=torch.float32, device=dev)
    for policy in (0, 2):
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, dA, k, m * k, dB, k, n * k, 0.0,
                                 dC, m, n * m, batch, policy)
        torch.cuda.synchronize()
        out = dC.cpu().numpy()
        for b in range(batch):
            _check(orc, out[b].T, A[b], Bt[b].T, policy)


def test_pack_then_gemm_reuses_operands(tc, orc, dev):
    m, n, k = 128, 64, 96
    rng = np.random.default_rng(44)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    Bt = rng.uniform(-1, 1, (n, k)).astype(np.float32)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(Bt).to(dev)
    pa = torch.empty(tc.pack_bytes(m, k), dtype=torch.uint8, device=dev)
    pb = torch.empty(tc.pack_bytes(n, k), dtype=torch.uint8, device=dev)
    tc.pack(0, m, k, dA, k, 1, pa)
    tc.pack(0, n, k, dB, k, 1, pb)
    dC = torch.zeros((n, m), dtype=torch.float32, device=dev)
    tc.gemm_packed(0, m, n, k, 1.0, pa, pb, 0.0, dC, m)
    torch.cuda.synchronize()
    assert np.array_equal(dC.cpu().numpy().T, _gemm(tc, dev, A, Bt.T, 0))
    # packed operand bytes: lane l of chunk (rb,kt,term) holds row 16*rb + l%16, k 32*kt+8*(l/16)..+7
    terms = orc.split(0, A)
    raw = pa.cpu().numpy().view(np.uint16).reshape(m // 16, -1, 2, 64, 8)
    KT = raw.shape[1]
    for rb, kt, t, lane in ((0, 0, 0, 0), (3, 1, 1, 37), (7, 2, 0, 63)):
        r, k0 = 16 * rb + lane % 16, 32 * kt + 8 * (lane // 16)
        assert np.array_equal(raw[rb, kt, t, lane], terms[t][r, k0:k0 + 8])
    assert KT == 3
    # rows and k beyond the matrix are zero filled
    m2, k2 = 20, 40
    p2 = torch.full((tc.pack_bytes(m2, k2),), 0xFF, dtype=torch.uint8, device=dev)
    tc.pack(0, m2, k2, dA, k, 1, p2)
    raw2 = p2.cpu().numpy().view(np.uint16).reshape(2, 2, 2, 64, 8)
    for rb, kt, lane in ((1, 0, 3), (1, 1, 20), (0, 1, 17), (1, 0, 4)):
        r, k0 = 16 * rb + lane % 16, 32 * kt + 8 * (lane // 16)
        for t in (0, 1):
            exp = np.zeros(8, dtype=np.uint16)
            if r < m2:
                for x in range(8):
                    if k0 + x < k2:
                        exp[x] = terms[t][r, k0 + x]
            assert np.array_equal(raw2[rb, kt, t, lane], exp)


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("trans", ["TN", "NT"])
def test_small_products_split_in_kernel_match_packed_path(tc, orc, dev, policy, trans):
    """Small products are split inside the GEMM kernel (no packed copy in memory; the path
    is forced here, the estimates take it for all of these but the one with k = 77 and three
    terms); the result is bit for bit that of pack + gemm_packed, also with the leading
    product accumulated outside the matrix core (policies that have that variant)."""
    rng = np.random.default_rng(91 + policy)
    rn = 1 if policy in (0, 2) and trans == "NT" else 0
    flags = rn | 4
    for m, n, k in ((64, 64, 64), (40, 24, 50), (256, 256, 256), (500, 130, 77), (512, 512, 33)):
        if (k, policy) != (77, 2):
            assert tc.sgemm_path(m, n, k, 1, policy, rn) == tc.PATH_FUSED
        A = rng.standard_normal((m, k)).astype(np.float32)
        B = rng.standard_normal((k, n)).astype(np.float32)
        C0 = rng.standard_normal((m, n)).astype(np.float32)
        for ld_pad in (0, 1):
            fused = _gemm(tc, dev, A, B, policy, alpha=1.25, beta=-0.5, C=C0, ta=trans[0], tb=trans[1],
                          ld_pad=ld_pad, flags=flags)
            dA = torch.from_numpy(A).to(dev)
            dB = torch.from_numpy(np.ascontiguousarray(B.T)).to(dev)
            pa = torch.empty(tc.pack_bytes(m, k, 1, policy), dtype=torch.uint8, device=dev)
            pb = torch.empty(tc.pack_bytes(n, k, 1, policy), dtype=torch.uint8, device=dev)
            tc.pack(policy, m, k, dA, k, 1, pa)
            tc.pack(policy, n, k, dB, k, 1, pb)
            dC = torch.from_numpy(np.ascontiguousarray(C0.T)).to(dev)
            tc.gemm_packed(policy, m, n, k, 1.25, pa, pb, -0.5, dC, m, flags=rn)
            torch.cuda.synchronize()
            assert np.array_equal(dC.cpu().numpy().T, fused), (m, n, k, ld_pad)
        _check(orc, fused, A, B, policy, C=C0, alpha=1.25, beta=-0.5)


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("mnk", [(64, 64, 8232), (200, 120, 16384), (256, 128, 32768)])
def test_split_k(tc, orc, dev, policy, mnk):
    """K-heavy shapes with few output tiles are cut into K slices (when the caller gives
    workspace for them); with and without the split the result meets the same gates."""
    m, n, k = mnk
    rng = np.random.default_rng(m + k + policy)
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    assert tc.gemm_packed_workspace_bytes(policy, m, n, k) > 0
    ws = torch.empty(tc.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
    C0 = rng.standard_normal((m, n)).astype(np.float32)
    split = _gemm(tc, dev, A, B, policy, alpha=0.5, beta=2.0, C=C0, workspace=ws, ld_pad=1)
    only_pack = torch.empty(tc.pack_bytes(m, k, 1, policy) + tc.pack_bytes(n, k, 1, policy),
                            dtype=torch.uint8, device=dev)
    unsplit = _gemm(tc, dev, A, B, policy, alpha=0.5, beta=2.0, C=C0, workspace=only_pack, ld_pad=1)
    ref = 0.5 * orc.gemm_f64(A, B) + 2.0 * C0
    e32 = orc.max_rel_err((0.5 * orc.gemm_f32(A, B) + 2.0 * C0).astype(np.float32), ref)
    for D in (split, unsplit):
        assert orc.max_rel_err(D, ref) <= 2 * e32
    assert np.abs(split - unsplit).max() <= 4 * e32 * np.abs(ref).max()   # both within the gate of each other
    # library-allocated workspace takes the same path as the explicit one
    assert np.array_equal(_gemm(tc, dev, A, B, policy, alpha=0.5, beta=2.0, C=C0, ld_pad=1), split)


def test_pointer_array_batched(tc, orc, dev):
    """The reference harness's calling convention: device arrays of matrix pointers
    (test/tcec/batch_gemm.cu:433-443), matrices scattered in memory, ramp inputs
    A[j] = j/k, B[j] = j/n of that harness for one entry."""
    batch, m, n, k = 7, 96, 64, 160
    rng = np.random.default_rng(55)
    As = [torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(dev) for _ in range(batch)]
    Bs = [torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).to(dev) for _ in range(batch)]
    As[3] = (torch.arange(m * k, dtype=torch.float32, device=dev) / k).reshape(m, k)
    Bs[3] = (torch.arange(k * n, dtype=torch.float32, device=dev) / n).reshape(n, k)
    Cs = [torch.full((n, m), 3.0, dtype=torch.float32, device=dev) for _ in range(batch)]
    pa = torch.tensor([t.data_ptr() for t in As], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in Bs], dtype=torch.int64, device=dev)
    pc = torch.tensor([t.data_ptr() for t in Cs], dtype=torch.int64, device=dev)
    for policy in (0, 2):
        for c in Cs:
            c.fill_(3.0)
        tc.sgemm_batched("T", "N", m, n, k, 2.0, pa, k, pb, k, -1.0, pc, m, batch, policy)
        torch.cuda.synchronize()
        for b in range(batch):
            a, bt = As[b].cpu().numpy(), Bs[b].cpu().numpy()
            ref = 2.0 * orc.gemm_f64(a, bt.T) - 3.0
            got = Cs[b].cpu().numpy().T
            e32 = orc.max_rel_err((2.0 * orc.gemm_f32(a, bt.T) - 3.0).astype(np.float32), ref)
            assert orc.max_rel_err(got, ref) <= 2 * e32 + 2.0**-21
            single = _gemm(tc, dev, a, bt.T, policy, alpha=2.0, beta=-1.0, C=np.full((m, n), 3.0, np.float32))
            assert np.array_equal(got, single)
        # Frobenius residual of the harness's ramp entry, as batch_gemm.cu:559-605 reports it
        ref3 = orc.gemm_f64(As[3].cpu().numpy(), Bs[3].cpu().numpy().T) * 2.0 - 3.0
        assert orc.frobenius_residual(Cs[3].cpu().numpy().T, ref3) < 3e-7


@pytest.mark.parametrize("type_ec", [(0, 1), (0, 0), (2, 1)])
def test_api_level_gemm_matches_driver(tc, orc, dev, type_ec):
    """A GEMM written only against the public tcec:: API (split at fragment load, as in
    the reference's bgemm_kernel) against the oracle and against the packed driver."""
    type_, ec = type_ec
    policy = {(0, 1): 0, (0, 0): 1, (2, 1): 2}[type_ec]
    m, n, k = 256, 384, 160
    rng = np.random.default_rng(77 + policy)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    Bt = rng.uniform(-1, 1, (n, k)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(Bt).to(dev)
    for alpha, beta in ((1.0, 0.0), (-0.5, 1.5)):
        dC = torch.from_numpy(np.ascontiguousarray(C0.T)).to(dev)
        tc.api_gemm(type_, ec, m, n, k, alpha, dA, k, dB, k, beta, dC, m)
        torch.cuda.synchronize()
        got = dC.cpu().numpy().T
        ref = alpha * orc.gemm_f64(A, Bt.T) + beta * C0
        _check(orc, got, A, Bt.T, policy, ref=ref, C=C0, alpha=alpha, beta=beta)
        # the kernel is tcec::mma_sync over k steps of 32 on a zero accumulator (round-to-nearest
        # adds of the leading product with error correction), then alpha / beta in fp32
        emu = orc.tcec_matmul(A, Bt.T, kind=POL_KIND[policy][0], ec=bool(ec), fk=32,
                              main_outside=bool(ec), hw_model=True)
        if (alpha, beta) == (1.0, 0.0):
            assert np.array_equal(got.view(np.uint32), emu.view(np.uint32)), np.abs(got - emu).max()
        else:
            expect = alpha * emu.astype(np.float64) + beta * C0
            assert (np.abs(got - expect) <= 2 * 2.0**-24 * (np.abs(alpha * emu) + np.abs(beta * C0))).all()
            # ... and exactly: beta * C rounded, then one fused multiply-add of alpha * (hi + lo / 2048)
            assert np.array_equal(got.view(np.uint32), orc.epilogue(emu, alpha, beta, C0, api_form=True).view(np.uint32))
        # the driver chains the leading product through the matrix core instead: two roundings
        # of the same sums
        drv = _gemm(tc, dev, A, Bt.T, policy, alpha=alpha, beta=beta, C=C0)
        assert np.abs(got - drv).max() <= 16 * 2.0**-24 * max(1.0, np.abs(ref).max())
        # the kernel with mma_rn_sync / mma_rz_sync in place of mma_sync: the model in that order
        if (alpha, beta) == (1.0, 0.0):
            for rounding in (1, 2):
                dC = torch.zeros((n, m), dtype=torch.float32, device=dev)
                tc.api_gemm(type_, ec, m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m, rounding=rounding)
                torch.cuda.synchronize()
                emu_r = orc.tcec_matmul(A, Bt.T, kind=POL_KIND[policy][0], ec=bool(ec), fk=32,
                                        main_outside=rounding == 1, hw_model=True)
                assert np.array_equal(dC.cpu().numpy().T.view(np.uint32), emu_r.view(np.uint32)), rounding
            # (chained, it gives the driver's bits)
            assert np.array_equal(dC.cpu().numpy().T, drv)
    from wmma_extension_amd._lib import WmmaeError
    with pytest.raises(WmmaeError) as e:
        tc.api_gemm(type_, ec, 100, n, k, 1.0, dA, k, dB, k, 0.0, dC, 100)
    assert e.value.status == -4


@pytest.mark.parametrize("type_ec", [(0, 1), (0, 0), (2, 1)])
def test_api_level_gemm_wide_exponent_range(tc, orc, dev, type_ec):
    """The kernel on the public API with operands over the whole exponent range of the policy's
    16-bit type, operands whose terms are subnormal there and fp32 subnormals: the split at the
    fragment load, the fp32 adds outside the matrix core and the store give the model's bits."""
    type_, ec = type_ec
    policy = {(0, 1): 0, (0, 0): 1, (2, 1): 2}[type_ec]
    f16 = type_ == 0
    m, n, k = 256, 384, 160
    for regime in ("wide", "tiny_a", "subnormal_a"):
        rng = np.random.default_rng(5 + policy + len(regime))
        if regime == "wide":
            lo, hi = (-40, 14) if f16 else (-60, 60)
            A, Bt = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (n, k), lo, hi)
        elif regime == "tiny_a":
            lo, hi = (-30, -10) if f16 else (-126, -100)
            A, Bt = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (n, k), -3, 3)
        else:
            A = (rng.integers(0, 1 << 24, (m, k)).astype(np.uint32)
                 | (rng.integers(0, 2, (m, k)).astype(np.uint32) << 31)).view(np.float32)
            Bt = _random_patterns(rng, (n, k), -3, 3)
        dC = torch.zeros((n, m), dtype=torch.float32, device=dev)
        tc.api_gemm(type_, ec, m, n, k, 1.0, torch.from_numpy(A).to(dev), k, torch.from_numpy(Bt).to(dev), k,
                    0.0, dC, m)
        torch.cuda.synchronize()
        got = dC.cpu().numpy().T
        emu = orc.tcec_matmul(A, Bt.T, kind=POL_KIND[policy][0], ec=bool(ec), fk=32, main_outside=bool(ec),
                              hw_model=True)
        assert np.isfinite(emu).all()
        assert np.array_equal(got.view(np.uint32), emu.view(np.uint32)), (regime, np.abs(got - emu).max())


@pytest.mark.parametrize("case", [(0, (128, 128, 20000), 0, (1.0, 0.0)), (0, (128, 96, 20000), 2, (-0.75, 1.5)),
                                  (0, (256, 128, 9999), 8, (1.0, 0.0)), (2, (200, 136, 8000), 2, (2.5, -1.0)),
                                  (3, (192, 128, 20000), 8, (1.0, 0.0)), (1, (96, 80, 30000), 0, (1.0, 1.0)),
                                  (0, (256, 256, 8192), 0, (1.0, 0.0))])
def test_k_slices_same_bits_as_the_model(tc, orc, dev, case):
    """A product cut into K slices: every slice is the product over its share of k (whole stages
    of 32, ceil(stages / slices) each) in the oracle's model of the matrix core, folded to
    main + err / scale in fp32; the slices are added in ascending order in double precision,
    rounded to fp32, and alpha and beta applied as by the other paths.  Same bits, on the packed
    path, the direct path and the library's choice."""
    policy, (m, n, k), flag, (alpha, beta) = case
    kind, ec = POL_KIND[policy]
    rng = np.random.default_rng(m + k)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    slices = tc.sgemm_k_slices(m, n, k, 1, policy, flag)
    assert slices > 1
    ws = torch.empty(tc.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
    D = _gemm(tc, dev, A, B, policy, alpha=alpha, beta=beta, C=C, flags=flag, workspace=ws)
    stages = (k + 31) // 32
    per = -(-stages // slices)
    total = np.zeros((m, n), np.float64)
    for s0 in range(0, stages, per):
        ka, kb = 32 * s0, min(k, 32 * (s0 + per))
        Ap = np.zeros((m, 32 * (-(-(kb - ka) // 32))), np.float32)          # the last stage padded with zeros
        Bp = np.zeros((Ap.shape[1], n), np.float32)
        Ap[:, :kb - ka], Bp[:kb - ka, :] = A[:, ka:kb], B[ka:kb, :]
        total += orc.tcec_matmul(Ap, Bp, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True).astype(np.float64)
    emu = orc.epilogue(total.astype(np.float32), alpha, beta, C)
    assert np.array_equal(D.view(np.uint32), emu.view(np.uint32)), int((D.view(np.uint32) != emu.view(np.uint32)).sum())


def test_gemm_kernel_events_inside_a_call(tc, dev):
    """wmmae_tcec_time_gemm_kernel: a call on the packed or the direct path records the caller's
    two events right around its MFMA GEMM kernel (and the fold of its K slices): the time between
    them is positive and shorter than the whole call's, which also runs the split pass; the
    result is the call's usual one; after the block nothing is recorded any more."""
    m = n = k = 2048
    g = torch.Generator(device=dev).manual_seed(3)
    A = torch.rand((m, k), generator=g, device=dev) * 2 - 1
    B = torch.rand((n, k), generator=g, device=dev) * 2 - 1
    ws = torch.empty(tc.workspace_bytes(m, n, k, 1, 0), dtype=torch.uint8, device=dev)
    for flag in (2, 8):
        C0 = torch.empty((n, m), device=dev)
        tc.sgemm("T", "N", m, n, k, 1.0, A, k, B, k, 0.0, C0, m, 0, flag, ws)
        torch.cuda.synchronize()
        C = torch.empty((n, m), device=dev)
        e0, e1, w0, w1 = (torch.cuda.Event(enable_timing=True) for _ in range(4))
        inner, whole = [], []
        for _ in range(5):
            w0.record()
            with tc.timed_gemm_kernel(e0, e1):
                tc.sgemm("T", "N", m, n, k, 1.0, A, k, B, k, 0.0, C, m, 0, flag, ws)
            w1.record()
            torch.cuda.synchronize()
            inner.append(e0.elapsed_time(e1))
            whole.append(w0.elapsed_time(w1))
        assert torch.equal(C, C0)
        assert 0.0 < min(inner) <= min(whole)
        if flag == 2:
            assert min(inner) < 0.95 * min(whole)          # the split pass is outside the two events
        # outside the block: the events keep their last times
        before = e0.elapsed_time(e1)
        tc.sgemm("T", "N", m, n, k, 1.0, A, k, B, k, 0.0, C, m, 0, flag, ws)
        torch.cuda.synchronize()
        assert e0.elapsed_time(e1) == before


@pytest.mark.parametrize("flag", [2, 8])
def test_fold_of_k_slices_is_the_same_with_any_layout_of_c(tc, dev, flag):
    """The kernel that adds the K slices takes 16 bytes per access where C allows it and single
    elements elsewhere (a padded leading dimension, a base that is no multiple of 16 bytes, a
    pointer array): same sums in the same order, same bits, with alpha and beta."""
    m, n, k, policy = 512, 384, 20000, 0
    assert tc.sgemm_k_slices(m, n, k, 1, policy, flag) > 1
    g = torch.Generator(device=dev).manual_seed(31)
    A = torch.rand((m, k), generator=g, device=dev) * 2 - 1
    B = torch.rand((n, k), generator=g, device=dev) * 2 - 1
    C0 = torch.rand((n, m), generator=g, device=dev) * 2 - 1
    ws = torch.empty(tc.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
    for alpha, beta in ((1.0, 0.0), (-0.75, 1.5)):
        outs = []
        for pad, shift in ((0, 0), (1, 0), (4, 0), (0, 1), (4, 3)):
            buf = torch.full((n * (m + pad) + 8,), 7.0, device=dev)
            C = buf[shift:shift + n * (m + pad)].view(n, m + pad)
            C[:, :m] = C0
            tc.sgemm("T", "N", m, n, k, alpha, A, k, B, k, beta, C, m + pad, policy, flag, ws)
            torch.cuda.synchronize()
            assert (C[:, m:] == 7.0).all() and (buf[:shift] == 7.0).all()
            outs.append(C[:, :m].clone())
        # ... and through an array of pointers
        C = C0.clone()
        ptr = lambda t: torch.tensor([t.data_ptr()], dtype=torch.int64, device=dev)   # noqa: E731
        tc.sgemm_batched("T", "N", m, n, k, alpha, ptr(A), k, ptr(B), k, beta, ptr(C), m, 1, policy, flag, ws)
        torch.cuda.synchronize()
        outs.append(C)
        assert all(torch.equal(outs[0], o) for o in outs[1:]), (alpha, beta)


def test_api_level_gemm_pointer_arrays(tc, orc, dev):
    """The API-level kernel on device arrays of matrix pointers (launch_bgemm's calling
    convention, batch_gemm.cu:433-443): every entry equals the single-matrix call bit for bit,
    and the reference harness's ramp inputs A[j] = j/k, B[j] = j/n (batch_gemm.cu:507-513) keep
    its residual gate."""
    batch, m, n, k = 5, 256, 128, 96
    rng = np.random.default_rng(4242)
    A = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
    Bt = rng.uniform(-1, 1, (batch, n, k)).astype(np.float32)
    A[0] = (np.arange(m * k, dtype=np.float32) / k).reshape(m, k)
    Bt[0] = (np.arange(n * k, dtype=np.float32) / n).reshape(n, k)
    dA = [torch.from_numpy(A[b]).to(dev) for b in range(batch)]
    dB = [torch.from_numpy(Bt[b]).to(dev) for b in range(batch)]
    dC = [torch.zeros((n, m), dtype=torch.float32, device=dev) for _ in range(batch)]
    pa = torch.tensor([t.data_ptr() for t in dA], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in dB], dtype=torch.int64, device=dev)
    pc = torch.tensor([t.data_ptr() for t in dC], dtype=torch.int64, device=dev)
    for type_, ec in ((0, 1), (2, 1), (0, 0)):
        tc.api_gemm_batched(type_, ec, m, n, k, 1.0, pa, k, pb, k, 0.0, pc, m, batch)
        torch.cuda.synchronize()
        for b in range(batch):
            single = torch.zeros((n, m), dtype=torch.float32, device=dev)
            tc.api_gemm(type_, ec, m, n, k, 1.0, dA[b], k, dB[b], k, 0.0, single, m)
            torch.cuda.synchronize()
            assert torch.equal(single, dC[b]), (type_, ec, b)
        if ec:
            got = dC[0].cpu().numpy().T.astype(np.float64)
            ref = orc.gemm_f64(A[0], Bt[0].T)
            assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 1e-6
    tc.api_gemm_batched(0, 1, m, n, k, 1.0, pa, k, pb, k, 0.0, pc, m, 0)     # empty batch: nothing to do


def test_api_level_gemm_fp32_policy(tc, orc, dev):
    """The same API-level GEMM with default_policy<float, without_ec, op_simt>: a plain
    fp32 product on the matrix core's fp32 path, the on-GPU comparator of the 2x gate."""
    m, n, k = 256, 128, 2048
    rng = np.random.default_rng(99)
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    Bt = rng.uniform(-1, 1, (n, k)).astype(np.float32)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(Bt).to(dev)
    dC = torch.zeros((n, m), dtype=torch.float32, device=dev)
    tc.api_gemm(3, 0, m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m)
    torch.cuda.synchronize()
    got = dC.cpu().numpy().T
    ref = orc.gemm_f64(A, Bt.T)
    e_gpu = orc.max_rel_err(got, ref)
    e_cpu = orc.max_rel_err(orc.gemm_f32(A, Bt.T), ref)
    # two fp32 summations in different orders: same error scale, neither exact
    assert e_gpu <= 4 * e_cpu and e_gpu > 0
    # the order of the matrix core's fused multiply-adds is known: the oracle's model, bit for bit
    emu = orc.fp32_policy_matmul(A, Bt.T)
    assert np.array_equal(got.view(np.uint32), emu.view(np.uint32)), np.abs(got - emu).max()
    # and TCEC with error correction on the same inputs is no worse than 2x either of them
    e_tcec = orc.max_rel_err(_gemm(tc, dev, A, Bt.T, 0), ref)
    assert e_tcec <= 2 * min(e_gpu, e_cpu)
    from wmma_extension_amd._lib import WmmaeError
    with pytest.raises(WmmaeError) as e:
        tc.api_gemm(3, 1, m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m)
    assert e.value.status == -4


def test_pointer_array_entries_with_any_alignment(tc, orc, dev):
    """Pointer-array entries that are only 4-byte aligned (matrices carved out of a
    larger buffer at odd offsets): the fused kernel finds out by itself and falls back
    to 4-byte requests; results equal the aligned call bit for bit."""
    batch, m, n, k = 9, 72, 40, 96
    rng = np.random.default_rng(123)
    A = rng.standard_normal((batch, m, k)).astype(np.float32)
    Bt = rng.standard_normal((batch, n, k)).astype(np.float32)
    for offsets in ([1] * batch, [0, 1, 2, 3, 0, 5, 0, 7, 0]):
        bufA = [torch.zeros(m * k + 8, dtype=torch.float32, device=dev) for _ in range(batch)]
        bufB = [torch.zeros(n * k + 8, dtype=torch.float32, device=dev) for _ in range(batch)]
        bufC = [torch.zeros(n * m + 8, dtype=torch.float32, device=dev) for _ in range(batch)]
        As, Bs, Cs = [], [], []
        for b, off in enumerate(offsets):
            As.append(bufA[b][off:off + m * k].view(m, k)); As[-1].copy_(torch.from_numpy(A[b]))
            Bs.append(bufB[b][off:off + n * k].view(n, k)); Bs[-1].copy_(torch.from_numpy(Bt[b]))
            Cs.append(bufC[b][off:off + n * m].view(n, m))
        pa = torch.tensor([t.data_ptr() for t in As], dtype=torch.int64, device=dev)
        pb = torch.tensor([t.data_ptr() for t in Bs], dtype=torch.int64, device=dev)
        pc = torch.tensor([t.data_ptr() for t in Cs], dtype=torch.int64, device=dev)
        for policy in (0, 2):
            tc.sgemm_batched("T", "N", m, n, k, 1.0, pa, k, pb, k, 0.0, pc, m, batch, policy)
            torch.cuda.synchronize()
            for b in range(batch):
                single = _gemm(tc, dev, A[b], Bt[b].T, policy)
                assert np.array_equal(Cs[b].cpu().numpy().T, single), (offsets[b], b, policy)
                # nothing was written outside the matrix
                off = offsets[b]
                raw = bufC[b].cpu().numpy()
                assert (raw[:off] == 0).all() and (raw[off + n * m:] == 0).all()


def test_sgemm_randomised_sweep(tc, orc, dev):
    """Forty seeded random problems over both GEMM paths: shapes from 1 to ~900 (ragged),
    all transposes, padded leading dimensions, random alpha/beta, all five policies."""
    rng = np.random.default_rng(2024)
    sizes = [1, 2, 7, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 257, 300,
             511, 512, 513, 640, 900]
    for case in range(40):
        m, n = (int(rng.choice(sizes)) for _ in range(2))
        k = int(rng.choice([1, 3, 8, 31, 32, 33, 64, 100, 129, 256, 500]))
        policy = int(rng.integers(0, 5))
        ta, tb = rng.choice(["N", "T"]), rng.choice(["N", "T"])
        alpha = float(rng.choice([1.0, -0.75, 2.5]))
        beta = float(rng.choice([0.0, 0.0, 1.0, -1.5]))
        ld_pad = int(rng.choice([0, 0, 1, 4]))
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
        D = _gemm(tc, dev, A, B, policy, alpha=alpha, beta=beta, C=C, ta=ta, tb=tb, ld_pad=ld_pad)
        kind, ec = POL_KIND[policy]
        emu = orc.tcec_matmul(A, B, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
        if tc.sgemm_path(m, n, k, 1, policy) == tc.PATH_PACKED_SPLIT_K:
            # K slices round their partial sums
            expect = alpha * emu.astype(np.float64) + beta * C
            tol = 32 * 2.0**-24 * max(1.0, np.abs(expect).max())
            assert (np.abs(D - expect) <= tol).all(), (case, m, n, k, policy, ta, tb, alpha, beta, ld_pad)
        else:
            # same sums as the emulator, and the same epilogue: one multiplication by alpha, one
            # fused multiply-add of beta * C - the same bits
            assert np.array_equal(D.view(np.uint32), orc.epilogue(emu, alpha, beta, C).view(np.uint32)), \
                (case, m, n, k, policy, ta, tb, alpha, beta, ld_pad)
        _check(orc, D, A, B, policy, C=C, alpha=alpha, beta=beta)
