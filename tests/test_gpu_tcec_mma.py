"""One-wave TCEC kernels on the GPU (device API of include/wmma_extension/tcec)
against the CPU emulator, the FP64 loop and the reference's thresholds."""
import itertools
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "primitive_kat.npz"))
TH_EC = float(KAT["threshold_with_ec"])
TH_NOEC = float(KAT["threshold_without_ec"])
KIND_OF_TYPE = {0: 0, 1: 1, 2: 2}           # half -> f16 split, bf16 -> bf16x2, tf32 -> bf16x3
INST_K = {0: 32, 1: 16, 2: 16}


def _dims(shape, inst):
    if shape == 0:
        return 32, 32, 32
    return (32, 64, 32) if inst == 2 else (16, 48, 64)


def _mem(x, col):
    """Dense memory image of matrix x in row- or column-major order."""
    return np.ascontiguousarray(x.T if col else x).reshape(-1)


def _run(tc, dev, shape, type_, ec, inst, A, B, C, a_col, b_col, c_col, d_col, rounding):
    m, n = A.shape[0], B.shape[1]
    d = torch.full((m * n,), float("nan"), dtype=torch.float32, device=dev)
    tc.mma_tile(shape, type_, ec, inst, torch.from_numpy(_mem(A, a_col)).to(dev),
                torch.from_numpy(_mem(B, b_col)).to(dev),
                None if C is None else torch.from_numpy(_mem(C, c_col)).to(dev),
                a_col, b_col, c_col, d_col, rounding, d)
    torch.cuda.synchronize()
    out = d.cpu().numpy()
    return out.reshape(n, m).T if d_col else out.reshape(m, n)


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("ec", [1, 0])
@pytest.mark.parametrize("inst", [0, 1, 2])
@pytest.mark.parametrize("shape", [0, 1])
@pytest.mark.parametrize("rounding", [0, 1, 2])
def test_mma_tile_all_layouts(tc, orc, dev, type_, ec, inst, shape, rounding):
    """Every memory-layout combination of A, B, C, D, with and without C
    (the matrix of test/tcec/mma.cu:186-3526), seeded uniform[-1,1], through mma_sync (the
    policy's default: mma_rn_sync with error correction, mma_rz_sync without,
    tcec.hpp:896-927, no_cor.hpp:858-897), mma_rn_sync and mma_rz_sync, each for both policies."""
    m, n, k = _dims(shape, inst)
    rng = np.random.default_rng(1000 * type_ + 100 * ec + 10 * inst + shape)
    kind = KIND_OF_TYPE[type_]
    # leading product added outside the matrix core (rn) or chained through it (rz)
    main_outside = bool(ec) if rounding == 0 else rounding == 1
    for a_col, b_col, c_col, d_col, with_c in itertools.product((0, 1), repeat=5):
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        C = rng.uniform(-1, 1, (m, n)).astype(np.float32) if with_c else None
        D = _run(tc, dev, shape, type_, ec, inst, A, B, C, a_col, b_col, c_col, d_col, rounding)
        ref = orc.gemm_f64(A, B) + (C if with_c else 0)
        err = orc.max_abs_err(D, ref)
        # the emulator follows the device function instruction by instruction, each instruction
        # in the measured accumulate arithmetic of the matrix core: same bits
        emu = orc.tcec_matmul(A, B, C, kind=kind, ec=bool(ec), fk=INST_K[inst],
                              main_outside=main_outside, hw_model=True)
        assert np.array_equal(D.view(np.uint32), emu.view(np.uint32)), \
            (a_col, b_col, c_col, d_col, with_c, np.abs(D - emu).max())
        if ec and type_ != 1:
            assert err < TH_EC                       # test/tcec/mma.cu:7-13
        elif ec:
            assert err < 1e-3                        # two bf16 terms: ~16 bits
        else:
            assert err < (TH_NOEC if type_ == 0 else 8 * TH_NOEC)   # bf16 has 3 fewer bits


def _random_patterns(rng, shape, emin, emax, zeros=0.02):
    """fp32 values with uniformly drawn sign, exponent (emin .. emax) and mantissa bits."""
    e = rng.integers(emin, emax + 1, shape)
    bits = ((rng.integers(0, 2, shape).astype(np.uint32) << 31) | ((e + 127).astype(np.uint32) << 23)
            | rng.integers(0, 1 << 23, shape).astype(np.uint32))
    v = bits.view(np.float32).copy()
    v[rng.random(shape) < zeros] = 0.0
    return v


def _subnormal_patterns(rng, shape, bits):
    return (rng.integers(0, 1 << bits, shape).astype(np.uint32)
            | (rng.integers(0, 2, shape).astype(np.uint32) << 31)).view(np.float32)


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("ec", [1, 0])
def test_mma_tile_wide_exponent_range(tc, orc, dev, type_, ec):
    """Operands far from [-1, 1] through the device API: the whole exponent range of the 16-bit
    type, operands whose terms are subnormal there, and fp32 subnormals (residual terms
    underflow, sums and the fp32 adds outside the matrix core end below 2^-126), with and
    without C, all three roundings and instruction shapes: the oracle's model, bit for bit."""
    kind = KIND_OF_TYPE[type_]
    f16 = kind == 0
    for inst, rounding, regime in itertools.product((0, 1, 2), (0, 1, 2), ("wide", "tiny_a", "subnormal_a")):
        m, n, k = _dims(0, inst)
        main_outside = bool(ec) if rounding == 0 else rounding == 1
        rng = np.random.default_rng(type_ * 1000 + ec * 100 + inst * 10 + rounding + len(regime))
        if regime == "wide":
            lo, hi = (-40, 14) if f16 else (-60, 60)
            A, B = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (k, n), lo, hi)
            C = _random_patterns(rng, (m, n), 2 * lo, 28 if f16 else 2 * hi)
        elif regime == "tiny_a":
            lo, hi = (-30, -10) if f16 else (-126, -100)
            A, B = _random_patterns(rng, (m, k), lo, hi), _random_patterns(rng, (k, n), -3, 3)
            C = _random_patterns(rng, (m, n), lo, hi)
        else:
            A, B = _subnormal_patterns(rng, (m, k), 24), _random_patterns(rng, (k, n), -3, 3)
            C = _subnormal_patterns(rng, (m, n), 25)
        for Cc in (None, C):
            D = _run(tc, dev, 0, type_, ec, inst, A, B, Cc, 0, 1, 1, 1, rounding)
            emu = orc.tcec_matmul(A, B, Cc, kind=kind, ec=bool(ec), fk=INST_K[inst],
                                  main_outside=main_outside, hw_model=True)
            fin = np.isfinite(emu)
            assert np.array_equal(np.isfinite(D), fin), (inst, rounding, regime)
            assert np.array_equal(D[fin].view(np.uint32), emu[fin].view(np.uint32)), \
                (inst, rounding, regime, Cc is not None)


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("ec", [1, 0])
def test_mma_tile_exact_cases(tc, orc, dev, type_, ec):
    """Inputs whose partial sums are all exact: bit-exact against the exact product
    for mma_sync, mma_rn_sync and mma_rz_sync alike."""
    rng = np.random.default_rng(77)
    A = (rng.integers(-8, 9, (32, 32)) * 0.25).astype(np.float32)
    B = (rng.integers(-8, 9, (32, 32)) * 0.5).astype(np.float32)
    C = rng.integers(-100, 100, (32, 32)).astype(np.float32)
    exact = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float32)
    for inst in (0, 1, 2):
        for rounding in (0, 1, 2):
            D = _run(tc, dev, 0, type_, ec, inst, A, B, C, 0, 1, 1, 1, rounding)
            assert np.array_equal(D, exact), (inst, rounding)
    # identity B returns the recombined split of A
    eye = np.eye(32, dtype=np.float32)
    A = rng.uniform(-1, 1, (32, 32)).astype(np.float32)
    D = _run(tc, dev, 0, type_, ec, 0, A, eye, None, 0, 0, 0, 0, 0)
    assert np.array_equal(D, orc.tcec_matmul(A, eye, kind=KIND_OF_TYPE[type_], ec=bool(ec)))


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("use", [0, 1])
def test_fragment_terms_from_a_swizzled_tile(tc, orc, dev, type_, use):
    """A tile staged in LDS with its 16-byte pieces permuted (tcec::row_major_swizzled for
    matrix_a, col_major_swizzled for matrix_b; written with utils::cp_async by the recipe of
    the layout) and loaded with that tag gives the same terms as the plain load of the same
    matrix, which test_fragment_terms_bit_exact pins against the oracle's split."""
    rng = np.random.default_rng(22 + type_)
    N = 32
    for ec, frag_col in itertools.product((1, 0), (0, 1)):
        X = rng.uniform(-1, 1, (N, N)).astype(np.float32)
        src = torch.from_numpy(_mem(X, use)).to(dev)      # A: rows of k; B: columns of k
        plain = tc.frag_dump(use, type_, ec, frag_col, src, 0, use).cpu().numpy()
        swz = tc.frag_dump(use, type_, ec, frag_col, src, 0, 2).cpu().numpy()
        assert plain.any() and np.array_equal(plain, swz), (ec, frag_col)


@pytest.mark.parametrize("type_", [0, 2])
def test_mma_tile_native_layout_overload(tc, orc, dev, type_):
    rng = np.random.default_rng(5)
    for ec, a_fc, b_fc, d_col in itertools.product((1, 0), (0, 1), (0, 1), (0, 1)):
        A = rng.uniform(-1, 1, (32, 32)).astype(np.float32)
        B = rng.uniform(-1, 1, (32, 32)).astype(np.float32)
        d = torch.empty(32 * 32, dtype=torch.float32, device=dev)
        tc.mma_tile_native(type_, ec, a_fc, b_fc, torch.from_numpy(_mem(A, a_fc)).to(dev),
                           torch.from_numpy(_mem(B, b_fc)).to(dev), d_col, d)
        out = d.cpu().numpy()
        D = out.reshape(32, 32).T if d_col else out.reshape(32, 32)
        err = orc.max_abs_err(D, orc.gemm_f64(A, B))
        assert err < (TH_EC if ec else (TH_NOEC if type_ == 0 else 8 * TH_NOEC))


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("ec", [1, 0])
def test_matvec(tc, orc, dev, type_, ec):
    """y = A x and y^T = x^T A through load_vector / store_vector
    (test/tcec/matvec.cu:21-50; its with_ec gate is 1e-5 as for mma)."""
    rng = np.random.default_rng(9)
    for a_col, left in itertools.product((0, 1), (0, 1)):
        A = rng.uniform(-1, 1, (32, 32)).astype(np.float32)
        x = rng.uniform(-1, 1, 32).astype(np.float32)
        y = tc.matvec(type_, ec, torch.from_numpy(_mem(A, a_col)).to(dev),
                      torch.from_numpy(x).to(dev), a_col, left).cpu().numpy()
        ref = (x.astype(np.float64) @ A.astype(np.float64)) if left else \
            (A.astype(np.float64) @ x.astype(np.float64))
        err = np.abs(y - ref).max()
        if ec and type_ != 1:
            assert err < TH_EC
        elif ec:
            assert err < 1e-3
        else:
            assert err < (TH_NOEC if type_ == 0 else 8 * TH_NOEC)
        # the vector is the first column (row) of an otherwise empty operand fragment: the same
        # matrix product in the oracle's model of the matrix core, bit for bit
        X = np.zeros((32, 32), np.float32)
        if left:
            X[0, :] = x
            emu = orc.tcec_matmul(X, A, kind=KIND_OF_TYPE[type_], ec=bool(ec), fk=32, main_outside=bool(ec),
                                  hw_model=True)[0, :]
        else:
            X[:, 0] = x
            emu = orc.tcec_matmul(A, X, kind=KIND_OF_TYPE[type_], ec=bool(ec), fk=32, main_outside=bool(ec),
                                  hw_model=True)[:, 0]
        assert np.array_equal(y.view(np.uint32), emu.view(np.uint32)), (a_col, left)


@pytest.mark.parametrize("type_", [0, 1, 2])
@pytest.mark.parametrize("use", [0, 1])
def test_fragment_terms_bit_exact(tc, orc, dev, type_, use):
    """The 16-bit terms a fragment holds after load_matrix_sync equal the oracle's
    split of the element the layout model assigns to that register, bit for bit;
    load_vector fills exactly the first column / row (test/tcec/vector.cu:109-199)."""
    rng = np.random.default_rng(21)
    kind = KIND_OF_TYPE[type_]
    N = 32
    fm = (16, 16, 32)
    ij = orc.frag_ij_table(use, *fm)             # (64, R, 2) for one sub-fragment
    R = ij.shape[1]
    sub_rows, sub_cols = (16, 32) if use == 0 else (32, 16)
    nbm, nbn = N // sub_rows, N // sub_cols
    for ec, frag_col, mem_col in itertools.product((1, 0), (0, 1), (0, 1)):
        X = rng.uniform(-1, 1, (N, N)).astype(np.float32)
        X[0, 0], X[1, 1], X[2, 3] = 0.0, 2.0**-16, 1.0
        got = tc.frag_dump(use, type_, ec, frag_col, torch.from_numpy(_mem(X, mem_col)).to(dev),
                           0, mem_col).cpu().numpy().view(np.uint16)
        terms = orc.split(kind, X)
        nterms = got.shape[0]
        for e in range(nbm * nbn * R):
            block, reg = divmod(e, R)
            bm, bn = block % nbm, block // nbm
            for lane in range(64):
                i = ij[lane, reg, 0] + bm * sub_rows
                j = ij[lane, reg, 1] + bn * sub_cols
                for t in range(nterms):
                    assert got[t, e, lane] == terms[t][i, j], (ec, frag_col, mem_col, e, lane, t)
        # load_vector: first column (col_major fragment) or first row (row_major)
        v = rng.uniform(-1, 1, N).astype(np.float32)
        gotv = tc.frag_dump(use, type_, ec, frag_col, torch.from_numpy(v).to(dev), 1, 0)
        gotv = gotv.cpu().numpy().view(np.uint16)
        dense = np.zeros((N, N), dtype=np.float32)
        if frag_col:
            dense[:, 0] = v
        else:
            dense[0, :] = v
        tv = orc.split(kind, dense)
        for e in range(nbm * nbn * R):
            block, reg = divmod(e, R)
            bm, bn = block % nbm, block // nbm
            for lane in range(64):
                i = ij[lane, reg, 0] + bm * sub_rows
                j = ij[lane, reg, 1] + bn * sub_cols
                for t in range(nterms):
                    assert gotv[t, e, lane] == tv[t][i, j]


@pytest.mark.parametrize("type_", [0, 2])
@pytest.mark.parametrize("ec", [1, 0])
@pytest.mark.parametrize("inst", [0, 1, 2])
def test_elementwise_accessors_neg_integrate(tc, orc, dev, type_, ec, inst):
    """x(i) / dx(i) address sub-fragment i / num_elements, register i % num_elements;
    fill_fragment sets the main part and clears the error part; neg negates both;
    integrate folds err/scale into main (test/tcec/elementwise.cu:7-26, tcec.hpp:40-98)."""
    fm, fn, fk = {0: (16, 16, 32), 1: (16, 16, 16), 2: (32, 32, 16)}[inst]
    ij = orc.frag_ij_table(2, fm, fn, fk)
    R = ij.shape[1]
    nbm = 32 // fm
    scale = 2048.0 if type_ == 0 else 1.0
    base = 2.5
    for do_neg, do_int in itertools.product((0, 1), (0, 1)):
        out = tc.elementwise(type_, ec, inst, base, do_neg, do_int, dev).cpu().numpy()
        got = out[:1024].reshape(32, 32).T                     # stored column-major
        nelem = (32 // fm) * (32 // fn) * R
        for lane in range(64):
            assert out[1024 + lane] == (base + lane * 100) + (base + lane * 100 + nelem - 1)
            for e in range(nelem):
                block, reg = divmod(e, R)
                bm, bn = block % nbm, block // nbm
                i = ij[lane, reg, 0] + bm * fm
                j = ij[lane, reg, 1] + bn * fn
                main = np.float32(base + lane * 100 + e)
                err = np.float32(e) if ec else np.float32(0)
                if do_neg:
                    main, err = -main, -err
                # store and integrate both evaluate main + err/scale in fp32
                expect = np.float32(main + np.float32(err / np.float32(scale)))
                assert got[i, j] == expect, (do_neg, do_int, lane, e)


# ---------------------------------------------------------------- fp32 policy (op_simt)
def test_fp32_policy_mma_tile(tc, orc, dev):
    """default_policy<float, without_ec, op_simt>: fp32 operands, no split
    (docs/mma_f32.md:139-152).  All layouts; the result is a plain fp32 product, so it
    sits within a few fp32 ulps of the oracle's fp32 loop and meets the with_ec gate of
    the reference's mma test although nothing is corrected."""
    for shape in (0, 1):
        m, n, k = _dims(shape, 1)
        rng = np.random.default_rng(300 + shape)
        for a_col, b_col, c_col, d_col, with_c in itertools.product((0, 1), repeat=5):
            A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
            B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
            C = rng.uniform(-1, 1, (m, n)).astype(np.float32) if with_c else None
            D = _run(tc, dev, shape, 3, 0, 1, A, B, C, a_col, b_col, c_col, d_col, 0)
            ref = orc.gemm_f64(A, B) + (C if with_c else 0)
            f32 = orc.gemm_f32(A, B) + (C if with_c else 0)
            assert orc.max_abs_err(D, ref) < TH_EC
            assert np.abs(D - f32).max() <= 16 * 2.0**-24 * max(1.0, np.abs(ref).max())
            # the matrix core's fp32 path is a chain of fused multiply-adds in a known order:
            # the oracle's model of it, bit for bit
            emu = orc.fp32_policy_matmul(A, B, C)
            assert np.array_equal(D.view(np.uint32), emu.view(np.uint32)), (shape, a_col, b_col, c_col, d_col, with_c)
            if a_col == b_col:
                # mma_rz_sync chains through the matrix core like the default; mma_rn_sync starts
                # every 16 of k from zero there and adds outside
                for rounding in (1, 2):
                    D2 = _run(tc, dev, shape, 3, 0, 1, A, B, C, a_col, b_col, c_col, d_col, rounding)
                    emu2 = orc.fp32_policy_matmul(A, B, C, main_outside=rounding == 1)
                    assert np.array_equal(D2.view(np.uint32), emu2.view(np.uint32)), (shape, rounding, with_c)
    # error correction does not exist for fp32 operands
    from wmma_extension_amd._lib import WmmaeError
    with pytest.raises(WmmaeError) as e:
        _run(tc, dev, 0, 3, 1, 1, A[:32, :32], B[:32, :32], None, 0, 0, 0, 0, 0)
    assert e.value.status == -4


def test_fp32_policy_exact_and_identity(tc, orc, dev):
    rng = np.random.default_rng(78)
    A = (rng.integers(-8, 9, (32, 32)) * 0.25).astype(np.float32)
    B = (rng.integers(-8, 9, (32, 32)) * 0.5).astype(np.float32)
    C = rng.integers(-100, 100, (32, 32)).astype(np.float32)
    exact = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float32)
    for rounding in (0, 1, 2):
        assert np.array_equal(_run(tc, dev, 0, 3, 0, 1, A, B, C, 0, 1, 1, 1, rounding), exact)
    # nothing is rounded away on the way in: B = I returns A bit for bit, including values
    # that no 16-bit split represents
    A = (rng.uniform(-1, 1, (32, 32)) * np.exp2(rng.integers(-60, 60, (32, 32)))).astype(np.float32)
    D = _run(tc, dev, 0, 3, 0, 1, A, np.eye(32, dtype=np.float32), None, 0, 0, 0, 0, 0)
    assert np.array_equal(D, A)


def test_fp32_policy_matvec(tc, orc, dev):
    rng = np.random.default_rng(10)
    for a_col, left in itertools.product((0, 1), (0, 1)):
        A = rng.uniform(-1, 1, (32, 32)).astype(np.float32)
        x = rng.uniform(-1, 1, 32).astype(np.float32)
        y = tc.matvec(3, 0, torch.from_numpy(_mem(A, a_col)).to(dev),
                      torch.from_numpy(x).to(dev), a_col, left).cpu().numpy()
        ref = (x.astype(np.float64) @ A.astype(np.float64)) if left else \
            (A.astype(np.float64) @ x.astype(np.float64))
        assert np.abs(y - ref).max() < TH_EC
        X = np.zeros((32, 32), np.float32)
        if left:
            X[0, :] = x
            emu = orc.fp32_policy_matmul(X, A)[0, :]
        else:
            X[:, 0] = x
            emu = orc.fp32_policy_matmul(A, X)[:, 0]
        assert np.array_equal(y.view(np.uint32), emu.view(np.uint32)), (a_col, left)


def test_fp32_policy_elementwise(tc, orc, dev):
    """x(i), fill_fragment, neg on the fp32 fragment (no error part; integrate is a no-op)."""
    ij = orc.frag_ij_table(2, 16, 16, 16)
    R = ij.shape[1]
    base = 2.5
    for do_neg, do_int in itertools.product((0, 1), (0, 1)):
        out = tc.elementwise(3, 0, 1, base, do_neg, do_int, dev).cpu().numpy()
        got = out[:1024].reshape(32, 32).T
        nelem = 4 * R
        for lane in range(64):
            for e in range(nelem):
                block, reg = divmod(e, R)
                i = ij[lane, reg, 0] + (block % 2) * 16
                j = ij[lane, reg, 1] + (block // 2) * 16
                main = np.float32(base + lane * 100 + e)
                assert got[i, j] == (-main if do_neg else main)
