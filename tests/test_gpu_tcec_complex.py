"""Complex TCEC (tcec::fragment_complex) on the GPU against an FP64 complex product, the
reference's thresholds (test/tcec/mma_complex.cu:7-20) and the composition of four real
TCEC products of the CPU emulator."""
import itertools
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
KIND_OF_TYPE = {0: 0, 1: 1, 2: 2}
N = 32


def _mem(z, col):
    """Interleaved (re, im) fp32 image of complex matrix z, row- or column-major."""
    zz = np.ascontiguousarray(z.T if col else z).astype(np.complex64)
    return zz.view(np.float32).reshape(-1).copy()


def _unmem(x, col):
    z = x.view(np.complex64).reshape(N, N)
    return z.T if col else z


def _run(tc, dev, type_, ec, A, B, C, a_col, b_col, c_col, d_col, rounding=0, mul=1.0):
    d = tc.mma_complex(type_, ec, torch.from_numpy(_mem(A, a_col)).to(dev),
                       torch.from_numpy(_mem(B, b_col)).to(dev),
                       None if C is None else torch.from_numpy(_mem(C, c_col)).to(dev),
                       a_col, b_col, c_col, d_col, rounding, mul)
    torch.cuda.synchronize()
    return _unmem(d.cpu().numpy(), d_col)


def _rand(rng):
    return (rng.uniform(-1, 1, (N, N)) + 1j * rng.uniform(-1, 1, (N, N))).astype(np.complex64)


def _threshold(type_, ec):
    if type_ == 3:
        return 4e-6                     # float, without_ec (mma_complex.cu:20)
    if ec:
        return 1e-5 if type_ != 1 else 1e-3
    return 1e-2 if type_ == 0 else 8e-2


@pytest.mark.parametrize("type_ec", [(0, 1), (0, 0), (1, 1), (2, 1), (2, 0), (3, 0)])
def test_complex_mma_all_layouts(tc, orc, dev, type_ec):
    type_, ec = type_ec
    rng = np.random.default_rng(40 + 10 * type_ + ec)
    for a_col, b_col, c_col, d_col, with_c in itertools.product((0, 1), repeat=5):
        A, B = _rand(rng), _rand(rng)
        C = _rand(rng) if with_c else None
        D = _run(tc, dev, type_, ec, A, B, C, a_col, b_col, c_col, d_col)
        ref = A.astype(np.complex128) @ B.astype(np.complex128) + (C if with_c else 0)
        err = max(np.abs(D.real - ref.real).max(), np.abs(D.imag - ref.imag).max())
        assert err < _threshold(type_, ec), (a_col, b_col, c_col, d_col, with_c, err)


@pytest.mark.parametrize("type_", [0, 2])
def test_complex_mma_matches_composed_real_products(tc, orc, dev, type_):
    """re = Ar Br - Ai Bi + Cr, im = Ai Br + Ar Bi + Ci with each real product done by
    the CPU TCEC emulator: agreement to a few fp32 ulps."""
    rng = np.random.default_rng(7 + type_)
    kind = KIND_OF_TYPE[type_]
    A, B, C = _rand(rng), _rand(rng), _rand(rng)
    D = _run(tc, dev, type_, 1, A, B, C, 0, 1, 1, 1)

    def f(x):
        return np.ascontiguousarray(x, dtype=np.float32)
    mm = lambda a, b, c: orc.tcec_matmul(f(a), f(b), f(c), kind=kind, ec=True, fk=32, main_outside=True)
    re = mm(A.imag, -B.imag, mm(A.real, B.real, C.real))
    im = mm(A.real, B.imag, mm(A.imag, B.real, C.imag))
    scale = 16 * 2.0**-24 * 32
    assert np.abs(D.real - re).max() <= scale and np.abs(D.imag - im).max() <= scale


@pytest.mark.parametrize("type_ec", [(0, 1), (0, 0), (1, 1), (1, 0), (2, 1), (2, 0), (3, 0)])
def test_complex_mma_bits_of_the_chained_real_products(tc, orc, dev, type_ec):
    """The four real products of a complex one run in pairs on one accumulator fragment each
    (complex.hpp:609-646: re = Ar Br + Cr, then - Ai Bi on top; im = Ai Br + Ci, then Ar Bi), the
    error part carried from the first product of a pair into the second and folded once at the
    store.  That is one real TCEC product over the joined operands [Ar | Ai] [Br ; -Bi] and
    [Ai | Ar] [Br ; Bi]: the oracle's model of the matrix core gives the same bits, for every
    rounding variant, with and without C, and for the fp32 policy."""
    type_, ec = type_ec

    def f(x):
        return np.ascontiguousarray(x, dtype=np.float32)
    for rounding, with_c in itertools.product((0, 1, 2), (0, 1)):
        rng = np.random.default_rng(type_ * 100 + ec * 10 + rounding + with_c)
        A, B = _rand(rng), _rand(rng)
        C = _rand(rng) if with_c else None
        D = _run(tc, dev, type_, ec, A, B, C, 0, 1, 1, 1, rounding)
        main_outside = bool(ec) if rounding == 0 else rounding == 1

        def mm(a1, a2, b1, b2, c):
            a, b = f(np.concatenate([a1, a2], axis=1)), f(np.concatenate([b1, b2], axis=0))
            c = None if c is None else f(c)
            if type_ == 3:
                return orc.fp32_policy_matmul(a, b, c, main_outside=rounding == 1)
            return orc.tcec_matmul(a, b, c, kind=KIND_OF_TYPE[type_], ec=bool(ec), fk=32,
                                   main_outside=main_outside, hw_model=True)
        re = mm(A.real, A.imag, B.real, -B.imag, C.real if with_c else None)
        im = mm(A.imag, A.real, B.real, B.imag, C.imag if with_c else None)
        assert np.array_equal(f(D.real).view(np.uint32), re.view(np.uint32)), (rounding, with_c)
        assert np.array_equal(f(D.imag).view(np.uint32), im.view(np.uint32)), (rounding, with_c)


@pytest.mark.parametrize("type_", [0, 2, 3])
def test_complex_exact_cases_roundings_and_scaled_io(tc, orc, dev, type_):
    rng = np.random.default_rng(11)
    ec = 0 if type_ == 3 else 1

    def small():
        return ((rng.integers(-8, 9, (N, N)) * 0.25) + 1j * (rng.integers(-8, 9, (N, N)) * 0.5)).astype(np.complex64)
    A, B, C = small(), small(), small()
    exact = (A.astype(np.complex128) @ B.astype(np.complex128) + C).astype(np.complex64)
    for rounding in (0, 1, 2):
        assert np.array_equal(_run(tc, dev, type_, ec, A, B, C, 0, 1, 1, 1, rounding), exact)
    # scaled load of A (x4) and scaled store (x1/4): exact for powers of two
    assert np.array_equal(_run(tc, dev, type_, ec, A, B, C, 1, 0, 0, 1, 0, mul=4.0), exact)
    assert np.array_equal(_run(tc, dev, type_, ec, A, B, None, 1, 0, 0, 0, 0, mul=0.5),
                          (A.astype(np.complex128) @ B.astype(np.complex128)).astype(np.complex64))
    # i * i = -1: A = i I, B = i I -> D = -I ; and multiplication by the identity returns
    # the recombined split of the other factor, component by component
    eye = np.eye(N).astype(np.complex64)
    D = _run(tc, dev, type_, ec, 1j * eye, 1j * eye, None, 0, 0, 0, 0)
    assert np.array_equal(D, -eye)
    Z = _rand(rng)
    D = _run(tc, dev, type_, ec, Z, eye, None, 0, 0, 0, 0)
    if type_ == 3:
        assert np.array_equal(D, Z)
    else:
        kind = KIND_OF_TYPE[type_]
        one = np.eye(N, dtype=np.float32)
        assert np.array_equal(D.real, orc.tcec_matmul(np.ascontiguousarray(Z.real), one, kind=kind, ec=True))
        assert np.array_equal(D.imag, orc.tcec_matmul(np.ascontiguousarray(Z.imag), one, kind=kind, ec=True))
