"""Fragment conveniences on the GPU: operators (test/primitive/operators.cu), add_eye /
make_identity_matrix (test/primitive/add_eye.cu) and direct-product fragments
(test/primitive/direct_product.cu), through the C-ABI harness entries."""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _round(x, elem):
    """fp32/fp64 array rounded once to the fragment's element type, back as float32."""
    x = np.asarray(x, dtype=np.float64)
    if elem == 0:
        return x.astype(np.float16).astype(np.float32)
    if elem == 1:
        return torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    return x.astype(np.float32)


@pytest.mark.parametrize("elem", [0, 1, 2])
@pytest.mark.parametrize("use", [0, 1, 2])
def test_fragment_operators(tc, dev, elem, use):
    """Every result element is the correctly rounded result of the operation on the
    (already rounded) operands; the reference's gate is a summed error below 1e-6
    (operators.cu:129), here the comparison is exact."""
    if use == 2 and elem != 2:
        from wmma_extension_amd._lib import WmmaeError
        with pytest.raises(WmmaeError) as e:
            tc.fragment_ops(0, use, elem, 1.0, torch.zeros(16, 16, device=dev), torch.zeros(16, 16, device=dev))
        assert e.value.status == -4
        return
    rng = np.random.default_rng(3 + elem + 10 * use)
    A = rng.uniform(-1, 1, (16, 16)).astype(np.float32)
    B = rng.uniform(-1, 1, (16, 16)).astype(np.float32)
    a, b = _round(A, elem).astype(np.float64), _round(B, elem).astype(np.float64)
    alpha = 1.5
    expect = {0: a + b, 1: a - b, 2: a * alpha, 3: a / alpha, 4: alpha * a + b, 5: a + alpha * b}
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    for op in range(6):
        got = tc.fragment_ops(op, use, elem, alpha, dA, dB).cpu().numpy()
        if elem == 1 and op >= 4:
            # bf16 fma: fp32 fused multiply-add, then one rounding to bf16
            x, y = (a, b) if op == 4 else (b, a)  # op 5 is a + alpha*b (operators.cu:211-225)
            want = _round(np.float32(alpha) * x.astype(np.float32) + y.astype(np.float32), 1)
            assert np.abs(got - want).max() <= 2.0**-8 * np.abs(want).max()
            continue
        if elem == 2 and op == 3:
            want = (a.astype(np.float32) / np.float32(alpha)).astype(np.float32)
        else:
            want = _round(expect[op], elem)
        assert np.array_equal(got, want), (op, np.abs(got - want).max())


def test_add_eye_and_identity(tc, dev):
    """fill(1) + add_eye(2) gives 3 on the diagonal and 1 elsewhere
    (add_eye.cu:37-44); make_identity_matrix overwrites whatever was there."""
    for shape, n in ((0, 16), (1, 32)):
        got = tc.fragment_eye(shape, 0, 2.0, dev).cpu().numpy()
        assert np.array_equal(got, np.ones((n, n), np.float32) + 2 * np.eye(n, dtype=np.float32))
        got = tc.fragment_eye(shape, 1, 0.0, dev).cpu().numpy()
        assert np.array_equal(got, np.eye(n, dtype=np.float32))


@pytest.mark.parametrize("elem", [0, 1])
@pytest.mark.parametrize("terms", [2, 3])
@pytest.mark.parametrize("from_float", [0, 1])
def test_direct_product(tc, orc, dev, elem, terms, from_float):
    """u v^T from one MMA on direct-product fragments: seeded uniform[0,1) vectors,
    error below 16 eps(fp32) for half (direct_product.cu:128-131); the exact sum of the
    products the fragments encode is reproduced to an fp32 rounding."""
    rng = np.random.default_rng(0)
    u = rng.uniform(0, 1, 16).astype(np.float32)
    v = rng.uniform(0, 1, 16).astype(np.float32)
    h = tc.direct_product(elem, terms, from_float, torch.from_numpy(u).to(dev),
                          torch.from_numpy(v).to(dev)).cpu().numpy()
    ref = np.outer(u.astype(np.float64), v.astype(np.float64))
    eps = 2.0**-23
    if elem == 0:
        assert np.abs(h - ref).max() < 16 * eps
    else:
        assert np.abs(h - ref).max() < 2.0**-15          # two bf16 terms carry ~16 bits
    # what the fragments hold: x = RN16(u), dx = RN16(u - x) (no scaling here)
    def parts(w):
        x = _round(w, elem).astype(np.float64)
        dx = _round(w.astype(np.float64) - x, elem).astype(np.float64)
        return x, dx
    xu, du = parts(u)
    xv, dv = parts(v)
    enc = np.outer(xu, xv) + np.outer(du, xv) + np.outer(xu, dv)
    if terms == 3:
        enc += np.outer(du, dv)
    assert np.abs(h - enc).max() <= 2.0**-23 * np.abs(enc).max()
    # and the third correction term is really there: it changes the encoded sum
    if terms == 3:
        assert np.abs(np.outer(du, dv)).max() > 0
