"""Seeded random products through every path of the driver against the oracle's model of the
matrix core, bit for bit: shapes that are no multiples of anything (k from 1 on), every policy,
alpha / beta, all four transpose combinations, padded leading dimensions, the round-to-nearest
flag, K slices where the driver cuts K.  Expected = every slice in the model (k padded with zeros to whole stages of 32, as the
kernels pad), slices added in double precision in ascending order, then the epilogue
(alpha, one fused multiply-add of beta * C)."""
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8
POL_KIND = {0: (0, True), 1: (0, False), 2: (2, True), 3: (1, True), 4: (1, False)}


def _model(orc, A, B, kind, ec, slices, rn):
    m, k = A.shape
    n = B.shape[1]
    stages = (k + 31) // 32
    per = -(-stages // slices)
    total = None
    for s0 in range(0, stages, per):
        ka, kb = 32 * s0, min(k, 32 * (s0 + per))
        ap = np.zeros((m, 32 * (-(-(kb - ka) // 32))), np.float32)
        bp = np.zeros((ap.shape[1], n), np.float32)
        ap[:, :kb - ka], bp[:kb - ka, :] = A[:, ka:kb], B[ka:kb, :]
        part = orc.tcec_matmul(ap, bp, kind=kind, ec=ec, fk=32, main_outside=rn, hw_model=True)
        if slices == 1:
            return part
        total = part.astype(np.float64) if total is None else total + part.astype(np.float64)
    return total.astype(np.float32)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_products_have_the_bits_of_the_model(tc, orc, dev, seed):
    from wmma_extension_amd._lib import WmmaeError
    rnd = random.Random(seed)
    rng = np.random.default_rng(seed)
    checked = 0
    for case in range(40):
        m = rnd.choice([1, 3, 16, 17, 40, 100, 129, 200, 257, 300, 400])
        n = rnd.choice([1, 5, 16, 31, 64, 100, 130, 200, 256, 333])
        k = rnd.choice([1, 2, 4, 5, 31, 32, 33, 64, 77, 100, 160, 255, 500, 1000, 3000, 9000])
        policy = rnd.choice([0, 0, 1, 2, 3, 4])
        alpha, beta = rnd.choice([(1.0, 0.0), (1.0, 0.0), (-0.75, 1.5), (2.5, -1.0)])
        pad = rnd.choice([0, 0, 1, 4])
        rn = rnd.random() < 0.2 and policy in (0, 2)
        ta, tb = rnd.choice([("T", "N")] * 3 + [("N", "N"), ("N", "T"), ("T", "T")])
        kind, ec = POL_KIND[policy]
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        C = rng.uniform(-1, 1, (m, n)).astype(np.float32)
        # column-major BLAS storage: op(A) = 'T' keeps A as m rows of k floats, 'N' as k rows of m
        a_store = A if ta == "T" else np.ascontiguousarray(A.T)
        b_store = np.ascontiguousarray(B.T) if tb == "N" else B
        dA = torch.zeros((a_store.shape[0], a_store.shape[1] + pad), device=dev)
        dB = torch.zeros((b_store.shape[0], b_store.shape[1] + pad), device=dev)
        dA[:, :a_store.shape[1]] = torch.from_numpy(a_store).to(dev)
        dB[:, :b_store.shape[1]] = torch.from_numpy(b_store).to(dev)
        models = {}
        for path in (0, PACKED, FUSED, DIRECT):
            flags = path | (1 if rn else 0)
            dC = torch.full((n, m + pad), 7.0, device=dev)
            dC[:, :m] = torch.from_numpy(np.ascontiguousarray(C.T)).to(dev)
            ws = torch.empty(max(16, tc.workspace_bytes(m, n, k, 1, policy)), dtype=torch.uint8, device=dev)
            try:
                slices = tc.sgemm_k_slices(m, n, k, 1, policy, flags)
                tc.sgemm(ta, tb, m, n, k, alpha, dA, dA.shape[1], dB, dB.shape[1], beta, dC, m + pad, policy,
                         flags, ws)
            except WmmaeError as e:
                assert e.status == -4 and path in (FUSED, DIRECT), (case, path, e)
                continue
            torch.cuda.synchronize()
            got = dC.cpu().numpy()
            assert (got[:, m:] == 7.0).all(), (case, path)
            if path == 0 and (pad % 4 != 0 or (ta, tb) != ("T", "N")):
                continue            # (the count the query reports holds for 'T', 'N' and tight leading dimensions)
            if slices not in models:
                models[slices] = orc.epilogue(_model(orc, A, B, kind, ec, slices, rn), alpha, beta, C)
            want = models[slices]
            D = np.ascontiguousarray(got[:, :m].T)
            assert np.array_equal(D.view(np.uint32), want.view(np.uint32)), \
                (case, (m, n, k), policy, path, slices, alpha, beta, pad, rn, ta, tb, int((D != want).sum()))
            checked += 1
    assert checked >= 80
