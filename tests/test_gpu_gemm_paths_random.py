"""Random products through every path of the driver (the library's choice, and the packed, the
single-kernel and the direct path forced), all four transpose combinations, padded leading
dimensions, alpha / beta, one to forty entries, dimensions that are no multiples of anything:

  * every result within the policy's tolerance of FP64 (reference metric, test/primitive/common.hpp:54-103);
  * the padding of C untouched;
  * the default call gives the bits of the forced path it reports (wmmae_tcec_sgemm_path);
  * the paths give each other's bits wherever they cut K alike (they issue the same products in the
    same order on the same accumulators); a case with much larger shapes, where the packed path
    also cuts K for the tiles of its last round, is compared with that cut switched off.
"""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8
TOL = {0: 4e-6, 1: 3e-3, 2: 4e-6, 3: 3e-4, 4: 3e-2}


def _cases(seed, count):
    rnd = random.Random(seed)

    def dim(lo, hi):
        return max(1, int(2 ** rnd.uniform(lo, hi)) + rnd.choice([0, 0, 0, 1, -1, 3, 5, 17]))
    out = []
    while len(out) < count:
        batch = rnd.choice([1, 1, 1, 2, 3, 5, 9, 17, 40])
        m, n = dim(3, 11.5), dim(3, 11.5)
        k = dim(2, 14.5) if batch == 1 else dim(2, 11)
        if (m * k + n * k + m * n) * batch * 4 > 3e8 or 2.0 * m * n * k * batch > 1e11:
            continue
        out.append(dict(m=m, n=n, k=k, batch=batch, policy=rnd.choice([0, 0, 1, 2, 3, 4]),
                        trans=rnd.choice([("T", "N")] * 3 + [("N", "N"), ("N", "T"), ("T", "T")]),
                        ab=rnd.choice([(1.0, 0.0), (1.0, 0.0), (1.5, -0.25), (-0.5, 1.0)]),
                        pad=rnd.choice([0, 0, 1, 4, 7])))
    return out


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_products_on_every_path(tc, dev, seed):
    from wmma_extension_amd._lib import WmmaeError
    for it, c in enumerate(_cases(seed, 60)):
        m, n, k, batch, policy, pad = c["m"], c["n"], c["k"], c["batch"], c["policy"], c["pad"]
        (ta, tb), (alpha, beta) = c["trans"], c["ab"]
        lda = (k if ta == "T" else m) + pad
        ldb = (k if tb == "N" else n) + pad
        ldc = m + pad
        g = torch.Generator(device="cpu").manual_seed(seed * 100003 + it)
        A = (torch.rand((batch, (m if ta == "T" else k), lda), generator=g) * 2 - 1).to(dev)
        B = (torch.rand((batch, (n if tb == "N" else k), ldb), generator=g) * 2 - 1).to(dev)
        C0 = (torch.rand((batch, n, ldc), generator=g) * 2 - 1).to(dev)
        a_op = A[:, :, :k].double() if ta == "T" else A[:, :, :m].double().transpose(1, 2)
        b_op = B[:, :, :k].double() if tb == "N" else B[:, :, :n].double().transpose(1, 2)
        ref = alpha * torch.bmm(b_op, a_op.transpose(1, 2)) + beta * C0[:, :, :m].double()
        scale = ref.abs().max().item() + 1e-30
        res, slices = {}, {}
        for flag in (0, PACKED, FUSED, DIRECT):
            C = C0.clone()
            ws = torch.empty(max(16, tc.workspace_bytes(m, n, k, batch, policy)), dtype=torch.uint8, device=dev)
            try:
                slices[flag] = tc.sgemm_k_slices(m, n, k, batch, policy, flag)
                tc.sgemm_strided_batched(ta, tb, m, n, k, alpha, A, lda, A.stride(0), B, ldb, B.stride(0),
                                         beta, C, ldc, n * ldc, batch, policy, flag, ws)
            except WmmaeError as e:
                # the direct kernel wants k contiguous in both operands, k >= 4, at most two terms
                assert flag == DIRECT and e.status == -4, (c, flag, e)
                assert (ta, tb) != ("T", "N") or k < 4 or policy == 2, c
                continue
            torch.cuda.synchronize()
            assert torch.equal(C[:, :, m:], C0[:, :, m:]), (c, flag)
            err = (C[:, :, :m].double() - ref).abs().max().item() / scale
            assert err <= TOL[policy] * (3 if beta != 0 else 1), (c, flag, err)
            res[flag] = C
        chosen = {0: FUSED, 1: PACKED, 2: PACKED, 3: DIRECT, 4: DIRECT}[tc.sgemm_path(m, n, k, batch, policy, 0)]
        if (ta, tb) == ("T", "N") and pad % 4 == 0:
            # (the path query assumes op(A) = 'T', op(B) = 'N', tight leading dimensions and
            # aligned bases: what the kernels can read 16 bytes at a time depends on those)
            assert torch.equal(res[0], res[chosen]), (c, chosen)
        # (a single large product may also cut K for the tiles of a partly empty last round, with
        # planes in the workspace: those tiles then sum in another order)
        tail_planes = slices[PACKED] == 1 and tc.gemm_packed_workspace_bytes(policy, m, n, k, batch) > 0
        if slices[PACKED] == 1 and not tail_planes:
            assert torch.equal(res[FUSED], res[PACKED]), c
        if DIRECT in res and slices[DIRECT] == slices[PACKED] and not tail_planes:
            assert torch.equal(res[DIRECT], res[PACKED]), c


def test_tail_slices_are_the_only_difference_on_a_large_single_product(tc, orc, dev):
    """2293 x 1802 x 5518: the packed path, given room for them, cuts K for the tiles of its partly
    empty last round, and those tiles come out with other last bits; with a workspace that only
    holds the packed operands it gives the bits of the direct and of the single kernel, with
    alpha and beta too."""
    m, n, k, policy = 2293, 1802, 5518, 0
    g = torch.Generator(device="cpu").manual_seed(5)
    A = (torch.rand((m, k), generator=g) * 2 - 1).to(dev)
    B = (torch.rand((n, k), generator=g) * 2 - 1).to(dev)
    C0 = (torch.rand((n, m), generator=g) * 2 - 1).to(dev)
    full = tc.workspace_bytes(m, n, k, 1, policy)
    operands = tc.pack_bytes(m, k, 1, policy) + tc.pack_bytes(n, k, 1, policy)
    assert full > operands and tc.sgemm_k_slices(m, n, k, 1, policy, PACKED) == 1
    for alpha, beta in ((1.0, 0.0), (-0.5, 1.0)):
        out = {}
        for name, flag, size in (("packed", PACKED, operands), ("tail", PACKED, full), ("direct", DIRECT, full),
                                 ("fused", FUSED, 0)):
            C = C0.clone()
            ws = torch.empty(size, dtype=torch.uint8, device=dev) if size else None
            tc.sgemm("T", "N", m, n, k, alpha, A, k, B, k, beta, C, m, policy, flag, ws)
            out[name] = C
        torch.cuda.synchronize()
        assert torch.equal(out["direct"], out["packed"]) and torch.equal(out["fused"], out["packed"])
        differing = int((out["tail"] != out["packed"]).sum())
        assert 0 < differing < m * n // 4
        scale = out["packed"].abs().max().item()
        assert (out["tail"] - out["packed"]).abs().max().item() < 1e-5 * scale
        if (alpha, beta) == (1.0, 0.0):
            _tail_tiles_follow_the_model(orc, A, B, out["packed"], out["tail"], k)


def _tail_tiles_follow_the_model(orc, A, B, whole, cut, k):
    """Sampled rows of the two results above against the oracle's model of the matrix core: the
    uncut run is the model over all of k; an element of the cut run is either that or the model
    over K slices of equal whole stages (2 .. 16 of them, one count for the whole product), the
    slices added in double precision - and both kinds occur (the cut tiles are the last of the
    walk through the tile grid: the bottom rows of C)."""
    import numpy as np
    m = A.shape[0]
    rows = [0, 777, m - 300, m - 130, m - 2, m - 1]
    a = A[rows].cpu().numpy()
    bt = B.cpu().numpy()
    got_whole = np.ascontiguousarray(whole[:, rows].cpu().numpy().T)
    got_cut = np.ascontiguousarray(cut[:, rows].cpu().numpy().T)

    def model(ka, kb):
        ap = np.zeros((len(rows), 32 * (-(-(kb - ka) // 32))), np.float32)
        bp = np.zeros((ap.shape[1], bt.shape[0]), np.float32)
        ap[:, :kb - ka], bp[:kb - ka, :] = a[:, ka:kb], bt[:, ka:kb].T
        return orc.tcec_matmul(ap, bp, kind=orc.SPLIT_F16, ec=True, fk=32, main_outside=False, hw_model=True)
    full = model(0, k)
    assert np.array_equal(got_whole.view(np.uint32), full.view(np.uint32))
    other = got_cut.view(np.uint32) != full.view(np.uint32)
    assert other.any() and not other.all()
    stages = (k + 31) // 32
    explained = []
    for count in range(2, 17):
        per = -(-stages // count)
        if -(-stages // per) != count:
            continue
        total = np.zeros(full.shape, np.float64)
        for s0 in range(0, stages, per):
            total += model(32 * s0, min(k, 32 * (s0 + per))).astype(np.float64)
        if np.array_equal(got_cut.view(np.uint32)[other], total.astype(np.float32).view(np.uint32)[other]):
            explained.append(count)
    assert len(explained) >= 1, "no slice count explains the cut tiles"
