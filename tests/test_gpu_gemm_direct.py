"""The third GEMM path: the packed path's MFMA kernel loading the fp32 operands itself and
splitting them on their way into LDS (WMMAE_FLAG_PATH_DIRECT forces it, the time estimates
choose it for batches of medium-sized matrices and K-heavy products).  It issues the same
products in the same order as the packed path, so every case compares bits with the packed
path forced on the same arguments; one case per group is also held against FP64.

Where K is cut into slices the two kernels plan the cut for their own tiles (256x128 only for
this kernel, 128x128 and 64x64 too for the packed path), and the slices' partial sums are
rounded: the direct path runs on its own plan, as a caller gets it, and the packed path is
given the same number of slices for the comparison."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8


def _uniform(shape, seed, dev):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.rand(shape, generator=g, dtype=torch.float32) * 2 - 1).to(dev)


def _both(tc, dev, m, n, k, batch, policy, lda=None, ldb=None, ldc=None, alpha=1.0, beta=0.0,
          a_off=0, b_off=0, workspace=True, seed=0):
    """Strided-batched 'T','N' call on the direct and on the packed path; returns both C."""
    lda, ldb, ldc = lda or k, ldb or k, ldc or m
    A = _uniform((batch * m * lda + a_off,), 11 + seed, dev)
    B = _uniform((batch * n * ldb + b_off,), 12 + seed, dev)
    C0 = _uniform((batch * n * ldc,), 13 + seed, dev)
    ws = (torch.empty(tc.workspace_bytes(m, n, k, batch, policy), dtype=torch.uint8, device=dev)
          if workspace else None)
    out = []
    slices = tc.sgemm_k_slices(m, n, k, batch, policy, DIRECT)
    for flag in (DIRECT, PACKED):
        C = C0.clone()
        with tc.forced_k_slices(slices if flag == PACKED else 0):
            tc.sgemm_strided_batched("T", "N", m, n, k, alpha, A[a_off:], lda, m * lda, B[b_off:],
                                     ldb, n * ldb, beta, C, ldc, n * ldc, batch, policy, flag, ws)
        out.append(C)
    torch.cuda.synchronize()
    return out, A[a_off:], B[b_off:], C0


@pytest.mark.parametrize("policy", [0, 1, 3, 4])
@pytest.mark.parametrize("shape", [(256, 128, 32, 1), (300, 200, 64, 1), (1000, 777, 256, 1),
                                   (1024, 1024, 96, 9), (520, 392, 1056, 5), (2048, 2304, 160, 1)])
def test_direct_path_gives_the_packed_path_bits(tc, orc, dev, policy, shape):
    """One, two, three, five and 33 stages; whole and ragged tiles; one entry, few entries
    (shared list) and nine (an XCD owns whole entries)."""
    m, n, k, batch = shape
    (d, p), A, B, _ = _both(tc, dev, m, n, k, batch, policy)
    assert torch.equal(d, p)
    if shape == (1000, 777, 256, 1):
        ref = orc.gemm_f64(A.view(m, k).cpu().numpy(), B.view(n, k).cpu().numpy().T)
        got = d.view(n, m).cpu().numpy().T
        assert orc.max_rel_err(got, ref) < {0: 4e-6, 1: 2e-3, 3: 2e-4, 4: 2e-2}[policy]


@pytest.mark.parametrize("policy", [0, 4])
def test_direct_path_any_leading_dimension_and_base(tc, dev, policy):
    """Rows that start at any float (leading dimensions that are no multiples of four, bases
    one and three floats into an allocation), a padded C, alpha and beta."""
    for (lda, ldb, a_off, b_off) in ((67, 64, 0, 0), (64, 71, 1, 0), (69, 65, 3, 1)):
        (d, p), _, _, C0 = _both(tc, dev, 300, 260, 64, 3, policy, lda=lda, ldb=ldb, ldc=304,
                                 alpha=1.5, beta=-0.25, a_off=a_off, b_off=b_off, seed=lda)
        assert torch.equal(d, p)
        pad = d.view(3, 260, 304)[:, :, 300:]
        assert torch.equal(pad, C0.view(3, 260, 304)[:, :, 300:])        # padding untouched


@pytest.mark.parametrize("policy", [0, 3])
def test_direct_path_k_slices(tc, orc, dev, policy):
    """A K-heavy product: on the same cut of K both paths fold the slices in the same order;
    without a workspace the direct path allocates the planes itself.  Then every slice count
    from one to nine forced on both paths."""
    m, n, k = 512, 384, 16384
    assert tc.sgemm_k_slices(m, n, k, 1, policy, DIRECT) > 1
    (d, p), A, B, _ = _both(tc, dev, m, n, k, 1, policy)
    assert torch.equal(d, p)
    (d2, _), _, _, _ = _both(tc, dev, m, n, k, 1, policy, workspace=False)
    assert torch.equal(d2, d)
    (d3, p3), _, _, _ = _both(tc, dev, m, n, k + 5, 1, policy)          # a shorter last stage
    assert torch.equal(d3, p3)
    (d4, _), _, _, _ = _both(tc, dev, m, n, k + 5, 1, policy, workspace=False)
    assert torch.equal(d4, d3)
    ref = orc.gemm_f64(A.view(m, k).cpu().numpy(), B.view(n, k).cpu().numpy().T)
    assert orc.max_rel_err(d.view(n, m).cpu().numpy().T, ref) < {0: 4e-6, 3: 2e-4}[policy]
    seen = set()
    for s in range(1, 10):
        res = []
        with tc.forced_k_slices(s):
            assert tc.sgemm_k_slices(m, n, k, 1, policy, DIRECT) == s
            ws = torch.empty(tc.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
            for flag in (DIRECT, PACKED):
                C = torch.zeros((n, m), dtype=torch.float32, device=dev)
                tc.sgemm("T", "N", m, n, k, 1.0, A[:m * k], k, B[:n * k], k, 0.0, C, m, policy, flag, ws)
                res.append(C)
        torch.cuda.synchronize()
        assert torch.equal(res[0], res[1]), s
        assert orc.max_rel_err(res[0].cpu().numpy().T, ref) < {0: 4e-6, 3: 2e-4}[policy]
        seen.add(res[0].cpu().numpy().tobytes())
    assert len(seen) > 1                     # the cut does show in the last bits
    assert tc.sgemm_k_slices(m, n, k, 1, policy, DIRECT) > 1      # the hook is off again


@pytest.mark.parametrize("policy", [0, 1, 3, 4])
def test_direct_path_k_not_a_multiple_of_32(tc, orc, dev, policy):
    """Any k from 4 on: the last stage of a row is shorter than 32 floats (one stage in all, a
    few, many; K slices; rows that end one to three floats into their last stage, or in the
    middle of a lane's four; rows that end at the allocation's last float)."""
    for (m, n, k, batch) in ((256, 128, 4, 1), (300, 200, 36, 3), (520, 392, 1000, 5),
                             (512, 384, 16388, 1), (1024, 1024, 100, 9), (256, 128, 5, 2),
                             (300, 200, 33, 3), (300, 200, 34, 1), (300, 200, 35, 2),
                             (520, 392, 1001, 5), (512, 384, 16387, 1), (384, 256, 31, 4),
                             (260, 130, 62, 3), (512, 512, 999, 16)):
        (d, p), A, B, _ = _both(tc, dev, m, n, k, batch, policy, seed=k)
        assert torch.equal(d, p), (m, n, k, batch)
    m, n, k = 300, 200, 36
    (d, _), A, B, _ = _both(tc, dev, m, n, k, 1, policy, seed=1)
    ref = orc.gemm_f64(A.view(m, k).cpu().numpy(), B.view(n, k).cpu().numpy().T)
    assert orc.max_rel_err(d.view(n, m).cpu().numpy().T, ref) < {0: 4e-6, 1: 2e-3, 3: 2e-4, 4: 2e-2}[policy]


def test_direct_path_staggered_start(tc, dev):
    """A launch bound by its bytes (many small matrices, two k stages a tile): the workgroups
    of an XCD start a little apart; nothing but their timing changes."""
    for policy in (0, 4):
        (d, p), _, _, _ = _both(tc, dev, 256, 256, 64, 1024, policy)
        assert torch.equal(d, p)


@pytest.mark.parametrize("k", [128, 100, 37])
def test_direct_path_pointer_arrays(tc, dev, k):
    """wmmae_tcec_sgemm_batched (device arrays of matrix pointers, test/tcec/batch_gemm.cu:433-443)
    with entries that are not 16-byte aligned; whole stages and a shorter last one."""
    m, n, batch = 384, 256, 10
    A = _uniform((batch, m * k + 3), 21, dev)
    B = _uniform((batch, n * k + 3), 22, dev)
    outs = []
    for flag in (DIRECT, PACKED):
        C = torch.zeros((batch, n * m), dtype=torch.float32, device=dev)
        pa = torch.tensor([A[e].data_ptr() + 4 * (e % 4) for e in range(batch)], dtype=torch.int64, device=dev)
        pb = torch.tensor([B[e].data_ptr() + 4 * ((e + 1) % 4) for e in range(batch)], dtype=torch.int64, device=dev)
        pc = torch.tensor([C[e].data_ptr() for e in range(batch)], dtype=torch.int64, device=dev)
        tc.sgemm_batched("T", "N", m, n, k, 1.0, pa, k, pb, k, 0.0, pc, m, batch, 0, flag)
        outs.append(C)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])


def test_direct_path_is_what_the_estimates_choose_for_the_harness_grid(tc, dev):
    """The reference harness's batched products (m = n = 512, 1024, 256 entries) and the
    K-heavy baseline product take the direct kernel; large single products do not; the
    default call gives the forced call's bits."""
    import ctypes
    from wmma_extension_amd import _lib
    out = ctypes.c_int(-1)
    for args, want in (((512, 512, 1024, 256, 0, 0), 3), ((1024, 1024, 4096, 256, 0, 0), 3),
                       ((1024, 1024, 262144, 1, 0, 0), 4), ((4096, 4096, 4096, 1, 0, 0), 1),
                       ((16384, 16384, 16384, 1, 2, 0), 1), ((2048, 2048, 2048, 1, 0, 0), 1)):
        assert _lib.lib().wmmae_tcec_sgemm_path(*args, ctypes.byref(out)) == 0
        assert out.value == want, args
    m, n, k, batch = 512, 512, 256, 24
    A = _uniform((batch, m, k), 31, dev)
    B = _uniform((batch, n, k), 32, dev)
    res = []
    for flag in (0, DIRECT):
        C = torch.zeros((batch, n, m), dtype=torch.float32, device=dev)
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, B, k, n * k, 0.0, C, m, n * m,
                                 batch, 0, flag)
        res.append(C)
    torch.cuda.synchronize()
    assert torch.equal(res[0], res[1])


def test_direct_path_turns_down_what_it_cannot_read(tc, dev):
    from wmma_extension_amd._lib import WmmaeError
    A = torch.zeros((64, 64), device=dev)
    C = torch.zeros((64, 64), device=dev)
    for kwargs in (dict(transa="N"), dict(k=3), dict(policy=2), dict(flags=DIRECT | 1)):
        a = dict(transa="T", k=64, policy=0, flags=DIRECT)
        a.update(kwargs)
        with pytest.raises(WmmaeError) as e:
            tc.sgemm(a["transa"], "N", 64, 64, a["k"], 1.0, A, 64, A, 64, 0.0, C, 64, a["policy"], a["flags"])
        assert e.value.status == -4
