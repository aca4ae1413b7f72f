"""The packed GEMM kernel hands its (tile, batch entry, K slice) items to workgroups in
three ways (persistent workgroups with XCD-owned batch entries, persistent workgroups on
one shared list, one workgroup per item).  Which one runs depends only on the shape, and
none of them may change a single bit of the result: every case below computes the same
product twice, once in a shape that takes the schedule under test and once cut into
pieces small enough for one workgroup per item, and compares the bytes.  One piece is also
checked against FP64 to the driver's accuracy bound."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TERMS = {0: 2, 1: 1, 2: 3, 3: 2, 4: 1}   # terms per operand element of each policy


def _uniform(shape, seed, dev):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.rand(shape, generator=g, dtype=torch.float32) * 2 - 1).to(dev)


def _pack(tc, policy, X, dev):
    """X: (batch, rows, k) fp32 on the device -> packed bytes, bytes per entry."""
    batch, rows, k = X.shape
    per = tc.pack_bytes(rows, k, 1, policy)
    assert tc.pack_bytes(rows, k, batch, policy) == per * batch
    p = torch.empty(per * batch, dtype=torch.uint8, device=dev)
    tc.pack(policy, rows, k, X, k, 1, p, batch, rows * k)
    return p, per


def _fp64_check(orc, A, B, C, policy):
    ref = orc.gemm_f64(A.cpu().numpy(), B.cpu().numpy().T)
    got = C.cpu().numpy().T
    assert orc.max_rel_err(got, ref) < {0: 4e-6, 2: 4e-6, 1: 2e-3, 3: 2e-4, 4: 2e-2}[policy]


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(1024, 1024, 160, 9), (520, 1000, 64, 21), (1024, 1024, 32, 9),
                                   (512, 512, 2080, 36)])
def test_xcd_owned_batch_entries_equal_single_entry_calls(tc, orc, dev, policy, shape):
    """8 or more entries and more items than resident workgroups: an XCD walks whole entries,
    requests run on into the next item (1, 2, 5 and 65 stages per item, odd and even)."""
    m, n, k, batch = shape
    A = _uniform((batch, m, k), 100 + k, dev)
    B = _uniform((batch, n, k), 200 + k, dev)
    C0 = _uniform((batch, n, m), 300 + k, dev)
    pa, per_a = _pack(tc, policy, A, dev)
    pb, per_b = _pack(tc, policy, B, dev)
    C = C0.clone()
    tc.gemm_packed(policy, m, n, k, 1.25, pa, pb, -0.5, C, m, batch, m * n)
    ref = C0.clone()
    for e in range(batch):
        tc.gemm_packed(policy, m, n, k, 1.25, pa[e * per_a:(e + 1) * per_a],
                       pb[e * per_b:(e + 1) * per_b], -0.5, ref[e], m)
    torch.cuda.synchronize()
    assert torch.equal(C, ref)
    e = batch - 1
    plain = torch.zeros((n, m), dtype=torch.float32, device=dev)
    tc.gemm_packed(policy, m, n, k, 1.0, pa[e * per_a:(e + 1) * per_a],
                   pb[e * per_b:(e + 1) * per_b], 0.0, plain, m)
    _fp64_check(orc, A[e], B[e], plain, policy)


@pytest.mark.parametrize("policy", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(4096, 4096, 96, 1), (2048, 3000, 40, 3), (4096, 2048, 1024, 2),
                                   (4096, 4096, 32, 1), (4096, 4096, 64, 1), (4096, 4096, 160, 1)])
def test_persistent_shared_list_equals_column_blocks(tc, orc, dev, policy, shape):
    """Few entries, short K loops, more tiles than resident workgroups: persistent
    workgroups on one list.  The same product from column blocks of 512 columns of B
    (few enough tiles for one workgroup each) has to agree bit for bit.  The whole products
    take the 256x128 tile (with three terms: one copy of the A fragments and a ring of two
    stages), the column blocks the 128x128 tile; 1, 2, 3, 5 and 32 stages per item."""
    m, n, k, batch = shape
    A = _uniform((batch, m, k), 400 + k, dev)
    B = _uniform((batch, n, k), 500 + k, dev)
    pa, per_a = _pack(tc, policy, A, dev)
    pb, per_b = _pack(tc, policy, B, dev)
    C = torch.full((batch, n, m), 7.0, dtype=torch.float32, device=dev)
    tc.gemm_packed(policy, m, n, k, 1.0, pa, pb, 0.0, C, m, batch, m * n)
    ref = torch.full((batch, n, m), 7.0, dtype=torch.float32, device=dev)
    kt = (k + 31) // 32
    rb_bytes = kt * TERMS[policy] * 1024            # one 16-row block of a packed operand
    blk = 512
    for e in range(batch):
        for c0 in range(0, n, blk):
            cols = min(blk, n - c0)
            pbe = pb[e * per_b + (c0 // 16) * rb_bytes:(e + 1) * per_b]
            tc.gemm_packed(policy, m, cols, k, 1.0, pa[e * per_a:(e + 1) * per_a], pbe, 0.0,
                           ref[e, c0:c0 + cols], m)
    torch.cuda.synchronize()
    assert torch.equal(C, ref)
    if m * n * k <= 4096 * 4096 * 96:
        _fp64_check(orc, A[0], B[0], C[0], policy)


@pytest.mark.parametrize("policy,slabs", [(0, 2), (2, 2), (2, 4)])
def test_one_workgroup_per_item_for_long_k(tc, orc, dev, policy, slabs):
    """Many tiles with 64 or more stages each and a single entry: one workgroup per item.
    Rows of A in two halves (the 256x128 tile again) or, with three terms, in four slabs
    of 1024 rows (256 tiles of 128x128: the smaller tile) give the same bits."""
    m, n, k = 4096, 4096, 2048 + 32
    A = _uniform((1, m, k), 7, dev)
    B = _uniform((1, n, k), 8, dev)
    pa, _ = _pack(tc, policy, A, dev)
    pb, _ = _pack(tc, policy, B, dev)
    C = torch.zeros((n, m), dtype=torch.float32, device=dev)
    tc.gemm_packed(policy, m, n, k, 1.0, pa, pb, 0.0, C, m)
    ref = torch.zeros((n, m), dtype=torch.float32, device=dev)
    part = m // slabs
    rb_bytes = ((k + 31) // 32) * TERMS[policy] * 1024
    for r0 in range(0, m, part):
        # rows r0 .. r0+part of C: the column-major slab starts at element r0 of every column
        tc.gemm_packed(policy, part, n, k, 1.0, pa[(r0 // 16) * rb_bytes:], pb, 0.0,
                       ref.view(-1)[r0:], m)
    torch.cuda.synchronize()
    assert torch.equal(C, ref)


@pytest.mark.parametrize("policy", [0, 2])
def test_pointer_arrays_through_packed_operands_and_xcd_owned_entries(tc, orc, dev, policy):
    """wmmae_tcec_sgemm_batched (device arrays of matrix pointers, test/tcec/batch_gemm.cu:433-443)
    on a batch that goes through packed operands with more items than resident workgroups,
    leading product accumulated outside the matrix core: same bits as the strided call on a
    copy of the same matrices, FP64 agreement on one entry."""
    batch, m, n, k = 10, 2048, 1792, 512
    assert tc.sgemm_path(m, n, k, batch, policy, 1) == tc.PATH_PACKED
    A = _uniform((batch, m, k), 31, dev)
    B = _uniform((batch, n, k), 32, dev)
    # entries scattered in memory, in another order than the strided copy
    As = [A[e].clone() for e in reversed(range(batch))][::-1]
    Bs = [B[e].clone() for e in range(batch)]
    Cs = [torch.full((n, m), 2.0, dtype=torch.float32, device=dev) for _ in range(batch)]
    pa = torch.tensor([t.data_ptr() for t in As], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in Bs], dtype=torch.int64, device=dev)
    pc = torch.tensor([t.data_ptr() for t in Cs], dtype=torch.int64, device=dev)
    ws = torch.empty(tc.workspace_bytes(m, n, k, batch, policy), dtype=torch.uint8, device=dev)
    tc.sgemm_batched("T", "N", m, n, k, 0.5, pa, k, pb, k, 1.5, pc, m, batch, policy, 1, ws)
    C = torch.full((batch, n, m), 2.0, dtype=torch.float32, device=dev)
    tc.sgemm_strided_batched("T", "N", m, n, k, 0.5, A, k, m * k, B, k, n * k, 1.5, C, m, m * n,
                             batch, policy, 1, ws)
    torch.cuda.synchronize()
    for e in range(batch):
        assert torch.equal(Cs[e], C[e]), e
    e = 7
    ref = 0.5 * orc.gemm_f64(A[e].cpu().numpy(), B[e].cpu().numpy().T) + 3.0
    assert orc.max_rel_err(C[e].cpu().numpy().T, ref) < 4e-6


def test_random_shapes_packed_path_and_driver_choice_agree(tc, orc, dev):
    """120 seeded problems (1..5000 rows and columns, 1..3000 of k, 1..40 entries, all five
    policies): pack + gemm_packed and the driver's own choice of path give the same bits
    wherever the driver does not cut the K loop into slices (the partial sums of slices are
    rounded on their own), and both stay within the policy's error bound of an FP64 product
    computed on the GPU."""
    import random
    rnd = random.Random(20240)
    bound = {0: 4e-6, 2: 4e-6, 1: 3e-3, 3: 3e-4, 4: 3e-2}
    sliced = 0
    for case in range(120):
        policy = rnd.choice([0, 0, 2, 2, 1, 3, 4])
        batch = rnd.choice([1, 1, 1, 2, 3, 9, 17, 40])
        big = rnd.random() < 0.5
        m = rnd.randint(1, 5000 if big else 700)
        n = rnd.randint(1, 5000 if big else 700)
        k = rnd.randint(1, 700 if batch * m * n > 4e6 else 3000)
        while batch * (m * k + n * k + m * n) * 4 > 1.0e9:
            batch = max(1, batch // 2)
            m = max(1, m // 2)
        A = _uniform((batch, m, k), 1000 + case, dev)
        B = _uniform((batch, n, k), 2000 + case, dev)
        ref = torch.matmul(A.double(), B.double().transpose(1, 2))
        scale = ref.abs().amax(dim=(1, 2)).clamp_min(1e-30)
        pa, _ = _pack(tc, policy, A, dev)
        pb, _ = _pack(tc, policy, B, dev)
        C = torch.full((batch, n, m), float("nan"), device=dev)
        tc.gemm_packed(policy, m, n, k, 1.0, pa, pb, 0.0, C, m, batch, m * n)
        C2 = torch.full((batch, n, m), float("nan"), device=dev)
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, B, k, n * k, 0.0, C2, m, m * n,
                                 batch, policy)
        err = ((C.transpose(1, 2).double() - ref).abs().amax(dim=(1, 2)) / scale).max().item()
        tag = (case, policy, batch, m, n, k)
        assert err < bound[policy], tag
        if tc.sgemm_path(m, n, k, batch, policy, 0) in (tc.PATH_PACKED_SPLIT_K, tc.PATH_DIRECT_SPLIT_K):
            sliced += 1
            err2 = ((C2.transpose(1, 2).double() - ref).abs().amax(dim=(1, 2)) / scale).max().item()
            assert err2 < bound[policy], tag
        else:
            assert torch.equal(C, C2), tag
    assert 0 < sliced < 40, sliced


@pytest.mark.parametrize("policy", [0, 2])
@pytest.mark.parametrize("shape", [(5120, 5120, 2304), (2304, 2304, 4096), (4000, 4500, 2100)])
def test_k_slices_for_the_last_round_of_tiles(tc, orc, dev, policy, shape):
    """Tile counts that leave the last round over the compute units mostly empty: with room
    in the workspace the tiles of that round are cut along K and folded afterwards.  The
    tiles of the whole rounds keep their bits, the cut ones agree with the uncut run to
    rounding of the partial sums, and both agree with FP64."""
    m, n, k = shape
    assert tc.gemm_packed_workspace_bytes(policy, m, n, k) > 0
    A = _uniform((1, m, k), 61, dev)
    B = _uniform((1, n, k), 62, dev)
    C0 = _uniform((n, m), 63, dev)
    pa, _ = _pack(tc, policy, A, dev)
    pb, _ = _pack(tc, policy, B, dev)
    plain = C0.clone()
    tc.gemm_packed(policy, m, n, k, 0.75, pa, pb, 0.5, plain, m)              # no workspace: uncut
    ws = torch.empty(tc.gemm_packed_workspace_bytes(policy, m, n, k), dtype=torch.uint8, device=dev)
    cut = C0.clone()
    tc.gemm_packed(policy, m, n, k, 0.75, pa, pb, 0.5, cut, m, workspace=ws)
    again = C0.clone()
    tc.gemm_packed(policy, m, n, k, 0.75, pa, pb, 0.5, again, m, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(cut, again)                                            # deterministic
    differ = (cut != plain)
    frac = differ.float().mean().item()
    assert 0.0 < frac < 0.5                      # only the last round's tiles were cut
    ref = 0.75 * torch.matmul(A[0].double(), B[0].double().T).T + 0.5 * C0.double()
    scale = ref.abs().max()
    assert ((cut.double() - ref).abs().max() / scale).item() < 4e-6
    assert ((plain.double() - ref).abs().max() / scale).item() < 4e-6
    assert ((cut - plain).abs().max().double() / scale).item() < 1e-6


def test_random_blas_arguments_against_fp64(tc, dev):
    """100 seeded calls of the strided-batched entry point the way a BLAS user makes them:
    both transposes of both operands, padded leading dimensions, alpha and beta other than
    1 and 0, the round-to-nearest flag, with and without a caller's workspace, shapes drawn
    so that all paths (fused, packed, packed with K slices, direct with and without K
    slices) are taken.  Each result is
    compared with alpha * op(A) op(B) + beta * C in FP64, and the padding rows of C
    (ldc > m) must keep their bytes."""
    import random
    rnd = random.Random(77)
    bound = {0: 4e-6, 2: 4e-6, 1: 3e-3, 3: 3e-4, 4: 3e-2}
    paths = [0, 0, 0, 0, 0]
    forced_direct = 0
    for case in range(100):
        policy = rnd.choice([0, 0, 2, 2, 1, 3, 4])
        batch = rnd.choice([1, 1, 1, 1, 2, 3, 9])
        kind = rnd.random()
        if kind < 0.4:      # small outputs, long k
            m, n, k = rnd.randint(1, 1200), rnd.randint(1, 1200), rnd.randint(1000, 30000)
        elif kind < 0.7:
            m, n, k = rnd.randint(1, 3000), rnd.randint(1, 3000), rnd.randint(1, 4000)
        else:
            m, n, k = rnd.randint(1, 600), rnd.randint(1, 600), rnd.randint(1, 600)
        while batch * (m * k + n * k + m * n) * 4 > 6.0e8:
            if batch > 1:
                batch //= 2
            else:
                k = max(1, k // 2)
        ta, tb = rnd.choice("NT"), rnd.choice("NT")
        readable = rnd.random() < 0.35  # what the direct kernel can read: 'T','N', k % 32 == 0
        if readable:
            ta, tb, k = "T", "N", max(32, k // 32 * 32)
        # column-major storage: A holds ra x ca elements, ra contiguous, in columns of lda
        ra, ca = (m, k) if ta == "N" else (k, m)
        rb, cb = (k, n) if tb == "N" else (n, k)
        lda, ldb, ldc = (x + rnd.choice([0, 0, 1, 3, 4, 16]) for x in (ra, rb, m))
        A = _uniform((batch, ca, lda), 5000 + case, dev)      # [entry, column, row]
        B = _uniform((batch, cb, ldb), 6000 + case, dev)
        C0 = _uniform((batch, n, ldc), 7000 + case, dev)
        alpha = rnd.choice([1.0, 1.0, -0.5, 2.25])
        beta = rnd.choice([0.0, 0.0, 1.0, -1.5])
        flags = rnd.choice([0, 0, 0, tc.FLAG_RN_MAIN]) if policy in (0, 2) else 0
        if readable and policy != 2 and flags == 0 and rnd.random() < 0.7:
            flags = tc.FLAG_PATH_DIRECT                       # else the estimates decide
            forced_direct += 1
        a_cm = A[:, :, :ra].double()                          # [entry, column, row]
        b_cm = B[:, :, :rb].double()
        op_a = a_cm.transpose(1, 2) if ta == "N" else a_cm    # (entry, m, k)
        op_b = b_cm.transpose(1, 2) if tb == "N" else b_cm    # (entry, k, n)
        prod = torch.matmul(op_a, op_b)
        ref = alpha * prod + beta * C0[:, :, :m].transpose(1, 2).double()
        scale = (abs(alpha) * prod.abs().amax(dim=(1, 2)) + abs(beta)).clamp_min(1e-30)
        ws = None
        if rnd.random() < 0.7:
            ws = torch.empty(max(16, tc.workspace_bytes(m, n, k, batch, policy)), dtype=torch.uint8,
                             device=dev)
        C = C0.clone()
        tc.sgemm_strided_batched(ta, tb, m, n, k, alpha, A, lda, ca * lda, B, ldb, cb * ldb, beta,
                                 C, ldc, n * ldc, batch, policy, flags, ws)
        err = ((C[:, :, :m].transpose(1, 2).double() - ref).abs().amax(dim=(1, 2)) / scale).max().item()
        tag = (case, policy, flags, batch, ta + tb, m, n, k, lda, ldb, ldc, alpha, beta, ws is not None)
        assert err < bound[policy], (tag, err)
        assert torch.equal(C[:, :, m:], C0[:, :, m:]), tag
        paths[tc.sgemm_path(m, n, k, batch, policy, flags & tc.FLAG_RN_MAIN)] += 1
    assert min(paths[:3]) >= 10 and forced_direct >= 10, (paths, forced_direct)
