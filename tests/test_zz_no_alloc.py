"""wmmae_tcec_sgemm_static (the entry point that allocates nothing) against
wmmae_tcec_sgemm on a caller-provided workspace: same bits, on two calls in a row,
the second with a smaller input so that the first call's leftovers in the shared
array would show."""
import gc

import pytest
import torch

from wmma_extension_amd import _lib, tcec

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    _lib.lib()
    return torch.device("cuda:0")


def _operands(dev, m, n, k, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    A = (torch.rand((m, k), generator=g) * 2 - 1).to(dev)
    Bt = (torch.rand((n, k), generator=g) * 2 - 1).to(dev)
    C0 = (torch.rand((n, m), generator=g) * 2 - 1).to(dev)
    return A, Bt, C0


def _both(dev, m, n, k, policy, alpha, beta, seed):
    A, Bt, C0 = _operands(dev, m, n, k, seed)
    ws = torch.empty(tcec.workspace_bytes(m, n, k, 1, policy), dtype=torch.uint8, device=dev)
    want = C0.clone()
    tcec.sgemm("T", "N", m, n, k, alpha, A, k, Bt, k, beta, want, m, policy, 0, ws)
    got = C0.clone()
    tcec.sgemm_static("T", "N", m, n, k, alpha, A, k, Bt, k, beta, got, m, policy, 0)
    torch.cuda.synchronize()
    return got, want


@pytest.mark.parametrize("policy", [tcec.Policy.F16_EC, tcec.Policy.BF16X3_EC])
def test_static_workspace_matches_caller_workspace(dev, policy):
    # first a product on packed operands with K slices, then a smaller one on packed operands,
    # then one the single kernel takes (no workspace at all)
    shapes = [(904, 1000, 1544, tcec.PATH_PACKED_SPLIT_K), (1160, 1544, 1056, tcec.PATH_PACKED),
              (200, 136, 328, tcec.PATH_FUSED)]
    for i, (m, n, k, path) in enumerate(shapes):
        assert tcec.sgemm_path(m, n, k, 1, policy) == path, (m, n, k)
        assert tcec.workspace_bytes(m, n, k, 1, policy) <= tcec.STATIC_SCRATCH_BYTES
        got, want = _both(dev, m, n, k, policy, 1.25, -0.5, 100 + i)
        assert torch.equal(got, want), (m, n, k, (got - want).abs().max().item())


DIRECT = 8


def test_static_workspace_on_the_path_that_reads_fp32_operands(dev):
    """Products the library runs on the fp32 operands directly use the array for K slices only,
    from its start (the packed path puts them behind the split operands): a product whose
    packed operands would not fit still succeeds, and the bits are those of the caller-workspace
    call.  Then the same kernel without K slices (forced), which does not touch the array."""
    pol = tcec.Policy.F16_EC
    m, n, k = 512, 384, 16384
    assert tcec.sgemm_path(m, n, k, 1, pol) == tcec.PATH_DIRECT_SPLIT_K
    assert tcec.workspace_bytes(m, n, k, 1, pol) > tcec.STATIC_SCRATCH_BYTES   # the upper bound
    assert tcec.gemm_packed_workspace_bytes(pol, m, n, k, 1) <= tcec.STATIC_SCRATCH_BYTES
    got, want = _both(dev, m, n, k, pol, 0.75, 0.5, 300)
    assert torch.equal(got, want), (got - want).abs().max().item()
    m, n, k = 1024, 520, 512
    A, Bt, C0 = _operands(dev, m, n, k, 301)
    want, got = C0.clone(), C0.clone()
    tcec.sgemm("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.0, want, m, pol, DIRECT, None)
    tcec.sgemm_static("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.0, got, m, pol, DIRECT)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_static_calls_back_to_back_share_the_array_in_stream_order(dev):
    """Calls of different paths one after the other on one stream, no synchronisation between
    them: packed operands in the array, then K-slice planes at its start, then packed operands
    again.  Stream order is all the calls need."""
    pol = tcec.Policy.F16_EC
    shapes = [(1160, 1544, 1056, 0), (512, 384, 16384, 0), (904, 1000, 1544, 0), (200, 136, 328, 0),
              (1024, 520, 512, DIRECT), (1160, 1544, 1056, 0)]
    ops = [_operands(dev, m, n, k, 400 + i) for i, (m, n, k, _) in enumerate(shapes)]
    want = []
    for (m, n, k, flags), (A, Bt, C0) in zip(shapes, ops):
        ws = torch.empty(tcec.workspace_bytes(m, n, k, 1, pol), dtype=torch.uint8, device=dev)
        c = C0.clone()
        tcec.sgemm("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.25, c, m, pol, flags, ws)
        want.append(c)
    torch.cuda.synchronize()
    got = [C0.clone() for (_, _, C0) in ops]
    torch.cuda.synchronize()
    for (m, n, k, flags), (A, Bt, _), c in zip(shapes, ops, got):
        tcec.sgemm_static("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.25, c, m, pol, flags)
    torch.cuda.synchronize()
    for sh, g, w in zip(shapes, got, want):
        assert torch.equal(g, w), (sh, (g - w).abs().max().item())


def test_static_calls_allocate_nothing(dev):
    """Device memory in use, as the runtime reports it (hipMemGetInfo) and as torch's allocator
    counts it, is the same before and after calls on every path (after one warm-up call each:
    the first launch of a kernel loads its code object)."""
    pol = tcec.Policy.F16_EC
    shapes = [(1160, 1544, 1056, 0), (512, 384, 16384, 0), (200, 136, 328, 0), (1024, 520, 512, DIRECT)]
    ops = [_operands(dev, m, n, k, 500 + i) for i, (m, n, k, _) in enumerate(shapes)]

    def run_all():
        for (m, n, k, flags), (A, Bt, C0) in zip(shapes, ops):
            tcec.sgemm_static("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.0, C0, m, pol, flags)
        torch.cuda.synchronize()
    run_all()
    gc.collect()          # tensors that earlier tests left to the collector go now, not below
    free0, _ = torch.cuda.mem_get_info(dev)
    alloc0, reserved0 = torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)
    for _ in range(3):
        run_all()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_allocated(dev) == alloc0
    assert torch.cuda.memory_reserved(dev) == reserved0


def test_static_workspace_result_is_right(dev):
    m, n, k = 1160, 1544, 1056
    A, Bt, _ = _operands(dev, m, n, k, 7)
    C = torch.empty((n, m), dtype=torch.float32, device=dev)
    tcec.sgemm_static("T", "N", m, n, k, 1.0, A, k, Bt, k, 0.0, C, m, tcec.Policy.F16_EC, 0)
    ref = (A.double() @ Bt.double().t()).t()
    err = ((C.double() - ref).abs().max() / ref.abs().max()).item()
    assert err < 2e-6, err


def test_static_workspace_rejects_what_does_not_fit(dev):
    m = n = k = 4096                      # 128 MiB of split operands
    assert tcec.sgemm_path(m, n, k, 1, tcec.Policy.F16_EC) != tcec.PATH_FUSED
    assert tcec.workspace_bytes(m, n, k, 1, tcec.Policy.F16_EC) > tcec.STATIC_SCRATCH_BYTES
    A = torch.zeros((m, k), device=dev)
    C = torch.full((n, m), 3.0, device=dev)
    with pytest.raises(_lib.WmmaeError) as e:
        tcec.sgemm_static("T", "N", m, n, k, 1.0, A, k, A, k, 0.0, C, m, tcec.Policy.F16_EC, 0)
    assert e.value.status == -5
    torch.cuda.synchronize()
    assert bool((C == 3.0).all())          # nothing was launched
