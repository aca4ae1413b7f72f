"""wmmae_tcec_sgemm_static (the entry point that allocates nothing) against
wmmae_tcec_sgemm on a caller-provided workspace: same bits, on two calls in a row,
the second with a smaller input so that the first call's leftovers in the shared
array would show."""
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
    shapes = [(520, 392, 8192, tcec.PATH_PACKED_SPLIT_K), (1160, 1544, 1056, tcec.PATH_PACKED),
              (200, 136, 328, tcec.PATH_FUSED)]
    for i, (m, n, k, path) in enumerate(shapes):
        assert tcec.sgemm_path(m, n, k, 1, policy) == path, (m, n, k)
        assert tcec.workspace_bytes(m, n, k, 1, policy) <= tcec.STATIC_SCRATCH_BYTES
        got, want = _both(dev, m, n, k, policy, 1.25, -0.5, 100 + i)
        assert torch.equal(got, want), (m, n, k, (got - want).abs().max().item())


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
