"""Products whose element counts and byte offsets pass 2^31 and 2^32: every index the kernels
form from a row, a column, a leading dimension or a batch stride has to be 64 bits wide.

  * C with more than 2^31 elements (46400 x 46400, 8.6 GB);
  * rows of an operand 64 MiB apart (a leading dimension of 2^24 + 4 floats);
  * batch entries 2^31 + 64 elements apart, in an operand and in C;
  * 200000 batch entries (more than a launch's grid holds in one dimension).

Each on the library's choice and on every path forced, against FP64 on the GPU (whole result, or
for the large C the first, last and some middle rows and columns).  The direct kernel keeps its
row offsets in 32 bits and turns leading dimensions of 2^24 floats and more down (status -4).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8


def _rel_err(got, ref):
    return (got.double() - ref).abs().max().item() / (ref.abs().max().item() + 1e-30)


def _each_path(tc, dev, m, n, k, batch, call, unsupported=()):
    from wmma_extension_amd._lib import WmmaeError
    ws = torch.empty(max(16, tc.workspace_bytes(m, n, k, batch, 0)), dtype=torch.uint8, device=dev)
    for flag in (0, PACKED, FUSED, DIRECT):
        if flag in unsupported:
            with pytest.raises(WmmaeError) as e:
                call(flag, ws)
            assert e.value.status == -4
            continue
        call(flag, ws)
        torch.cuda.synchronize()
        yield flag


def test_result_with_more_than_2_31_elements(tc, dev):
    m = n = 46400
    k = 64
    g = torch.Generator(device=dev).manual_seed(1)
    A = torch.rand((m, k), generator=g, device=dev) * 2 - 1
    B = torch.rand((n, k), generator=g, device=dev) * 2 - 1
    C = torch.empty((n, m), device=dev)
    assert C.numel() > 1 << 31
    pick = torch.tensor([0, 1, 255, 256, 12345, 23199, 23200, 46143, 46144, 46398, 46399], device=dev)
    rows_ref = B.double() @ A[pick].double().t()         # columns `pick` of the stored (n, m) array
    cols_ref = B[pick].double() @ A.double().t()

    def call(flag, ws):
        C.fill_(7.0)
        tc.sgemm("T", "N", m, n, k, 1.0, A, k, B, k, 0.0, C, m, 0, flag, ws)
    for flag in _each_path(tc, dev, m, n, k, 1, call):
        assert _rel_err(C[:, pick], rows_ref) < 1e-6, flag
        assert _rel_err(C[pick, :], cols_ref) < 1e-6, flag


def test_rows_64_mib_apart(tc, dev):
    m = n = 256
    k = 128
    lda = (1 << 24) + 4
    g = torch.Generator(device=dev).manual_seed(2)
    Abuf = torch.empty((m, lda), device=dev)
    Abuf[:, :k] = torch.rand((m, k), generator=g, device=dev) * 2 - 1
    B = torch.rand((n, k), generator=g, device=dev) * 2 - 1
    ref = B.double() @ Abuf[:, :k].double().t()
    C = torch.empty((n, m), device=dev)

    def call(flag, ws):
        C.fill_(7.0)
        tc.sgemm("T", "N", m, n, k, 1.0, Abuf, lda, B, k, 0.0, C, m, 0, flag, ws)
    for flag in _each_path(tc, dev, m, n, k, 1, call, unsupported=(DIRECT,)):
        assert _rel_err(C, ref) < 1e-6, flag


def test_batch_entries_2_31_elements_apart(tc, dev):
    batch, m, n, k = 3, 128, 128, 128
    stride = (1 << 31) + 64
    g = torch.Generator(device=dev).manual_seed(3)
    Abuf = torch.empty((2 * stride + m * k,), device=dev)
    Cbuf = torch.empty((2 * stride + m * n,), device=dev)
    B = torch.rand((batch, n, k), generator=g, device=dev) * 2 - 1
    refs = []
    for b in range(batch):
        a = torch.rand((m, k), generator=g, device=dev) * 2 - 1
        Abuf[b * stride: b * stride + m * k] = a.reshape(-1)
        refs.append(B[b].double() @ a.double().t())

    def call(flag, ws):
        for b in range(batch):
            Cbuf[b * stride: b * stride + m * n] = 7.0
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, Abuf, k, stride, B, k, n * k, 0.0,
                                 Cbuf, m, stride, batch, 0, flag, ws)
    for flag in _each_path(tc, dev, m, n, k, batch, call):
        for b in range(batch):
            assert _rel_err(Cbuf[b * stride: b * stride + m * n].reshape(n, m), refs[b]) < 1e-6, (flag, b)


def test_two_hundred_thousand_entries(tc, dev):
    batch, m, n, k = 200000, 24, 24, 24
    g = torch.Generator(device=dev).manual_seed(4)
    A = torch.rand((batch, m, k), generator=g, device=dev) * 2 - 1
    B = torch.rand((batch, n, k), generator=g, device=dev) * 2 - 1
    ref = torch.bmm(B.double(), A.double().transpose(1, 2))
    C = torch.empty((batch, n, m), device=dev)

    def call(flag, ws):
        C.fill_(7.0)
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, B, k, n * k, 0.0,
                                 C, m, n * m, batch, 0, flag, ws)
    for flag in _each_path(tc, dev, m, n, k, batch, call):
        assert _rel_err(C, ref) < 1e-6, flag
