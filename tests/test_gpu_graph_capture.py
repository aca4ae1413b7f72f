"""The driver under HIP graph capture.  With a workspace from the caller - or through the entry
point that allocates nothing - a call is kernel launches only (no allocation, no memset, no
host synchronisation), so it can be captured once and replayed: every path of the driver, K
slices included, replayed four times with new operands in the same buffers, the program's own
eager work and synchronisations in between, gives the bits of the eager calls.  One eager call
per kernel comes first (the first launch of a kernel sets its LDS limit, the first use of the
fixed array looks it up)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8
CASES = [(0, 700, 520, 1000, 1, 0), (2, 1288, 1032, 1000, 1, PACKED), (0, 256, 256, 256, 64, DIRECT),
         (0, 128, 128, 20000, 1, 0), (1, 96, 80, 72, 9, FUSED), (0, 1024, 1024, 8192, 1, DIRECT)]


def test_captured_calls_replay_with_the_eager_bits(tc, dev):
    g = torch.Generator(device=dev).manual_seed(9)
    bufs = []
    for (policy, m, n, k, batch, _) in CASES:
        bufs.append((torch.rand((batch, m, k), generator=g, device=dev) * 2 - 1,
                     torch.rand((batch, n, k), generator=g, device=dev) * 2 - 1,
                     torch.full((batch, n, m), 5.0, device=dev),
                     torch.empty(max(16, tc.workspace_bytes(m, n, k, batch, policy)), dtype=torch.uint8, device=dev)))
    c_static = torch.full((520, 700), 5.0, device=dev)

    def run_all():
        for (policy, m, n, k, batch, flag), (A, B, C, ws) in zip(CASES, bufs):
            tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, B, k, n * k, 0.0, C, m, n * m,
                                     batch, policy, flag, ws)
        tc.sgemm_static("T", "N", 700, 520, 1000, 1.0, bufs[0][0], 1000, bufs[0][1], 1000, 0.0, c_static, 700, 0, 0)
    run_all()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all()
    torch.cuda.synchronize()
    for rep in range(4):
        for (A, B, C, ws) in bufs:
            A.copy_(torch.rand(A.shape, generator=g, device=dev) * 2 - 1)
            B.copy_(torch.rand(B.shape, generator=g, device=dev) * 2 - 1)
            C.fill_(float(rep))
            ws.fill_(rep)                                 # nothing left over from the last run is relied on
        c_static.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        got = [b[2].clone() for b in bufs] + [c_static.clone()]
        for b in bufs:
            b[2].fill_(9.0)
        c_static.fill_(9.0)
        run_all()
        torch.cuda.synchronize()
        want = [b[2] for b in bufs] + [c_static]
        assert all(torch.equal(x, y) for x, y in zip(got, want)), rep
