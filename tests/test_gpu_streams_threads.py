"""Calls on several streams and from several host threads at once.  The C-ABI keeps no state
between calls (the entry point that allocates nothing aside, which documents its one shared
buffer): the same products issued on two side streams in turn, and from four host threads with a
stream each, with the caller's workspace or with one the call allocates on its stream, give the
bits of the same calls made one after the other on the default stream."""
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu

PACKED, FUSED, DIRECT = 2, 4, 8
# (policy, m, n, k, entries, path flag): every path, K slices, tail slices, batches
CASES = [(0, 700, 520, 1000, 1, 0), (2, 1288, 1032, 1000, 1, PACKED), (0, 256, 256, 256, 64, DIRECT),
         (0, 128, 128, 20000, 1, 0), (3, 300, 200, 4000, 3, 0), (1, 96, 80, 72, 9, FUSED),
         (0, 1024, 1024, 8192, 1, DIRECT), (4, 2000, 100, 333, 1, 0)]


def _run_all(tc, dev, data, own_workspace):
    outs = []
    for (policy, m, n, k, batch, flag), (A, B) in zip(CASES, data):
        C = torch.full((batch, n, m), 5.0, device=dev)
        ws = (torch.empty(max(16, tc.workspace_bytes(m, n, k, batch, policy)), dtype=torch.uint8, device=dev)
              if own_workspace else None)
        tc.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, B, k, n * k, 0.0, C, m, n * m,
                                 batch, policy, flag, ws)
        outs.append(C)
    return outs


def _same(a, b):
    return all(torch.equal(x, y) for x, y in zip(a, b))


def test_streams_and_threads_give_the_serial_bits(tc, dev):
    g = torch.Generator(device=dev).manual_seed(9)
    data = [(torch.rand((b, m, k), generator=g, device=dev) * 2 - 1, torch.rand((b, n, k), generator=g, device=dev) * 2 - 1)
            for (_, m, n, k, b, _) in CASES]
    base = _run_all(tc, dev, data, True)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()      # default priority
    for rep in range(3):
        with torch.cuda.stream(s1):
            o1 = _run_all(tc, dev, data, rep % 2 == 0)
        with torch.cuda.stream(s2):
            o2 = _run_all(tc, dev, data, rep % 2 == 1)
        torch.cuda.synchronize()
        assert _same(base, o1) and _same(base, o2), rep
    results, errors = {}, []

    def worker(i):
        try:
            torch.cuda.set_device(dev)
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for rep in range(3):
                    results[(i, rep)] = _run_all(tc, dev, data, (i + rep) % 2 == 0)
            s.synchronize()
        except Exception as e:                               # noqa: BLE001 - reported below
            errors.append((i, repr(e)))
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    assert len(results) == 12 and all(_same(base, o) for o in results.values())
