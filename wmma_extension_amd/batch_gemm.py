"""The reference's batched-GEMM harness as a command (test/tcec/batch_gemm.cu:447-664).

    python -m wmma_extension_amd.batch_gemm [--m 512 1024] [--k 128 ... 16384] [--batch 256]
                                            [--policy F16_EC] [--count 32] [--rn-main] [--vendor]

For every (m = n, k) of the grid it allocates `batch` separate A (m x k, row major), B (k x n,
column major) and C (m x n, column major) matrices, fills A[j] = j / k, B[j] = j / n, C = 0
(batch_gemm.cu:505-520), runs the pointer-array product once, takes the relative Frobenius
residual of the last entry against an FP64 product (:559-575), then times `count` launches
with the wall clock (:582-597) and prints the reference's CSV line
`wmmae,m,n,k,batch_size,residual,throughput` (:604, header :657), throughput in TFLOPS =
2 m n k batch / t.  Where the reference calls `launch_bgemm` this calls
`wmmae_tcec_sgemm_batched` with the same arguments.  The FP64 product runs on the GPU
(the reference uses a host OpenMP loop).  `--vendor` adds the line the reference prints when
built with TEST_CUBLAS (:609-637), `vendor,m,n,k,batch_size,-,throughput`: the vendor library's
fp32 batched GEMM on the same operands (torch.bmm on one strided copy of them)."""
import argparse
import sys
import time

import torch

from . import tcec


def run_vendor(m, n, k, batch, count, dev, out=sys.stdout):
    """fp32 batched GEMM of the vendor library on the harness's operands."""
    a = (torch.arange(m * k, dtype=torch.float32, device=dev) / float(k)).reshape(1, m, k)
    b = (torch.arange(k * n, dtype=torch.float32, device=dev) / float(n)).reshape(1, n, k)
    A = a.repeat(batch, 1, 1)
    Bt = b.repeat(batch, 1, 1).transpose(1, 2)          # (batch, k, n), k contiguous as in the harness
    C = torch.empty((batch, m, n), dtype=torch.float32, device=dev)
    torch.bmm(A, Bt, out=C)
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(count):
        torch.bmm(A, Bt, out=C)
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - start) / count
    tflops = 2.0 * m * n * k * batch / elapsed / 1e12
    print("vendor,%u,%u,%u,%u,-,%e" % (m, n, k, batch, tflops), file=out, flush=True)
    return tflops


def run_case(m, n, k, batch, policy, count, dev, out=sys.stdout, flags=0):
    a = (torch.arange(m * k, dtype=torch.float32, device=dev) / float(k)).reshape(m, k)
    b = (torch.arange(k * n, dtype=torch.float32, device=dev) / float(n)).reshape(n, k)
    As = [a.clone() for _ in range(batch)]
    Bs = [b.clone() for _ in range(batch)]
    Cs = [torch.zeros((n, m), dtype=torch.float32, device=dev) for _ in range(batch)]
    pa = torch.tensor([t.data_ptr() for t in As], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in Bs], dtype=torch.int64, device=dev)
    pc = torch.tensor([t.data_ptr() for t in Cs], dtype=torch.int64, device=dev)
    ws_bytes = tcec.workspace_bytes(m, n, k, batch, policy)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None

    def launch():
        tcec.sgemm_batched("T", "N", m, n, k, 1.0, pa, k, pb, k, 0.0, pc, m, batch, policy, flags, ws)

    launch()
    torch.cuda.synchronize()
    ref = torch.matmul(As[-1].double(), Bs[-1].double().T)          # (m, n)
    diff = Cs[-1].T.double() - ref
    residual = float(torch.sqrt((diff * diff).sum() / (ref * ref).sum()))

    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(count):
        launch()
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - start) / count
    tflops = 2.0 * m * n * k * batch / elapsed / 1e12
    print("wmmae,%u,%u,%u,%u,%e,%e" % (m, n, k, batch, residual, tflops), file=out, flush=True)
    return residual, tflops


def main(argv=None, out=sys.stdout):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--m", type=int, nargs="+", default=[1 << 9, 1 << 10], help="m = n of the grid")
    ap.add_argument("--k", type=int, nargs="+", default=[1 << e for e in range(7, 15)])
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--policy", default="F16_EC", choices=[p.name for p in tcec.Policy])
    ap.add_argument("--count", type=int, default=32, help="timed launches per case")
    ap.add_argument("--rn-main", action="store_true",
                    help="accumulate the leading product with fp32 adds outside the matrix core "
                         "(the reference's mma_rn_sync, tcec/tcec.hpp:673-694)")
    ap.add_argument("--vendor", action="store_true",
                    help="also time the vendor library's fp32 batched GEMM (the reference's "
                         "TEST_CUBLAS lines)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("batch_gemm: no GPU")
    dev = torch.device("cuda:0")
    policy = tcec.Policy[args.policy]
    print("mode,m,n,k,batch_size,residual,throughput", file=out, flush=True)
    for m in args.m:
        for k in args.k:
            run_case(m, m, k, args.batch, policy, args.count, dev, out,
                     tcec.FLAG_RN_MAIN if args.rn_main else 0)
            if args.vendor:
                run_vendor(m, m, k, args.batch, args.count, dev, out)


if __name__ == "__main__":
    main()
