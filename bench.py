#!/usr/bin/env python3
"""Benchmark of the TCEC SGEMM hot path on one MI355X.

One "step" = one full product C = A*B on synthetic seeded fp32 inputs that are
already resident in HBM: one call of the library's SGEMM entry point, on the
path its time estimates choose for the shape - the split+pack of both operands
and the MFMA GEMM on the packed path (large single products, the headline
workload), or the one kernel that splits the fp32 operands itself (batches of
medium-sized matrices, K-heavy products).  The workspace is allocated once,
outside the timed region.

Prints ONE JSON line: effective fp32 TFLOPS (2*M*N*K*batch / t), the MFMA
roofline of the GEMM kernel measured with HIP events inside the timed region,
the accuracy against an FP64 reference on a row sample, and the CPU oracle's
plain fp32 GEMM timed on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (M, N, K, batch, policy name, distribution, MFMA flop multiplier)
    "c3": dict(m=4096, n=4096, k=4096, batch=1, policy="F16_EC", dist="uniform", mult=3,
               desc="TCEC SGEMM fp16 hi+lo with EC, M=N=K=4096, A row-major, B col-major"),
    "c4": dict(m=16384, n=16384, k=16384, batch=1, policy="BF16X3_EC", dist="exp", mult=6,
               desc="TCEC SGEMM bf16 three-term split (tf32-policy replacement), M=N=K=16384"),
    "c4f16": dict(m=16384, n=16384, k=16384, batch=1, policy="F16_EC", dist="uniform", mult=3,
                  desc="TCEC SGEMM fp16 hi+lo with EC, M=N=K=16384"),
    "c2": dict(kind="prim", tiles=1 << 20, dist="uniform",
               desc="fragment primitives over 1,048,576 16x16 tiles (foreach_ij fills of A/B row+col, "
                    "accumulator store, load_vector/store_vector)"),
    "c5a": dict(m=256, n=256, k=256, batch=1024, policy="F16_EC", dist="normal", mult=3,
                desc="strided-batched TCEC SGEMM, 1024 x 256^3"),
    "c5a_fused": dict(m=256, n=256, k=256, batch=1024, policy="F16_EC", dist="normal", mult=3, path_flag=4,
                      desc="strided-batched TCEC SGEMM, 1024 x 256^3, forced onto the single (fused) kernel"),
    "c5a_packed": dict(m=256, n=256, k=256, batch=1024, policy="F16_EC", dist="normal", mult=3, path_flag=2,
                       desc="strided-batched TCEC SGEMM, 1024 x 256^3, forced through packed operands"),
    "c5b": dict(m=1024, n=1024, k=262144, batch=1, policy="F16_EC", dist="normal", mult=3,
                desc="K-heavy TCEC SGEMM, M=N=1024, K=262144"),
    "api": dict(kind="api", m=4096, n=4096, k=4096, dist="uniform",
                desc="GEMM written against the public tcec:: device API only, fp16 hi+lo with EC, M=N=K=4096"),
}
# a timed region of a few milliseconds is measured while the power management still ramps
DEFAULT_STEPS = {"c3": 200, "c5a": 400, "c5a_fused": 400, "c5a_packed": 200, "c5b": 50, "c2": 100, "api": 200}
PEAK_MFMA_TFLOPS = 2500.0      # dense fp16 / bf16 MFMA, MI355X
PEAK_HBM_GBS = 8000.0
# workloads whose dominant kernel is bound by HBM rather than by the matrix cores
HBM_BOUND = {"c2", "c5a", "c5a_fused", "c5a_packed"}
# Bytes per launch of the dominant kernel that crossed the fabric side of L2 come from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE, with --calibrate), whose
# summary under profiles/ ends in a line
#     traffic: fetch_kib=<n> write_kib=<n> sources=<sha>
# `sources` is the hash (below) of the kernel sources the figures were measured on: when the
# sources have changed since, the figure is stale and `traffic` is reported as null.
TRAFFIC_PROFILES = {
    "c4": "tcec_gemm_kernel_c4_16384_bf16x3.md",
    "c3": "tcec_gemm_kernel_c3_4096_f16.md",
    "c5a": "tcec_gemm_kernel_direct_c5a_1024x256_f16.md",
    "c5a_fused": "tcec_gemm_fused_kernel_c5a_1024x256_f16.md",
    "c5b": "tcec_gemm_kernel_c5b_1024x1024x262144_f16.md",
    "c2": "primitive_tiles_kernel_c2_1M_tiles.md",
    "api": "tcec_api_gemm_kernel_api_4096_f16.md",
}
KERNEL_SOURCES = {
    "api": ["tcec_api_gemm_kernel.hpp", "include/wmma_extension/tcec/tcec.hpp",
            "include/wmma_extension/tcec/detail/split.hpp", "include/wmma_extension/utils.hpp",
            "include/wmma_extension/wmma_extension.hpp", "include/wmma_extension/detail/mfma.hpp"],
    "c4": ["tcec_gemm_kernels.hpp"], "c3": ["tcec_gemm_kernels.hpp"], "c5b": ["tcec_gemm_kernels.hpp"],
    "c5a": ["tcec_gemm_kernels.hpp"], "c5a_fused": ["tcec_gemm_kernels.hpp", "tcec_gemm_fused_kernel.hpp"],
    "c2": ["harness_kernels.hpp"],
}


def kernel_sources_hash(workload):
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES.get(workload, []):
        path = os.path.join(ROOT, name) if "/" in name else os.path.join(ROOT, "wmma_extension_amd", "csrc", name)
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def measured_traffic(workload):
    """(bytes or None, where it came from) for the workload's dominant kernel."""
    import re
    name = TRAFFIC_PROFILES.get(workload)
    if name is None:
        return None, None
    path = os.path.join(ROOT, "profiles", name)
    try:
        text = open(path).read()
    except OSError:
        return None, None
    m = re.search(r"traffic:\s*fetch_kib=(\d+)\s+write_kib=(\d+)\s+sources=([0-9a-f]+)", text)
    if m is None:
        return None, f"profiles/{name}: no traffic line"
    if m.group(3) != kernel_sources_hash(workload):
        return None, f"profiles/{name} was measured on other kernel sources ({m.group(3)}): stale, not reported"
    return (int(m.group(1)) + int(m.group(2))) * 1024, f"profiles/{name} (sources {m.group(3)})"


def make_inputs(torch, w, dev, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    shape_a = (w["batch"], w["m"], w["k"])
    shape_b = (w["batch"], w["n"], w["k"])

    def draw(shape):
        if w["dist"] == "zeros":
            return torch.zeros(shape, device=dev, dtype=torch.float32)
        if w["dist"] == "uniform":
            return torch.rand(shape, generator=g, device=dev, dtype=torch.float32) * 2 - 1
        if w["dist"] == "normal":
            return torch.randn(shape, generator=g, device=dev, dtype=torch.float32)
        # +-x * 2^e, x ~ U[1,2), e ~ U{-15..15}
        x = torch.rand(shape, generator=g, device=dev, dtype=torch.float32) + 1
        e = torch.randint(-15, 16, shape, generator=g, device=dev).to(torch.float32)
        s = torch.randint(0, 2, shape, generator=g, device=dev).to(torch.float32) * 2 - 1
        return s * x * torch.exp2(e)
    return draw(shape_a), draw(shape_b)


def cpu_baseline(orc, w, target_s=15.0):
    """Plain fp32 GEMM loop of the oracle on the host cores, on a sample of the
    workload sized for about target_s seconds (full K, a square block of C)."""
    import numpy as np
    rng = np.random.default_rng(1)
    # full K where the output block is small enough for the time budget
    k = w["k"] if w["m"] * w["n"] <= (1 << 20) else min(w["k"], 16384)
    if w["batch"] > 1:
        # batched workload: whole batch entries, as many as fit the time budget
        m, n = w["m"], w["n"]
        a = rng.standard_normal((8, m, k)).astype(np.float32)
        b = rng.standard_normal((8, n, k)).astype(np.float32)
        orc.gemm_f32_tn(a[0], b[0])
        done, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < target_s:
            orc.gemm_f32_tn(a[done % 8], b[done % 8])
            done += 1
        dt = time.perf_counter() - t0
        return {"value": 2.0 * m * n * k * done / dt / 1e12, "unit": "TFLOPS", "cores": orc.num_threads(),
                "kind": "port",
                "sample": f"fp32 triple loop (OpenMP collapse(2), float accumulator) on {done} batch entries "
                          f"({m}x{n}x{k} each; the workload has {w['batch']}), {dt:.2f} s"}
    probe = 256
    a = rng.uniform(-1, 1, (probe, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (probe, k)).astype(np.float32)
    t0 = time.perf_counter()
    orc.gemm_f32_tn(a, b)
    dt = time.perf_counter() - t0
    rate = 2.0 * probe * probe * k / dt
    side = int((rate * target_s / (2.0 * k)) ** 0.5)
    side = max(256, min(side, w["m"], w["n"], 8192) // 64 * 64)
    a = rng.uniform(-1, 1, (side, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (side, k)).astype(np.float32)
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        orc.gemm_f32_tn(a, b)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {"value": 2.0 * side * side * k / best / 1e12, "unit": "TFLOPS", "cores": orc.num_threads(),
            "kind": "port",
            "sample": f"fp32 triple loop (OpenMP collapse(2), float accumulator) on a {side}x{side}x{k} "
                      f"block of the workload, best of 2, {best:.2f} s"}


def calibration_copy(torch, dev):
    """One elementwise kernel that reads 1 GiB and writes 1 GiB: the known-size copy
    that the FETCH_SIZE / WRITE_SIZE counters are scaled with."""
    src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    torch.add(src, 1.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def bench_primitives(args, torch, tcec, dev, w, steps=None, warmup=None, cpu=None):
    """Workload c2: the fragment-primitive kernel over a stream of tiles (HBM bound).
    Returns the JSON line's fields."""
    import ctypes
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    cpu = (not args.no_cpu) if cpu is None else cpu
    from wmma_extension_amd import _lib
    T = w["tiles"]
    g = torch.Generator(device=dev)
    g.manual_seed(0x5EED + 2)
    tiles = torch.rand((T, 256), generator=g, device=dev, dtype=torch.float32) * 2 - 1
    out = tcec.primitive_tiles(tiles)
    h = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptrs = [ctypes.c_void_p(out[k].data_ptr()) for k in ("a_row", "a_col", "b_row", "b_col", "acc", "vec")]

    def step():
        st = h.wmmae_primitive_tiles(ctypes.c_void_p(tiles.data_ptr()), T, *ptrs, stream)
        assert st == 0
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    if args.calibrate:
        calibration_copy(torch, dev)
    kernel_ms = e0.elapsed_time(e1) / steps
    # per tile: 1024 B fp32 in, 4 x 512 B fp16 fragment dumps, 1024 B accumulator, 2 x 64 B vectors
    nbytes = T * (1024 + 4 * 512 + 1024 + 128)
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    res = {
        "metric": "fragment-primitive tile stream, algorithmic GB/s", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"c2: {w['desc']}", "tiles": T},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": measured_traffic("c2")[0],
                     "traffic_source": measured_traffic("c2")[1],
                     "kernel": "primitive_tiles_kernel",
                     "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes": nbytes},
        "tiles_per_s": round(T / (kernel_ms * 1e-3), 1),
        "cpu_baseline": None,
    }
    if cpu:
        # the oracle's layout tables applied with numpy to a sample of the tiles
        import numpy as np
        from oracle import oracle as orc
        sample = min(T, 1 << 20)
        x = tiles[:sample].cpu().numpy()
        tables = [orc.foreach_tables(use, 16, 16, 16, col)[0] for use, col in ((0, 0), (0, 1), (1, 0), (1, 1))]
        t0 = time.perf_counter()
        x16 = x.astype(np.float16)
        outs = [x16[:, tb] for tb in tables]
        acc = np.ascontiguousarray(x.reshape(-1, 16, 16).transpose(0, 2, 1))
        vec = x[:, :32].copy()
        dt = time.perf_counter() - t0
        del outs, acc, vec
        res["cpu_baseline"] = {"value": round(sample * (1024 + 4 * 512 + 1024 + 128) / dt / 1e9, 3), "unit": "GB/s",
                               "cores": 1, "kind": "port",
                               "sample": f"oracle layout tables applied with numpy to {sample} tiles, {dt:.2f} s"}
    del tiles, out
    return res


POLICY_MODEL = {"F16_EC": (0, True), "F16_NOEC": (0, False), "BF16X3_EC": (2, True), "BF16X2_EC": (1, True),
                "BF16_NOEC": (1, False)}


def model_bits_block(orc, a, bt, c, policy_name, slices):
    """Two of the sampled rows, every 16th column: the result against the oracle's model of the
    matrix core (each MFMA in its measured arithmetic, in the driver's order; K slices folded in
    double precision as the library folds them).  The model gives the library's bits, so this
    reads true or names the number of differing elements."""
    import numpy as np
    kind, ec = POLICY_MODEL[policy_name]
    a2, bt2 = np.ascontiguousarray(a[:2]), np.ascontiguousarray(bt[::16])
    got = np.ascontiguousarray(c[:2, ::16])
    k = a2.shape[1]
    stages = (k + 31) // 32
    per = -(-stages // max(slices, 1))
    total = np.zeros(got.shape, np.float64)
    for s0 in range(0, stages, per):
        ka, kb = 32 * s0, min(k, 32 * (s0 + per))
        ap = np.zeros((2, 32 * (-(-(kb - ka) // 32))), np.float32)
        bp = np.zeros((ap.shape[1], bt2.shape[0]), np.float32)
        ap[:, :kb - ka], bp[:kb - ka, :] = a2[:, ka:kb], bt2[:, ka:kb].T
        part = orc.tcec_matmul(ap, bp, kind=kind, ec=ec, fk=32, main_outside=False, hw_model=True)
        total = part if slices <= 1 else total + part.astype(np.float64)
    want = np.ascontiguousarray(total.astype(np.float32))
    differing = int((got.view(np.uint32) != want.view(np.uint32)).sum())
    return {"equal": differing == 0, "differing": differing, "elements": int(got.size), "k_slices": int(slices),
            "what": "2 sampled rows x every 16th column of C against the oracle's bit-level model of the "
                    "gfx950 matrix core in the driver's instruction order"}


def accuracy_block(torch, tcec, orc, A, Bt, Ct, rows, model=None):
    """max|C - C64| / max|C64| on `rows` seeded full rows of batch 0 for the TCEC result and for
    three plain fp32 products of the same rows: the oracle's sequential CPU loop, the vendor's
    fp32 GEMM on the GPU and this library's fp32 policy (the API-level GEMM on the matrix core's
    fp32 path).  The gate "no worse than 2x plain fp32" is reported against each."""
    import numpy as np
    m, k = A.shape[1], A.shape[2]
    n = Bt.shape[1]
    rows = min(rows, m)
    g = torch.Generator().manual_seed(1234)
    idx = torch.randperm(m, generator=g)[:rows].sort().values
    a_rows = A[0][idx.to(A.device)].contiguous()                   # (rows, k)
    a = a_rows.cpu().numpy()
    bt = Bt[0].cpu().numpy()
    c = Ct[0][:, idx.to(Ct.device)].cpu().numpy().T               # (rows, n)
    ref = orc.gemm_f64(a, bt.T)
    err = orc.max_rel_err(np.ascontiguousarray(c), ref)
    plain = {"cpu_loop": orc.max_rel_err(np.ascontiguousarray(orc.gemm_f32_tn(a, bt).T), ref)}
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        vend = torch.matmul(a_rows, Bt[0].t())
        torch.cuda.synchronize()
        plain["vendor_fp32_gemm_gpu"] = orc.max_rel_err(np.ascontiguousarray(vend.cpu().numpy()), ref)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    if rows % 128 == 0 and n % 128 == 0 and k % 32 == 0:
        out = torch.empty((n, rows), dtype=torch.float32, device=A.device)
        tcec.api_gemm(3, 0, rows, n, k, 1.0, a_rows, k, Bt[0], k, 0.0, out, rows)
        torch.cuda.synchronize()
        plain["fp32_policy_api_gemm_gpu"] = orc.max_rel_err(np.ascontiguousarray(out.cpu().numpy().T), ref)
    extra = {}
    if model is not None:
        extra["same_bits_as_matrix_core_model"] = model_bits_block(orc, a, bt, np.ascontiguousarray(c), *model)
    return {
        **extra,
        "max_rel_err_vs_fp64": float(f"{err:.4e}"),
        "plain_fp32_max_rel_err_vs_fp64": float(f"{plain['cpu_loop']:.4e}"),
        "plain_fp32_comparators": {k_: float(f"{v:.4e}") for k_, v in plain.items()},
        "gate_2x_plain_fp32": {k_: bool(err <= 2 * v) for k_, v in plain.items()},
        "accuracy_sample": f"{rows} seeded full rows of C (batch 0), FP64 host loop",
    }


def cpu_config1(orc):
    """The fixed CPU point: the oracle's fp32 loop at M=N=K=1024, uniform[-1,1], best of 3."""
    import numpy as np
    rng = np.random.default_rng(0x5EED + 1)
    a = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    b = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        orc.gemm_f32_tn(a, b)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {"m": 1024, "n": 1024, "k": 1024, "best_of": 3, "seconds": round(best, 5),
            "gflops": round(2.0 * 1024 ** 3 / best / 1e9, 2)}


def run_gemm_workload(args, torch, tcec, dev, name, steps, warmup):
    """Times `steps` whole products of workload `name`; returns the fields of the JSON line that
    describe it, plus the tensors the accuracy check needs."""
    w = dict(WORKLOADS[name])
    if args.dist is not None:
        w["dist"] = args.dist
    policy = tcec.Policy[w["policy"]]
    m, n, k, batch = w["m"], w["n"], w["k"], w["batch"]
    A, Bt = make_inputs(torch, w, dev, 0x5EED + 3)
    Ct = torch.empty((batch, n, m), dtype=torch.float32, device=dev)
    # The step is the product the way the library runs it: ONE wmmae_tcec_sgemm_strided_batched
    # call on the path its time estimates choose for the shape (a workload may force another
    # one), inputs and workspace resident in HBM.  On the packed path the call launches the
    # split pass of both operands and then the MFMA GEMM kernel; the library records the two
    # events right around that kernel (wmmae_tcec_time_gemm_kernel), so that the roofline is
    # the GEMM kernel's alone while the value is the whole call's.  The other paths are one
    # kernel (plus the fold of the K slices where there are any), bracketed from outside.
    flags = args.flags | w.get("path_flag", 0)
    path = {2: tcec.PATH_PACKED, 4: tcec.PATH_FUSED, 8: tcec.PATH_DIRECT}.get(
        flags & 14, tcec.sgemm_path(m, n, k, batch, policy, flags & 1))
    packed = path in (tcec.PATH_PACKED, tcec.PATH_PACKED_SPLIT_K)
    fused = path == tcec.PATH_FUSED
    # packed operands, or the planes of K slices (the tail planes of the packed path included)
    ws_bytes = tcec.workspace_bytes(m, n, k, batch, policy)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    call_flags = flags | (2 if packed else 0)    # (the path is fixed above: no second choice inside)

    def step(ev=None):
        if packed and ev is not None:
            with tcec.timed_gemm_kernel(ev[0], ev[1]):
                tcec.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, Bt, k, n * k, 0.0,
                                           Ct, m, n * m, batch, policy, call_flags, ws)
            return
        if ev is not None:
            ev[0].record()
        tcec.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, Bt, k, n * k, 0.0,
                                   Ct, m, n * m, batch, policy, call_flags, ws)
        if ev is not None:
            ev[1].record()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(steps)]
    trace = None
    if args.clock_trace:
        # one more untimed step gives the length of the region to cover
        t0 = time.perf_counter()
        step()
        torch.cuda.synchronize()
        est_ms = (time.perf_counter() - t0) * 1e3 * steps
        period = 10_000                                   # 100 us of the 100 MHz counter
        nsamples = int(min(50_000, (est_ms * 1.5 + 30.0) / 0.1))
        side = torch.cuda.Stream()
        trace = tcec.clock_samples(nsamples, period, side)
        time.sleep(0.005)                                 # a few idle samples first
        mark0 = tcec.clock_samples(1, 0)                  # GPU time stamps of the region, main stream
    if trace is None:
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(events[i])
    if trace is not None:
        mark1 = tcec.clock_samples(1, 0)
        torch.cuda.current_stream().synchronize()      # the sampler may run on for a while
    else:
        torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    torch.cuda.synchronize()

    flops = 2.0 * m * n * k * batch
    ms_per_step = elapsed / steps * 1e3
    value = flops / (elapsed / steps) / 1e12
    gemm_ms = sum(e0.elapsed_time(e1) for e0, e1 in events) / steps
    achieved = flops * w["mult"] / (gemm_ms * 1e-3) / 1e12
    bytes_min = 4.0 * (m * k + k * n + m * n) * batch
    traffic, traffic_source = measured_traffic(name)
    kernel_name = ("tcec_gemm_fused_kernel" if fused else
                   "tcec_gemm_kernel" if packed else "tcec_gemm_kernel (DIRECT: fp32 operands split in the kernel)")

    if name in HBM_BOUND:
        # packed operands in (2*terms bytes per element), C out: the GEMM kernel's own minimum
        terms = {"F16_EC": 2, "BF16X3_EC": 3, "BF16X2_EC": 2, "F16_NOEC": 1, "BF16_NOEC": 1}[w["policy"]]
        kbytes = (2.0 * terms * (m * k + k * n) + 4.0 * m * n) * batch
        if not packed:
            kbytes = bytes_min              # fp32 A and B in, fp32 C out
        hbm = kbytes / (gemm_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(hbm, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(hbm / PEAK_HBM_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                    "kernel": kernel_name,
                    "kernel_ms": round(gemm_ms, 4), "algorithmic_bytes": kbytes, "mfma_frac": round(achieved / PEAK_MFMA_TFLOPS, 4)}
    else:
        roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_MFMA_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(achieved / PEAK_MFMA_TFLOPS, 4),
                    "traffic": traffic, "traffic_source": traffic_source,
                    "kernel": kernel_name, "kernel_ms": round(gemm_ms, 4),
                    "issued_flop_multiplier": w["mult"],
                    "hbm_frac_of_min_traffic": round(bytes_min / (gemm_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    out = {
        "value": round(value, 3),
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "dtype": "bf16" if "BF16" in w["policy"] else "f16",
        "config": {"workload": f"{name}: {w['desc']}", "m": m, "n": n, "k": k, "batch": batch,
                   "policy": w["policy"], "distribution": w["dist"], "flags": args.flags,
                   "path": {0: "fused", 1: "packed", 2: "packed + K slices", 3: "direct",
                            4: "direct + K slices"}[path],
                   "step": ("one wmmae_tcec_sgemm_strided_batched call: split+pack of A and B (one launch), MFMA "
                            "GEMM; inputs and workspace resident in HBM; the roofline's events are recorded by "
                            "the library right around the GEMM kernel"
                            if packed else
                            "one wmmae_tcec_sgemm_strided_batched call (one kernel splits the fp32 operands "
                            "and multiplies; plus the fold of K slices if any); inputs resident in HBM")},
        "roofline": roofline,
        "gemm_only_effective_tflops": round(flops / (gemm_ms * 1e-3) / 1e12, 3),
    }
    if path in (tcec.PATH_PACKED_SPLIT_K, tcec.PATH_DIRECT_SPLIT_K):
        roofline["kernel_ms_covers"] = "the GEMM kernel and the fold of its K slices (the events bracket the call)"
    if trace is not None:
        import numpy as np
        tr = trace.cpu().numpy()
        w0, w1 = int(mark0[0, 0]), int(mark1[0, 0])
        tr = tr[tr[:, 0] > 0]
        mhz = np.diff(tr[:, 1]) / np.maximum(np.diff(tr[:, 0]), 1) * 100.0
        mid = (tr[1:, 0] + tr[:-1, 0]) / 2
        busy = mhz[(mid >= w0) & (mid <= w1)]
        idle = mhz[mid < w0]
        out["shader_clock_mhz"] = {
            "idle": round(float(idle.max()), 0) if idle.size else None,
            "timed_region_mean": round(float(busy.mean()), 0) if busy.size else None,
            "timed_region_min": round(float(busy.min()), 0) if busy.size else None,
            "timed_region_max": round(float(busy.max()), 0) if busy.size else None,
            "samples": int(busy.size), "sample_period_us": 100,
            "note": "one extra wave on a second stream reads the shader cycle counter against the constant "
                    "100 MHz counter; the timed region is delimited by two stamps on the work stream"}
    if not args.no_accuracy:
        from oracle import oracle as orc
        slices = tcec.sgemm_k_slices(m, n, k, batch, policy, flags & 14)
        # (the tiles of a partly empty last round may be cut into K slices of their own: not modelled here)
        tail = packed and slices == 1 and tcec.gemm_packed_workspace_bytes(policy, m, n, k, batch) > 0
        out.update(accuracy_block(torch, tcec, orc, A, Bt, Ct, 128 if k >= 8192 else 256,
                                  model=None if tail or (flags & 1) else (w["policy"], slices)))
    return out, w


def bench_api_gemm(torch, tcec, dev, n=4096, steps=100, warmup=10, also_rz=True):
    """The GEMM written only against the public tcec:: device API (what a user of the headers
    gets), fp16 hi+lo with error correction, uniform[-1,1], M=N=K=n: with tcec::mma_sync, the
    reference's default (the figure), and with mma_rz_sync, which on this hardware is as accurate
    (`with_mma_rz_sync`)."""
    g = torch.Generator(device=dev)
    g.manual_seed(0x5EED + 3)
    A = torch.rand((n, n), generator=g, device=dev, dtype=torch.float32) * 2 - 1
    Bt = torch.rand((n, n), generator=g, device=dev, dtype=torch.float32) * 2 - 1
    C = torch.empty((n, n), dtype=torch.float32, device=dev)

    def timed(rounding):
        for _ in range(warmup):
            tcec.api_gemm(0, 1, n, n, n, 1.0, A, n, Bt, n, 0.0, C, n, rounding=rounding)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            tcec.api_gemm(0, 1, n, n, n, 1.0, A, n, Bt, n, 0.0, C, n, rounding=rounding)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        return ms, 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    ms, tf = timed(0)
    out = {"kernel": "tcec_api_gemm_kernel (tcec::load_matrix_sync / mma_sync / utils::cp_async only)",
           "workload": f"M=N=K={n}, fp16 hi+lo with EC, uniform[-1,1]", "steps": steps,
           "ms_per_step": round(ms, 4), "value": round(tf, 2), "unit": "TFLOPS",
           "mfma_frac": round(3 * tf / PEAK_MFMA_TFLOPS, 4)}
    if also_rz:
        ms_rz, tf_rz = timed(2)
        out["with_mma_rz_sync"] = {"ms_per_step": round(ms_rz, 4), "value": round(tf_rz, 2),
                                   "mfma_frac": round(3 * tf_rz / PEAK_MFMA_TFLOPS, 4)}
    return out


# Pinned shapes for the guard of the fitted path / tile / slice choices: (m, n, k, entries,
# policy).  The reference harness's grid (test/tcec/batch_gemm.cu:655-664: m = n in {512, 1024},
# k = 128 .. 16384, 256 entries) at its corners, the baseline workloads, ragged and skinny shapes.
PATHCHECK_SHAPES = [
    (512, 512, 128, 256, "F16_EC"), (512, 512, 1024, 256, "F16_EC"),
    (1024, 1024, 128, 256, "F16_EC"), (1024, 1024, 4096, 256, "F16_EC"),
    (4096, 4096, 4096, 1, "F16_EC"), (256, 256, 256, 1024, "F16_EC"), (1024, 1024, 262144, 1, "F16_EC"),
    (1000, 900, 50000, 2, "F16_EC"), (777, 1333, 515, 7, "F16_EC"),
    (48, 832, 1376, 40, "F16_EC"), (4096, 64, 4096, 1, "F16_EC"),
    (2048, 2048, 2048, 1, "BF16X3_EC"), (1024, 1024, 1024, 1, "BF16X3_EC"), (384, 384, 384, 100, "BF16X3_EC"),
]
PATH_NAMES = {0: "chosen", 2: "packed", 4: "fused", 8: "direct"}


def vendor_mfma_yardstick(torch, dev, names=("c3", "c4")):
    """What ONE plain half-precision product of the vendor library (torch.matmul -> hipBLASLt) reaches
    on the leading terms of the same operands, same box, same minute: how much of the nominal
    matrix peak a tuned kernel sustains on this data under the power limit.  A yardstick beside the
    roofline fractions of this library's kernels (which issue 3 or 6 such products per result and
    accumulate the error terms apart); never part of `value`."""
    out = {}
    for name in names:
        w = dict(WORKLOADS[name])
        m, n, k = w["m"], w["n"], w["k"]
        dt = torch.bfloat16 if "BF16" in w["policy"] else torch.float16
        A, Bt = make_inputs(torch, w, dev, 0x5EED + 3)
        a, b = A[0].to(dt), Bt[0].to(dt).t()                 # row-major A, column-major B, as the workload
        del A, Bt
        flops = 2.0 * m * n * k
        steps = max(10, min(400, int(1.5e15 / flops)))       # about one second
        c = torch.matmul(a, b)
        for _ in range(max(3, steps // 10)):
            torch.matmul(a, b, out=c)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.matmul(a, b, out=c)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        tf = flops / (ms * 1e-3) / 1e12
        out[name] = {"what": f"torch.matmul, {str(dt).split('.')[-1]} in and out, {m}x{n}x{k}, "
                             f"{w['dist']} operands rounded to the type", "steps": steps,
                     "ms": round(ms, 4), "tflops": round(tf, 1), "frac_of_mfma_peak": round(tf / PEAK_MFMA_TFLOPS, 4)}
        del a, b, c
        torch.cuda.empty_cache()
    return out


def random_path_shapes(count, seed):
    """Seeded random products for the path check: m, n = 45 .. 5000, k = 32 .. 32768, 1 .. 1024
    entries, 1e8 .. 4e11 flop, half of them with dimensions that are multiples of nothing, all
    five policies (the distribution the estimates' constants were fitted on, another seed)."""
    import random
    rnd = random.Random(seed)
    names = ["F16_EC", "F16_EC", "F16_EC", "F16_NOEC", "BF16X3_EC", "BF16X3_EC", "BF16X2_EC", "BF16_NOEC", "BF16_NOEC"]
    shapes = []
    while len(shapes) < count:
        batch = rnd.choice([1, 1, 1, 2, 4, 8, 16, 32, 64, 128, 256, 1024])
        m, n, k = int(2 ** rnd.uniform(5.5, 12.3)), int(2 ** rnd.uniform(5.5, 12.3)), int(2 ** rnd.uniform(5, 15))
        r = rnd.random()
        if r < 0.5:
            m, n, k = (m + 15) // 16 * 16, (n + 15) // 16 * 16, (k + 31) // 32 * 32
        elif r < 0.75:
            k = (k + 3) // 4 * 4
        flop = 2.0 * m * n * k * batch
        if flop > 4e11 or flop < 1e8 or (m * k + n * k + m * n) * batch * 4 > 2e9:
            continue
        shapes.append((m, n, k, batch, rnd.choice(names)))
    return shapes


def bench_pathcheck(torch, tcec, dev, rounds=3, shapes=None):
    """Every pinned shape as one whole library call (workspace resident) on the path the time
    estimates choose and on every path forced; the variants of a shape are timed in alternation,
    the fastest round of each counts.  ratio = chosen / fastest (>= 1 by construction: the chosen
    call is one of the candidates)."""
    from wmma_extension_amd._lib import WmmaeError
    rows, worst = [], 1.0
    for (m, n, k, batch, pol) in (PATHCHECK_SHAPES if shapes is None else shapes):
        policy = tcec.Policy[pol]
        g = torch.Generator(device=dev)
        g.manual_seed(0x5EED + 6)
        A = torch.randn((batch, m, k), generator=g, device=dev, dtype=torch.float32)
        Bt = torch.randn((batch, n, k), generator=g, device=dev, dtype=torch.float32)
        Ct = torch.empty((batch, n, m), dtype=torch.float32, device=dev)
        ws_bytes = tcec.workspace_bytes(m, n, k, batch, policy)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None

        def call(flags):
            tcec.sgemm_strided_batched("T", "N", m, n, k, 1.0, A, k, m * k, Bt, k, n * k, 0.0,
                                       Ct, m, n * m, batch, policy, flags, ws)
        variants, reps = [], {}
        for flags in (0, 2, 4, 8):
            try:
                call(flags)                                  # also the warm-up
            except WmmaeError as e:
                if e.status != -4:
                    raise
                continue
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            call(flags)
            torch.cuda.synchronize()
            est = time.perf_counter() - t0
            variants.append(flags)
            reps[flags] = int(max(5, min(200, 4e-3 / max(est, 1e-5))))
        best = {f: float("inf") for f in variants}
        for _ in range(rounds):
            for f in variants:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(reps[f]):
                    call(f)
                e1.record()
                torch.cuda.synchronize()
                best[f] = min(best[f], e0.elapsed_time(e1) / reps[f])
        fastest = min(best.values())
        ratio = best[0] / fastest
        worst = max(worst, ratio)
        path = tcec.sgemm_path(m, n, k, batch, policy)
        rows.append({"m": m, "n": n, "k": k, "entries": batch, "policy": pol,
                     "chosen_path": {0: "fused", 1: "packed", 2: "packed + K slices", 3: "direct",
                                     4: "direct + K slices"}[path],
                     "ms": {PATH_NAMES[f]: round(best[f], 4) for f in variants},
                     "chosen_over_best": round(ratio, 3),
                     "effective_tflops": round(2.0 * m * n * k * batch / (best[0] * 1e-3) / 1e12, 1)})
        del A, Bt, Ct, ws
        torch.cuda.empty_cache()
    ratios = sorted(r["chosen_over_best"] for r in rows)
    return {"worst_ratio": round(worst, 3), "mean_ratio": round(sum(ratios) / len(ratios), 4),
            "above_1.10": sum(1 for x in ratios if x > 1.10), "count": len(ratios), "shapes": rows,
            "what": "whole wmmae_tcec_sgemm_strided_batched calls, N(0,1) operands, workspace resident; "
                    "each shape on the path the estimates choose and on every path forced, variants "
                    f"alternating, fastest of {rounds} rounds each"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps; default 80 (about 3 s) for the 16384^3 workloads and more for the short "
                         "ones, so that the timed region lasts long enough for the clocks to settle")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps; default 2 (20 for the short workloads)")
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS) + ["pathcheck"],
                    help="pathcheck: pinned shapes, each timed on every path the driver has "
                         "(the guard of the fitted path choices; also part of the default run)")
    ap.add_argument("--random-shapes", type=int, default=0, metavar="N",
                    help="with --workload pathcheck: N seeded random products instead of the pinned shapes "
                         "(value = mean ratio; the worst and the number above 1.10 are in the line too)")
    ap.add_argument("--seed", type=int, default=2024, help="seed of --random-shapes")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-accuracy", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="with the default workload: skip the 4096^3 half of the metric (c3), the "
                         "API-level GEMM figure, the batched / K-heavy configurations (c5a, c5b), the "
                         "primitive tile stream (c2), the path check and the vendor library's "
                         "half-precision yardstick")
    ap.add_argument("--flags", type=int, default=0)
    ap.add_argument("--dist", default=None, choices=["uniform", "normal", "exp", "zeros"],
                    help="override the workload's input distribution (zeros: what the kernel reaches "
                         "when the matrix cores are not power limited; not a valid benchmark value)")
    ap.add_argument("--clock-trace", action="store_true",
                    help="sample the shader clock on a second stream during the timed region and add "
                         "its statistics to the JSON line (the matrix cores are power limited); the sampling "
                         "wave holds one SIMD, which a launch of one persistent workgroup per compute unit "
                         "(c5a, c5b) pays for with up to twice its time: not a benchmark value there")
    ap.add_argument("--calibrate", action="store_true",
                    help="after the timed region run one 1 GiB read + 1 GiB write elementwise kernel "
                         "(the known-size copy that rocprofv3 FETCH_SIZE / WRITE_SIZE are scaled with)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; --gpus must be 1 "
              "(the path would shard by blocks of C or by batch entry, with no exchange)", file=sys.stderr)
        sys.exit(2)

    import torch
    from wmma_extension_amd import _lib, tcec
    _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "pathcheck":
        shapes = random_path_shapes(args.random_shapes, args.seed) if args.random_shapes > 0 else None
        r = bench_pathcheck(torch, tcec, dev, shapes=shapes)
        if shapes is not None:
            r["what"] = f"{len(shapes)} random products (seed {args.seed}); " + r["what"]
            r["shapes"] = sorted(r["shapes"], key=lambda x: -x["chosen_over_best"])[:12]   # the worst ones
        print(json.dumps({
            "metric": ("time of the chosen path over the fastest forced path, "
                       + ("mean over random products" if shapes is not None else "worst of the pinned shapes")),
            "value": r["mean_ratio"] if shapes is not None else r["worst_ratio"],
            "unit": "ratio", "n_gpus": 1, "steps": 3, "warmup": 1,
            "ms_per_step": None, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "f16", "data": "synthetic", "config": {"workload": "pathcheck: " + r["what"]},
            "pathcheck": r, "roofline": None, "cpu_baseline": None}))
        return
    w = dict(WORKLOADS[args.workload])
    if args.warmup is None:
        args.warmup = 20 if args.workload in DEFAULT_STEPS else 2
    if args.steps is None:
        args.steps = DEFAULT_STEPS.get(args.workload, 80)
    if w.get("kind") == "prim":
        if args.dist is not None:
            w["dist"] = args.dist
        print(json.dumps(bench_primitives(args, torch, tcec, dev, w)))
        return
    if w.get("kind") == "api":
        # (only the kernel with the reference's default here: the profiles of this workload
        # are taken from this command, one kernel per summary)
        r = bench_api_gemm(torch, tcec, dev, w["m"], args.steps, args.warmup, also_rz=False)
        if args.calibrate:
            calibration_copy(torch, dev)
        traffic, traffic_source = measured_traffic("api")
        print(json.dumps({
            "metric": "TCEC SGEMM effective fp32 TFLOPS", "value": r["value"], "unit": "TFLOPS", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": f"api: {w['desc']}"},
            "roofline": {"bound": "mfma", "achieved": round(3 * r["value"], 2), "peak": PEAK_MFMA_TFLOPS,
                         "unit": "TFLOP/s", "frac": r["mfma_frac"], "traffic": traffic,
                         "traffic_source": traffic_source, "kernel": "tcec_api_gemm_kernel", "kernel_ms": r["ms_per_step"],
                         "issued_flop_multiplier": 3},
            "cpu_baseline": None}))
        return

    main_out, w = run_gemm_workload(args, torch, tcec, dev, args.workload, args.steps, args.warmup)
    if args.calibrate:
        calibration_copy(torch, dev)
    out = {
        "metric": "TCEC SGEMM effective fp32 TFLOPS",
        "value": main_out.pop("value"),
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": main_out.pop("steps"),
        "warmup": main_out.pop("warmup"),
        "ms_per_step": main_out.pop("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": main_out.pop("dtype"),
        "data": "synthetic",
    }
    out.update(main_out)
    out["fp32_vector_peak_tflops"] = 157.3
    if args.workload == "c4" and not args.no_secondary and args.dist is None:
        # the other half of the metric (4096^3, fp16 hi+lo) and the drop-in API's own GEMM
        torch.cuda.empty_cache()
        sec, _ = run_gemm_workload(args, torch, tcec, dev, "c3", DEFAULT_STEPS["c3"], 20)
        sec["unit"] = "TFLOPS"
        out["secondary"] = sec
        out["api_level_gemm"] = bench_api_gemm(torch, tcec, dev)
        # the two batched / K-heavy baseline configurations, each on the path the library chooses
        out["other_configs"] = {}
        for name in ("c5a", "c5b"):
            torch.cuda.empty_cache()
            o, _ = run_gemm_workload(args, torch, tcec, dev, name, DEFAULT_STEPS[name], 20)
            o["unit"] = "TFLOPS"
            out["other_configs"][name] = o
        # the fragment-primitive tile stream (its own metric: algorithmic GB/s)
        torch.cuda.empty_cache()
        c2 = bench_primitives(args, torch, tcec, dev, dict(WORKLOADS["c2"]), DEFAULT_STEPS["c2"], 20,
                              cpu=not args.no_cpu)
        for key in ("n_gpus", "higher_is_better", "scaling", "vs_baseline", "data"):
            c2.pop(key, None)
        out["other_configs"]["c2"] = c2
        # the guard of the fitted path choices: chosen path against every forced one
        torch.cuda.empty_cache()
        pc = bench_pathcheck(torch, tcec, dev)
        out["pathcheck"] = {"worst_ratio": pc["worst_ratio"], "what": pc["what"],
                            "shapes": [{"shape": f"{r['m']}x{r['n']}x{r['k']} x{r['entries']} {r['policy']}",
                                        "chosen_path": r["chosen_path"], "chosen_over_best": r["chosen_over_best"],
                                        "ms": r["ms"]} for r in pc["shapes"]]}
        # the vendor library's single half-precision product on the same data (a yardstick for the
        # roofline fractions above: what the power limit leaves a tuned kernel of this part)
        torch.cuda.empty_cache()
        out["vendor_mfma_yardstick"] = vendor_mfma_yardstick(torch, dev)
    if not args.no_cpu:
        from oracle import oracle as orc
        out["cpu_baseline"] = cpu_baseline(orc, w)
        out["cpu_baseline"]["config1_1024_cubed"] = cpu_config1(orc)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
