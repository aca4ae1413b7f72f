"""Fragment-mapping primitives on the GPU against the CPU layout model (bit exact),
and the layout model against silicon (multiply and compare)."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [(16, 16, 16), (16, 16, 32), (32, 32, 8), (32, 32, 16)]
KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "primitive_kat.npz"))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("use", [0, 1, 2])
@pytest.mark.parametrize("col", [0, 1])
def test_integer_tables_bit_exact(tc, orc, dev, shape, use, col):
    """foreach_ij, foreach, foreach_v and map tables from the device headers equal
    the oracle's (reference semantics: wmma_extension.hpp:27-123)."""
    M, N, K = shape
    ij, mem, vidx, tid, fid = [t.cpu().numpy() for t in tc.layout_dump(use, M, N, K, col, dev)]
    assert np.array_equal(ij, orc.frag_ij_table(use, M, N, K))
    omem, ovidx = orc.foreach_tables(use, M, N, K, col)
    assert np.array_equal(mem, omem)
    assert np.array_equal(vidx, ovidx)
    otid, ofid = orc.frag_map_table(use, M, N, K)
    assert np.array_equal(tid, otid) and np.array_equal(fid, ofid)


def _expected_tiles(orc, tiles):
    """Oracle prediction of wmmae_primitive_tiles for (T,256) fp32 tiles."""
    T = tiles.shape[0]
    shape = (16, 16, 16)
    out = {}
    with np.errstate(all="ignore"):
        t16 = tiles.astype(np.float16)
    for name, use, col in (("a_row", 0, 0), ("a_col", 0, 1), ("b_row", 1, 0), ("b_col", 1, 1)):
        mem, _ = orc.foreach_tables(use, *shape, col)
        out[name] = t16[:, mem]                                     # (T,64,4)
    out["acc"] = tiles.reshape(T, 16, 16).transpose(0, 2, 1).reshape(T, 256)
    out["vec"] = tiles[:, :32].copy()
    return out


def _check_tiles(tc, orc, dev, tiles):
    got = tc.primitive_tiles(torch.from_numpy(tiles).to(dev))
    torch.cuda.synchronize()
    exp = _expected_tiles(orc, tiles)
    for name in ("a_row", "a_col", "b_row", "b_col"):
        g = got[name].cpu().numpy().view(np.uint16)
        assert np.array_equal(g, exp[name].view(np.uint16)), name
    assert np.array_equal(got["acc"].cpu().numpy(), exp["acc"])
    assert np.array_equal(got["vec"].cpu().numpy(), exp["vec"])


def test_primitive_tiles_small(tc, orc, dev):
    rng = np.random.default_rng(11)
    for T in (1, 3, 4, 5, 1000):
        _check_tiles(tc, orc, dev, rng.uniform(-1, 1, (T, 256)).astype(np.float32))
    # empty input
    assert tc.primitive_tiles(torch.zeros((0, 256), device=dev))["acc"].numel() == 0


def test_primitive_tiles_reference_known_answers(tc, orc, dev):
    tiles = np.stack([KAT["foreach_ij_src"], KAT["map_value"].reshape(-1),
                      KAT["load_vector_tile"], KAT["store_vector_src"], KAT["gevm_eye"]])
    _check_tiles(tc, orc, dev, tiles.astype(np.float32))


def test_primitive_tiles_full_size(tc, orc, dev):
    """1,048,576 tiles: checked in full against the oracle prediction."""
    T = 1 << 20
    g = torch.Generator(device="cpu").manual_seed(0x5EED + 2)
    tiles = (torch.rand((T, 256), generator=g, dtype=torch.float32) * 2 - 1)
    got = tc.primitive_tiles(tiles.to(dev))
    torch.cuda.synchronize()
    tiles_np = tiles.numpy()
    step = 1 << 17
    shape = (16, 16, 16)
    tables = {name: orc.foreach_tables(use, *shape, col)[0]
              for name, use, col in (("a_row", 0, 0), ("a_col", 0, 1), ("b_row", 1, 0), ("b_col", 1, 1))}
    for s in range(0, T, step):
        blk = tiles_np[s:s + step]
        t16 = blk.astype(np.float16)
        for name, mem in tables.items():
            g_ = got[name][s:s + step].cpu().numpy().view(np.uint16)
            assert np.array_equal(g_, t16[:, mem].view(np.uint16)), (name, s)
        acc = got["acc"][s:s + step].cpu().numpy()
        assert np.array_equal(acc, blk.reshape(-1, 16, 16).transpose(0, 2, 1).reshape(-1, 256))
        assert np.array_equal(got["vec"][s:s + step].cpu().numpy(), blk[:, :32])


@pytest.mark.parametrize("type_", [0, 1])
@pytest.mark.parametrize("shape", SHAPES)
def test_layout_model_matches_silicon(tc, orc, dev, type_, shape):
    """Fill A and B through foreach_ij, run one real MFMA, compare with the exact
    product: a wrong lane/register assignment of A, B or D cannot pass
    (the pattern of test/primitive/foreach.cu:24-80 and mma.cu:11-45).  Small
    integer inputs make every partial sum exact, so the comparison is bit exact."""
    M, N, K = shape
    rng = np.random.default_rng(100 + type_)
    a = rng.integers(-7, 8, (M, K)).astype(np.float32)
    b = rng.integers(-7, 8, (K, N)).astype(np.float32)
    c = rng.integers(-50, 50, (M, N)).astype(np.float32)
    if type_ == 0:
        abits, bbits = a.astype(np.float16).view(np.int16), b.astype(np.float16).view(np.int16)
    else:
        abits = (a.view(np.uint32) >> 16).astype(np.uint16).view(np.int16)
        bbits = (b.view(np.uint32) >> 16).astype(np.uint16).view(np.int16)
    d = tc.mfma_probe(type_, M, N, K, torch.from_numpy(abits).to(dev),
                      torch.from_numpy(bbits).to(dev), torch.from_numpy(c).to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy(), a @ b + c)


@pytest.mark.parametrize("type_", [0, 1])
@pytest.mark.parametrize("shape", [(16, 16, 32), (16, 16, 16), (32, 32, 16), (32, 32, 8)])
def test_raw_mfma_matches_oracle_model_bit_for_bit(tc, orc, dev, type_, shape):
    """Fresh random bit patterns, exponents spread far wider than the 24-bit window of a
    product: one raw MFMA on the GPU equals the oracle's model of the matrix core's accumulate
    arithmetic in every bit (the recorded vectors of tests/golden/mfma_kat.npz pin the same
    model on the CPU)."""
    M, N, K = shape
    rng = np.random.default_rng(9000 + 10 * type_ + K + M)
    for trial in range(6):
        spread = (-12, 8) if type_ == 0 else (-30, 30)
        ea, eb = rng.integers(*spread, (M, K)), rng.integers(*spread, (K, N))
        if trial % 3 == 0:
            ea, eb = ea // 6, eb // 6
        bits = 10 if type_ == 0 else 7
        a = (rng.choice([-1.0, 1.0], (M, K)) * (1 + rng.integers(0, 1 << bits, (M, K)) / float(1 << bits))
             * np.exp2(ea)).astype(np.float32)
        b = (rng.choice([-1.0, 1.0], (K, N)) * (1 + rng.integers(0, 1 << bits, (K, N)) / float(1 << bits))
             * np.exp2(eb)).astype(np.float32)
        if trial % 3 == 2:
            a[:, 1::2] = -a[:, 0::2]
            b[1::2, :] = b[0::2, :]
        c = (rng.choice([-1.0, 1.0], (M, N)) * (1 + rng.random((M, N)))
             * np.exp2(rng.integers(-20, 20, (M, N)))).astype(np.float32)
        if type_ == 0:
            abits, bbits = a.astype(np.float16).view(np.uint16), b.astype(np.float16).view(np.uint16)
        else:
            abits = (a.view(np.uint32) >> 16).astype(np.uint16)      # exact: 7 mantissa bits drawn
            bbits = (b.view(np.uint32) >> 16).astype(np.uint16)
        d = tc.mfma_probe(type_, M, N, K, torch.from_numpy(abits.view(np.int16)).to(dev),
                          torch.from_numpy(bbits.view(np.int16)).to(dev), torch.from_numpy(c).to(dev))
        torch.cuda.synchronize()
        want = orc.mfma_tile(type_, abits, bbits, c)
        assert np.array_equal(d.cpu().numpy().view(np.uint32), want.view(np.uint32)), trial


# ---------------------------------------------------------------- the reference's MMA-and-compare tests
def _img(x, col):
    return np.ascontiguousarray(x.T if col else x).reshape(-1).astype(np.float32)


@pytest.mark.parametrize("elem", [0, 1, 2])
@pytest.mark.parametrize("shape", [0, 1, 2, 3])
def test_primitive_mma_all_shapes(tc, orc, dev, elem, shape):
    """mma::load_matrix_sync -> mma_sync -> mma::store_matrix_sync on uniform[-1,1] inputs:
    max|diff|/max|ref| below 16 eps of the operand type (test/primitive/mma.cu:103-105),
    for every layout combination, with and without C."""
    import itertools
    from wmma_extension_amd import tcec as T
    from wmma_extension_amd._lib import WmmaeError
    m, n, k = T.PRIMITIVE_SHAPES[shape]
    if elem == 2 and shape in (1, 3):
        with pytest.raises(WmmaeError) as e:
            z = torch.zeros(m * k, device=dev)
            tc.primitive_mma(elem, shape, z, torch.zeros(k * n, device=dev), None, 0, 0, 0, 0)
        assert e.value.status == -4
        return
    eps = {0: 2.0**-10, 1: 2.0**-7, 2: 2.0**-23}[elem]
    rng = np.random.default_rng(17 + 4 * elem + shape)
    for a_col, b_col, c_col, d_col, with_c in itertools.product((0, 1), repeat=5):
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        C = rng.uniform(-1, 1, (m, n)).astype(np.float32) if with_c else None
        d = tc.primitive_mma(elem, shape, torch.from_numpy(_img(A, a_col)).to(dev),
                             torch.from_numpy(_img(B, b_col)).to(dev),
                             None if C is None else torch.from_numpy(_img(C, c_col)).to(dev),
                             a_col, b_col, c_col, d_col).cpu().numpy()
        D = d.reshape(n, m).T if d_col else d.reshape(m, n)
        ref = orc.gemm_f64(A, B) + (C if with_c else 0)
        assert orc.max_rel_err(D, ref) < 16 * eps, (a_col, b_col, c_col, d_col, with_c)
        # the same MMA through tcec::detail's foreach(_ij)_wrapper + compute_mem_offset,
        # load_matrix_sync_wrapper / fill_fragment_wrapper, mma_sync_wrapper and
        # store_matrix_sync_wrapper (tcec/detail/functions.hpp:10-348): same bits
        dw = tc.primitive_mma(elem, shape, torch.from_numpy(_img(A, a_col)).to(dev),
                              torch.from_numpy(_img(B, b_col)).to(dev),
                              None if C is None else torch.from_numpy(_img(C, c_col)).to(dev),
                              a_col, b_col, c_col, d_col, wrappers=True).cpu().numpy()
        assert np.array_equal(d.view(np.uint32), dw.view(np.uint32)), (a_col, b_col, c_col, d_col, with_c)


@pytest.mark.parametrize("shape", [0, 2])
def test_accumulator_load_store_aligned_and_not(tc, dev, shape):
    """Column-major accumulator tiles at a 16-byte aligned base move with 16-byte accesses,
    any other base element by element: C read from, and D written to, views that start one,
    two and three floats into an allocation give the bytes of the aligned call, and the
    floats around D keep theirs."""
    from wmma_extension_amd import tcec as T
    m, n, k = T.PRIMITIVE_SHAPES[shape]
    rng = np.random.default_rng(300 + shape)
    a = torch.from_numpy(rng.integers(-4, 5, m * k).astype(np.float32)).to(dev)
    b = torch.from_numpy(rng.integers(-4, 5, k * n).astype(np.float32)).to(dev)
    c = torch.from_numpy(rng.integers(-9, 10, m * n).astype(np.float32)).to(dev)
    for c_col, d_col in ((1, 1), (1, 0), (0, 1)):
        want = tc.primitive_mma(2, shape, a, b, c, 0, 0, c_col, d_col)
        for off in (1, 2, 3):
            c_buf = torch.zeros(m * n + 8, device=dev)
            c_buf[off:off + m * n] = c
            d_buf = torch.full((m * n + 8,), -77.0, device=dev)
            got = tc.primitive_mma(2, shape, a, b, c_buf[off:off + m * n], 0, 0, c_col, d_col,
                                   d=d_buf[off:off + m * n])
            assert got.data_ptr() % 16 == 4 * off
            assert torch.equal(got, want), (c_col, d_col, off)
            assert torch.all(d_buf[:off] == -77.0) and torch.all(d_buf[off + m * n:] == -77.0)


def test_foreach_error_corrected_product(tc, orc, dev):
    """A, dA, B, dB filled through foreach's mem_index, three MMAs: error below 1e-6
    against FP64 on uniform[-1,1] inputs (test/primitive/foreach.cu:24-80, :120)."""
    rng = np.random.default_rng(1)
    A = rng.uniform(-1, 1, (16, 16)).astype(np.float32)
    B = rng.uniform(-1, 1, (16, 16)).astype(np.float32)
    d = tc.foreach_ec(torch.from_numpy(_img(A, 1)).to(dev), torch.from_numpy(_img(B, 0)).to(dev)).cpu().numpy()
    D = d.reshape(16, 16).T
    assert np.abs(D - orc.gemm_f64(A, B)).max() < 1e-6
    # without the two correction products the error is a thousand times larger
    h = lambda x: x.astype(np.float16).astype(np.float64)
    assert np.abs(h(A) @ h(B) - orc.gemm_f64(A, B)).max() > 1e-4


def test_gevm_identity_and_general(tc, orc, dev):
    """Identity times a load_vector fragment returns the (fp16-rounded) vector through
    store_vector (test/primitive/gevm.cu:22-43, eye at i%17==0); a general matrix gives
    the row-vector product."""
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, 16).astype(np.float32)
    eye = np.zeros(256, dtype=np.float32)
    eye[np.arange(256) % 17 == 0] = 1.0
    y = tc.gevm(torch.from_numpy(x).to(dev), torch.from_numpy(eye).to(dev)).cpu().numpy()
    assert np.array_equal(y, x.astype(np.float16).astype(np.float32))
    E = rng.uniform(-1, 1, (16, 16)).astype(np.float32)
    y = tc.gevm(torch.from_numpy(x).to(dev), torch.from_numpy(_img(E, 1)).to(dev)).cpu().numpy()
    h = lambda v: v.astype(np.float16).astype(np.float64)
    assert np.abs(y - h(x) @ h(E)).max() < 1e-6


def test_print_fragment_runs_and_prints_every_lane(dev):
    """print_fragment of both layers in a one-wave kernel (test/primitive/print_fragment.cu):
    run in a child process, whose stdout receives the device printf."""
    import subprocess
    import sys
    code = (
        "import torch, sys; sys.path.insert(0, %r)\n"
        "from wmma_extension_amd import tcec\n"
        "src = (torch.arange(256, dtype=torch.float32, device='cuda:0') / 4)\n"
        "tcec.print_fragment(0, 1, src, 1.5)\n"
        "torch.cuda.synchronize()\n") % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [ln for ln in out.stdout.splitlines() if ln.strip()]
    assert lines[0] == "prim_a = " and lines[65] == "tcec_acc = " and len(lines) == 130
    # lane 0 of the matrix_a fragment holds row 0, k = 0..3 of the tile: 0, 0.25, 0.5, 0.75
    assert lines[1].split() == ["+0.000e+00", "+2.500e-01", "+5.000e-01", "+7.500e-01"]
    # lane 5 of the accumulator: 16 elements "(main)+(error / 2048)" = (1.5)+(5)
    assert lines[66 + 5].split() == ["(+1.500e+00)+(+5.000e+00)"] * 16


@pytest.mark.parametrize("producer", [0, 1])
def test_a_register_written_right_before_a_hand_placed_mfma_is_read_stale(tc, dev, producer):
    """The hardware fact behind wmma_extension_amd/isa_check.py: a vector-ALU write (v_mov_b32, or
    the v_accvgpr_read_b32 of a reload from an AGPR spill copy) of a source register directly in
    front of an MFMA is not interlocked - the MFMA multiplies the old contents (32 = 32 x 1 x 1);
    one wait state or any instruction in between, and it sees the new ones (40 = 24 + 8 x 2).
    The compiler spaces its own MFMAs; inside an asm statement nobody does, hence the check of
    the generated code.  (Should a later part interlock this, the first assertion fails and the
    check can go.)"""
    for _ in range(20):
        stale = tc.mfma_source_hazard_probe(producer, 0, dev)
        assert bool((stale == 32.0).all()), stale
    for gap in (1, 2, 3):
        fresh = tc.mfma_source_hazard_probe(producer, gap, dev)
        assert bool((fresh == 40.0).all()), (gap, fresh)
