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
