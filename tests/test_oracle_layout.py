"""Pins the oracle's gfx950 fragment layout model by what the mathematics fixes
and by the known-answer inputs of the reference's primitive tests (CPU only)."""
import os

import numpy as np
import pytest

SHAPES = [(16, 16, 16), (16, 16, 32), (32, 32, 8), (32, 32, 16)]
KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "primitive_kat.npz"))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("use", [0, 1, 2])
def test_layout_is_a_bijection_and_map_inverts_it(orc, shape, use):
    M, N, K = shape
    rows, cols, R = orc.frag_shape(use, M, N, K)
    assert rows * cols == 64 * R
    ij = orc.frag_ij_table(use, M, N, K)
    flat = ij[..., 0] * cols + ij[..., 1]
    assert sorted(flat.reshape(-1).tolist()) == list(range(rows * cols))
    tid, fid = orc.frag_map_table(use, M, N, K)
    for lane in range(64):
        for reg in range(R):
            i, j = ij[lane, reg]
            assert tid[i, j] == lane and fid[i, j] == reg


@pytest.mark.parametrize("shape", SHAPES)
def test_layout_matches_mfma_register_facts(orc, shape):
    """Independent statement of the vendor layout (ck_tile kAMLane/kABKLane/
    kABKPerLane/kCM1PerLane): A rows and B columns run over lane % M, k runs in
    K-per-lane consecutive values per lane group, a C lane holds 4 consecutive rows."""
    M, N, K = shape
    a = orc.frag_ij_table(0, M, N, K)
    b = orc.frag_ij_table(1, M, N, K)
    c = orc.frag_ij_table(2, M, N, K)
    P = K * M // 64
    for lane in range(64):
        assert (a[lane, :, 0] == lane % M).all()
        assert (a[lane, :, 1] == P * (lane // M) + np.arange(P)).all()
        assert (b[lane, :, 1] == lane % N).all()
        assert (b[lane, :, 0] == a[lane, :, 1]).all()      # A and B pair the same k
        assert (c[lane, :, 1] == lane % N).all()
        rows = c[lane, :, 0].reshape(-1, 4)
        assert (rows == rows[:, :1] + np.arange(4)).all()
        assert (rows[:, 0] == 4 * (lane // N) + (256 // N) * np.arange(rows.shape[0])).all()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("use", [0, 1, 2])
@pytest.mark.parametrize("col", [0, 1])
def test_foreach_and_foreach_v_follow_foreach_ij(orc, shape, use, col):
    M, N, K = shape
    rows, cols, R = orc.frag_shape(use, M, N, K)
    ij = orc.frag_ij_table(use, M, N, K)
    mem, vidx = orc.foreach_tables(use, M, N, K, col)
    i, j = ij[..., 0], ij[..., 1]
    assert (mem == (i + j * rows if col else i * cols + j)).all()
    if col:
        assert (vidx == np.where(j == 0, i, -1)).all()
        assert sorted(vidx[vidx >= 0].tolist()) == list(range(rows))
    else:
        assert (vidx == np.where(i == 0, j, -1)).all()
        assert sorted(vidx[vidx >= 0].tolist()) == list(range(cols))


def _load_dense(orc, use, shape, tile, col):
    """Fragment registers of a dense tile read in the given layout."""
    M, N, K = shape
    mem, _ = orc.foreach_tables(use, M, N, K, col)
    return tile[mem]


def test_reference_known_answer_inputs(orc):
    shape = (16, 16, 16)
    # foreach_ij / foreach agree on the i/32 ramp (test/primitive/foreach_ij.cu:104)
    src = KAT["foreach_ij_src"]
    for use in (0, 1, 2):
        for col in (0, 1):
            ij = orc.frag_ij_table(use, *shape)
            via_ij = src[ij[..., 0] + 16 * ij[..., 1]] if col else src[ij[..., 0] * 16 + ij[..., 1]]
            assert (via_ij == _load_dense(orc, use, shape, src, col)).all()
    # map: the register map(i,j) names holds the value stored at (i,j) (map.cu:28, 47)
    val = KAT["map_value"]                      # val[i,j] = i + j*M
    for use in (0, 1, 2):
        ij = orc.frag_ij_table(use, *shape)
        frag = val[ij[..., 0], ij[..., 1]]
        tid, fid = orc.frag_map_table(use, *shape)
        assert (frag[tid, fid] == val).all()
    # load_vector: fragment == load of the tile whose first 16 elements are v
    v, tile = KAT["load_vector_v"], KAT["load_vector_tile"]
    for use in (0, 1, 2):
        for col in (0, 1):
            _, vidx = orc.foreach_tables(use, *shape, col)
            frag = np.where(vidx >= 0, v[np.maximum(vidx, 0)], 0).astype(np.float32)
            assert (frag == _load_dense(orc, use, shape, tile, col)).all()
    # store_vector: first 16 memory elements of the i ramp come back
    src = KAT["store_vector_src"]
    for col in (0, 1):
        frag = _load_dense(orc, 2, shape, src, col)
        _, vidx = orc.foreach_tables(2, *shape, col)
        out = np.full(16, -1, dtype=np.float32)
        out[vidx[vidx >= 0]] = frag[vidx >= 0]
        assert (out == KAT["store_vector_expect"]).all()
