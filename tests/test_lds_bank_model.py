"""Host-side LDS bank analysis of the layouts the GEMM kernels use (the reference does
this on the device for its shared-memory skew, research/bank-conflict/main.cu:38-71).

Model: 64 banks of 4 bytes; a 128-bit read is served sixteen lanes at a time, each lane
touching four consecutive banks; the conflict degree of a phase is the largest number of
lanes that hit one bank.  rocprofv3's SQ_LDS_BANK_CONFLICT reads 0 for all three kernels
on the GPU; this test shows why, and that the obvious alternatives would not."""
import numpy as np


def _degree_b128(byte_addr):
    """Worst conflict degree over the four 16-lane phases of a 64-lane ds_read_b128."""
    worst = 0
    for phase in range(4):
        hits = np.zeros(64, dtype=int)
        for lane in range(16 * phase, 16 * phase + 16):
            first = (byte_addr[lane] // 4) % 64
            for b in range(4):
                hits[(first + b) % 64] += 1
        worst = max(worst, hits.max())
    return worst


def test_fragment_major_chunks_are_conflict_free():
    """Packed operands and the fused kernel's term buffers: lane l reads base + 16*l."""
    lane = np.arange(64)
    assert _degree_b128(16 * lane) == 1


def test_fused_kernel_raw_layout():
    """Raw fp32 row block of the fused kernel: 16 rows x 128 bytes.  Lane l converts row
    r = l%16, floats 8*(l/16) .. +7.  Stored row-major, all sixteen rows of a phase start
    in the same banks; with the pieces of a row permuted as the kernel does
    (32-byte pair index XOR (r/2)%4, halves swapped for r >= 8) every phase covers all
    banks exactly once."""
    lane = np.arange(64)
    r, g = lane % 16, lane // 16
    plain = r * 128 + g * 32
    assert _degree_b128(plain) == 8 and _degree_b128(plain + 16) == 8
    base = r * 128 + 32 * (g ^ ((r >> 1) & 3))
    lo = base + 16 * (r >> 3)
    hi = base + 16 * (1 - (r >> 3))
    assert _degree_b128(lo) == 1 and _degree_b128(hi) == 1
    # the permutation is the one the requests write: lane l of request h fetches row
    # 8h + l/8, piece (l%8) ^ (2*((l/16)%4) + h) into slot h*1024 + 16*l
    where = {}
    for h in range(2):
        for l in range(64):
            row = 8 * h + l // 8
            piece = (l % 8) ^ (2 * ((l // 16) % 4) + h)
            where[(row, piece)] = h * 1024 + 16 * l
    assert len(where) == 128                                    # every piece of every row once
    for l in range(64):
        assert where[(r[l], 2 * g[l])] == lo[l]                  # floats 8g .. 8g+3
        assert where[(r[l], 2 * g[l] + 1)] == hi[l]              # floats 8g+4 .. 8g+7


def test_api_level_kernel_skew():
    """The API-level GEMM stages fp32 tiles with a leading dimension of 32 + 4 floats
    (the reference settles on a skew of 8 floats for its 32-lane warps, batch_gemm.cu:11).
    A fragment load takes lane l's eight floats of row l%16 from k = 8*(l/16) on, as two
    128-bit reads: with the skew of 4 the sixteen rows of a phase start 36 banks apart and
    cover all banks once; unpadded they all start in the same or the opposite half."""
    lane = np.arange(64)

    def degree(ld):
        addr = ((lane % 16) * ld + 8 * (lane // 16)) * 4
        return max(_degree_b128(addr), _degree_b128(addr + 16))
    assert degree(36) == 1
    assert degree(32) == 8
    assert degree(40) > 1          # the reference's skew of 8 does not suit 64 banks
