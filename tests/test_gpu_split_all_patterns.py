"""The device's split of an fp32 operand into 16-bit terms against the oracle's, for EVERY fp32
bit pattern (2^32 values per split, zeros, subnormals, infinities and NaNs included).

The split under test is the one `wmmae_tcec_pack` runs (the reference's rule, tcec/tcec.hpp:219-223
with tcec/detail/scale.hpp:8-20: leading term = the value rounded to nearest even, residual term =
the rounded, scaled remainder; the three-term bf16 split repeats the step); the kernels that split
inside the GEMM use the same helper functions and are tied to this one by the bit-equality tests
of the driver's paths.  The bar is bit equality of every term; where a term is a NaN, any NaN
pattern of the 16-bit type counts (the payload of a NaN is not part of the reference's contract).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LOG_CHUNK = 26            # patterns per pass: 256 MiB of operands
K = 4096


def _nan_mask(bits, f16):
    if f16:
        return ((bits & 0x7C00) == 0x7C00) & ((bits & 0x03FF) != 0)
    return ((bits & 0x7F80) == 0x7F80) & ((bits & 0x007F) != 0)


@pytest.mark.parametrize("policy,kind_name,terms", [(0, "SPLIT_F16", 2), (2, "SPLIT_BF16X3", 3)])
def test_split_of_every_fp32_pattern(tc, orc, dev, policy, kind_name, terms):
    kind = getattr(orc, kind_name)
    count = 1 << LOG_CHUNK
    rows = count // K
    packed = torch.empty(tc.pack_bytes(rows, K, 1, policy), dtype=torch.uint8, device=dev)
    assert packed.numel() == count * 2 * terms
    for chunk in range((1 << 32) >> LOG_CHUNK):
        base = chunk << LOG_CHUNK
        bits = torch.arange(base, base + count, dtype=torch.int64, device=dev).to(torch.int32)
        tc.pack(policy, rows, K, bits.view(torch.float32).reshape(rows, K), K, 1, packed)
        # packed operand: chunk (row block, k stage, term), lane l holds row 16*rb + l % 16,
        # k = 32*stage + 8*(l / 16) .. + 7  ->  back to (term, row, k)
        got = (packed.view(torch.int16).reshape(rows // 16, K // 32, terms, 4, 16, 8)
               .permute(2, 0, 4, 1, 3, 5).reshape(terms, count).cpu().numpy().view(np.uint16))
        v = np.arange(base, base + count, dtype=np.uint64).astype(np.uint32).view(np.float32)
        want = orc.split(kind, v)
        for t in range(terms):
            differ = got[t] != want[t]
            if differ.any():
                f16 = kind == orc.SPLIT_F16
                differ &= ~(_nan_mask(got[t], f16) & _nan_mask(want[t], f16))
            if differ.any():
                i = int(np.flatnonzero(differ)[0])
                raise AssertionError(
                    f"policy {policy} term {t}: fp32 pattern {base + i:#010x} -> device {int(got[t][i]):#06x}, "
                    f"oracle {int(want[t][i]):#06x} ({int(differ.sum())} patterns of this pass differ)")


def test_cast_of_every_fp32_pattern(tc, orc, dev):
    """utils `cast` to half, bfloat16 and tf32 (the reference's detail/common.hpp:22-61 and its
    cvt.rna, :73-91) for every fp32 bit pattern.  half / bfloat16: against torch's own conversions
    (round to nearest even; NaNs by class).  tf32: against the oracle's rule in integer arithmetic
    (add half a step of the 13 dropped bits to the magnitude, clear them: ties away from zero;
    infinities and NaNs pass through) - on the device for all patterns, and the oracle's own
    function on a strided sample of each pass."""
    log_chunk = 27
    count = 1 << log_chunk
    for chunk in range((1 << 32) >> log_chunk):
        base = chunk << log_chunk
        bits = torch.arange(base, base + count, dtype=torch.int64, device=dev)
        x = bits.to(torch.int32).view(torch.float32)
        for dst, tdt, exp_mask, man_mask in ((0, torch.float16, 0x7C00, 0x03FF), (1, torch.bfloat16, 0x7F80, 0x007F)):
            got = tc.utils_cast(dst, x).to(torch.int32) & 0xFFFF
            want = x.to(tdt).view(torch.int16).to(torch.int32) & 0xFFFF
            nan = ((got & exp_mask) == exp_mask) & ((got & man_mask) != 0)
            nan_w = ((want & exp_mask) == exp_mask) & ((want & man_mask) != 0)
            assert torch.equal(nan, nan_w), (chunk, dst)
            assert torch.equal(got[~nan], want[~nan]), (chunk, dst)
        t = tc.utils_cast(2, x).view(torch.int32).to(torch.int64) & 0xFFFFFFFF
        nonfinite = (bits & 0x7F800000) == 0x7F800000
        rule = torch.where(nonfinite, bits, (bits + 0x1000) & 0xFFFFE000)
        assert torch.equal(t, rule), chunk
        sample = x[::65537].cpu().numpy()
        fin = np.isfinite(sample)
        want = np.array([orc.to_tf32(e) for e in sample[fin]], dtype=np.float32)
        got = tc.utils_cast(2, x[::65537].contiguous()).cpu().numpy()[fin]
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), chunk
