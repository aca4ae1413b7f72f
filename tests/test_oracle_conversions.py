"""Pins the oracle's 16-bit conversions and operand splits (CPU only)."""
import numpy as np
import pytest
import torch


def _structured_bits():
    """fp32 bit patterns around every rounding boundary of fp16 and bf16."""
    rng = np.random.default_rng(1234)
    parts = [rng.integers(0, 2**32, size=400_000, dtype=np.uint64).astype(np.uint32)]
    # every exponent, mantissas at/around the fp16 (bit 13) and bf16 (bit 16) ties
    exps = np.arange(0, 256, dtype=np.uint32) << 23
    mans = []
    for tie_bit in (12, 15):
        base = np.uint32(1 << tie_bit)
        for hi in (0, 1, 2, 3, 0x3ff, 0x7f):
            upper = np.uint32((hi << (tie_bit + 1)) & 0x7fffff)
            for d in (-1, 0, 1):
                mans.append(np.uint32((int(upper) | int(base)) + d) & np.uint32(0x7fffff))
    mans = np.array(sorted(set(int(x) for x in mans)) + [0, 1, 0x7fffff, 0x7ffffe], dtype=np.uint32)
    grid = (exps[:, None] | mans[None, :]).reshape(-1)
    parts += [grid, grid | np.uint32(0x80000000)]
    return np.concatenate(parts)


def test_f16_conversion_matches_numpy(orc):
    bits = _structured_bits()
    v = bits.view(np.float32)
    hi = orc.split(orc.SPLIT_F16, v)[0]
    with np.errstate(all="ignore"):
        ref = v.astype(np.float16).view(np.uint16)
    ok = np.isnan(v) | (hi == ref)
    assert ok.all(), f"{np.count_nonzero(~ok)} mismatches, first {hex(bits[~ok][0])}"
    # NaN stays NaN
    assert np.isnan(orc.f16_bits_to_f32(hi[np.isnan(v)])).all()


def test_bf16_conversion_matches_torch(orc):
    bits = _structured_bits()
    v = bits.view(np.float32)
    hi = orc.split(orc.SPLIT_BF16X2, v)[0]
    ref = torch.from_numpy(v.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    ok = np.isnan(v) | (hi == ref)
    assert ok.all(), f"{np.count_nonzero(~ok)} mismatches"


def test_f16_conversion_sweep(orc):
    """fp32 -> fp16 of the oracle against numpy over the whole 32-bit pattern space:
    every 61st pattern by default (70 M values, all exponents, ties and subnormals
    included through the halfway patterns added below); all 2^32 patterns with
    WMMAE_EXHAUSTIVE=1 (about ten minutes)."""
    import os
    stride = 1 if os.environ.get("WMMAE_EXHAUSTIVE") == "1" else 61
    step = 1 << 26
    for start in range(0, 1 << 32, step):
        bits = np.arange(start, start + step, stride, dtype=np.uint64).astype(np.uint32)
        v = bits.view(np.float32)
        hi = orc.split(orc.SPLIT_F16, v)[0]
        with np.errstate(all="ignore"):
            ref = v.astype(np.float16).view(np.uint16)
        assert (np.isnan(v) | (hi == ref)).all()
    # every exact halfway case and its two neighbours, for all exponents and both signs:
    # mantissa patterns x * 2^13 + {2^12 - 1, 2^12, 2^12 + 1} (normal range) and the wider
    # ties of the fp16 subnormal range
    expo = np.arange(0, 256, dtype=np.uint32)[:, None, None] << np.uint32(23)
    hi10 = np.arange(0, 1024, dtype=np.uint32)[None, :, None] << np.uint32(13)
    for shift in range(12, 24):
        half = np.uint32(1) << np.uint32(shift)
        tail = np.array([half - 1, half, half + 1], dtype=np.uint32)[None, None, :]
        bits = ((expo | hi10) & ~np.uint32((1 << (shift + 1)) - 1) & np.uint32(0x7FFFFFFF)) | tail
        for sign in (np.uint32(0), np.uint32(0x80000000)):
            v = (bits | sign).ravel().view(np.float32)
            got = orc.split(orc.SPLIT_F16, v)[0]
            with np.errstate(all="ignore"):
                ref = v.astype(np.float16).view(np.uint16)
            assert (np.isnan(v) | (got == ref)).all()


def test_f16_split_closed_form(orc):
    """hi = RN16(v), lo = RN16((v-hi)*2048): hi + lo/2048 recovers v to 2^-22
    relative in fp16's normal range; exactly representable v gives lo == 0
    (reference: tcec/tcec.hpp:219-223, tcec/detail/scale.hpp:8-20)."""
    rng = np.random.default_rng(7)
    v = rng.uniform(-1, 1, 200_000).astype(np.float32)
    v = v[np.abs(v) > 2.0**-10]
    hi, lo = orc.split(orc.SPLIT_F16, v)
    hif, lof = orc.f16_bits_to_f32(hi), orc.f16_bits_to_f32(lo)
    # independent restatement with numpy float16 (numpy converts float64 -> float16 RN-even)
    hi_np = v.astype(np.float16)
    lo_np = ((v - hi_np.astype(np.float32)) * np.float32(2048)).astype(np.float16)
    assert (hi == hi_np.view(np.uint16)).all() and (lo == lo_np.view(np.uint16)).all()
    rec = hif.astype(np.float64) + lof.astype(np.float64) / 2048
    rel = np.abs(rec - v.astype(np.float64)) / np.abs(v.astype(np.float64))
    assert rel.max() <= 2.0**-21
    # |lo/2048| is at most half an fp16 ulp of hi
    assert (np.abs(lof) / 2048 <= np.abs(hif) * 2.0**-11 * 1.0000001).all()
    # representable values: lo == 0
    rep = rng.uniform(-4, 4, 1000).astype(np.float16).astype(np.float32)
    hi, lo = orc.split(orc.SPLIT_F16, rep)
    assert (orc.f16_bits_to_f32(hi) == rep).all() and (lo & 0x7fff == 0).all()


def test_bf16_splits_closed_form(orc):
    rng = np.random.default_rng(8)
    e = rng.integers(-15, 16, 100_000)
    v = (rng.uniform(1, 2, 100_000) * np.exp2(e) * rng.choice([-1, 1], 100_000)).astype(np.float32)
    t2 = [orc.bf16_bits_to_f32(t).astype(np.float64) for t in orc.split(orc.SPLIT_BF16X2, v)]
    t3 = [orc.bf16_bits_to_f32(t).astype(np.float64) for t in orc.split(orc.SPLIT_BF16X3, v)]
    v64 = np.abs(v.astype(np.float64))
    assert (np.abs(t2[0] + t2[1] - v) / v64).max() <= 2.0**-16
    # three bf16 terms carry 24 significand bits: exact for every fp32 value here
    assert (t3[0] + t3[1] + t3[2] == v.astype(np.float64)).all()
    # the first two terms of the 3-split are the 2-split
    assert (t3[0] == t2[0]).all() and (t3[1] == t2[1]).all()
    assert orc.split_scale(orc.SPLIT_F16) == 2048.0 and orc.split_scale(orc.SPLIT_BF16X3) == 1.0


def test_split_special_values(orc):
    v = np.array([0.0, -0.0, 1.0, -1.0, 2.0**-14, 2.0**-15, 2.0**-24, 65504.0, 2.0e-8],
                 dtype=np.float32)
    hi, lo = orc.split(orc.SPLIT_F16, v)
    hif, lof = orc.f16_bits_to_f32(hi), orc.f16_bits_to_f32(lo)
    assert hif[2] == 1.0 and lof[2] == 0.0
    assert hif[4] == 2.0**-14 and hif[5] == 2.0**-15 and hif[6] == 2.0**-24  # subnormal hi kept
    assert hif[7] == 65504.0 and lof[7] == 0
    # a value below half the smallest fp16 subnormal: hi = 0, lo carries it scaled
    assert hif[8] == 0.0 and abs(lof[8] / 2048 - 2.0e-8) < 2.0e-8 * 2.0**-10


def test_to_tf32_ties_away_literals():
    """cvt.rna.tf32.f32 of the reference (detail/common.hpp:36-48): nearest, ties away from
    zero, low 13 bits cleared.  Bit patterns written out."""
    from oracle import oracle as orc

    def bits(u):
        return np.array([u], dtype=np.uint32).view(np.float32)[0]
    cases = [
        (0x3F800000, 0x3F800000),   # 1.0
        (0x3F800FFF, 0x3F800000),   # just below half a unit: down
        (0x3F801000, 0x3F802000),   # exactly half, even mantissa below: away (nearest-even would stay)
        (0x3F801001, 0x3F802000),
        (0x3F803000, 0x3F804000),   # exactly half, odd mantissa below: up under both rules
        (0xBF801000, 0xBF802000),   # negative tie: away from zero
        (0xBF800FFF, 0xBF800000),
        (0x00001000, 0x00002000),   # subnormal tie
        (0x00000FFF, 0x00000000),
        (0x7F7FF000, 0x7F800000),   # rounds up to infinity
        (0x7F800000, 0x7F800000),   # inf stays
        (0x80000000, 0x80000000),   # -0 stays
    ]
    for src, want in cases:
        got = np.float32(orc.to_tf32(bits(src))).view(np.uint32)
        assert got == want, (hex(src), hex(got), hex(want))


def test_to_tf32_against_float64_arithmetic():
    from oracle import oracle as orc
    rng = np.random.default_rng(11)
    v = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    v = v[np.isfinite(v)]
    x = v.astype(np.float64)
    e = np.maximum(np.floor(np.log2(np.maximum(np.abs(x), 2.0**-140))), -126.0)
    ulp = np.exp2(e - 10)
    want = np.sign(x) * np.floor(np.abs(x) / ulp + 0.5) * ulp
    got = np.array([orc.to_tf32(t) for t in v], dtype=np.float32).astype(np.float64)
    ok = np.abs(want) < 3.4028235e38
    assert np.array_equal(got[ok], want[ok])
