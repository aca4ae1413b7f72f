"""utils::cp_async and utils::cast on the GPU (reference: test/utils/cp_async.cu,
test/utils/cast.cu), through the C-ABI harness entries."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("size", [4, 8, 16])
@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4, 5])
def test_cp_async_copies_every_byte(tc, dev, size, mode):
    """The reference's check: input word i holds float(i); the copy through LDS returns
    it unchanged (error = 0), for lane-linear, scattered, partially masked and pipelined use,
    and for cp_async_lane_linear (modes 4, 5: full and partially masked waves)."""
    words = 256 * size // 4
    src = torch.arange(words, dtype=torch.float32, device=dev)
    if mode >= 4 and size == 8:
        from wmma_extension_amd._lib import WmmaeError
        with pytest.raises(WmmaeError) as e:
            tc.utils_cp_async(size, mode, src)
        assert e.value.status == -4
        return
    got = tc.utils_cp_async(size, mode, src).cpu().numpy()
    expect = np.arange(words, dtype=np.float32)
    if mode in (2, 5):
        elem = (np.arange(words) // (size // 4)) % 128
        expect = np.where(elem % 3 != 0, expect, 0.0).astype(np.float32)
    assert np.array_equal(got, expect)


@pytest.mark.parametrize("size", [4, 16])
@pytest.mark.parametrize("copies", [1, 3, 4])
def test_cp_async_three_stage_pipeline_keeps_two_groups_in_flight(tc, dev, size, copies):
    """cp_async / commit / wait_group<2> as a three-stage pipeline (the use the reference's
    utils.hpp:29-64 is made for): every byte arrives, and wait_group<2> waits for exactly the
    oldest group - right after it the wave's own counter of outstanding vector-memory
    instructions (read from the hardware) is at most the two younger groups' copies, and above
    zero at least once: later groups are still in flight while the first is consumed."""
    groups = 8
    words = groups * copies * 64 * size // 4
    src = torch.arange(words, dtype=torch.float32, device=dev)
    junk = torch.empty(1 << 28, dtype=torch.float32, device=dev)
    in_flight = 0
    for attempt in range(5):
        # push the source out of the caches (1 GiB written behind it), so that the copies take a
        # round trip to HBM, much longer than the wave needs to issue three groups
        junk.fill_(float(attempt))
        torch.cuda.synchronize()
        got, pending = tc.utils_cp_async_pipeline(size, copies, groups, src)
        torch.cuda.synchronize()
        assert torch.equal(got, src)
        p = pending.cpu().numpy()
        assert 0 <= p[0] <= 3 * copies                     # three groups issued, nothing awaited
        assert (p[1:1 + groups] >= 0).all() and (p[1:1 + groups] <= 2 * copies).all(), p
        assert p[1 + groups] == 0                          # wait_all
        in_flight = max(in_flight, int(p[1:1 + groups].max()))
        if in_flight > 0:
            break
    # groups of a few hundred bytes share their HBM bursts and may all arrive together; larger
    # ones were still in flight behind the awaited group in one of the attempts at least
    if copies * 64 * size >= 4096:
        assert in_flight > 0


def test_cp_async_pipeline_register_path_has_nothing_pending(tc, dev):
    """Size 8 has no direct global -> LDS load: the copies go through registers, are complete when
    cp_async returns and are not counted as pending."""
    src = torch.arange(6 * 2 * 64 * 2, dtype=torch.float32, device=dev)
    got, pending = tc.utils_cp_async_pipeline(8, 2, 6, src)
    assert torch.equal(got, src)
    assert (pending.cpu().numpy()[1:] == 0).all()


def test_cp_async_argument_checks(tc, dev):
    from wmma_extension_amd._lib import WmmaeError
    src = torch.zeros(1024, dtype=torch.float32, device=dev)
    with pytest.raises(WmmaeError) as e:
        tc.utils_cp_async(12, 0, src)
    assert e.value.status == -1
    with pytest.raises(WmmaeError) as e:
        tc.utils_cp_async(16, 0, src[1:])
    assert e.value.status == -7


def test_cast_matches_oracle_conversions(tc, orc, dev):
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 2**32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    v = bits.view(np.float32)
    v = v[np.isfinite(v)]
    special = np.array([0.0, -0.0, 1.0, 65504.0, 65520.0, 2.0**-24, 2.0**-25, 1.0 + 2.0**-11,
                        1.0 + 3 * 2.0**-11, 3.0e38], dtype=np.float32)
    v = np.concatenate([v, special])
    x = torch.from_numpy(v).to(dev)
    h = tc.utils_cast(0, x).cpu().numpy().view(np.uint16)
    assert np.array_equal(h, orc.split(orc.SPLIT_F16, v)[0])
    b = tc.utils_cast(1, x).cpu().numpy().view(np.uint16)
    assert np.array_equal(b, orc.split(orc.SPLIT_BF16X2, v)[0])
    # tf32: 10 mantissa bits in an fp32 container, ties away from zero (cvt.rna in the reference)
    t = tc.utils_cast(2, x).cpu().numpy()
    want = np.array([orc.to_tf32(e) for e in v[:4096]] + [orc.to_tf32(e) for e in special], dtype=np.float32)
    got = np.concatenate([t[:4096], t[-special.size:]])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert (t.view(np.uint32) & 0x1FFF == 0).all()
    # in float64 over the whole sample: scale to the kept precision, floor(|x| + 1/2), scale back
    x64 = v.astype(np.float64)
    e = np.maximum(np.floor(np.log2(np.maximum(np.abs(x64), 2.0**-140))), -126.0)
    ulp = np.exp2(e - 10)
    r64 = np.sign(x64) * np.floor(np.abs(x64) / ulp + 0.5) * ulp
    ok = np.abs(r64) < 3.4028235e38
    assert np.array_equal(t[ok].astype(np.float64), r64[ok])
    f = tc.utils_cast(3, x).cpu().numpy()
    assert np.array_equal(f.view(np.uint32), v.view(np.uint32))
