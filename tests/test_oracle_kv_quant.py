"""The narrower block-32 cache types CRISPASR_KV_QUANT accepts (src/core/attention.h:79-105): Q4_0, Q4_1, Q5_0, Q5_1.
ggml is absent from the reference's tree, so the oracle's layouts and arithmetic are ggml's as recalled; what holds
them here: blocks worked out by hand from the formats' definitions (scale from the signed extreme, offset 8 / 16,
low nibbles = first half of the block, fifth bits in qh), a numpy restatement over random data, and the bounds of
the reference's own round-trip test on that test's own input stream (tests/test-kv-quant-roundtrip.cpp:43-53, 184-199)."""
import numpy as np
import pytest

import oracle as ora

F16 = lambda v: np.float32(np.float16(np.float32(v)))


def _fields(type_, raw):
    """(d, m or None, q[32]) per block, unpacked here without the oracle's code"""
    bs = ora.TYPE_SIZE[type_]
    out = []
    for b in np.ascontiguousarray(raw, np.uint8).reshape(-1, bs):
        o = 0
        d = np.float32(b[0:2].view(np.float16)[0]); o = 2
        m = None
        if type_ in (ora.Q4_1, ora.Q5_1):
            m = np.float32(b[2:4].view(np.float16)[0]); o = 4
        qh = 0
        if type_ in (ora.Q5_0, ora.Q5_1):
            qh = int(b[o:o + 4].copy().view("<u4")[0]); o += 4
        qs = b[o:o + 16].astype(np.int64)
        q = np.concatenate([qs & 15, qs >> 4])
        q |= ((qh >> np.arange(32)) & 1) << 4
        out.append((d, m, q))
    return out


def test_block_sizes():
    assert [ora.lib().ora_block_bytes(t) for t in (ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1, ora.Q8_0, ora.F16)] == [18, 20, 22, 24, 34, 0]


def test_q4_0_known_block_negative_extreme():
    # extreme value -4: d = -4 / -8 = 0.5, q = trunc(x/0.5 + 8.5): the ramp -4, -3.5, .. 3.5 maps to 0..15 exactly
    x = np.zeros(32, np.float32)
    x[:16] = (np.arange(16) - 8) * 0.5
    x[16:] = x[:16][::-1]
    raw = ora.quantize(ora.Q4_0, x)
    assert raw.size == 18
    assert raw[0:2].view(np.float16)[0] == np.float16(0.5)
    want_q = np.concatenate([np.arange(16), np.arange(16)[::-1]])
    assert list(raw[2:]) == [int(want_q[j] | (want_q[j + 16] << 4)) for j in range(16)]
    assert np.array_equal(ora.dequantize(ora.Q4_0, raw), x)                       # every value is on the grid


def test_q4_0_known_block_positive_extreme_clips_the_other_end():
    # extreme value +4: d = 4 / -8 = -0.5; +4 -> quant 0, -4 would be quant 16 and clips to 15 -> -3.5
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2], x[17] = 4.0, -4.0, 1.0, -0.5
    raw = ora.quantize(ora.Q4_0, x)
    assert raw[0:2].view(np.float16)[0] == np.float16(-0.5)
    (d, _, q), = _fields(ora.Q4_0, raw)
    assert q[0] == 0 and q[1] == 15 and q[2] == 6 and q[17] == 9 and q[3] == 8
    y = ora.dequantize(ora.Q4_0, raw)
    assert y[0] == 4.0 and y[1] == -3.5 and y[2] == 1.0 and y[17] == -0.5 and y[3] == 0.0
    # the first of two equal magnitudes decides the sign of the scale
    x2 = x.copy(); x2[0], x2[1] = -4.0, 4.0
    assert ora.quantize(ora.Q4_0, x2)[0:2].view(np.float16)[0] == np.float16(0.5)


def test_q5_0_known_block_and_the_fifth_bits():
    # extreme -8: d = -8 / -16 = 0.5; the ramp -8, -7.5, .. 7.5 maps to 0..31; fifth bit set for q >= 16
    x = ((np.arange(32) - 16) * 0.5).astype(np.float32)
    raw = ora.quantize(ora.Q5_0, x)
    assert raw.size == 22 and raw[0:2].view(np.float16)[0] == np.float16(0.5)
    assert int(raw[2:6].copy().view("<u4")[0]) == 0xFFFF0000                     # elements 16..31 carry the bit
    assert list(raw[6:]) == [j | (j << 4) for j in range(16)]                    # low nibbles of j and j + 16 are equal
    assert np.array_equal(ora.dequantize(ora.Q5_0, raw), x)
    # a permutation moves the bits with the elements: element e <-> bit e
    perm = np.random.default_rng(5).permutation(32)
    (_, _, q), = _fields(ora.Q5_0, ora.quantize(ora.Q5_0, x[perm]))
    assert np.array_equal(q, np.arange(32)[perm])


def test_q4_1_and_q5_1_known_blocks():
    # min 1, max 8.5: d = 7.5 / 15 = 0.5, m = 1; the ramp 1, 1.5, .. 8.5 maps to 0..15 twice over
    x = np.concatenate([1 + 0.5 * np.arange(16), 8.5 - 0.5 * np.arange(16)]).astype(np.float32)
    raw = ora.quantize(ora.Q4_1, x)
    assert raw.size == 20
    assert raw[0:2].view(np.float16)[0] == np.float16(0.5) and raw[2:4].view(np.float16)[0] == np.float16(1.0)
    assert list(raw[4:]) == [j | ((15 - j) << 4) for j in range(16)]
    assert np.array_equal(ora.dequantize(ora.Q4_1, raw), x)
    # Q5_1: min -2, max 13.5: d = 15.5 / 31 = 0.5, m = -2
    x = (-2 + 0.5 * np.arange(32)).astype(np.float32)
    raw = ora.quantize(ora.Q5_1, x)
    assert raw.size == 24
    assert raw[0:2].view(np.float16)[0] == np.float16(0.5) and raw[2:4].view(np.float16)[0] == np.float16(-2.0)
    assert int(raw[4:8].copy().view("<u4")[0]) == 0xFFFF0000
    assert list(raw[8:]) == [j | (j << 4) for j in range(16)]
    assert np.array_equal(ora.dequantize(ora.Q5_1, raw), x)


@pytest.mark.parametrize("type_", [ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1])
def test_constant_and_zero_blocks(type_):
    z = ora.quantize(type_, np.zeros(32, np.float32))
    assert np.array_equal(ora.dequantize(type_, z), np.zeros(32, np.float32))
    c = np.full(32, 0.75, np.float32)
    y = ora.dequantize(type_, ora.quantize(type_, c))
    # a constant block: the types with a minimum return it exactly (d = 0, m = c); the symmetric ones put it on quant 0
    assert np.array_equal(y, c)


@pytest.mark.parametrize("type_", [ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1])
def test_numpy_restatement_on_random_rows(type_):
    x = (ora.randn(17 + type_, (96, 128)) * 1.7).reshape(-1, 32)
    levels = 16 if type_ in (ora.Q4_0, ora.Q4_1) else 32
    got = _fields(type_, ora.quantize(type_, x))
    for xb, (d, m, q) in zip(x, got):
        if type_ in (ora.Q4_0, ora.Q5_0):
            ext = xb[np.argmax(np.abs(xb))]                                       # first of the largest magnitudes
            df = np.float32(ext) / np.float32(-(levels // 2))
            t = xb * (np.float32(1) / df) + np.float32(levels // 2 + 0.5)
            assert m is None
        else:
            lo, hi = xb.min(), xb.max()
            df = (hi - lo) / np.float32(levels - 1)
            t = (xb - lo) * (np.float32(1) / df) + np.float32(0.5)
            assert m == F16(lo)
        assert d == F16(df)
        assert np.array_equal(q, np.minimum(levels - 1, np.trunc(t.astype(np.float32)).astype(np.int64)))
    y = ora.dequantize(type_, ora.quantize(type_, x)).reshape(-1, 32)
    for yb, (d, m, q) in zip(y, got):
        want = (q - levels // 2).astype(np.float32) * d if m is None else q.astype(np.float32) * d + m
        assert np.array_equal(yb, want.astype(np.float32))


def _reference_test_stream(seed, n):
    """the generator of tests/test-kv-quant-roundtrip.cpp:43-53: xorshift64, (next % 20001) / 10000 - 1"""
    s, out = seed, np.empty(n, np.float32)
    M = (1 << 64) - 1
    for i in range(n):
        s ^= (s << 13) & M
        s ^= s >> 7
        s ^= (s << 17) & M
        out[i] = np.float32(((s >> 11) & 0xFFFFFFFF) % 20001 / 10000.0 - 1.0)
    return out


# tolerances of tests/test-kv-quant-roundtrip.cpp:190-199
REF_TOL = {ora.F16: 1e-3, ora.Q8_0: 0.02, ora.Q5_1: 0.10, ora.Q5_0: 0.10, ora.Q4_1: 0.20, ora.Q4_0: 0.20}


@pytest.mark.parametrize("type_", sorted(REF_TOL))
def test_reference_roundtrip_bounds_on_the_reference_tests_own_input(type_):
    x = _reference_test_stream(0x370, 128 * 8 * 2)                                # kHeadDim x kWrite x kKvHeads
    assert -1.0 <= x.min() and x.max() <= 1.0 and abs(float(x.mean())) < 0.05
    t = ora.from_f32(x.reshape(1, 2, 8, 128), type_)
    y = np.empty(x.size, np.float32)
    if type_ == ora.F16:
        y = ora.fp16_to_fp32(t.buf.view(np.uint16))
    else:
        y = ora.dequantize(type_, t.buf)
    err = np.abs(x - y)
    assert err.max() <= REF_TOL[type_]
    if type_ in (ora.Q4_0, ora.Q5_0, ora.Q4_1, ora.Q5_1):
        # what the formats imply: half a step, except at the clipped end of a symmetric type (a whole step)
        xb = x.reshape(-1, 32)
        levels = 16 if type_ in (ora.Q4_0, ora.Q4_1) else 32
        if type_ in (ora.Q4_0, ora.Q5_0):
            step = np.abs(xb).max(axis=1) / (levels // 2)
            bound = step * 1.0
        else:
            step = (xb.max(axis=1) - xb.min(axis=1)) / (levels - 1)
            bound = step * 0.5
        slack = (np.abs(xb).max(axis=1) + step * levels) * 2.0 ** -10           # fp16 rounding of d and m
        assert np.all(err.reshape(-1, 32).max(axis=1) <= bound + slack)
        # and they are worth their bits: the error is not far below the bound either
        assert err.max() >= 0.2 * bound.max()
