"""The CPU oracle against the committed golden vectors (tests/golden/, written with numpy alone: float64 textbook
attention on the decoded operands, numpy.float16 conversions, Q8_0 known-answer blocks, the relative-position mask
through numpy's strided view).  The reference holds no vectors of its own for this op."""
import numpy as np
import pytest

import oracle as ora
from cases import errors
from golden_util import FATTN, load_conversions, load_fattn, load_relpos


@pytest.mark.parametrize("name", FATTN)
def test_oracle_exact_mode_matches_golden(name):
    case, want = load_fattn(name)
    got = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"], 0.0, 0.0, ora.MODE_EXACT)
    max_abs, rel = errors(got, want)
    assert max_abs <= 2e-6 and rel <= 1e-6, (name, max_abs, rel)      # both are float64 arithmetic on the same operands


@pytest.mark.parametrize("name", FATTN)
def test_oracle_ggml_like_mode_stays_near_golden(name):
    case, want = load_fattn(name)
    got = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"], 0.0, 0.0, ora.MODE_GGML_LIKE)
    max_abs, rel = errors(got, want)
    # this mode carries the roundings ggml-cpu is recalled to make (f16 accumulator for F16 V, the query row quantised
    # to Q8_0 for Q8_0 K): it is the less accurate side, a few 1e-3 from the exact result
    assert max_abs <= 8e-3 and rel <= 6e-3, (name, max_abs, rel)


def test_conversions_match_golden():
    z = load_conversions()
    assert np.array_equal(ora.fp32_to_fp16(z["f32"]), z["f16_bits"])
    x, raw, dec = z["q8_x"], z["q8_raw"], z["q8_dec"]
    got = ora.quantize_q8_0(x.reshape(-1)).reshape(raw.shape)
    assert np.array_equal(got, raw)
    assert np.array_equal(ora.dequantize_q8_0(raw.reshape(-1)).reshape(dec.shape), dec)


def test_relpos_bias_matches_golden():
    t, want = load_relpos()
    got = ora.relpos_bias(t["qv"], t["r"], t["add"], t["scale"], t["n_kv"]).buf.view(np.uint16).reshape(want.shape)
    neg_inf = want == 0xFC00
    assert np.array_equal(got == 0xFC00, neg_inf)
    g, w = ora.fp16_to_fp32(got[~neg_inf]), ora.fp16_to_fp32(want[~neg_inf])
    # same arithmetic (float64 dot rounded to f32, f32 scale and add, one f16 rounding); a dot that lands within an
    # f32 ulp of a rounding boundary may fall the other way: an f16 ulp on a handful of elements at most
    assert (got[~neg_inf] != want[~neg_inf]).mean() < 1e-3
    assert np.abs(g - w).max() <= 2e-3 * np.maximum(1.0, np.abs(w)).max()
