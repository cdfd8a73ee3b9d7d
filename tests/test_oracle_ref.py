"""The oracle against compiled reference code: the reference's own scalar attention helpers
(src/core/cpu_attention.h, built into oracle/_ref/ by oracle/Makefile from where the header lies in the reference
tree) driven the way its hand-written CPU backends drive them (src/wav2vec2-ggml.cpp:1908-1924,
src/firered_asr.cpp:1525-1577).  ggml's own FLASH_ATTN_EXT cannot be built here; these helpers are the reference
code for the same mathematics that can.  Skipped where oracle/_ref/ has not been built."""
import math

import numpy as np
import pytest

import oracle as ora
from cases import MAX_ABS_TOL, REL_L2_TOL, errors

pytestmark = pytest.mark.skipif(ora.ref_lib() is None, reason="oracle/_ref not built (needs the reference tree)")


def _heads_view(x: np.ndarray, n_heads: int) -> ora.Tensor:
    """[T, n_heads*hd] row-major -> ggml view ne [hd, T, n_heads, 1] over the same bytes"""
    T, H = x.shape
    hd = H // n_heads
    return ora.Tensor(x.view(np.uint8).reshape(-1).copy(), ora.F32, (hd, T, n_heads, 1), (4, 4 * H, 4 * hd, 4 * H * T))


@pytest.mark.parametrize("T,n_heads,hd", [(57, 3, 64), (33, 2, 80), (70, 2, 128), (1, 1, 8)])
def test_attention_oracle_matches_the_reference_helpers(T, n_heads, hd):
    H = n_heads * hd
    q, k, v = (ora.randn(9100 + i, (T, H)) for i in range(3))
    scale = 1.0 / math.sqrt(hd)
    want = ora.ref_mha(q, k, v, n_heads, scale)
    for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
        got = ora.flash_attn_ext(_heads_view(q, n_heads), _heads_view(k, n_heads), _heads_view(v, n_heads), None,
                                 scale, 0.0, 0.0, mode)                      # [1, T, n_heads, hd]
        max_abs, rel = errors(got.reshape(T, H), want)
        assert max_abs < 2e-5 and rel < 1e-5, (mode, max_abs, rel)          # f32 accumulation on the reference's side


def test_relpos_mask_plus_attention_matches_the_reference_relpos_attention():
    # FireRed's conformer attention: score = ((q + bu).k + (q + bv).p[T-1-tq+tk]) / sqrt(hd).  The same block through
    # the restated FastConformer graph: mask = f16(scale * rel_shift(P^T (q + bv))), then attention on q + bu.
    T, n_heads, hd = 41, 2, 64
    d = n_heads * hd
    q, k, v = (0.7 * ora.randn(9200 + i, (T, d)) for i in range(3))
    p = 0.7 * ora.randn(9203, (2 * T - 1, d))
    bu, bv = 0.3 * ora.randn(9204, (n_heads, hd)), 0.3 * ora.randn(9205, (n_heads, hd))
    want = ora.ref_relpos_mha(q, k, v, p, bu, bv, n_heads)
    scale = 1.0 / math.sqrt(hd)
    qu = (q.reshape(T, n_heads, hd) + bu[None]).reshape(T, d).astype(np.float32)
    qv = (q.reshape(T, n_heads, hd) + bv[None]).reshape(T, d).astype(np.float32)
    mask = ora.relpos_bias(_heads_view(qv, n_heads), _heads_view(p, n_heads), None, scale, T)
    got = ora.flash_attn_ext(_heads_view(qu, n_heads), _heads_view(k, n_heads), _heads_view(v, n_heads), mask, scale,
                             0.0, 0.0, ora.MODE_EXACT)
    max_abs, rel = errors(got.reshape(T, d), want)
    # the mask is the graph's f16 tensor: its rounding (2^-11 relative on each bias) is the only difference
    assert max_abs <= MAX_ABS_TOL and rel <= REL_L2_TOL, (max_abs, rel)
    # and the bias values themselves, before that rounding matters: scale * <qv[i], p[T-1-i+j]>
    m = ora.fp16_to_fp32(mask.buf.view(np.uint16)).reshape(n_heads, T, T)               # [h, i, j]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    for h in range(n_heads):
        bd = np.einsum("id,ijd->ij", qv[:, h * hd:(h + 1) * hd].astype(np.float64),
                       p[T - 1 - i + j][:, :, h * hd:(h + 1) * hd].astype(np.float64)) * scale
        assert np.abs(m[h] - bd).max() <= 2e-3 * max(1.0, np.abs(bd).max())
