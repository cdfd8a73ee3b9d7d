"""The HIP kernels against the committed golden vectors (tests/golden/): an anchor that does not pass through the
oracle's C code."""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from gpu_util import assert_parity, run_gpu, upload
from golden_util import FATTN, load_conversions, load_fattn, load_relpos

pytestmark = pytest.mark.gpu

K = ca.ggml


@pytest.mark.parametrize("name", FATTN)
@pytest.mark.parametrize("kernel", [K.KERNEL_AUTO, K.KERNEL_VEC])
def test_kernels_match_golden(name, kernel):
    case, want = load_fattn(name)
    print("golden", name, "kernel", kernel, K.flash_attn_plan(upload(case["q"]), upload(case["k"]), upload(case["v"]),
          upload(case["mask"]) if case["mask"] is not None else None, case["scale"], kernel=kernel), flush=True)
    assert_parity(run_gpu(case, kernel), want, name)


def test_copies_match_golden_conversions():
    z = load_conversions()
    f = z["f32"]
    src = ora.from_f32(f.reshape(1, 1, 1, -1), ora.F32)
    dst = ca.Tensor.empty(ca.F16, (f.size, 1, 1, 1))
    ca.cpy(upload(src), dst)
    torch.cuda.synchronize()
    assert np.array_equal(dst.to_host()[:2 * f.size].view(np.uint16), z["f16_bits"])
    x, raw = z["q8_x"], z["q8_raw"]
    dq = ca.Tensor.empty(ca.Q8_0, (32, x.shape[0], 1, 1))
    ca.cpy(upload(ora.from_f32(x.reshape(1, 1, x.shape[0], 32), ora.F32)), dq)
    torch.cuda.synchronize()
    assert np.array_equal(dq.to_host()[:raw.size].reshape(raw.shape), raw)


def test_relpos_bias_matches_golden():
    t, want = load_relpos()
    out = K.relpos_bias(upload(t["qv"]), upload(t["r"]), upload(t["add"]), t["scale"], t["n_kv"])
    torch.cuda.synchronize()
    got = out.to_host()[:2 * want.size].view(np.uint16).reshape(want.shape)
    neg_inf = want == 0xFC00
    assert np.array_equal(got == 0xFC00, neg_inf)
    g, w = ora.fp16_to_fp32(got[~neg_inf]), ora.fp16_to_fp32(want[~neg_inf])
    err = np.abs(g - w)
    # the kernel rounds Q_v and R to f16 before an f32 accumulation: a few f16 ulps at most, under one on average
    assert (err <= 4e-3 * np.maximum(1.0, np.abs(w))).all() and err.mean() < 6e-4, (err.max(), err.mean())


@pytest.mark.skipif(ora.ref_lib() is None, reason="oracle/_ref not built (needs the reference tree)")
@pytest.mark.parametrize("T,n_heads,hd,kernel", [(300, 3, 64, K.KERNEL_MMA), (150, 2, 128, K.KERNEL_MMA),
                                                  (40, 2, 80, K.KERNEL_VEC), (12, 4, 64, K.KERNEL_AUTO)])
def test_kernels_match_the_reference_scalar_attention(T, n_heads, hd, kernel):
    # compiled reference code as the checker: src/core/cpu_attention.h driven as src/wav2vec2-ggml.cpp:1908-1924 does,
    # Q/K/V [T, n_heads*hd] row-major F32 (the kernels see them as strided ggml views of the same bytes)
    H = n_heads * hd
    q, k, v = (ora.randn(9400 + i, (T, H)) for i in range(3))
    scale = 1.0 / np.sqrt(hd)
    want = ora.ref_mha(q, k, v, n_heads, scale)

    def heads(x):
        return upload(ora.Tensor(x.view(np.uint8).reshape(-1).copy(), ora.F32, (hd, T, n_heads, 1), (4, 4 * H, 4 * hd, 4 * H * T)))

    print("kernel", kernel, "vs reference scalar attention", T, n_heads, hd, flush=True)
    out = ca.flash_attn_ext(heads(q), heads(k), heads(v), None, float(scale), kernel=kernel)
    assert_parity(out.numpy_f32().reshape(T, H), want, "vs reference scalar attention")
