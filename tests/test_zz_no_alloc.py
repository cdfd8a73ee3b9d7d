"""mi355x_flash_attn_ext_noalloc - the entry point for callers that cannot allocate - against mi355x_flash_attn_ext,
through the C ABI: same bits (the same kernels run, the scratch is the library's static device array), on two calls in
a row, the second with a smaller input, plus the size limit."""
import numpy as np
import pytest
import torch

import oracle as ora
from cases import make_case
from crispasr_amd import ggml
from gpu_util import assert_parity, run_oracle, upload

pytestmark = pytest.mark.gpu

CALLS = [
    # larger first: Q8_0 K/V rounded to f16 copies in the scratch (tile kernel), then split-KV partials (decode kernel),
    # then the query rows staged as Q8_0 in front of the partials
    (dict(seed=801, D=128, Nq=300, Nkv=1100, Hq=8, Hkv=2, ktype=ora.Q8_0, mask="causal"), {}),
    (dict(seed=802, D=64, Nq=5, Nkv=1500, Hq=20, q_layout="thd", kv_layout="thd", scale=0.35355339), {}),
    (dict(seed=803, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0), dict(q_quant=ggml.Q8_0)),
    # a head size the tile kernel takes on zero-padded f16 copies, which go to the scratch as well
    (dict(seed=804, D=80, Nq=200, Nkv=300, Hq=8, ktype=ora.F32, mask="causal"), {}),
]


def _free_bytes():
    torch.cuda.synchronize()
    return ggml.device_info(torch.cuda.current_device())["free_memory"]


def test_noalloc_entry_point_matches_the_ordinary_one_and_allocates_nothing():
    cases = [(make_case(**spec), kw) for spec, kw in CALLS]
    dev = []
    for case, kw in cases:
        q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
        m = upload(case["mask"]) if case["mask"] is not None else None
        need = ggml.flash_attn_workspace_size(q, k, v, m, case["scale"], **kw)
        assert 0 < need <= ggml.NOALLOC_SCRATCH_BYTES, need            # every call here really uses the scratch
        out = ggml.Tensor.empty(ggml.F32, (v.ne[0], q.ne[2], q.ne[1], q.ne[3]))
        dev.append((q, k, v, m, out, need))
    # first round, larger call first: set-up (the array's address on this device) and each kernel's first launch, which
    # may make the runtime itself take memory
    got = []
    for (case, kw), (q, k, v, m, out, need) in zip(cases, dev):
        out.buf.fill_(0xFF)                                            # NaN bits: every element must be written
        print("noalloc call", need, "bytes of scratch", flush=True)
        ggml.flash_attn_ext(q, k, v, m, case["scale"], out=out, no_alloc=True, **kw)
    for (case, kw), (q, k, v, m, out, need) in zip(cases, dev):
        got.append(out.numpy_f32())
    # second round the other way round (smaller first), back to back: no device memory may be taken by these calls
    free0 = _free_bytes()
    for (case, kw), (q, k, v, m, out, need) in reversed(list(zip(cases, dev))):
        out.buf.fill_(0xFF)
        ggml.flash_attn_ext(q, k, v, m, case["scale"], out=out, no_alloc=True, **kw)
    assert _free_bytes() == free0
    # against the ordinary entry point (same bits) and the oracle
    for i, ((case, kw), (q, k, v, m, out, need)) in enumerate(zip(cases, dev)):
        again = out.numpy_f32()
        want = ggml.flash_attn_ext(q, k, v, m, case["scale"], **kw).numpy_f32()
        assert np.array_equal(got[i], want), i
        assert np.array_equal(again, want), i
        if not kw:
            assert_parity(got[i], run_oracle(case), "noalloc call %d against the oracle" % i)
        else:
            assert_parity(got[i], run_oracle(case, ora.MODE_GGML_LIKE), "noalloc q_quant call against the ggml-like oracle")


def test_noalloc_entry_point_refuses_what_its_scratch_cannot_hold():
    """F32 K/V of 4096 keys x 128 x 8 heads x 5 sequences need 40 MiB of f16 copies: refused with a message, nothing
    launched, the destination untouched; the ordinary entry point takes the same call."""
    D, Nq, Nkv, H, B = 128, 128, 4096, 8, 5
    q = ggml.Tensor(torch.randn(B * H * Nq * D, device="cuda").view(torch.uint8), ggml.F32, (D, Nq, H, B))
    k = ggml.Tensor(torch.randn(B * H * Nkv * D, device="cuda").view(torch.uint8), ggml.F32, (D, Nkv, H, B))
    v = ggml.Tensor(torch.randn(B * H * Nkv * D, device="cuda").view(torch.uint8), ggml.F32, (D, Nkv, H, B))
    assert ggml.flash_attn_workspace_size(q, k, v, None, 0.1) > ggml.NOALLOC_SCRATCH_BYTES
    out = ggml.Tensor.empty(ggml.F32, (D, H, Nq, B))
    out.buf.fill_(0x5A)
    with pytest.raises(ggml.Mi355xError) as err:
        ggml.flash_attn_ext(q, k, v, None, 0.1, out=out, no_alloc=True)
    assert err.value.status == ggml.ERR_WORKSPACE and "allocation-free" in str(err.value)
    torch.cuda.synchronize()
    assert bool((out.buf == 0x5A).all())
    ref = ggml.flash_attn_ext(q, k, v, None, 0.1).numpy_f32()
    assert np.isfinite(ref).all()
