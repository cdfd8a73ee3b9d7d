"""GPU parity with every tensor in pinned, GPU-mapped host memory.

A backend that implements one op has to leave weights and KV caches readable by ggml-cpu, so its default
buffer type is host memory with is_host = true (the runtimes put both there: src/crispasr.cpp:1940-1944,
3942-3971; src/voxtral.cpp:1137-1145) and the kernels read q/k/v/mask and write dst through host pointers.
Each case runs once on such buffers and once on device buffers: the results must match the oracle within the
path's tolerance and each other bit for bit, and must be visible to the CPU after a stream synchronise.
"""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import make_case
from gpu_util import assert_parity, run_gpu, run_oracle

pytestmark = pytest.mark.gpu

K = ca.ggml


def in_host(t: ora.Tensor) -> ca.Tensor:
    return ca.Tensor.in_host_buffer(t.buf, t.type, t.ne, t.nb, t.offset)


CASES = [
    ("tile kernel, f16 K/V, Whisper strides", K.KERNEL_MMA,
     dict(seed=801, D=64, Nq=300, Nkv=200, Hq=4, q_layout="thd", kv_layout="thd")),
    ("tile kernel, per-head f16 bias with -inf pads (mask fetched by global->LDS loads)", K.KERNEL_MMA,
     dict(seed=802, D=128, Nq=192, Nkv=192, Hq=2, B=2, mask="bias_perhead_pad", lengths=[150, 192])),
    ("tile kernel, Q8_0 K/V rounded to f16 in the workspace first, causal mask", K.KERNEL_MMA,
     dict(seed=803, D=128, Nq=160, Nkv=200, Hq=8, Hkv=2, ktype=ora.Q8_0, mask="causal")),
    ("decode kernel, Q8_0 cache, 32 q / 8 kv heads", K.KERNEL_DECODE_MMA,
     dict(seed=804, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0)),
    ("decode, 5 beams with their own masks", K.KERNEL_AUTO,
     dict(seed=805, D=64, Nq=1, Nkv=224, Hq=20, B=5, mask="random_inf_batched", scale=1.0, std=0.35)),
    ("vector kernel, F32 K/V, head size 80", K.KERNEL_VEC,
     dict(seed=806, D=80, Nq=3, Nkv=77, Hq=4, ktype=ora.F32)),
]


@pytest.mark.parametrize("what,kernel,spec", CASES, ids=[c[0].split(",")[0] + f" {i}" for i, c in enumerate(CASES)])
def test_flash_attn_on_host_buffers(what, kernel, spec):
    case = make_case(**spec)
    print("host buffers:", what, spec, flush=True)
    q, k, v = in_host(case["q"]), in_host(case["k"]), in_host(case["v"])
    m = in_host(case["mask"]) if case["mask"] is not None else None
    ne = (v.ne[0], q.ne[2], q.ne[1], q.ne[3])
    out = ca.Tensor(ca.HostBuffer(4 * ne[0] * ne[1] * ne[2] * ne[3]), ca.F32, ne)
    out.buf.array[:] = 0xFF                                   # NaN bytes: every element must be written
    ca.flash_attn_ext(q, k, v, m, case["scale"], case["max_bias"], case["softcap"], kernel=kernel, out=out)
    torch.cuda.synchronize()
    got = out.numpy_f32().copy()                               # read by the CPU, in place
    assert_parity(got, run_oracle(case), what)
    assert np.array_equal(got, run_gpu(case, kernel)), "host-buffer and device-buffer results differ"


@pytest.mark.parametrize("dtype", [ora.F16, ora.Q8_0])
def test_kv_write_into_a_host_buffer_cache(dtype):
    # ggml_cpy of new K rows into a cache view (src/core/attention.h:342-378) when the cache lives in host memory
    D, T, H, ctx, n_past = 128, 9, 4, 32, 5
    src = ora.from_f32(2.0 * ora.randn(811, (1, H, T, D)), ora.F32)
    rs = ora.row_size(dtype, D)
    cache = np.full(H * ctx * rs, 0xAB, np.uint8)
    nb = (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs)
    want = ora.Tensor(cache.copy(), dtype, (D, T, H, 1), nb, n_past * rs)
    ora.cpy_f32(src, want)
    dst = ca.Tensor.in_host_buffer(cache, dtype, (D, T, H, 1), nb, n_past * rs)
    print("cpy into host cache", dtype, flush=True)
    ca.cpy(in_host(src), dst)
    torch.cuda.synchronize()
    assert np.array_equal(dst.buf.array[:cache.size], want.buf)
