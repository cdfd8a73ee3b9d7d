"""The Voxtral-style LLM decoder attention as a loop: a 407-token causal prefill, then 256 single-token steps against
the growing Q8_0 cache (GQA 32 query / 8 KV heads, head size 128).

Every step does what core_attn::kv_self_attn does with a quantised cache (src/core/attention.h:850-867, 917-920; driven
by src/voxtral.cpp:1176-1209): ggml_set_rows writes the step's K and V rows (F32 -> Q8_0) at their positions into the
layer's slice of a [hd, max_ctx, n_kv, n_layers] cache, and flash_attn_ext reads the first Lk rows of that slice - here
directly as Q8_0 blocks with native GQA, the form the op's contract allows (src/canary.cpp:953-972 reads its cache that
way).  Each step's output is held to the exact oracle over the oracle's own quantised cache, and at the end the two
caches must hold the same bytes."""
import numpy as np
import pytest
import torch

import oracle as ora
from cases import errors, MAX_ABS_TOL, REL_L2_TOL
from crispasr_amd import ggml

pytestmark = pytest.mark.gpu

HD, N_Q, N_KV, N_LAYERS = 128, 32, 8, 2
T_PROMPT, N_STEPS, MAX_CTX = 407, 256, 704           # 375 audio + 32 text tokens, 256 generated
LAYER = 1                                              # the layer whose slice the loop uses (a non-zero offset)


def _kv_new(seed, T):
    """the step's new K or V rows as the graph has them: [hd, n_kv, T] memory viewed as ne [hd, T, n_kv]"""
    x = ora.randn(seed, (T, N_KV, HD))
    return x, ora.Tensor(x.view(np.uint8).reshape(-1), ora.F32, (HD, T, N_KV), (4, 4 * HD * N_KV, 4 * HD, 4 * HD * N_KV * T))


@pytest.mark.parametrize("ktype", [ora.Q8_0, ora.F16, ora.Q4_0])
def test_prefill_then_256_steps_against_the_growing_cache(ktype):
    rs = ora.row_size(ktype, HD)
    nb = (ora.TYPE_SIZE[ktype], rs, rs * MAX_CTX, rs * MAX_CTX * N_KV)
    layer_off = LAYER * nb[3]
    nbytes = nb[3] * N_LAYERS
    # the device caches start out as garbage the way an uncleared allocation does (src/voxtral.cpp:1137-1145): only
    # rows that have been written are ever visible
    dev_k = ggml.Tensor(torch.full((nbytes,), 0xFF, dtype=torch.uint8, device="cuda"), ktype, (HD, MAX_CTX, N_KV, N_LAYERS), nb)
    dev_v = ggml.Tensor(torch.full((nbytes,), 0xFF, dtype=torch.uint8, device="cuda"), ktype, (HD, MAX_CTX, N_KV, N_LAYERS), nb)
    host_k = np.full(nbytes, 0xFF, np.uint8)
    host_v = np.full(nbytes, 0xFF, np.uint8)
    scale = HD ** -0.5
    plans = set()

    def step(seed, n_past, T, causal):
        positions = np.arange(n_past, n_past + T, dtype=np.int64)
        idx = torch.from_numpy(positions).cuda()
        for s, (dcache, hcache) in ((seed + 1, (dev_k, host_k)), (seed + 2, (dev_v, host_v))):
            x, src = _kv_new(s, T)
            dsrc = ggml.Tensor.from_host(src.buf, ggml.F32, src.ne, src.nb)
            # k_layer = view_3d(kv_k, hd, max_ctx, n_kv, nb1, nb2, il * nb3); set_rows(k_layer, K_new_perm, positions)
            ggml.set_rows(dcache.view((HD, MAX_CTX, N_KV), nb[:3] + (0,), layer_off), dsrc, idx)
            for i, p in enumerate(positions):
                row = ora.Tensor(src.buf, ora.F32, (HD, 1, N_KV), src.nb, i * src.nb[1])
                ora.cpy_f32(row, ora.Tensor(hcache, ktype, (HD, 1, N_KV), nb[:3] + (0,), layer_off + int(p) * nb[1]))
        Lk = n_past + T
        q = ora.from_f32(ora.randn(seed + 3, (1, N_Q, T, HD)))
        mask = None
        if causal:
            m = np.zeros((1, 1, T, Lk), np.float32)
            m[0, 0][np.arange(Lk)[None, :] > np.arange(T)[:, None] + n_past] = -np.inf
            mask = ora.from_f32(m, ora.F16)
        hk = ora.Tensor(host_k, ktype, (HD, Lk, N_KV), nb[:3] + (0,), layer_off)
        hv = ora.Tensor(host_v, ktype, (HD, Lk, N_KV), nb[:3] + (0,), layer_off)
        ref = ora.flash_attn_ext(q, hk, hv, mask, scale)
        dq = ggml.Tensor.from_host(q.buf, ggml.F32, q.ne, q.nb)
        dk = dev_k.view((HD, Lk, N_KV), nb[:3] + (0,), layer_off)
        dv = dev_v.view((HD, Lk, N_KV), nb[:3] + (0,), layer_off)
        dm = ggml.Tensor.from_host(mask.buf, ggml.F16, mask.ne, mask.nb) if mask is not None else None
        plans.add(ggml.flash_attn_plan(dq, dk, dv, dm, scale))
        got = ggml.flash_attn_ext(dq, dk, dv, dm, scale).numpy_f32()
        assert not np.isnan(got).any(), (n_past, T)
        max_abs, rel = errors(got, ref)
        assert max_abs <= MAX_ABS_TOL and rel <= REL_L2_TOL, "n_past %d T %d: max_abs %.3e rel_l2 %.3e" % (n_past, T, max_abs, rel)
        return max_abs

    print("prefill", T_PROMPT, "tokens, type", ktype, flush=True)
    worst = step(5000, 0, T_PROMPT, True)
    for t in range(N_STEPS):
        worst = max(worst, step(6000 + 10 * t, T_PROMPT + t, 1, False))
    print("worst max_abs over the loop %.3e; (kernel, splits) seen:" % worst, sorted(plans), flush=True)
    assert np.array_equal(dev_k.to_host(), host_k) and np.array_equal(dev_v.to_host(), host_v)
    # the decode steps ran on the split-KV MFMA kernel, and the planner changed its split count along the way
    dec = {ns for kern, ns in plans if kern == ggml.KERNEL_DECODE_MMA}
    assert len(dec) >= 2, plans
