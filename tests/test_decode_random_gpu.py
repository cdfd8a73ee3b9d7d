"""Randomised decode shapes: few query rows per KV head against long caches of every type, so that the decode kernel's
key ranges, partial last steps, streamed and strided row paths and the merge pass meet in every combination."""
import numpy as np
import pytest

import oracle as ora
from cases import make_case, sweep_seeds
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_gpu, run_oracle

pytestmark = pytest.mark.gpu

TYPES = [ora.F16, ora.Q8_0, ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1]


def draw(seed: int) -> dict:
    r = np.random.default_rng(77000 + seed)
    gqa = int(r.choice([1, 2, 4, 8]))
    Hkv = int(r.integers(1, 4))
    B = int(r.integers(1, 4))
    return dict(seed=88000 + seed, D=int(r.choice([64, 128])), Nq=int(r.integers(1, 1 + 16 // gqa)),
                Nkv=int(r.choice([int(r.integers(17, 6000)), 32 * int(r.integers(1, 160)), 4096])),
                Hq=Hkv * gqa, Hkv=Hkv, B=B, Bk=B if r.random() < 0.7 else 1, ktype=int(r.choice(TYPES)),
                mask=[None, None, "random_inf", "random_inf_batched", "causal"][int(r.integers(0, 5))],
                kv_layout=str(r.choice(["contig", "contig", "gap", "thd"])))


@pytest.mark.parametrize("seed", sweep_seeds("DECODE_RANDOM_CASES", 40))
def test_random_decode_shape_matches_oracle(seed):
    spec = draw(seed)
    print("decode case", spec, flush=True)
    case = make_case(**spec)
    ref = run_oracle(case)
    plan = plan_details(case)
    # <= 16 rows per KV head, more than 16 keys: the decode kernel - except 9 .. 16 queries (no GQA) over an f16 cache of
    # 128-wide heads or of 2048 keys and more, which the tile kernel takes
    to_tile = spec["ktype"] == ora.F16 and spec["Hq"] == spec["Hkv"] and spec["Nq"] > 8 and (spec["D"] == 128 or spec["Nkv"] >= 2048)
    assert plan["kernel"] == (ggml.KERNEL_MMA if to_tile else ggml.KERNEL_DECODE_MMA), plan
    # (a causal mask over more keys than queries leaves every row at least Nkv - Nq + 1 keys)
    got = run_gpu(case)
    assert_parity(got, ref, "auto %s" % spec)
    for ns in (0, 1, 3):                                           # the planner's count, unsplit, and an odd number of key ranges
        assert_parity(run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA, n_splits=ns), ref, "%d ranges %s" % (ns, spec))
    assert_parity(run_gpu(case, kernel=ggml.KERNEL_VEC), ref, "vector kernel %s" % spec)
