"""The shapes that the planner's rules were measured on, at full size: which kernel and form AUTO takes there, and parity
of what it computes against the CPU oracle (the rules themselves are pinned without a GPU in tests/test_host.py)."""
import pytest

import oracle as ora
from cases import make_case
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_gpu, run_oracle

pytestmark = pytest.mark.gpu

VEC, MMA, DEC = ggml.KERNEL_VEC, ggml.KERNEL_MMA, ggml.KERNEL_DECODE_MMA

SHAPES = [
    # a short prompt against a long Q8_0 cache, four and eight 16-row chunks per KV head: the decode kernel, by price
    (dict(seed=901, D=64, Nq=16, Nkv=4096, Hq=32, Hkv=8, B=5, ktype=ora.Q8_0, mask="causal"), DEC, None),
    (dict(seed=902, D=128, Nq=32, Nkv=4096, Hq=32, Hkv=8, B=5, ktype=ora.Q8_0, mask="causal"), DEC, None),
    # a long cache under few heads: no more key ranges than their merge is worth
    (dict(seed=903, D=128, Nq=1, Nkv=8192, Hq=8, B=1, ktype=ora.F16), DEC, dict(max_splits=24)),
    # 16 query rows of one head over an f16 cache of 128-wide heads: the tile kernel, in key ranges of its own
    (dict(seed=904, D=128, Nq=16, Nkv=8192, Hq=8, B=1, ktype=ora.F16, mask="causal"), MMA, dict(min_splits=8)),
    # 160 key-split workgroups against a long cache: cut towards two workgroups per CU
    (dict(seed=905, D=128, Nq=256, Nkv=4096, Hq=40, B=1, ktype=ora.F16, mask="causal"), MMA, dict(min_splits=3, max_splits=3, key_split=2)),
    # F32 K/V under four queries: the tile kernel from 40k (row, key) pairs on
    (dict(seed=906, D=64, Nq=4, Nkv=1024, Hq=32, Hkv=8, B=5, ktype=ora.F32), MMA, None),
    # ... and a single query: the vector kernel, in at most 8 ranges
    (dict(seed=907, D=128, Nq=1, Nkv=4096, Hq=32, B=1, ktype=ora.F32), VEC, dict(max_splits=8)),
    # 300 queries: 128-query workgroups (256-query ones would carry 512 slots)
    (dict(seed=908, D=64, Nq=300, Nkv=300, Hq=64, B=1, ktype=ora.F16, mask="causal"), MMA, dict(query_blocks=1, key_split=1)),
    # a small f16 call with 16 chunks per KV head: one round of the decode kernel
    (dict(seed=909, D=64, Nq=64, Nkv=256, Hq=32, Hkv=8, B=1, ktype=ora.F16, mask="causal"), DEC, None),
    # a masked 64-wide call at one 128-query workgroup per CU and 900 keys: the key-split form
    (dict(seed=910, D=64, Nq=900, Nkv=900, Hq=32, B=1, ktype=ora.F16, mask="bias_perhead"), MMA, dict(key_split=2)),
    # the vector kernel's short ranges for wide heads, and a GQA group counted once
    (dict(seed=911, D=128, Nq=1, Nkv=408, Hq=32, Hkv=8, B=1, ktype=ora.F32), VEC, dict(min_splits=8, max_splits=8)),
]


@pytest.mark.parametrize("spec,kernel,want", SHAPES, ids=lambda x: "seed%d" % x["seed"] if isinstance(x, dict) and "seed" in x else None)
def test_planned_shape_runs_where_it_was_measured_and_matches_the_oracle(spec, kernel, want):
    case = make_case(**spec)
    plan = plan_details(case)
    print("planned shape", spec, {k: plan[k] for k in ("kernel", "n_splits", "key_split", "query_blocks")}, flush=True)
    assert plan["kernel"] == kernel, plan
    want = want or {}
    assert want.get("min_splits", 1) <= plan["n_splits"] <= want.get("max_splits", 1 << 20), plan
    for field in ("key_split", "query_blocks"):
        if field in want:
            assert plan[field] == want[field], plan
    ref = run_oracle(case)
    assert_parity(run_gpu(case), ref, str(spec))
