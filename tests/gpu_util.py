"""Helpers of the GPU parity tests: upload an oracle case and run it through the C-ABI."""
from __future__ import annotations

import numpy as np

import crispasr_amd as ca
import oracle as ora
from cases import MAX_ABS_TOL, REL_L2_TOL, errors


def upload(t: ora.Tensor) -> ca.Tensor:
    return ca.Tensor.from_host(t.buf, t.type, t.ne, t.nb, t.offset)


def run_gpu(case: dict, kernel: int = ca.ggml.KERNEL_AUTO, n_splits: int = 0, tile_variant: int = 0) -> np.ndarray:
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    m = upload(case["mask"]) if case["mask"] is not None else None
    out = ca.flash_attn_ext(q, k, v, m, case["scale"], case["max_bias"], case["softcap"],
                            kernel=kernel, n_splits=n_splits, tile_variant=tile_variant)
    return out.numpy_f32()          # [B, Nq, Hq, DV]


def plan_details(case: dict, **kw) -> dict:
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    m = upload(case["mask"]) if case["mask"] is not None else None
    return ca.ggml.flash_attn_plan_details(q, k, v, m, case["scale"], case["max_bias"], case["softcap"], **kw)


def run_oracle(case: dict, mode: int = ora.MODE_EXACT) -> np.ndarray:
    return ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"],
                              case["max_bias"], case["softcap"], mode)


def assert_parity(got: np.ndarray, ref: np.ndarray, what: str = "", max_abs_tol: float = MAX_ABS_TOL,
                  rel_l2_tol: float = REL_L2_TOL):
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert not np.isnan(got).any(), f"{what}: NaN in output"
    max_abs, rel = errors(got, ref)
    assert max_abs <= max_abs_tol and rel <= rel_l2_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"
    return max_abs, rel
