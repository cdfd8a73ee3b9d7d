"""Loads the committed fixtures of tests/golden/ (written by tests/golden/make_golden.py with numpy alone) as
oracle.Tensor views, in the form the oracle and GPU helpers take."""
from __future__ import annotations

import os

import numpy as np

import oracle as ora

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FATTN = ["mha_f16", "gqa_causal_q8_0", "bias_pad_f32", "decode_beams_f16", "decode_gqa_q8_0", "tile_f16_d128"]


def _bytes(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()


def load_fattn(name: str):
    """-> (case dict as tests/cases.make_case builds it, expected output [B, Nq, Hq, D] f32)"""
    z = np.load(os.path.join(GOLDEN, f"fattn_{name}.npz"))          # arrays only: allow_pickle stays False
    q = z["q"]
    B, Hq, Nq, D = q.shape
    ktype = int(z["ktype"])
    Bk, Hkv, Nkv, _ = z["k_raw"].shape
    case = {
        "q": ora.Tensor(_bytes(q), ora.F32, (D, Nq, Hq, B)),
        "k": ora.Tensor(_bytes(z["k_raw"]), ktype, (D, Nkv, Hkv, Bk)),
        "v": ora.Tensor(_bytes(z["v_raw"]), ktype, (D, Nkv, Hkv, Bk)),
        "mask": None, "scale": float(z["scale"]), "max_bias": 0.0, "softcap": 0.0,
    }
    if "mask" in z.files:
        m = z["mask"]                                               # uint16 [Bm, Hm, Nq, Nkv]
        case["mask"] = ora.Tensor(_bytes(m), ora.F16, (m.shape[3], m.shape[2], m.shape[1], m.shape[0]))
    return case, z["out"]


def load_relpos():
    z = np.load(os.path.join(GOLDEN, "relpos_bias.npz"))
    qv, r, add = z["qv"], z["r"], z["add"]
    B, H, T, D = qv.shape
    t = {
        "qv": ora.Tensor(_bytes(qv), ora.F32, (D, T, H, B)),
        "r": ora.Tensor(_bytes(r), ora.F32, (D, r.shape[2], H, 1)),
        "add": ora.Tensor(_bytes(add), ora.F32, (T, T, 1, B)),
        "scale": float(z["scale"]), "n_kv": T,
    }
    return t, z["mask"]                                             # f16 bits [B, H, Nq, Nkv]


def load_conversions():
    return np.load(os.path.join(GOLDEN, "conversions.npz"))
