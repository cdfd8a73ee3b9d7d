"""Seeded FLASH_ATTN_EXT cases shared by the oracle tests and the GPU parity tests.

A case is a dict of oracle.Tensor views (host bytes) plus the scalar op parameters; the GPU
tests upload the same bytes and call the HIP path through the C-ABI.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import numpy as np

import oracle as ora

NEG_INF_H = np.uint16(0xFC00)


def sweep_seeds(count_variable: str, default: int) -> range:
    """Seeds of a randomised test: `default` of them, or as many as the environment variable says (a longer hunt), from
    RANDOM_FIRST_SEED on (0 by default: the cases every run repeats)."""
    first = int(os.environ.get("RANDOM_FIRST_SEED", "0"))
    return range(first, first + int(os.environ.get(count_variable, str(default))))


def _store(x_f32: np.ndarray, type_: int, layout: str, pad_rows: int = 0) -> ora.Tensor:
    """x_f32 is numpy [B, H, N, D].  Layouts:
    contig : ggml ne [D, N, H, B] contiguous
    thd    : memory order [B][N][H][D] viewed as ne [D, N, H, B] - the permuted views the
             runtimes pass (nb1 = H*rowsize, nb2 = rowsize; src/crispasr.cpp:2806-2819)
    pad_rows > 0 appends that many zero rows to N (Whisper's n_ctx padded to 1536,
    src/crispasr.cpp:2733) and reports them in ne[1].
    """
    B, H, N, D = x_f32.shape
    if pad_rows:
        x_f32 = np.concatenate([x_f32, np.zeros((B, H, pad_rows, D), np.float32)], axis=2)
        N += pad_rows
    rs = ora.row_size(type_, D)
    if layout == "contig":
        t = ora.from_f32(x_f32, type_)
        return t
    if layout == "thd":
        xt = np.ascontiguousarray(x_f32.transpose(0, 2, 1, 3))      # [B, N, H, D]
        t = ora.from_f32(xt, type_)
        return ora.Tensor(t.buf, type_, (D, N, H, B), (ora.TYPE_SIZE[type_], H * rs, rs, N * H * rs))
    if layout == "gap":
        # rows padded to a larger pitch and a leading byte offset (a view into a bigger cache)
        pitch = rs + 64
        lead = 128
        t = ora.from_f32(x_f32, type_)
        raw = np.zeros(lead + B * H * N * pitch, np.uint8)
        src = t.buf.reshape(B * H * N, rs)
        dst = raw[lead:].reshape(B * H * N, pitch)
        dst[:, :rs] = src
        return ora.Tensor(raw, type_, (D, N, H, B), (ora.TYPE_SIZE[type_], pitch, N * pitch, H * N * pitch), lead)
    raise ValueError(layout)


def make_mask(kind: Optional[str], seed: int, Nq: int, Nkv: int, Hq: int, B: int,
              lengths=None) -> Optional[ora.Tensor]:
    """f16 mask [Nkv, Nq, Hm, Bm] (ggml ne order), contiguous."""
    if kind is None:
        return None
    if kind == "causal":          # LLM prefill: key j visible to query i iff j <= i + (Nkv - Nq)
        m = np.zeros((1, 1, Nq, Nkv), np.float32)
        off = Nkv - Nq
        jj = np.arange(Nkv)[None, :]
        ii = np.arange(Nq)[:, None]
        m[0, 0][jj > ii + off] = -np.inf
    elif kind == "random_inf":    # beam-style arbitrary visibility (src/crispasr.cpp:3485-3487)
        r = ora.randn(seed + 7001, (1, 1, Nq, Nkv))
        m = np.where(r > 0.3, -np.inf, 0.0).astype(np.float32)
        m[..., 0] = 0.0           # keep one key visible per row
    elif kind == "random_inf_batched":
        r = ora.randn(seed + 7002, (B, 1, Nq, Nkv))
        m = np.where(r > 0.3, -np.inf, 0.0).astype(np.float32)
        m[..., 0] = 0.0
    elif kind == "bias":          # additive f16 bias, shared by heads
        m = 0.5 * ora.randn(seed + 7003, (1, 1, Nq, Nkv))
    elif kind == "bias_perhead":  # FastConformer rel-pos bias [T,T,H] (src/core/fastconformer.h:918)
        m = 0.5 * ora.randn(seed + 7004, (1, Hq, Nq, Nkv))
    elif kind == "bias_perhead_pad":   # per-head bias per sequence + -inf pad keys
        m = 0.5 * ora.randn(seed + 7005, (B, Hq, Nq, Nkv))
        for b in range(B):
            L = lengths[b]
            m[b, :, :, L:] = -np.inf
    elif kind == "all_masked_rows":
        m = np.zeros((1, 1, Nq, Nkv), np.float32)
        m[0, 0, ::3, :] = -np.inf
    else:
        raise ValueError(kind)
    return ora.from_f32(m.astype(np.float32), ora.F16)


def make_case(seed: int, D: int, Nq: int, Nkv: int, Hq: int, Hkv: Optional[int] = None, B: int = 1,
              Bk: Optional[int] = None, ktype: int = ora.F16, vtype: Optional[int] = None,
              mask: Optional[str] = None, scale: Optional[float] = None, max_bias: float = 0.0,
              softcap: float = 0.0, q_layout: str = "contig", kv_layout: str = "contig",
              kv_pad_rows: int = 0, std: float = 1.0, lengths=None) -> dict:
    Hkv = Hkv or Hq
    Bk = Bk or B
    vtype = ktype if vtype is None else vtype
    q = std * ora.randn(seed * 10 + 1, (B, Hq, Nq, D))
    k = std * ora.randn(seed * 10 + 2, (Bk, Hkv, Nkv, D))
    v = std * ora.randn(seed * 10 + 3, (Bk, Hkv, Nkv, D))
    case = {
        "q": _store(q, ora.F32, q_layout),
        "k": _store(k, ktype, kv_layout, kv_pad_rows),
        "v": _store(v, vtype, kv_layout, kv_pad_rows),
        "mask": make_mask(mask, seed, Nq, Nkv + kv_pad_rows, Hq, B, lengths),
        "scale": float(scale if scale is not None else 1.0 / math.sqrt(D)),
        "max_bias": float(max_bias),
        "softcap": float(softcap),
    }
    return case


def to_f32(t: ora.Tensor) -> np.ndarray:
    """Materialise a view as numpy f32 [ne3, ne2, ne1, ne0] (exact for every storage type)."""
    ne0, ne1, ne2, ne3 = t.ne
    out = np.empty((ne3, ne2, ne1, ne0), np.float32)
    rs = ora.row_size(t.type, ne0)
    for i3 in range(ne3):
        for i2 in range(ne2):
            for i1 in range(ne1):
                o = t.offset + i1 * t.nb[1] + i2 * t.nb[2] + i3 * t.nb[3]
                raw = t.buf[o:o + rs]
                if t.type == ora.F32:
                    out[i3, i2, i1] = raw.view(np.float32)
                elif t.type == ora.F16:
                    out[i3, i2, i1] = raw.view(np.float16).astype(np.float32)
                else:
                    out[i3, i2, i1] = ora.dequantize(t.type, raw)
    return out


def textbook_attention(case: dict) -> np.ndarray:
    """fp64 softmax(scale*QK^T [softcap] + slope*mask) V with numpy only - written
    independently of the C oracle.  Returns [B, Nq, Hq, DV]."""
    q = to_f32(case["q"]).astype(np.float64)        # [B, Hq, Nq, D]
    k = to_f32(case["k"]).astype(np.float64)        # [Bk, Hkv, Nkv, D]
    v = to_f32(case["v"]).astype(np.float64)
    B, Hq, Nq, D = q.shape
    Bk, Hkv, Nkv, _ = k.shape
    k = np.repeat(np.repeat(k, Hq // Hkv, axis=1), B // Bk, axis=0)
    v = np.repeat(np.repeat(v, Hq // Hkv, axis=1), B // Bk, axis=0)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * case["scale"]
    if case["softcap"]:
        s = case["softcap"] * np.tanh(s / case["softcap"])
    if case["mask"] is not None:
        m = to_f32(case["mask"]).astype(np.float64)[:, :, :Nq, :Nkv]   # [Bm, Hm, Nq, Nkv]
        m = np.tile(m, (B // m.shape[0], Hq // m.shape[1], 1, 1))       # index b % Bm, h % Hm
        if case["max_bias"] > 0:
            n2 = 2 ** math.floor(math.log2(Hq))
            m0 = 2.0 ** (-case["max_bias"] / n2)
            m1 = 2.0 ** (-(case["max_bias"] / 2.0) / n2)
            slopes = np.array([m0 ** (h + 1) if h < n2 else m1 ** (2 * (h - n2) + 1) for h in range(Hq)])
            with np.errstate(invalid="ignore"):
                m = m * slopes[None, :, None, None]
        s = s + m
    smax = s.max(axis=-1, keepdims=True)
    smax = np.where(np.isfinite(smax), smax, 0.0)
    p = np.exp(s - smax)
    den = p.sum(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        p = np.where(den > 0, p / den, 0.0)
    o = np.einsum("bhqk,bhkd->bhqd", p, v)
    return np.ascontiguousarray(o.transpose(0, 2, 1, 3)).astype(np.float32)


def errors(got: np.ndarray, ref: np.ndarray):
    got = got.astype(np.float64).reshape(-1)
    ref = ref.astype(np.float64).reshape(-1)
    max_abs = float(np.max(np.abs(got - ref))) if got.size else 0.0
    den = float(np.linalg.norm(ref))
    rel_l2 = float(np.linalg.norm(got - ref) / den) if den > 0 else float(np.linalg.norm(got - ref))
    return max_abs, rel_l2


# the tolerance the task states for this path (f32 output vs ggml-cpu semantics)
MAX_ABS_TOL = 2e-3
REL_L2_TOL = 1e-3


def poison_rows(t: ora.Tensor, keys, pattern: int, head=None, batch=None):
    """overwrite rows `keys` (dimension 1) of a K or V tensor - of every head and batch, or of one - with non-finite bit patterns"""
    D, N, H, B = t.ne
    rs = ora.row_size(t.type, D)
    if t.type == ora.F16:
        words = np.array([[0x7E00, 0xFFFF, 0x7C00, 0xFC00], [0x7C00, 0x7C00, 0xFC00, 0x7E01]][pattern], np.uint16)
        row = np.resize(words, D).view(np.uint8)
    elif t.type == ora.F32:
        words = np.array([[0x7FC00000, 0xFFFFFFFF, 0x7F800000, 0xFF800000], [0x7F800000, 0x7F800000, 0xFF800000, 0x7FC00001]][pattern], np.uint32)
        row = np.resize(words, D).view(np.uint8)
    else:
        bs = ora.TYPE_SIZE[t.type]
        blk = np.full(bs, 0x5A, np.uint8)                       # arbitrary quants
        blk[0:2] = np.array([[0x7E00], [0x7C00]][pattern], np.uint16).view(np.uint8)     # d = NaN / +inf
        if t.type in (ora.Q4_1, ora.Q5_1):
            blk[2:4] = np.array([[0xFC00], [0x7E00]][pattern], np.uint16).view(np.uint8)  # m = -inf / NaN
        if t.type == ora.Q8_0 and pattern == 1:
            blk[2:10] = 0                                       # inf * 0 quants as well
        row = np.tile(blk, D // 32)
    assert row.size == rs
    for b in (range(B) if batch is None else [batch]):
        for h in (range(H) if head is None else [head]):
            for j in keys:
                o = t.offset + j * t.nb[1] + h * t.nb[2] + b * t.nb[3]
                t.buf[o:o + rs] = row
