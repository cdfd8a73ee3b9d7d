#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.  numpy only: nothing here imports the oracle, the HIP
library or the reference, so the vectors are an independent statement of what the op computes.

The reference holds no output vectors for GGML_OP_FLASH_ATTN_EXT, so these fix the results by the
mathematics the call sites rely on: dst = softmax(scale * q.k^T + mask) . v in float64 on the exact
values of the stored operands (f16 and Q8_0 decoded by numpy), with ggml's layouts:
q [D, Nq, Hq, B] f32, k/v [D, Nkv, Hkv, Bk], mask f16 [Nkv, Nq, Hm, Bm], dst [D, Hq, Nq, B]
(dimension 0 fastest; numpy arrays below are the reverse order).  Also: f32 -> f16 known answers
(numpy.float16, round to nearest even), Q8_0 known-answer blocks (d = amax / 127 in f32, stored as f16;
q = round-to-nearest-even(x * (1 / d))), and FastConformer's relative-position mask
f16(scale * rel_shift(R^T Q_v) + add) (src/core/fastconformer.h:98-102, 880-918) through numpy's
as_strided view with the strides of the graph's own view.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
from numpy.lib.stride_tricks import as_strided

HERE = os.path.dirname(os.path.abspath(__file__))


def q8_0_quantize(x):
    """x f32 [..., D] -> raw bytes [..., D/32 * 34] (fp16 d, 32 int8) and the decoded f32 values"""
    xb = x.reshape(x.shape[:-1] + (x.shape[-1] // 32, 32)).astype(np.float32)
    amax = np.abs(xb).max(axis=-1, keepdims=True).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, np.float32(1.0)), np.float32(0.0)).astype(np.float32)
    q = np.rint((xb * inv).astype(np.float32)).astype(np.int8)
    dh = d.astype(np.float16)
    raw = np.concatenate([dh.view(np.uint8).reshape(dh.shape[:-1] + (2,)), q.view(np.uint8)], axis=-1)
    dec = (q.astype(np.float32) * dh.astype(np.float32)).astype(np.float32)
    return raw.reshape(x.shape[:-1] + (-1,)), dec.reshape(x.shape)


def attention(q, k, v, mask, scale):
    """q [B,Hq,Nq,D], k/v [Bk,Hkv,Nkv,D] exact values, mask [Bm,Hm,Nq,Nkv] or None -> [B,Nq,Hq,D] float64
    (stored rounded to f32: 6e-8 relative, far below the 2e-3 the kernels are held to)"""
    B, Hq, Nq, D = q.shape
    Bk, Hkv, Nkv, _ = k.shape
    out = np.zeros((B, Nq, Hq, D))
    for b in range(B):
        for h in range(Hq):
            kk = k[b // (B // Bk), h // (Hq // Hkv)].astype(np.float64)
            vv = v[b // (B // Bk), h // (Hq // Hkv)].astype(np.float64)
            s = scale * (q[b, h].astype(np.float64) @ kk.T)
            if mask is not None:
                s = s + mask[b % mask.shape[0], h % mask.shape[1]].astype(np.float64)
            m = s.max(axis=1, keepdims=True)
            dead = np.isneginf(m)                       # every key excluded: the row is zero
            p = np.exp(s - np.where(dead, 0.0, m))
            l = p.sum(axis=1, keepdims=True)
            out[b, :, h] = np.where(dead, 0.0, (p @ vv) / np.where(l == 0, 1.0, l))
    return out


def fattn_case(name, rng, D, Nq, Nkv, Hq, Hkv, B, Bk, ktype, mask_kind, scale=None):
    q = rng.standard_normal((B, Hq, Nq, D)).astype(np.float32)
    k = rng.standard_normal((Bk, Hkv, Nkv, D)).astype(np.float32)
    v = rng.standard_normal((Bk, Hkv, Nkv, D)).astype(np.float32)
    if ktype == "f16":
        kraw, vraw = k.astype(np.float16), v.astype(np.float16)
        kx, vx = kraw.astype(np.float32), vraw.astype(np.float32)
        kraw, vraw = kraw.view(np.uint8), vraw.view(np.uint8)
    elif ktype == "q8_0":
        kraw, kx = q8_0_quantize(k)
        vraw, vx = q8_0_quantize(v)
    else:
        kraw, vraw, kx, vx = k.view(np.uint8), v.view(np.uint8), k, v
    mask = None
    if mask_kind == "causal":
        mask = np.zeros((1, 1, Nq, Nkv), np.float16)
        mask[0, 0][np.arange(Nkv)[None, :] > np.arange(Nq)[:, None] + (Nkv - Nq)] = -np.inf
    elif mask_kind == "bias_pad":                        # per-head bias, -inf beyond each sequence's length, one dead row
        mask = (0.5 * rng.standard_normal((B, Hq, Nq, Nkv))).astype(np.float16)
        for b in range(B):
            mask[b, :, :, Nkv - 3 - 5 * b:] = -np.inf
        mask[0, 0, 1, :] = -np.inf
    elif mask_kind == "beams":                           # arbitrary visibility per batch entry, shared by heads
        mask = np.where(rng.random((B, 1, Nq, Nkv)) > 0.6, -np.inf, 0.0).astype(np.float16)
        mask[..., 0] = 0.0
    scale = float(scale if scale is not None else 1.0 / np.sqrt(D))
    out = attention(q, kx, vx, mask, scale)
    d = {"q": q, "k_raw": np.ascontiguousarray(kraw).reshape(Bk, Hkv, Nkv, -1), "v_raw": np.ascontiguousarray(vraw).reshape(Bk, Hkv, Nkv, -1),
         "ktype": np.array({"f32": 0, "f16": 1, "q8_0": 8}[ktype]), "scale": np.array(scale, np.float64), "out": out.astype(np.float32)}
    if mask is not None:
        d["mask"] = mask.view(np.uint16)
    np.savez_compressed(os.path.join(HERE, f"fattn_{name}.npz"), **d)


def relpos_case(rng):
    D, T, H, B = 64, 37, 2, 2
    qv = rng.standard_normal((B, H, T, D)).astype(np.float32)
    r = rng.standard_normal((1, H, 2 * T - 1, D)).astype(np.float32)
    add = np.zeros((B, 1, T, T), np.float32)
    add[1, 0, :, T - 6:] = -np.inf                       # pad keys of the second sequence
    add[0, 0][np.abs(np.arange(T)[:, None] - np.arange(T)[None, :]) > 20] = -1e9      # a local-attention window
    scale = np.float32(1.0 / np.sqrt(D))
    out = np.zeros((B, H, T, T), np.float16)
    bd32 = np.zeros((B, H, T, T), np.float32)
    for b in range(B):
        for h in range(H):
            # mul_mat(cont(R), Q_v): raw[i, n] = <Q_v[i], R[n]>, ne = [2T-1, T]
            raw = (qv[b, h].astype(np.float64) @ r[0, h].astype(np.float64).T).astype(np.float32)
            nb0, nb1 = raw.strides[1], raw.strides[0]
            # rel_shift: view ne = [T, T], nb1 = nb1_raw - nb0, offset (T-1)*nb0
            flat = raw.reshape(-1)
            view = as_strided(flat[T - 1:], shape=(T, T), strides=(nb1 - nb0, nb0))
            bd = np.ascontiguousarray(view)              # [i, j]
            bd32[b, h] = bd
            with np.errstate(over="ignore"):            # -1e9 becomes -inf in f16, as in the graph's cast
                out[b, h] = ((bd * scale).astype(np.float32) + add[b, 0]).astype(np.float16)
    np.savez_compressed(os.path.join(HERE, "relpos_bias.npz"), qv=qv, r=r, add=add, scale=np.array(scale), bd_f32=bd32,
                        mask=out.view(np.uint16))


def conversions():
    f = np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 1e5, -1e5, np.inf, -np.inf,
                  5.9604645e-08, 2.9802322e-08, 2.9802325e-08, 8.940697e-08, 6.1035156e-05, 6.0975552e-05,
                  1.0009766, 1.00048828125, 1.00146484375, 0.1, 0.333333, 3.14159265, 2049.0, 2051.0, 1e-10], np.float32)
    rng = np.random.default_rng(11)
    f = np.concatenate([f, rng.standard_normal(200).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 5, 200).astype(np.float32)])
    with np.errstate(over="ignore"):
        h = f.astype(np.float16)
    x = rng.standard_normal((6, 32)).astype(np.float32)
    x[0] = 0.0                                           # all-zero block: d = 0, q = 0
    x[1] = np.linspace(-127, 127, 32)                    # amax = 127: d = 1, integers survive
    x[2, :] = (np.arange(32) - 15.5)                     # every value a tie at d = 15.5/127
    x[3, 5] = 1000.0                                     # one outlier sets the scale
    x[4] *= 1e-6
    raw, dec = q8_0_quantize(x)
    np.savez_compressed(os.path.join(HERE, "conversions.npz"), f32=f, f16_bits=h.view(np.uint16), q8_x=x, q8_raw=raw, q8_dec=dec)


def main():
    rng = np.random.default_rng(20240607)
    fattn_case("mha_f16", rng, D=64, Nq=33, Nkv=70, Hq=2, Hkv=2, B=1, Bk=1, ktype="f16", mask_kind=None, scale=0.125)
    fattn_case("gqa_causal_q8_0", rng, D=128, Nq=20, Nkv=64, Hq=4, Hkv=2, B=2, Bk=1, ktype="q8_0", mask_kind="causal")
    fattn_case("bias_pad_f32", rng, D=128, Nq=24, Nkv=24, Hq=2, Hkv=2, B=2, Bk=2, ktype="f32", mask_kind="bias_pad")
    fattn_case("decode_beams_f16", rng, D=64, Nq=1, Nkv=224, Hq=2, Hkv=2, B=3, Bk=3, ktype="f16", mask_kind="beams", scale=1.0)
    fattn_case("decode_gqa_q8_0", rng, D=128, Nq=1, Nkv=200, Hq=8, Hkv=2, B=1, Bk=1, ktype="q8_0", mask_kind=None)
    fattn_case("tile_f16_d128", rng, D=128, Nq=130, Nkv=70, Hq=1, Hkv=1, B=1, Bk=1, ktype="f16", mask_kind=None)
    relpos_case(rng)
    conversions()


if __name__ == "__main__":
    main()
