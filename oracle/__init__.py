"""ctypes front end of the CPU oracle (``oracle/fattn_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the shipped package never imports it.

A tensor here is a ggml-style view over host bytes: ``type`` (ggml type id), ``ne`` (elements
per dimension, dimension 0 fastest), ``nb`` (byte strides) and a byte ``offset`` into ``buf``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass, field
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0 = 0, 1, 2, 3, 6, 7, 8
BLOCK_TYPES = (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0)
MODE_EXACT, MODE_GGML_LIKE = 0, 1
ROUND_NEAREST_EVEN, ROUND_HALF_AWAY = 0, 1
QK8_0 = 32
BLOCK_Q8_0_BYTES = 34

TYPE_SIZE = {F32: 4, F16: 2, Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: BLOCK_Q8_0_BYTES}
BLOCK_SIZE = {F32: 1, F16: 1, Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: QK8_0}


def build() -> str:
    """Compile liboracle.so with the committed Makefile."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


REFERENCE_HEADER = "/root/reference/src/core/cpu_attention.h"
_REF_LIB_PATH = os.path.join(_HERE, "_ref", "libref_cpu_attention.so")


def build_ref() -> Optional[str]:
    """Compile the reference's own scalar attention helpers into oracle/_ref/ (only where the reference tree is
    present); returns the library's path, or None when there is nothing to build from."""
    if not os.path.exists(REFERENCE_HEADER):
        return _REF_LIB_PATH if os.path.exists(_REF_LIB_PATH) else None
    subprocess.check_call(["make", "-C", _HERE, "-B", "ref"], stdout=subprocess.DEVNULL)
    return _REF_LIB_PATH


_ref_lib = None


def ref_lib() -> Optional[ctypes.CDLL]:
    """The compiled reference helpers, or None when they have not been built."""
    global _ref_lib
    if _ref_lib is None and os.path.exists(_REF_LIB_PATH):
        L = ctypes.CDLL(_REF_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        L.ref_mha_f32.restype = None
        L.ref_mha_f32.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, fp, fp, fp, ctypes.c_float, fp]
        L.ref_relpos_mha_f32.restype = None
        L.ref_relpos_mha_f32.argtypes = [ctypes.c_int] * 4 + [fp] * 7
        _ref_lib = L
    return _ref_lib


def _fp(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def ref_mha(q: np.ndarray, k: np.ndarray, v: np.ndarray, n_heads: int, scale: float) -> np.ndarray:
    """q, k, v f32 [T, n_heads*head_dim] -> [T, n_heads*head_dim] by the reference's compiled helpers"""
    T, H = q.shape
    out = np.zeros((T, H), np.float32)
    ref_lib().ref_mha_f32(T, n_heads, H // n_heads, _fp(q), _fp(k), _fp(v), float(scale), _fp(out))
    return out


def ref_relpos_mha(q, k, v, p, bu, bv, n_heads: int) -> np.ndarray:
    """FireRed's relative-position attention: q, k, v [T, d], p [T_pe, d], bu / bv [n_heads, head_dim]"""
    T, d = q.shape
    out = np.zeros((T, d), np.float32)
    ref_lib().ref_relpos_mha_f32(T, p.shape[0], n_heads, d // n_heads, _fp(q), _fp(k), _fp(v), _fp(p), _fp(bu), _fp(bv), _fp(out))
    return out


class _CTensor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("type", ctypes.c_int32),
        ("ne", ctypes.c_int64 * 4),
        ("nb", ctypes.c_int64 * 4),
    ]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.ora_fp32_to_fp16.restype = ctypes.c_uint16
        L.ora_fp32_to_fp16.argtypes = [ctypes.c_float]
        L.ora_fp16_to_fp32.restype = ctypes.c_float
        L.ora_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        for name in ("ora_fp32_to_fp16_row", "ora_fp16_to_fp32_row"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.ora_quantize_row_q8_0.restype = None
        L.ora_quantize_row_q8_0.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int]
        L.ora_dequantize_row_q8_0.restype = None
        L.ora_quantize_row.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.ora_dequantize_row.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.ora_block_bytes.restype = ctypes.c_size_t
        L.ora_block_bytes.argtypes = [ctypes.c_int]
        L.ora_dequantize_row_q8_0.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.ora_randn.restype = None
        L.ora_randn.argtypes = [ctypes.c_uint64, ctypes.c_int64, ctypes.c_void_p]
        L.ora_randint.restype = ctypes.c_int64
        L.ora_randint.argtypes = [ctypes.c_uint64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
        L.ora_flash_attn_ext.restype = ctypes.c_int
        L.ora_flash_attn_ext.argtypes = [
            ctypes.POINTER(_CTensor), ctypes.POINTER(_CTensor), ctypes.POINTER(_CTensor),
            ctypes.POINTER(_CTensor), ctypes.c_void_p,
            ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int,
        ]
        L.ora_cpy_f32.restype = ctypes.c_int
        L.ora_cpy_f32.argtypes = [ctypes.POINTER(_CTensor), ctypes.c_void_p, ctypes.c_int32,
                                  ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
        L.ora_relpos_bias.restype = ctypes.c_int
        L.ora_relpos_bias.argtypes = [ctypes.POINTER(_CTensor), ctypes.POINTER(_CTensor), ctypes.POINTER(_CTensor),
                                      ctypes.c_float, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int]
        L.ora_alibi_slope.restype = ctypes.c_float
        L.ora_alibi_slope.argtypes = [ctypes.c_float, ctypes.c_int64, ctypes.c_int64]
        L.ora_vec_dot_q8_0_q8_0.restype = ctypes.c_float
        L.ora_vec_dot_q8_0_q8_0.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.ora_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def row_size(type_: int, ne0: int) -> int:
    return TYPE_SIZE[type_] * (ne0 // BLOCK_SIZE[type_])


def contiguous_nb(type_: int, ne: Sequence[int]) -> tuple:
    nb0 = TYPE_SIZE[type_]
    nb1 = row_size(type_, ne[0])
    nb2 = nb1 * ne[1]
    nb3 = nb2 * ne[2]
    return (nb0, nb1, nb2, nb3)


@dataclass
class Tensor:
    """A ggml-style strided view over a host byte buffer."""
    buf: np.ndarray                      # uint8, 1-D, owns the bytes
    type: int
    ne: tuple
    nb: tuple = field(default=None)
    offset: int = 0

    def __post_init__(self):
        self.ne = tuple(int(x) for x in self.ne) + (1,) * (4 - len(self.ne))
        if self.nb is None:
            self.nb = contiguous_nb(self.type, self.ne)
        self.nb = tuple(int(x) for x in self.nb)
        assert self.buf.dtype == np.uint8 and self.buf.ndim == 1 and self.buf.flags.c_contiguous

    def span(self) -> int:
        """bytes from offset to one past the last byte the view touches"""
        if any(n == 0 for n in self.ne):
            return 0
        last = (self.ne[0] // BLOCK_SIZE[self.type] - 1) * self.nb[0]
        last += sum((self.ne[i] - 1) * self.nb[i] for i in (1, 2, 3))
        return last + TYPE_SIZE[self.type]

    def c(self) -> _CTensor:
        assert self.offset + self.span() <= self.buf.nbytes, "view exceeds its buffer"
        t = _CTensor()
        t.data = self.buf.ctypes.data + self.offset
        t.type = self.type
        t.ne = (ctypes.c_int64 * 4)(*self.ne)
        t.nb = (ctypes.c_int64 * 4)(*self.nb)
        return t


def from_f32(x: np.ndarray, type_: int = F32, rounding: int = ROUND_NEAREST_EVEN) -> Tensor:
    """Contiguous tensor of the given storage type from an f32 array whose numpy shape is
    ggml's ne reversed (numpy [B, H, N, D] -> ne [D, N, H, B])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    ne = tuple(reversed(x.shape))
    if type_ == F32:
        raw = x.view(np.uint8).reshape(-1).copy()
    elif type_ == F16:
        raw = fp32_to_fp16(x).view(np.uint8).reshape(-1).copy()
    elif type_ == Q8_0:
        raw = quantize_q8_0(x.reshape(-1), rounding)
    elif type_ in BLOCK_TYPES:
        raw = quantize(type_, x.reshape(-1))
    else:
        raise ValueError(type_)
    return Tensor(raw, type_, ne)


def fp32_to_fp16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().ora_fp32_to_fp16_row(x.ctypes.data, y.ctypes.data, x.size)
    return y


def fp16_to_fp32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    y = np.empty(h.shape, dtype=np.float32)
    lib().ora_fp16_to_fp32_row(h.ctypes.data, y.ctypes.data, h.size)
    return y


def fp32_to_fp16_scalar(f: float) -> int:
    return int(lib().ora_fp32_to_fp16(float(f)))


def fp16_to_fp32_scalar(h: int) -> float:
    return float(lib().ora_fp16_to_fp32(int(h)))


def quantize_q8_0(x: np.ndarray, rounding: int = ROUND_NEAREST_EVEN) -> np.ndarray:
    """f32[n] (n % 32 == 0) -> uint8[n/32*34] of block_q8_0"""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    assert x.size % QK8_0 == 0
    out = np.empty(x.size // QK8_0 * BLOCK_Q8_0_BYTES, dtype=np.uint8)
    lib().ora_quantize_row_q8_0(x.ctypes.data, out.ctypes.data, x.size, rounding)
    return out


def dequantize_q8_0(raw: np.ndarray) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    assert raw.size % BLOCK_Q8_0_BYTES == 0
    n = raw.size // BLOCK_Q8_0_BYTES * QK8_0
    out = np.empty(n, dtype=np.float32)
    lib().ora_dequantize_row_q8_0(raw.ctypes.data, out.ctypes.data, n)
    return out


def quantize(type_: int, x: np.ndarray) -> np.ndarray:
    """f32[n] (n % 32 == 0) -> the bytes of n/32 blocks of a block-32 type (Q8_0: round to nearest even)"""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    assert x.size % 32 == 0 and type_ in BLOCK_TYPES
    out = np.empty(x.size // 32 * TYPE_SIZE[type_], dtype=np.uint8)
    assert lib().ora_quantize_row(type_, x.ctypes.data, out.ctypes.data, x.size) == 0
    return out


def dequantize(type_: int, raw: np.ndarray) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    assert type_ in BLOCK_TYPES and raw.size % TYPE_SIZE[type_] == 0
    n = raw.size // TYPE_SIZE[type_] * 32
    out = np.empty(n, dtype=np.float32)
    assert lib().ora_dequantize_row(type_, raw.ctypes.data, out.ctypes.data, n) == 0
    return out


def alibi_slope(max_bias: float, h: int, n_head: int) -> float:
    """the factor the oracle multiplies head h's mask by"""
    return float(lib().ora_alibi_slope(float(max_bias), int(h), int(n_head)))


def vec_dot_q8_0_q8_0(x_raw: np.ndarray, y_raw: np.ndarray) -> float:
    """dot product of two rows of block_q8_0 (uint8[n/32*34] each), as ggml-like mode takes it for Q8_0 K"""
    x_raw = np.ascontiguousarray(x_raw, dtype=np.uint8).reshape(-1)
    y_raw = np.ascontiguousarray(y_raw, dtype=np.uint8).reshape(-1)
    assert x_raw.size == y_raw.size and x_raw.size % BLOCK_Q8_0_BYTES == 0
    return float(lib().ora_vec_dot_q8_0_q8_0(x_raw.ctypes.data, y_raw.ctypes.data, x_raw.size // BLOCK_Q8_0_BYTES * QK8_0))


def randn(seed: int, shape) -> np.ndarray:
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    lib().ora_randn(int(seed), n, out.ctypes.data)
    return out.reshape(shape)


def randint(seed: int, i: int, lo: int, hi: int) -> int:
    return int(lib().ora_randint(int(seed), int(i), int(lo), int(hi)))


def max_threads() -> int:
    return int(lib().ora_max_threads())


def flash_attn_ext(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor], scale: float,
                   max_bias: float = 0.0, logit_softcap: float = 0.0,
                   mode: int = MODE_EXACT, n_threads: int = 0) -> np.ndarray:
    """Returns f32 numpy [B, Nq, Hq, DV] (= ggml ne [DV, Hq, Nq, B])."""
    DV, Nq, Hq, B = v.ne[0], q.ne[1], q.ne[2], q.ne[3]
    out = np.zeros((B, Nq, Hq, DV), dtype=np.float32)
    if n_threads <= 0:
        n_threads = max_threads()
    cq, ck, cv = q.c(), k.c(), v.c()
    cm = mask.c() if mask is not None else None
    rc = lib().ora_flash_attn_ext(ctypes.byref(cq), ctypes.byref(ck), ctypes.byref(cv),
                                  ctypes.byref(cm) if cm is not None else None,
                                  out.ctypes.data, scale, max_bias, logit_softcap, mode, n_threads)
    if rc != 0:
        raise ValueError(f"ora_flash_attn_ext rejected the arguments (code {rc})")
    return out


def cpy_f32(src: Tensor, dst: Tensor, rounding: int = ROUND_NEAREST_EVEN) -> None:
    """ggml_cpy(src F32 -> dst view), writes into dst.buf"""
    assert src.ne == dst.ne
    assert dst.offset + dst.span() <= dst.buf.nbytes
    cs = src.c()
    nb = (ctypes.c_int64 * 4)(*dst.nb)
    rc = lib().ora_cpy_f32(ctypes.byref(cs), dst.buf.ctypes.data + dst.offset, dst.type, nb, rounding)
    if rc != 0:
        raise ValueError(f"ora_cpy_f32 rejected the arguments (code {rc})")


def relpos_bias(qv: Tensor, r: Tensor, add: Optional[Tensor], scale: float, n_kv: int, n_threads: int = 0) -> Tensor:
    """FastConformer's rel-pos mask f16(scale * rel_shift(R^T Q_v) + add) as an F16 tensor ne [n_kv, Nq, H, B]."""
    Nq, H, B = qv.ne[1], qv.ne[2], qv.ne[3]
    out = np.zeros(B * H * Nq * n_kv, dtype=np.uint16)
    if n_threads <= 0:
        n_threads = max_threads()
    cq, cr = qv.c(), r.c()
    ca = add.c() if add is not None else None
    rc = lib().ora_relpos_bias(ctypes.byref(cq), ctypes.byref(cr), ctypes.byref(ca) if ca is not None else None,
                               scale, n_kv, out.ctypes.data, n_threads)
    if rc != 0:
        raise ValueError(f"ora_relpos_bias rejected the arguments (code {rc})")
    return Tensor(out.view(np.uint8).reshape(-1), F16, (n_kv, Nq, H, B))
