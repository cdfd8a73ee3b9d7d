"""Host-side mirror of the ggml operator interface for the attention path.

``Tensor`` carries what a ``ggml_tensor`` carries for this path - type, ``ne`` (elements
per dimension, dimension 0 fastest), ``nb`` (byte strides), a byte offset into a device
buffer - and ``flash_attn_ext`` / ``cpy`` / ``set_rows`` take the same arguments, with the
same meaning and the same contract checks, as ``ggml_flash_attn_ext`` (call sites:
src/crispasr.cpp:2821, 3220, 3280; src/core/attention.h:992; src/core/fastconformer.h:924-934),
``ggml_cpy`` (src/crispasr.cpp:2810-2811) and ``ggml_set_rows`` (src/core/attention.h:366-376)
in the reference.  All arithmetic happens in libmi355x_fattn.so; torch only owns the device
memory and the stream.  There is no CPU fallback: without the built library every op raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import numpy as np
import torch

F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0 = 0, 1, 2, 3, 6, 7, 8
QK8_0 = 32
TYPE_SIZE = {F32: 4, F16: 2, Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34}
BLOCK_SIZE = {F32: 1, F16: 1, Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: QK8_0}

KERNEL_AUTO, KERNEL_VEC, KERNEL_MMA, KERNEL_DECODE_MMA = 0, 1, 2, 3
PREC_DEFAULT, PREC_F32 = 0, 10
# tile_variant values: 16 * key_split + query_blocks
TILE_Q256, TILE_Q128, TILE_Q64_KEYSPLIT = 16 + 2, 16 + 1, 32 + 1

OK, ERR_UNSUPPORTED, ERR_INVALID, ERR_HIP, ERR_NO_DEVICE, ERR_WORKSPACE = range(6)
NOALLOC_SCRATCH_BYTES = 32 << 20

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355X_FATTN_LIB points at an alternative build of the same library (e.g. one compiled with other flags)
LIB_PATH = os.environ.get("MI355X_FATTN_LIB") or os.path.join(_HERE, "libmi355x_fattn.so")


class Mi355xError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"mi355x status {status}: {message}")
        self.status = status


class UnsupportedError(Mi355xError):
    """The op is valid but outside the kernels' coverage (a backend would route it to CPU)."""


class InvalidError(Mi355xError, ValueError):
    """The arguments break the op's contract (ggml would assert)."""


class CTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("type", ctypes.c_int32),
                ("ne", ctypes.c_int64 * 4), ("nb", ctypes.c_size_t * 4)]


class CParams(ctypes.Structure):
    _fields_ = [("scale", ctypes.c_float), ("max_bias", ctypes.c_float), ("logit_softcap", ctypes.c_float),
                ("prec", ctypes.c_int32), ("kernel", ctypes.c_int32), ("n_splits", ctypes.c_int32),
                ("workspace", ctypes.c_void_p), ("workspace_size", ctypes.c_size_t), ("q_quant", ctypes.c_int32),
                ("tile_variant", ctypes.c_int32)]


class CPlanInfo(ctypes.Structure):
    _fields_ = [("kernel", ctypes.c_int32), ("n_splits", ctypes.c_int32), ("keys_per_split", ctypes.c_int32),
                ("kv_to_f16", ctypes.c_int32), ("workspace", ctypes.c_size_t),
                ("queries_per_workgroup", ctypes.c_int32), ("query_blocks", ctypes.c_int32), ("key_split", ctypes.c_int32),
                ("direct", ctypes.c_int32), ("mask_dma", ctypes.c_int32), ("merge_in_kernel", ctypes.c_int32),
                ("head_pad", ctypes.c_int32)]


class CDeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 32),
                ("compute_units", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
                ("memory_clock_khz", ctypes.c_int32), ("memory_bus_bits", ctypes.c_int32),
                ("total_memory", ctypes.c_uint64), ("free_memory", ctypes.c_uint64),
                ("lds_bytes_per_block", ctypes.c_int32), ("wavefront_size", ctypes.c_int32)]


# every symbol include/mi355x_fattn.h declares
EXPORTS = [
    "mi355x_api_version", "mi355x_status_string", "mi355x_last_error",
    "mi355x_device_count", "mi355x_device_get_info", "mi355x_set_device", "mi355x_stream_synchronize",
    "mi355x_fattn_supports", "mi355x_flash_attn_ext", "mi355x_flash_attn_ext_noalloc", "mi355x_fattn_workspace_size", "mi355x_fattn_plan", "mi355x_fattn_plan_details",
    "mi355x_relpos_bias_supports", "mi355x_relpos_bias", "mi355x_relpos_bias_workspace_size", "mi355x_flash_attn_relpos", "mi355x_fattn_relpos_workspace_size",
    "mi355x_cpy_supports", "mi355x_cpy", "mi355x_set_rows", "mi355x_set_rows_supports",
    "mi355x_buffer_alloc", "mi355x_buffer_free", "mi355x_host_buffer_alloc", "mi355x_host_buffer_free", "mi355x_host_buffer_mirror_stats", "mi355x_host_buffer_invalidate", "mi355x_buffer_memset", "mi355x_buffer_set",
    "mi355x_buffer_get", "mi355x_buffer_copy",
]

_lib = None


def lib() -> ctypes.CDLL:
    """The C-ABI library; raises when it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, --offload-arch=gfx950). There is no CPU fallback for this path.")
        L = ctypes.CDLL(LIB_PATH)
        PT, PP = ctypes.POINTER(CTensor), ctypes.POINTER(CParams)
        L.mi355x_api_version.restype = ctypes.c_int
        L.mi355x_status_string.restype = ctypes.c_char_p
        L.mi355x_status_string.argtypes = [ctypes.c_int]
        L.mi355x_last_error.restype = ctypes.c_char_p
        L.mi355x_device_count.argtypes = [ctypes.POINTER(ctypes.c_int)]
        L.mi355x_device_get_info.argtypes = [ctypes.c_int, ctypes.POINTER(CDeviceInfo)]
        L.mi355x_set_device.argtypes = [ctypes.c_int]
        L.mi355x_stream_synchronize.argtypes = [ctypes.c_void_p]
        L.mi355x_fattn_supports.argtypes = [PT, PT, PT, PT, PT, PP]
        L.mi355x_flash_attn_ext.argtypes = [PT, PT, PT, PT, PT, PP, ctypes.c_void_p]
        L.mi355x_flash_attn_ext_noalloc.argtypes = [PT, PT, PT, PT, PT, PP, ctypes.c_void_p]
        L.mi355x_fattn_workspace_size.argtypes = [PT, PT, PT, PT, PP, ctypes.POINTER(ctypes.c_size_t)]
        L.mi355x_fattn_plan.argtypes = [PT, PT, PT, PT, PP, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]
        L.mi355x_fattn_plan_details.argtypes = [PT, PT, PT, PT, PP, ctypes.POINTER(CPlanInfo)]
        L.mi355x_relpos_bias_supports.argtypes = [PT, PT, PT, PT]
        L.mi355x_relpos_bias.argtypes = [PT, PT, PT, PT, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.mi355x_relpos_bias_workspace_size.argtypes = [PT, ctypes.POINTER(ctypes.c_size_t)]
        L.mi355x_set_rows_supports.argtypes = [PT, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64), PT]
        L.mi355x_flash_attn_relpos.argtypes = [PT, PT, PT, PT, PT, PT, PT, PP, ctypes.c_void_p]
        L.mi355x_fattn_relpos_workspace_size.argtypes = [PT, PT, PT, PT, PT, PT, PP, ctypes.POINTER(ctypes.c_size_t)]
        L.mi355x_cpy_supports.argtypes = [PT, PT]
        L.mi355x_cpy.argtypes = [PT, PT, ctypes.c_void_p]
        L.mi355x_set_rows.argtypes = [PT, ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64),
                                      ctypes.POINTER(ctypes.c_size_t), PT, ctypes.c_void_p]
        L.mi355x_buffer_alloc.argtypes = [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
        L.mi355x_buffer_free.argtypes = [ctypes.c_void_p]
        L.mi355x_host_buffer_alloc.argtypes = [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
        L.mi355x_host_buffer_free.argtypes = [ctypes.c_void_p]
        L.mi355x_host_buffer_mirror_stats.argtypes = [ctypes.c_void_p] + [ctypes.POINTER(ctypes.c_size_t)] * 3
        L.mi355x_host_buffer_invalidate.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        L.mi355x_buffer_memset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
        L.mi355x_buffer_set.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.mi355x_buffer_get.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.mi355x_buffer_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        for name in EXPORTS:
            fn = getattr(L, name)
            if name not in ("mi355x_status_string", "mi355x_last_error"):
                fn.restype = ctypes.c_int
        _lib = L
    return _lib


def _check(status: int) -> None:
    if status == OK:
        return
    msg = lib().mi355x_last_error().decode(errors="replace")
    if status == ERR_UNSUPPORTED:
        raise UnsupportedError(status, msg)
    if status == ERR_INVALID:
        raise InvalidError(status, msg)
    raise Mi355xError(status, msg)


def row_size(type_: int, ne0: int) -> int:
    """ggml_row_size"""
    return TYPE_SIZE[type_] * (ne0 // BLOCK_SIZE[type_])


def contiguous_nb(type_: int, ne: Sequence[int]) -> tuple:
    nb1 = row_size(type_, ne[0])
    return (TYPE_SIZE[type_], nb1, nb1 * ne[1], nb1 * ne[1] * ne[2])


class HostBuffer:
    """Pinned host memory that the GPU addresses at the same pointer (mi355x_host_buffer_alloc): the
    is_host buffer type a one-op backend gives ggml, so that ggml-cpu keeps running every other op on the
    tensors in it.  ``array`` is the CPU's view of the bytes; the kernels read and write them in place."""

    def __init__(self, nbytes: int, device=None):
        self.device = torch.device("cuda", torch.cuda.current_device() if device is None else torch.device(device).index or 0)
        self.nbytes = max(int(nbytes), 1)
        p = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            _check(lib().mi355x_host_buffer_alloc(self.nbytes, ctypes.byref(p)))
        self.ptr = p.value
        self.array = np.ctypeslib.as_array((ctypes.c_uint8 * self.nbytes).from_address(self.ptr))

    def numel(self) -> int:
        return self.nbytes

    def data_ptr(self) -> int:
        return self.ptr

    def mirror_stats(self) -> dict:
        """the buffer's mirror in HBM: its size (0: none yet), the bytes that are up to date, the bytes fetched so far"""
        m, v, u = ctypes.c_size_t(0), ctypes.c_size_t(0), ctypes.c_size_t(0)
        _check(lib().mi355x_host_buffer_mirror_stats(self.ptr, ctypes.byref(m), ctypes.byref(v), ctypes.byref(u)))
        return {"mirror_bytes": m.value, "valid_bytes": v.value, "uploaded_bytes": u.value}

    def invalidate(self, offset: int = 0, nbytes: Optional[int] = None) -> None:
        """the CPU has written [offset, offset + nbytes) through `array`: the mirror's pages there are stale"""
        _check(lib().mi355x_host_buffer_invalidate(self.ptr + offset, self.nbytes - offset if nbytes is None else nbytes))

    def __del__(self):
        if getattr(self, "ptr", None):
            self.array = None
            lib().mi355x_host_buffer_free(self.ptr)
            self.ptr = None


class Tensor:
    """A ggml tensor (or view) living in a device buffer (a torch uint8 tensor) or in a HostBuffer."""

    def __init__(self, buf, type_: int, ne: Sequence[int],
                 nb: Optional[Sequence[int]] = None, offset: int = 0):
        self.buf = buf                      # 1-D uint8 device tensor, a HostBuffer, or None (planning only)
        self.type = int(type_)
        self.ne = tuple(int(x) for x in ne) + (1,) * (4 - len(ne))
        self.nb = tuple(int(x) for x in (nb if nb is not None else contiguous_nb(self.type, self.ne)))
        self.offset = int(offset)
        self._c = None                      # the C descriptor, built once: a view never changes
        if buf is not None and not isinstance(buf, HostBuffer):
            assert buf.dtype == torch.uint8 and buf.dim() == 1 and buf.is_contiguous()

    # -- construction ---------------------------------------------------------------------
    @staticmethod
    def empty(type_: int, ne: Sequence[int], device="cuda") -> "Tensor":
        """ggml_new_tensor + allocation in a device buffer"""
        ne4 = tuple(int(x) for x in ne) + (1,) * (4 - len(ne))
        nbytes = row_size(type_, ne4[0]) * ne4[1] * ne4[2] * ne4[3]
        return Tensor(torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device), type_, ne4)

    @staticmethod
    def from_host(raw: np.ndarray, type_: int, ne, nb=None, offset: int = 0, device="cuda") -> "Tensor":
        """ggml_backend_tensor_set of a whole buffer; the view (ne, nb, offset) is kept as is"""
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        buf = torch.from_numpy(raw.copy()).to(device)
        if buf.numel() == 0:
            buf = torch.zeros(1, dtype=torch.uint8, device=device)
        return Tensor(buf, type_, ne, nb, offset)

    @staticmethod
    def in_host_buffer(raw: np.ndarray, type_: int, ne, nb=None, offset: int = 0) -> "Tensor":
        """the same view over a fresh HostBuffer: set_tensor on an is_host buffer is a memcpy by the CPU"""
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        buf = HostBuffer(raw.size)
        buf.array[:raw.size] = raw
        return Tensor(buf, type_, ne, nb, offset)

    def view(self, ne, nb, offset: int = 0, type_: Optional[int] = None) -> "Tensor":
        """ggml_view_{1,2,3,4}d: same buffer, new extents/strides, offset relative to this view"""
        return Tensor(self.buf, self.type if type_ is None else type_, ne, nb, self.offset + offset)

    # -- access -----------------------------------------------------------------------------
    def span(self) -> int:
        if any(n == 0 for n in self.ne):
            return 0
        last = (self.ne[0] // BLOCK_SIZE[self.type] - 1) * self.nb[0]
        last += sum((self.ne[i] - 1) * self.nb[i] for i in (1, 2, 3))
        return last + TYPE_SIZE[self.type]

    def data_ptr(self) -> int:
        if self.buf is None:
            # planning before allocation: the predicates never dereference, they only look at the address's low bits
            # (buffers start on 256 bytes, so the view's offset modulo 256 stands for them)
            return self.offset % 256
        if self.offset + self.span() > self.buf.numel():
            raise InvalidError(ERR_INVALID, "tensor view exceeds its buffer")
        return self.buf.data_ptr() + self.offset

    def c(self) -> CTensor:
        if self._c is None:
            t = CTensor()
            t.data = self.data_ptr()
            t.type = self.type
            t.ne = (ctypes.c_int64 * 4)(*self.ne)
            t.nb = (ctypes.c_size_t * 4)(*self.nb)
            self._c = (t, ctypes.byref(t))
        return self._c[0]

    def ref(self):
        """pointer to the C descriptor, as the entry points take it"""
        self.c()
        return self._c[1]

    def to_host(self) -> np.ndarray:
        """ggml_backend_tensor_get of the whole underlying buffer (uint8)"""
        if isinstance(self.buf, HostBuffer):
            return self.buf.array.copy()
        return self.buf.cpu().numpy()

    def numpy_f32(self) -> np.ndarray:
        """contiguous F32 tensor -> numpy [ne3, ne2, ne1, ne0]"""
        assert self.type == F32 and self.nb == contiguous_nb(F32, self.ne)
        n = self.ne[0] * self.ne[1] * self.ne[2] * self.ne[3]
        if isinstance(self.buf, HostBuffer):
            raw = self.buf.array[self.offset:self.offset + 4 * n]
        else:
            raw = self.buf[self.offset:self.offset + 4 * n].cpu().numpy()
        return raw.view(np.float32).reshape(self.ne[3], self.ne[2], self.ne[1], self.ne[0]).copy()


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device):
    """make `device` current for the call; no context switch when it already is"""
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _stream_handle(stream) -> int:
    if stream is None:
        stream = torch.cuda.current_stream()
    return int(stream.cuda_stream)


def _params(scale, max_bias, logit_softcap, prec, kernel, n_splits, workspace, q_quant=0, tile_variant=0) -> CParams:
    p = CParams()
    p.q_quant = int(q_quant)
    p.tile_variant = int(tile_variant)
    p.scale, p.max_bias, p.logit_softcap = float(scale), float(max_bias), float(logit_softcap)
    p.prec, p.kernel, p.n_splits = int(prec), int(kernel), int(n_splits)
    if workspace is not None:
        p.workspace = workspace.data_ptr()
        p.workspace_size = workspace.numel() * workspace.element_size()
    else:
        p.workspace, p.workspace_size = None, 0
    return p


def _opt(t: Optional[Tensor]):
    return ctypes.byref(t.c()) if t is not None else None


def flash_attn_supports(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None, scale: float = 1.0,
                        max_bias: float = 0.0, logit_softcap: float = 0.0, prec: int = PREC_DEFAULT) -> int:
    """What the backend's supports_op asks: OK, ERR_UNSUPPORTED or ERR_INVALID.  Touches no device."""
    p = _params(scale, max_bias, logit_softcap, prec, KERNEL_AUTO, 0, None)
    cq, ck, cv = q.c(), k.c(), v.c()
    cm = mask.c() if mask is not None else None
    return lib().mi355x_fattn_supports(ctypes.byref(cq), ctypes.byref(ck), ctypes.byref(cv),
                                       ctypes.byref(cm) if cm is not None else None, None, ctypes.byref(p))


def flash_attn_plan(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None, scale: float = 1.0,
                    max_bias: float = 0.0, logit_softcap: float = 0.0, kernel: int = KERNEL_AUTO,
                    n_splits: int = 0):
    p = _params(scale, max_bias, logit_softcap, PREC_DEFAULT, kernel, n_splits, None)
    cq, ck, cv = q.c(), k.c(), v.c()
    cm = mask.c() if mask is not None else None
    kern, ns = ctypes.c_int32(0), ctypes.c_int32(0)
    _check(lib().mi355x_fattn_plan(ctypes.byref(cq), ctypes.byref(ck), ctypes.byref(cv),
                                   ctypes.byref(cm) if cm is not None else None, ctypes.byref(p),
                                   ctypes.byref(kern), ctypes.byref(ns)))
    return kern.value, ns.value


def flash_attn_plan_details(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None, scale: float = 1.0,
                            max_bias: float = 0.0, logit_softcap: float = 0.0, kernel: int = KERNEL_AUTO,
                            n_splits: int = 0, tile_variant: int = 0, workspace: Optional[torch.Tensor] = None) -> dict:
    """Kernel, split count and - for the tile kernel - the instantiation the call takes."""
    p = _params(scale, max_bias, logit_softcap, PREC_DEFAULT, kernel, n_splits, workspace, 0, tile_variant)
    info = CPlanInfo()
    _check(lib().mi355x_fattn_plan_details(q.ref(), k.ref(), v.ref(), mask.ref() if mask is not None else None,
                                           ctypes.byref(p), ctypes.byref(info)))
    return {f: getattr(info, f) for f, _ in CPlanInfo._fields_}


def flash_attn_workspace_size(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None, scale: float = 1.0,
                              max_bias: float = 0.0, logit_softcap: float = 0.0, kernel: int = KERNEL_AUTO,
                              n_splits: int = 0, q_quant: int = 0) -> int:
    """Bytes of workspace the call would use (split-KV partials, f16 copies of F32 / Q8_0 K/V); 0 if none."""
    p = _params(scale, max_bias, logit_softcap, PREC_DEFAULT, kernel, n_splits, None, q_quant)
    n = ctypes.c_size_t(0)
    _check(lib().mi355x_fattn_workspace_size(q.ref(), k.ref(), v.ref(), mask.ref() if mask is not None else None,
                                             ctypes.byref(p), ctypes.byref(n)))
    return n.value


def flash_attn_ext(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor], scale: float,
                   max_bias: float = 0.0, logit_softcap: float = 0.0, *, prec: int = PREC_DEFAULT,
                   kernel: int = KERNEL_AUTO, n_splits: int = 0, out: Optional[Tensor] = None,
                   workspace: Optional[torch.Tensor] = None, stream=None, q_quant: int = 0,
                   tile_variant: int = 0, no_alloc: bool = False) -> Tensor:
    """ggml_flash_attn_ext(ctx, q, k, v, mask, scale, max_bias, logit_softcap) computed on the GPU.
    q_quant = Q8_0 rounds the query rows to Q8_0 blocks first (ggml-cpu's recalled arithmetic for Q8_0 K; comparison runs).

    Returns the F32 result tensor with ne = [DV, Hq, Nq, B] (what the reference's callers
    immediately reshape_2d to [DV*Hq, Nq])."""
    if out is None:
        out = Tensor.empty(F32, (v.ne[0], q.ne[2], q.ne[1], q.ne[3]), device=q.buf.device)
    p = _params(scale, max_bias, logit_softcap, prec, kernel, n_splits, workspace, q_quant, tile_variant)
    # no_alloc: the entry point that takes its scratch from the library's static device array (pass `out`: the result
    # tensor is the caller's to provide there)
    entry = lib().mi355x_flash_attn_ext_noalloc if no_alloc else lib().mi355x_flash_attn_ext
    with _on_device(q.buf.device):
        _check(entry(q.ref(), k.ref(), v.ref(), mask.ref() if mask is not None else None,
                     out.ref(), ctypes.byref(p), _stream_handle(stream)))
    return out


def relpos_bias_workspace_size(r: Tensor) -> int:
    """Bytes of workspace relpos_bias uses for this table (0: an F16 table with contiguous rows is read in place)."""
    n = ctypes.c_size_t(0)
    _check(lib().mi355x_relpos_bias_workspace_size(r.ref(), ctypes.byref(n)))
    return n.value


def relpos_bias(q_v: Tensor, r: Tensor, add: Optional[Tensor], scale: float, n_kv: Optional[int] = None, *,
                out: Optional[Tensor] = None, workspace: Optional[torch.Tensor] = None, stream=None) -> Tensor:
    """The F16 mask core_conformer::build_block builds for its flash-attention call (src/core/fastconformer.h:880-918):
    cast_f16(scale * rel_shift(mul_mat(cont(R), Q_v)) [+ add]).  Returns it with ne = [n_kv, Nq, H, B]."""
    if out is None:
        if n_kv is None:
            n_kv = r.ne[1] - q_v.ne[1] + 1
        out = Tensor.empty(F16, (n_kv, q_v.ne[1], q_v.ne[2], q_v.ne[3]), device=q_v.buf.device)
    with _on_device(q_v.buf.device):
        _check(lib().mi355x_relpos_bias(q_v.ref(), r.ref(), add.ref() if add is not None else None, out.ref(),
                                        float(scale), workspace.data_ptr() if workspace is not None else None,
                                        workspace.numel() * workspace.element_size() if workspace is not None else 0,
                                        _stream_handle(stream)))
    return out


def flash_attn_relpos(q_u: Tensor, q_v: Tensor, k: Tensor, v: Tensor, r: Tensor, add: Optional[Tensor], scale: float, *,
                      kernel: int = KERNEL_AUTO, n_splits: int = 0, out: Optional[Tensor] = None,
                      workspace: Optional[torch.Tensor] = None, stream=None) -> Tensor:
    """The flash branch of a FastConformer attention block (src/core/fastconformer.h:876-934) in one call:
    softmax(scale * (q_u.k^T + rel_shift(q_v.r^T)) + add) . v, result ne = [DV, H, Nq, B]."""
    if out is None:
        out = Tensor.empty(F32, (v.ne[0], q_u.ne[2], q_u.ne[1], q_u.ne[3]), device=q_u.buf.device)
    p = _params(scale, 0.0, 0.0, PREC_DEFAULT, kernel, n_splits, workspace)
    with _on_device(q_u.buf.device):
        _check(lib().mi355x_flash_attn_relpos(q_u.ref(), q_v.ref(), k.ref(), v.ref(), r.ref(),
                                              add.ref() if add is not None else None, out.ref(), ctypes.byref(p),
                                              _stream_handle(stream)))
    return out


def flash_attn_relpos_workspace_size(q_u: Tensor, q_v: Tensor, k: Tensor, v: Tensor, r: Tensor, add: Optional[Tensor],
                                     scale: float, kernel: int = KERNEL_AUTO, n_splits: int = 0) -> int:
    p = _params(scale, 0.0, 0.0, PREC_DEFAULT, kernel, n_splits, None)
    n = ctypes.c_size_t(0)
    _check(lib().mi355x_fattn_relpos_workspace_size(q_u.ref(), q_v.ref(), k.ref(), v.ref(), r.ref(),
                                                    add.ref() if add is not None else None, ctypes.byref(p), ctypes.byref(n)))
    return n.value


def cpy(src: Tensor, dst: Tensor, stream=None) -> Tensor:
    """ggml_cpy(ctx, src, dst): convert src's elements into dst's type and layout"""
    cs, cd = src.c(), dst.c()
    with torch.cuda.device(dst.buf.device):
        _check(lib().mi355x_cpy(ctypes.byref(cs), ctypes.byref(cd), _stream_handle(stream)))
    return dst


def set_rows_supports(dst: Tensor, src: Tensor, n_idx: Sequence[int], idx_bits: int = 64) -> int:
    """planning predicate of set_rows: idx extents [n_rows, I1, I2] in ggml order, idx type 64 or 32"""
    ine3 = tuple(int(x) for x in n_idx) + (1,) * (3 - len(n_idx))
    return lib().mi355x_set_rows_supports(src.ref(), idx_bits, (ctypes.c_int64 * 3)(*ine3), dst.ref())


def set_rows(dst: Tensor, src: Tensor, idx: torch.Tensor, stream=None) -> Tensor:
    """ggml_set_rows(ctx, dst, src, idx): dst[:, idx[i], ...] = src[:, i, ...]; idx int64/int32 device tensor
    of shape [n_rows] (or [I2, I1, n_rows] in numpy order, broadcast over dims 2 and 3)"""
    assert idx.dtype in (torch.int64, torch.int32) and idx.is_contiguous()
    shape = (1,) * (3 - idx.dim()) + tuple(idx.shape)
    ine = (ctypes.c_int64 * 3)(shape[2], shape[1], shape[0])
    es = idx.element_size()
    inb = (ctypes.c_size_t * 3)(es, es * shape[2], es * shape[2] * shape[1])
    cs, cd = src.c(), dst.c()
    with torch.cuda.device(dst.buf.device):
        _check(lib().mi355x_set_rows(ctypes.byref(cs), idx.data_ptr(), 64 if idx.dtype == torch.int64 else 32,
                                     ine, inb, ctypes.byref(cd), _stream_handle(stream)))
    return dst


def device_info(device: int = 0) -> dict:
    info = CDeviceInfo()
    _check(lib().mi355x_device_get_info(device, ctypes.byref(info)))
    return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes) else getattr(info, f))
            for f, _ in CDeviceInfo._fields_}


def device_count() -> int:
    n = ctypes.c_int(0)
    lib().mi355x_device_count(ctypes.byref(n))
    return n.value
