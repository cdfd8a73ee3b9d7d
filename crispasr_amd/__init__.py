"""MI355X-native attention hot path of CrispASR's ggml graphs (GGML_OP_FLASH_ATTN_EXT).

The product is ``libmi355x_fattn.so`` (hand-written HIP for gfx950 behind a C ABI, see
``include/mi355x_fattn.h``).  This package is the thin host side the tests and the
benchmark drive it through: ``ggml`` mirrors the reference's operator interface for this
path (``ggml_flash_attn_ext``, ``ggml_cpy``, ``ggml_set_rows`` on strided tensor views).
"""
from . import ggml  # noqa: F401
from .ggml import (F16, F32, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, HostBuffer, Tensor, cpy, flash_attn_ext, set_rows)  # noqa: F401

__all__ = ["ggml", "Tensor", "HostBuffer", "F32", "F16", "Q8_0", "Q4_0", "Q4_1", "Q5_0", "Q5_1", "flash_attn_ext", "cpy", "set_rows"]
