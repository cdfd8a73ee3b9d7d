"""CPU-side checks of the drop-in boundary: the C-ABI library loads, exports every symbol the
header declares, and its supports/plan predicates (which touch no device) answer like the
op's contract says.  No compute call is made here."""
import ctypes
import os
import re

import pytest

import crispasr_amd as ca
from crispasr_amd import ggml

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi355x_fattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355x_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = ggml.lib()
    names = _declared_symbols()
    assert len(names) >= 18
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/mi355x_fattn.h but not exported"
    assert sorted(ggml.EXPORTS) == names
    assert L.mi355x_api_version() == 6
    assert L.mi355x_status_string(0) == b"ok"


def _t(type_, ne, nb=None):
    return ca.Tensor(None, type_, ne, nb)


def test_supports_accepts_the_reference_call_shapes():
    # Whisper encoder: strided [token][head][dim] views, K/V padded to 1536 (src/crispasr.cpp:2806-2821)
    H, n_state = 20, 1280
    q = _t(ca.F32, (64, 1500, H, 1), (4, 4 * n_state, 256, 4 * n_state * 1500))
    k = _t(ca.F16, (64, 1536, H, 1), (2, 2 * n_state, 128, 2 * n_state * 1536))
    assert ggml.flash_attn_supports(q, k, k, None, 0.125) == ggml.OK
    # Whisper decoder self-attn with an F16 mask [n_kv, n_tok]
    q = _t(ca.F32, (64, 5, H, 1), (4, 4 * n_state, 256, 4 * n_state * 5))
    k = _t(ca.F16, (64, 224, H, 1), (2, 2 * n_state, 128, 2 * n_state * 224))
    m = _t(ca.F16, (224, 5, 1, 1))
    assert ggml.flash_attn_supports(q, k, k, m, 1.0) == ggml.OK
    # Canary decoder: quantised cache view straight into the op (src/canary.cpp:966-972)
    q = _t(ca.F32, (128, 1, 8, 1))
    k = _t(ca.Q8_0, (128, 300, 8, 1), (34, 136, 136 * 1024, 136 * 1024 * 8))
    assert ggml.flash_attn_supports(q, k, k, None, 128 ** -0.5) == ggml.OK
    # FastConformer: F32 K/V strided into a fused QKV buffer, per-head F16 mask [T,T,H]
    T, d = 750, 1024
    q = _t(ca.F32, (128, T, 8, 1), (4, 3 * d * 4, 128 * 4, 3 * d * 4 * T))
    m = _t(ca.F16, (T, T, 8, 1))
    assert ggml.flash_attn_supports(q, q, q, m, 128 ** -0.5) == ggml.OK
    # GQA, native
    q = _t(ca.F32, (128, 407, 32, 1))
    k = _t(ca.Q8_0, (128, 407, 8, 1))
    m = _t(ca.F16, (407, 407, 1, 1))
    assert ggml.flash_attn_supports(q, k, k, m, 128 ** -0.5) == ggml.OK


def test_supports_rejects_contract_violations_and_uncovered_ops():
    q = _t(ca.F32, (64, 4, 8, 1))
    k = _t(ca.F16, (64, 16, 8, 1))
    assert ggml.flash_attn_supports(q, _t(ca.F16, (128, 16, 8, 1)), k, None) == ggml.ERR_INVALID        # D mismatch
    assert ggml.flash_attn_supports(q, _t(ca.F16, (64, 16, 3, 1)), _t(ca.F16, (64, 16, 3, 1)), None) == ggml.ERR_INVALID
    assert ggml.flash_attn_supports(q, k, _t(ca.F16, (64, 17, 8, 1)), None) == ggml.ERR_INVALID          # Nkv mismatch
    assert ggml.flash_attn_supports(q, k, k, None, max_bias=1.0) == ggml.ERR_INVALID                     # needs a mask
    assert ggml.flash_attn_supports(q, k, k, _t(ca.F16, (8, 4, 1, 1))) == ggml.ERR_INVALID               # mask too narrow
    assert ggml.flash_attn_supports(q, k, k, _t(ca.F16, (16, 4, 3, 1))) == ggml.ERR_INVALID              # 8 % 3
    # valid for ggml, outside these kernels: goes to the CPU backend
    assert ggml.flash_attn_supports(q, k, _t(ca.F32, (64, 16, 8, 1)), None) == ggml.OK                   # a K and a V of different types: both rounded to f16 first
    assert ggml.flash_attn_supports(q, k, _t(30, (64, 16, 8, 1), (2, 128, 2048, 16384)), None) == ggml.ERR_UNSUPPORTED    # a V type outside the cache types
    assert ggml.flash_attn_supports(_t(ca.F16, (64, 4, 8, 1)), k, k, None) == ggml.ERR_UNSUPPORTED       # q not F32
    k4 = _t(ca.Q4_0, (64, 16, 8, 1), (18, 36, 576, 4608))
    assert ggml.flash_attn_supports(q, k4, k4, None) == ggml.OK                                          # Q4_0 cache view
    assert ggml.flash_attn_supports(q, k4, _t(ca.Q5_1, (64, 16, 8, 1)), None) == ggml.OK                 # -ctk q4_0 -ctv q5_1
    assert ggml.flash_attn_supports(_t(ca.F32, (48, 4, 8, 1)), _t(ca.Q4_0, (32, 16, 8, 1), (18, 18, 288, 2304)),
                                    _t(ca.Q4_0, (32, 16, 8, 1), (18, 18, 288, 2304)), None) == ggml.ERR_INVALID
    k12 = ca.Tensor.__new__(ca.Tensor); k12.__dict__.update(_t(ca.F16, (64, 16, 8, 1)).__dict__); k12.type = 12   # a k-quant
    assert ggml.flash_attn_supports(q, k12, k12, None) == ggml.ERR_UNSUPPORTED
    assert ggml.flash_attn_supports(q, k, k, _t(ca.F32, (16, 4, 1, 1))) == ggml.ERR_UNSUPPORTED          # F32 mask
    # head sizes: multiples of 4 (Moonshine's 36 and 52, src/core/cross_attn.h:119-153) with K and V of one plain type
    q36 = _t(ca.F32, (36, 4, 8, 1))
    assert ggml.flash_attn_supports(q36, _t(ca.F16, (36, 16, 8, 1)), _t(ca.F16, (36, 16, 8, 1)), None) == ggml.OK
    assert ggml.flash_attn_supports(q36, _t(ca.F32, (36, 16, 8, 1)), _t(ca.F32, (36, 16, 8, 1)), None) == ggml.OK
    assert ggml.flash_attn_supports(q36, _t(ca.F16, (36, 16, 8, 1)), _t(ca.F32, (36, 16, 8, 1)), None) == ggml.ERR_UNSUPPORTED
    assert ggml.flash_attn_plan(q36, _t(ca.F16, (36, 16, 8, 1)), _t(ca.F16, (36, 16, 8, 1)), None, 1.0)[0] == ggml.KERNEL_VEC
    q38 = _t(ca.F32, (38, 4, 8, 1))
    assert ggml.flash_attn_supports(q38, _t(ca.F16, (38, 16, 8, 1)), _t(ca.F16, (38, 16, 8, 1)), None) == ggml.ERR_UNSUPPORTED
    assert ggml.flash_attn_supports(q, k, _t(ca.F16, (32, 16, 8, 1)), None) == ggml.ERR_UNSUPPORTED      # DV != DK
    assert ggml.lib().mi355x_last_error() != b""


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(ggml, "_lib", None)
    monkeypatch.setattr(ggml, "LIB_PATH", "/nonexistent/libmi355x_fattn.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ggml.lib()


def test_cpy_supports_matrix():
    L = ggml.lib()
    def ok(s, d, ne_s=(64, 4, 2, 1), ne_d=None):
        a, b = _t(s, ne_s).c(), _t(d, ne_d or ne_s).c()
        return L.mi355x_cpy_supports(ctypes.byref(a), ctypes.byref(b))
    assert ok(ca.F32, ca.F16) == ok(ca.F32, ca.Q8_0) == ok(ca.F32, ca.F32) == ggml.OK
    assert ok(ca.F16, ca.F32) == ok(ca.Q8_0, ca.F32) == ok(ca.Q8_0, ca.Q8_0) == ggml.OK
    assert ok(ca.F16, ca.Q8_0) == ggml.ERR_UNSUPPORTED
    for t in (ca.Q4_0, ca.Q4_1, ca.Q5_0, ca.Q5_1):
        assert ok(ca.F32, t) == ok(t, ca.F32) == ok(t, t) == ggml.OK
        assert ok(t, ca.F16) == ok(t, ca.Q8_0) == ok(ca.F16, t) == ggml.ERR_UNSUPPORTED
    assert ok(ca.F32, ca.F16, (64, 4, 2, 1), (512, 1, 1, 1)) == ggml.OK          # reshape with equal counts
    assert ok(ca.F32, ca.F16, (64, 4, 2, 1), (64, 5, 2, 1)) == ggml.ERR_INVALID
    assert ok(ca.F32, ca.Q8_0, (48, 4, 2, 1)) == ggml.ERR_INVALID


@pytest.mark.gpu
def test_native_host_driver_runs_the_bench_protocol():
    """The C++ driver links only the C-ABI library, checks one masked call against its own double-precision loop
    and runs the reference's decode protocol at attention level; exit code 0 = self-check within 2e-3."""
    import json
    import subprocess
    exe = os.path.join(ROOT, "crispasr_amd", "host", "mi355x_attn_protocol")
    assert os.path.exists(exe), "host driver not built (python -c 'import __graft_entry__ as g; g.build()')"
    res = subprocess.run([exe, "4"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    out = json.loads(res.stdout.strip().splitlines()[-1])
    assert out["layers"] == 4 and out["self_check_max_abs"] <= 2e-3
    assert out["single_token_x256"]["us_per_attention_call"] > 0


def test_relpos_bias_supports_predicate():
    """the predicate a backend's supports_op would ask before claiming FastConformer's mask-building node chain"""
    L = ggml.lib()

    def sup(qv, r, add, dst):
        return L.mi355x_relpos_bias_supports(qv.ref(), r.ref(), add.ref() if add is not None else None, dst.ref())

    T, H = 750, 8
    qv = _t(ca.F32, (128, T, H, 1), (4, 1024 * 4, 128 * 4, T * 1024 * 4))          # permuted view of a [1024, T] activation
    r = _t(ca.F32, (128, 2 * T - 1, H, 1), (4, 1024 * 4, 128 * 4, (2 * T - 1) * 1024 * 4))
    dst = _t(ca.F16, (T, T, H, 1))
    assert sup(qv, r, None, dst) == ggml.OK
    assert sup(qv, r, _t(ca.F32, (T, T, 1, 1)), dst) == ggml.OK                      # pad / window mask, all heads
    assert sup(qv, _t(ca.F16, (128, 2 * T - 1, H, 1)), None, dst) == ggml.OK
    assert sup(qv, _t(ca.F32, (128, 2 * T - 2, H, 1)), None, dst) == ggml.ERR_INVALID    # table one row short
    assert sup(qv, r, _t(ca.F32, (T - 1, T, 1, 1)), dst) == ggml.ERR_INVALID             # add narrower than the keys
    assert sup(qv, r, None, _t(ca.F32, (T, T, H, 1))) == ggml.ERR_INVALID                # the mask is F16
    assert sup(qv, r, None, _t(ca.F16, (T, T, H, 2))) == ggml.ERR_INVALID                # batch mismatch
    q80 = _t(ca.F32, (80, 16, 2, 1))
    assert sup(q80, _t(ca.F32, (80, 31, 2, 1)), None, _t(ca.F16, (16, 16, 2, 1))) == ggml.ERR_UNSUPPORTED   # head size
    assert sup(_t(ca.F16, (128, T, H, 1)), r, None, dst) == ggml.ERR_UNSUPPORTED         # Q_v must be F32


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_planning_sees_the_alignment_a_view_will_have():
    """supports_op runs before allocation: the predicates take the low bits of the future address in the data
    field (never dereferenced), so a view that would be refused at launch is refused at planning already."""
    H, D = 8, 64
    q = _t(ca.F32, (D, 4, H, 1))
    k = _t(ca.F16, (D, 32, H, 1))
    assert ggml.flash_attn_supports(q, k, k, None) == ggml.OK
    for off, want in ((0, ggml.OK), (256, ggml.OK), (16, ggml.OK), (2, ggml.OK), (1, ggml.ERR_UNSUPPORTED), (7, ggml.ERR_UNSUPPORTED)):
        kv = ca.Tensor(None, ca.F16, (D, 32, H, 1), offset=off)
        assert ggml.flash_attn_supports(q, kv, kv, None) == want, off
    assert ggml.flash_attn_supports(ca.Tensor(None, ca.F32, (D, 4, H, 1), offset=4), k, k, None) == ggml.OK
    assert ggml.flash_attn_supports(ca.Tensor(None, ca.F32, (D, 4, H, 1), offset=2), k, k, None) == ggml.ERR_UNSUPPORTED
    # the plan follows the alignment too: the tile kernel's direct-to-LDS loads need 16-byte rows
    qb = _t(ca.F32, (D, 256, H, 1))
    kb = _t(ca.F16, (D, 512, H, 1))
    assert ggml.flash_attn_plan_details(qb, kb, kb, None, kernel=ggml.KERNEL_MMA)["direct"] == 1
    ko = ca.Tensor(None, ca.F16, (D, 512, H, 1), offset=2)
    assert ggml.flash_attn_plan_details(qb, ko, ko, None, kernel=ggml.KERNEL_MMA)["direct"] == 0
    # Q8_0 blocks are 34 bytes: the kernels read them in 2-byte units
    kq = ca.Tensor(None, ca.Q8_0, (D, 32, H, 1), offset=34)
    assert ggml.flash_attn_supports(q, kq, kq, None) == ggml.OK
    kq = ca.Tensor(None, ca.Q8_0, (D, 32, H, 1), offset=35)
    assert ggml.flash_attn_supports(q, kq, kq, None) == ggml.ERR_UNSUPPORTED
    # the copies
    cpy_supports = lambda a, b: ggml.lib().mi355x_cpy_supports(a.ref(), b.ref())
    src = _t(ca.F32, (D, 4, H, 1))
    assert cpy_supports(src, ca.Tensor(None, ca.F16, (D, 4, H, 1), offset=2)) == ggml.OK
    assert cpy_supports(src, ca.Tensor(None, ca.F16, (D, 4, H, 1), offset=1)) == ggml.ERR_UNSUPPORTED
    assert cpy_supports(ca.Tensor(None, ca.F32, (D, 4, H, 1), offset=2), _t(ca.F16, (D, 4, H, 1))) == ggml.ERR_UNSUPPORTED


def test_planning_of_the_narrow_cache_types():
    """Q4_0 .. Q5_1 K/V: up to 16 query rows per KV head go to the decode kernel (head sizes 64 / 128, no soft cap), more
    rows to the tile kernel through f16 copies in the workspace, everything else to the vector kernel."""
    for t, bb in ((ca.Q4_0, 18), (ca.Q4_1, 20), (ca.Q5_0, 22), (ca.Q5_1, 24)):
        for D in (64, 128):
            rs = D // 32 * bb
            k = _t(t, (D, 700, 2, 1), (bb, rs, rs * 700, rs * 1400))
            one = ggml.flash_attn_plan_details(_t(ca.F32, (D, 1, 8, 1)), k, k, None)              # 4 rows per KV head
            assert one["kernel"] == ggml.KERNEL_DECODE_MMA and one["kv_to_f16"] == 0, (t, D, one)
            many = ggml.flash_attn_plan_details(_t(ca.F32, (D, 40, 8, 1)), k, k, None)
            assert many["kernel"] == ggml.KERNEL_MMA and many["kv_to_f16"] == 1, (t, D, many)
            assert many["workspace"] >= 2 * D * 700 * 2 * 2
            capped = ggml.flash_attn_plan_details(_t(ca.F32, (D, 1, 8, 1)), k, k, None, logit_softcap=30.0)
            assert capped["kernel"] == ggml.KERNEL_VEC, (t, D, capped)
        k96 = _t(t, (96, 700, 2, 1), (bb, 3 * bb, 3 * bb * 700, 3 * bb * 1400))
        assert ggml.flash_attn_plan_details(_t(ca.F32, (96, 1, 8, 1)), k96, k96, None)["kernel"] == ggml.KERNEL_VEC
        few = _t(t, (128, 9, 2, 1), (bb, 4 * bb, 4 * bb * 9, 4 * bb * 18))                        # a handful of keys: exact values
        assert ggml.flash_attn_plan_details(_t(ca.F32, (128, 1, 8, 1)), few, few, None)["kernel"] == ggml.KERNEL_VEC


def test_set_rows_supports_checks_shapes_types_and_alignment():
    D, rows = 128, 64
    dst = _t(ca.Q8_0, (D, rows, 8, 1))
    src = _t(ca.F32, (D, 3, 8, 1))
    assert ggml.set_rows_supports(dst, src, (3,)) == ggml.OK
    assert ggml.set_rows_supports(dst, src, (3,), 32) == ggml.OK
    assert ggml.set_rows_supports(dst, src, (3,), 16) != ggml.OK                               # no such index type
    assert ggml.set_rows_supports(dst, src, (4,)) == ggml.ERR_INVALID                          # one index per source row
    assert ggml.set_rows_supports(dst, _t(ca.F32, (64, 3, 8, 1)), (3,)) == ggml.ERR_INVALID    # row length
    assert ggml.set_rows_supports(dst, _t(ca.F32, (D, 3, 4, 1)), (3,)) == ggml.ERR_INVALID     # planes
    assert ggml.set_rows_supports(dst, src, (3, 3)) == ggml.ERR_INVALID                        # 8 % 3: index planes must divide
    assert ggml.set_rows_supports(dst, src, (3, 2)) == ggml.OK
    assert ggml.set_rows_supports(dst, _t(ca.F16, (D, 3, 8, 1)), (3,)) == ggml.ERR_UNSUPPORTED # source must be F32
    assert ggml.set_rows_supports(_t(ca.F16, (D, rows, 8, 1)), src, (3,)) == ggml.OK
    assert ggml.set_rows_supports(_t(ca.F32, (D, rows, 8, 1)), src, (3,)) == ggml.OK
    assert ggml.set_rows_supports(ca.Tensor(None, ca.Q8_0, (D, rows, 8, 1), offset=1), src, (3,)) == ggml.ERR_UNSUPPORTED
    assert ggml.set_rows_supports(dst, ca.Tensor(None, ca.F32, (D, 3, 8, 1), offset=2), (3,)) == ggml.ERR_UNSUPPORTED
    # zero rows: nothing to do, still a supported node
    assert ggml.set_rows_supports(dst, _t(ca.F32, (D, 0, 8, 1)), (0,)) == ggml.OK


@pytest.mark.parametrize("kernel", [ggml.KERNEL_AUTO, ggml.KERNEL_VEC, ggml.KERNEL_MMA, ggml.KERNEL_DECODE_MMA])
@pytest.mark.parametrize("nq,nkv", [(0, 32), (4, 0), (0, 0)])
def test_planning_an_empty_op_with_any_forced_kernel(kernel, nq, nkv):
    """a forced kernel on a shape with no queries or no keys used to divide by zero while planning"""
    q = _t(ca.F32, (64, nq, 8, 1))
    k = _t(ca.F16, (64, nkv, 8, 1))
    for ns in (0, 1, 4):
        try:
            kern, n = ggml.flash_attn_plan(q, k, k, None, kernel=kernel, n_splits=ns)
            assert n >= 1
            assert ggml.flash_attn_workspace_size(q, k, k, None, kernel=kernel, n_splits=ns) >= 0
        except ggml.Mi355xError:
            pass            # a refusal is fine; the process must survive


def test_relpos_workspace_size_is_the_f16_copy_of_the_table():
    D, NR = 128, 149
    r32 = _t(ca.F32, (D, NR, 8, 1))
    assert ggml.relpos_bias_workspace_size(r32) == (D * NR * 8 * 2 + 255) // 256 * 256
    assert ggml.relpos_bias_workspace_size(_t(ca.F16, (D, NR, 8, 1))) == 0
    assert ggml.relpos_bias_workspace_size(_t(ca.F16, (D, NR, 8, 1), (2, 512, 512 * NR, 512 * NR * 8))) > 0     # padded rows


def test_public_header_is_plain_c(tmp_path):
    """the boundary is a C ABI: the header must compile as C99 and as C++11 with nothing but itself"""
    import shutil
    import subprocess
    src = tmp_path / "chk.c"
    src.write_text('#include "mi355x_fattn.h"\nint main(void) { mi355x_fattn_params p; mi355x_fattn_plan_info i; (void)p; (void)i; '
                   'return MI355X_FATTN_API_VERSION > 0 ? 0 : 1; }\n')
    inc = os.path.join(ROOT, "include")
    for cc, std, extra in (("gcc", "-std=c99", []), ("g++", "-std=c++11", ["-x", "c++"])):
        if shutil.which(cc) is None:
            pytest.skip(cc + " not installed")
        res = subprocess.run([cc, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, *extra, "-c", str(src), "-o", str(tmp_path / "chk.o")],
                             capture_output=True, text=True)
        assert res.returncode == 0, res.stderr


def _split_top_level(args: str):
    """the comma-separated pieces of an argument or parameter list, commas inside brackets left alone"""
    parts, depth, cur = [], 0, ""
    for ch in args:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip() and cur.strip() != "void":
        parts.append(cur.strip())
    return parts


def _balanced(text: str, open_at: int) -> str:
    depth = 0
    for i in range(open_at, len(text)):
        depth += text[i] == "("
        depth -= text[i] == ")"
        if depth == 0:
            return text[open_at + 1:i]
    raise AssertionError("unbalanced parentheses")


def test_backend_glue_source_calls_the_library_as_the_header_declares_it():
    """crispasr_amd/ggml-mi355x/ggml-mi355x.cpp needs ggml's headers and is not compiled here: what can be held in step
    without them is that every library name it uses is declared by the public header and that every call passes as many
    arguments as the prototype has parameters"""
    strip = lambda s: re.sub(r"//[^\n]*", "", re.sub(r"/\*.*?\*/", "", s, flags=re.S))
    header = strip(open(os.path.join(ROOT, "include", "mi355x_fattn.h")).read())
    glue = strip(open(os.path.join(ROOT, "crispasr_amd", "ggml-mi355x", "ggml-mi355x.cpp")).read())
    glue = re.sub(r'"(?:\\.|[^"\\])*"', '""', glue)                        # string literals may hold commas and brackets
    protos = {}
    for m in re.finditer(r"\b(mi355x_[a-z0-9_]+)\s*\(", header):
        protos[m.group(1)] = len(_split_top_level(_balanced(header, m.end() - 1)))
    assert set(protos) == set(_declared_symbols())
    declared = set(re.findall(r"\b(?:mi355x|MI355X)_\w+\b", header))
    own = set(re.findall(r"\b(?:static|struct)\s+(?:[\w:<>\*&]+\s+)*?((?:mi355x|MI355X)_\w+)\b", glue))
    used = set(re.findall(r"\b(?:mi355x|MI355X)_\w+\b", glue))
    unknown = sorted(n for n in used - declared - own)
    assert not unknown, f"the glue uses names that the header does not declare: {unknown}"
    calls = 0
    for m in re.finditer(r"\b(mi355x_[a-z0-9_]+)\s*\(", glue):
        name = m.group(1)
        if name not in protos:
            continue                                                       # one of the glue's own functions
        n = len(_split_top_level(_balanced(glue, m.end() - 1)))
        assert n == protos[name], f"{name}: called with {n} arguments, declared with {protos[name]}"
        calls += 1
    assert calls >= 15
    # the entry points a backend cannot do without are all bound
    for name in ("mi355x_api_version", "mi355x_fattn_supports", "mi355x_flash_attn_ext", "mi355x_cpy", "mi355x_set_rows",
                 "mi355x_host_buffer_alloc", "mi355x_buffer_alloc"):
        assert name in used, name


def test_tile_kernel_instantiation_follows_the_grid_and_the_query_padding():
    """which form of the tile kernel a shape takes (planning needs no GPU; 256 CUs are assumed without one): two query blocks
    per wave from one workgroup per CU on and only where 256-query workgroups pad the queries no worse than 128-query
    ones; the key split where 128-query workgroups would leave CUs empty or alone"""
    def form(D, N, H, B=1, Hkv=None, kernel=ggml.KERNEL_MMA):
        q = _t(ca.F32, (D, N, H, B))
        k = _t(ca.F16, (D, N, Hkv or H, B))
        info = ggml.flash_attn_plan_details(q, k, k, None, kernel=kernel)
        return info["query_blocks"], info["key_split"], info["queries_per_workgroup"]
    assert form(64, 1500, 20, 4) == (2, 1, 256)          # Whisper large-v3 encoder, four windows: 480 workgroups
    assert form(64, 1500, 20, 1) == (1, 2, 64)           # one window: 240 workgroups of 128 queries, long key loop
    assert form(64, 1500, 8, 1) == (1, 2, 64)            # Whisper base
    assert form(64, 300, 64) == (1, 1, 128)              # 256-query workgroups would carry 512 slots for 300 queries
    assert form(64, 128, 160) == (1, 1, 128)
    assert form(64, 448, 64) == (1, 1, 128)              # one workgroup per CU and 7 key tiles: the split's merge does not pay
    assert form(64, 750, 20) == (1, 2, 64)
    assert form(128, 407, 32, Hkv=8) == (1, 2, 64)       # Voxtral prefill: 128 workgroups of 128 queries
    assert form(128, 300, 64) == (1, 1, 128)             # 192 workgroups of 128 queries: more than half the CUs
    assert form(128, 2500, 8) == (1, 2, 64)              # ... unless the key loop is long
    assert form(128, 750, 8, 8) == (1, 1, 128)           # FastConformer block


def test_decode_kernel_key_ranges_follow_the_priced_plan():
    """how many key ranges a decode call is cut into (planning needs no GPU; 256 CUs assumed without one): the measured
    optima of the BASELINE shapes, and no more than the merge is worth on long caches under few heads"""
    def plan(D, Nq, Hq, Hkv, B, Nkv, kt=ca.F16):
        q = _t(ca.F32, (D, Nq, Hq, B))
        k = _t(kt, (D, Nkv, Hkv, B))
        info = ggml.flash_attn_plan_details(q, k, k, None)
        return info["kernel"], info["n_splits"]
    dec = ggml.KERNEL_DECODE_MMA
    assert plan(64, 5, 20, 20, 1, 1500) == (dec, 8)                 # Whisper cross-attention, 5 beams: 8 ranges of 192
    assert plan(64, 1, 20, 20, 5, 224) == (dec, 1)                  # ... self-attention: unsplit
    assert plan(128, 1, 32, 8, 1, 663, ca.Q8_0) == (dec, 7)         # Voxtral step at the end of the 256: 7 of 96
    assert plan(128, 1, 32, 32, 1, 663) == (dec, 7)                 # the same with the heads expanded, f16
    assert plan(128, 1, 32, 8, 64, 4096, ca.Q8_0) == (dec, 1)       # 64 sequences fill the chip unsplit
    # short caches (timed with K/V that no cache holds): whole up to 384 keys at 64-wide heads and 256 at 128-wide ones,
    # then 3 ranges or more - 2 were almost never the best count
    assert plan(64, 1, 20, 20, 1, 384) == (dec, 1)
    assert plan(64, 1, 20, 20, 1, 448) == (dec, 3)
    assert plan(128, 1, 32, 8, 1, 256) == (dec, 1)
    assert plan(128, 1, 32, 8, 1, 320) == (dec, 4)
    k, n = plan(128, 1, 8, 8, 1, 4096)                              # 8 heads alone: bounded by the merge (43 before)
    assert k == dec and 12 <= n <= 20, n
    k, n = plan(128, 16, 8, 8, 1, 8192, ca.Q8_0)
    assert k == dec and 12 <= n <= 24, n
    # 9 .. 16 rows per KV head over an f16 cache: the tile kernel at 128-wide heads, and at 64-wide ones from 2048 keys on
    assert plan(128, 16, 8, 8, 1, 8192)[0] == ggml.KERNEL_MMA
    assert plan(128, 4, 32, 8, 1, 256)[0] == dec                        # 4 queries x 4 query heads per KV head: not these
    assert plan(128, 8, 8, 8, 1, 256)[0] == dec
    assert plan(64, 16, 20, 20, 1, 4096)[0] == ggml.KERNEL_MMA
    assert plan(64, 16, 20, 20, 1, 1024)[0] == dec
    # a short prompt against a long Q8_0 cache, several 16-row chunks per KV head: the decode kernel where the tile kernel
    # would dequantise the cache once per query head, the tile kernel where its own key split makes it cheap
    assert plan(64, 16, 32, 8, 5, 4096, ca.Q8_0)[0] == dec
    assert plan(128, 32, 32, 8, 5, 4096, ca.Q8_0)[0] == dec
    assert plan(128, 64, 8, 8, 1, 4096, ca.Q8_0)[0] == ggml.KERNEL_MMA
    assert plan(64, 100, 20, 20, 5, 4096, ca.Q8_0)[0] == ggml.KERNEL_MMA


def test_key_ranges_of_the_vector_and_tile_kernels():
    """the other two split plans (256 CUs assumed without a GPU): the vector kernel keeps to few, power-of-two ranges; the
    tile kernel cuts long caches under small grids"""
    def plan(D, Nq, H, B, Nkv, kt, **kw):
        q = _t(ca.F32, (D, Nq, H, B))
        k = _t(kt, (D, Nkv, H, B))
        info = ggml.flash_attn_plan_details(q, k, k, None, **kw)
        return info["kernel"], info["n_splits"]
    vec, mma = ggml.KERNEL_VEC, ggml.KERNEL_MMA
    assert plan(128, 1, 32, 1, 663, ca.F32) == (vec, 6)              # Voxtral's step with F32 K/V repeated to 32 heads
    assert plan(128, 1, 32, 1, 224, ca.F32) == (vec, 4)              # 56 keys a range for wide heads, 112 beyond 448 keys
    assert plan(128, 1, 32, 1, 408, ca.F32) == (vec, 8)
    assert plan(64, 1, 20, 1, 224, ca.F32) == (vec, 1)               # 128 keys a range for 64-wide ones, and no cut under two ranges' worth
    assert plan(64, 1, 20, 1, 663, ca.F32) == (vec, 6)
    assert plan(64, 1, 20, 1, 408, ca.F32) == (vec, 4)
    assert plan(128, 1, 32, 1, 64, ca.F32) == (vec, 1)
    assert plan(128, 1, 32, 1, 4096, ca.F32) == (vec, 8)             # 32 before
    assert plan(64, 1, 20, 1, 4096, ca.F32) == (vec, 16)             # fewer rows: up to 16 from 4096 keys on
    assert plan(128, 2, 32, 4, 1024, ca.F32, kernel=vec) == (vec, 2) # 256 rows: 4 before
    assert plan(128, 1, 32, 4, 1024, ca.F32) == (vec, 2)
    assert plan(128, 256, 40, 1, 8192, ca.F16) == (mma, 3)           # 160 workgroups of 64 queries: towards two per CU
    assert plan(128, 256, 40, 1, 1024, ca.F16) == (mma, 1)           # ... but no range under 16 tiles there
    assert plan(128, 32, 8, 1, 1024, ca.F16, kernel=mma) == (mma, 8) # 8 workgroups: ranges of two tiles
    assert plan(64, 1500, 8, 1, 1500, ca.F16) == (mma, 1)            # Whisper base: 192 key-split workgroups x 24 tiles, whole
    assert plan(128, 407, 32, 1, 407, ca.F16) == (mma, 1)            # the 407-token prefill


def test_other_head_sizes_are_planned_onto_zero_padded_forms():
    """multiples of 8 below 128 other than 64.  Prompts and encoder windows: the tile kernel on f16 copies of K/V padded to
    64 or 128 - one query block per wave, the copies in the workspace.  Decode-shaped calls over f16 caches: the decode
    kernel, which reads the rows where they lie.  F32 and quantised caches under few query rows, small calls, other head
    sizes and MI355X_FATTN_VEC by name keep the vector kernel."""
    mma, dec, vec = ggml.KERNEL_MMA, ggml.KERNEL_DECODE_MMA, ggml.KERNEL_VEC
    def details(D, Nq, H, Nkv, kt=ca.F16, **kw):
        q = _t(ca.F32, (D, Nq, H, 1))
        k = _t(kt, (D, Nkv, H, 1))
        return ggml.flash_attn_plan_details(q, k, k, None, **kw)
    for D, pad in ((32, 64), (48, 64), (80, 128), (96, 128), (120, 128)):
        p = details(D, 1100, 16, 1100)
        assert (p["kernel"], p["head_pad"], p["kv_to_f16"], p["n_splits"], p["query_blocks"]) == (mma, pad, 1, 1, 1), (D, p)
        assert p["workspace"] == 2 * pad * 1100 * 16 * 2, (D, p)
        assert details(D, 1100, 16, 1100, kernel=vec)["head_pad"] == 0
        # up to 64 chunks of 16 rows per KV head in three rounds of workgroups: the decode kernel in place, no copy launch
        p = details(D, 300, 16, 300)
        assert (p["kernel"], p["head_pad"], p["kv_to_f16"]) == (dec, pad, 0), (D, p)
        assert details(D, 300, 16, 300, ca.F32)["kernel"] == mma
        # one query row per head: the decode kernel in place (no copies; partial rows of the padded size when it splits)
        p = details(D, 1, 16, 1500)
        assert (p["kernel"], p["head_pad"], p["kv_to_f16"]) == (dec, pad, 0), (D, p)
        assert p["n_splits"] > 1 and p["workspace"] == 16 * p["n_splits"] * (pad + 2) * 4, (D, p)
        assert details(D, 1, 16, 1500, ca.F32)["kernel"] == vec                    # (the decode kernel does not read F32)
    assert details(96, 300, 16, 300, ca.Q8_0)["head_pad"] == 128
    assert details(96, 1, 16, 300, ca.Q8_0)["kernel"] == vec
    p = details(80, 32, 4, 8192, kernel=mma)                         # a small grid against a long cache: key ranges, partial rows of 128
    assert p["n_splits"] > 1 and p["workspace"] == 2 * 128 * 8192 * 4 * 2 + 32 * 4 * p["n_splits"] * (128 + 2) * 4, p
    for D in (36, 52, 64, 128, 160):
        assert details(D, 300, 16, 300)["head_pad"] == 0, D
    # f16 calls in 16-row chunks: the decode kernel while a head's chunks see no more than 64k keys between them
    assert details(48, 300, 1, 200)["kernel"] == dec
    assert details(48, 300, 1, 3000)["kernel"] == dec                # 19 chunks x 3000 keys
    assert details(80, 300, 1, 2000)["kernel"] == dec
    assert details(80, 300, 1, 4000)["kernel"] == mma
    assert details(80, 600, 16, 600)["kernel"] == dec                # 38 chunks per head, 608 in all: three rounds
    assert details(80, 16, 16, 4096)["kernel"] == dec                # 16 rows per head: never the tile kernel, which would need the copies
    assert details(80, 1, 16, 64)["kernel"] == dec
    assert details(48, 1, 16, 64)["kernel"] == dec
    assert details(48, 3000, 1, 400)["kernel"] == mma                # 188 chunks on one KV head
    # F32 caches: too small to pay for the copy launch (100k query-key pairs); 2 .. 15 queries only above 64, from 150k pairs on
    assert details(48, 300, 1, 200, ca.F32)["kernel"] == vec
    assert (details(80, 8, 16, 4096, ca.F32)["kernel"], details(80, 8, 16, 4096, ca.F32)["head_pad"]) == (mma, 128)
    assert details(80, 8, 16, 1024, ca.F32)["kernel"] == vec
    assert details(32, 8, 16, 4096, ca.F32)["kernel"] == vec
    assert details(80, 8, 16, 4096)["kernel"] == dec


def test_a_call_is_sized_the_same_with_and_without_its_data_pointers():
    """graph planning asks for a call's workspace before its tensors have addresses (data NULL): the plan - kernel, form,
    key ranges, bytes - must not depend on whether the mask's pointer is there yet, only on whether the call has a mask"""
    for D, N, H in ((64, 900, 32), (64, 600, 40), (64, 2048, 4), (128, 256, 40), (64, 128, 64)):
        q = _t(ca.F32, (D, N, H, 1))
        k = _t(ca.F16, (D, N if D == 64 else 8192, H, 1))
        nkv = k.ne[1]
        pitch = (2 * nkv + 31) // 32 * 32
        for off in (0, 32):                         # no address yet / an address with the alignment the buffer will give
            m = ca.Tensor(None, ca.F16, (nkv, N, 1, 1), (2, pitch, pitch * N, pitch * N), offset=off)
            info = ggml.flash_attn_plan_details(q, k, k, m)
            size = ggml.flash_attn_workspace_size(q, k, k, m)
            if off == 0:
                first = (info["kernel"], info["n_splits"], info["key_split"], info["query_blocks"], size)
            else:
                assert (info["kernel"], info["n_splits"], info["key_split"], info["query_blocks"], size) == first, (D, N, H)
        unmasked = ggml.flash_attn_plan_details(q, k, k, None)
        if (D, N, H) == (64, 900, 32):
            assert first[2] == 2 and unmasked["key_split"] == 1          # the mask is what decides the form here
