"""The planning entry points of the C ABI on arbitrary descriptors: a backend's supports_op is called with whatever the
graph holds, so these must answer with a status code - never crash, never touch a device - for any extents, strides,
types and null pointers."""
import ctypes

from hypothesis import given, settings, strategies as st

from crispasr_amd import ggml

STATUS = {ggml.OK, ggml.ERR_UNSUPPORTED, ggml.ERR_INVALID, ggml.ERR_WORKSPACE}

dims = st.one_of(st.integers(-2, 3), st.sampled_from([0, 1, 5, 8, 16, 31, 32, 64, 80, 128, 256, 257, 1500, 1 << 20, 1 << 40]))
strides = st.one_of(st.integers(0, 4096), st.sampled_from([2, 4, 34, 68, 136, 256, 5120, 1 << 33]))
types = st.sampled_from([0, 1, 2, 3, 6, 7, 8, 30, -1, 1000])


@st.composite
def tensors(draw, planning=True):
    t = ggml.CTensor()
    # planning calls never dereference: NULL, or the low bits the address will have
    t.data = draw(st.sampled_from([None, None, 1, 2, 8, 16, 34, 255])) if planning else draw(st.sampled_from([1, 2, 16, 4096]))
    t.type = draw(types)
    t.ne = (ctypes.c_int64 * 4)(*[draw(dims) for _ in range(4)])
    t.nb = (ctypes.c_size_t * 4)(*[draw(strides) for _ in range(4)])
    return t


def _p(t):
    return ctypes.byref(t) if t is not None else None


@settings(max_examples=int(__import__("os").environ.get("ABI_FUZZ_EXAMPLES", "400")), deadline=None)
@given(q=tensors(), k=tensors(), v=tensors(), m=st.one_of(st.none(), tensors()), d=st.one_of(st.none(), tensors()),
       scale=st.floats(-2, 2), max_bias=st.sampled_from([0.0, 8.0, -1.0]), softcap=st.sampled_from([0.0, 20.0]),
       prec=st.sampled_from([0, 10, 3]), kernel=st.integers(0, 6), n_splits=st.integers(-1, 300), qq=st.sampled_from([0, 8, 5]),
       null=st.integers(0, 7))
def test_attention_planning_calls_answer_with_a_status(q, k, v, m, d, scale, max_bias, softcap, prec, kernel, n_splits, qq, null):
    p = ggml._params(scale, max_bias, softcap, prec, kernel, n_splits, None, qq)
    L = ggml.lib()
    qp, kp, vp = (None if null == 1 else _p(q)), (None if null == 2 else _p(k)), (None if null == 3 else _p(v))
    pp = None if null == 4 else ctypes.byref(p)
    assert L.mi355x_fattn_supports(qp, kp, vp, _p(m), _p(d), pp) in STATUS
    n = ctypes.c_size_t(0)
    assert L.mi355x_fattn_workspace_size(qp, kp, vp, _p(m), pp, ctypes.byref(n)) in STATUS
    kern, ns = ctypes.c_int32(0), ctypes.c_int32(0)
    rc = L.mi355x_fattn_plan(qp, kp, vp, _p(m), pp, ctypes.byref(kern), ctypes.byref(ns))
    assert rc in STATUS
    if rc == ggml.OK:
        assert 1 <= kern.value <= 3 and ns.value >= 1
    info = ggml.CPlanInfo()
    rc2 = L.mi355x_fattn_plan_details(qp, kp, vp, _p(m), pp, ctypes.byref(info))
    assert rc2 == rc
    if rc2 == ggml.OK:
        assert info.kernel == kern.value and info.n_splits == ns.value and info.query_blocks in (0, 1, 2) and info.key_split in (0, 1, 2)
    # the relative-position call plans through the same checks (q doubles as q_v, k as the table)
    assert L.mi355x_fattn_relpos_workspace_size(qp, qp, kp, vp, kp, _p(m), pp, ctypes.byref(n)) in STATUS


@settings(max_examples=int(__import__("os").environ.get("ABI_FUZZ_EXAMPLES", "300")), deadline=None)
@given(a=tensors(), b=tensors(), c=st.one_of(st.none(), tensors()), d=tensors(), null=st.integers(0, 4))
def test_copy_and_relpos_predicates_answer_with_a_status(a, b, c, d, null):
    L = ggml.lib()
    assert L.mi355x_cpy_supports(None if null == 1 else _p(a), None if null == 2 else _p(b)) in STATUS
    assert L.mi355x_relpos_bias_supports(None if null == 1 else _p(a), None if null == 2 else _p(b), _p(c),
                                         None if null == 3 else _p(d)) in STATUS
    n = ctypes.c_size_t(0)
    assert L.mi355x_relpos_bias_workspace_size(None if null == 1 else _p(a), ctypes.byref(n)) in STATUS
    ine = (ctypes.c_int64 * 3)(*[int(a.ne[1]), int(b.ne[2]) % 5, int(b.ne[3]) % 3])
    for bits in (64, 32, 7):
        assert L.mi355x_set_rows_supports(None if null == 1 else _p(a), bits, None if null == 4 else ine,
                                          None if null == 2 else _p(b)) in STATUS
