"""The C ABI without a GPU: the library loads, exports exactly what include/vrl.h declares, and every
argument error is caught on the host before anything could be launched."""

import ctypes
import os
import re

import pytest

from verl_amd import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "vrl.h")


def _declarations():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char\*)\s+(vrl_\w+)\s*\(([^)]*)\)\s*;", text):
        args = m.group(2).strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        decls[m.group(1)] = n
    return decls


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_header_and_binding_declare_the_same_entry_points():
    decls = _declarations()
    assert set(decls) == set(_lib.SIGNATURES), (sorted(decls), sorted(_lib.SIGNATURES))
    for name, nargs in decls.items():
        assert len(_lib.SIGNATURES[name][1]) == nargs, name


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declarations():
        assert hasattr(raw, name), name
    assert lib.vrl_abi_version() == _lib.ABI_VERSION
    m = re.search(r"#define VRL_ABI_VERSION (\d+)", open(HEADER).read())
    assert int(m.group(1)) == _lib.ABI_VERSION


def test_status_codes_match_header_and_have_text(lib):
    text = open(HEADER).read()
    for name in ("VRL_OK", "VRL_ERR_NULL", "VRL_ERR_DTYPE", "VRL_ERR_SHAPE", "VRL_ERR_ALIGN", "VRL_ERR_HIP", "VRL_ERR_ARG",
                 "VRL_ERR_SCRATCH"):
        m = re.search(rf"#define {name} \(?(-?\d+)\)?", text)
        assert int(m.group(1)) == getattr(_lib, name), name
        assert lib.vrl_strerror(getattr(_lib, name)).decode() not in ("", "unknown vrl status")
    assert lib.vrl_strerror(-99).decode() == "unknown vrl status"
    assert lib.vrl_last_hip_error().decode() == ""


# Fake, suitably aligned "device pointers": every call below must return before touching them.
P = 0x10000


def test_rowscore_argument_errors(lib):
    f = lib.vrl_rowscore
    ok = dict(logits=P, dtype=_lib.VRL_BF16, n=4, V=100, stride=100, labels=P, temp=None, lp=P, h=P, flag=P)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["logits"], a["dtype"], a["n"], a["V"], a["stride"], a["labels"], a["temp"], a["lp"], a["h"], a.get("q"), a.get("lse"), a["flag"], None)

    assert call(dtype=7) == _lib.VRL_ERR_DTYPE
    assert call(n=-1) == _lib.VRL_ERR_SHAPE
    assert call(V=0) == _lib.VRL_ERR_SHAPE
    assert call(stride=99) == _lib.VRL_ERR_SHAPE
    assert call(n=2**31) == _lib.VRL_ERR_SHAPE
    assert call(lp=None, h=None) == _lib.VRL_ERR_ARG
    assert call(logits=None) == _lib.VRL_ERR_NULL
    assert call(labels=None) == _lib.VRL_ERR_NULL
    assert call(flag=None) == _lib.VRL_ERR_NULL
    assert call(logits=P + 1) == _lib.VRL_ERR_ALIGN
    assert call(dtype=_lib.VRL_F32, logits=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(labels=P + 4) == _lib.VRL_ERR_ALIGN
    assert call(lp=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(temp=P + 1) == _lib.VRL_ERR_ALIGN
    # nothing to do is not an error, and needs no pointers
    assert call(q=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(lse=P + 1) == _lib.VRL_ERR_ALIGN
    assert call(lp=None, h=None, labels=None, flag=None, lse=None) == _lib.VRL_ERR_ARG
    assert f(None, _lib.VRL_F32, 0, 100, 100, None, None, None, P, None, None, None, None) == _lib.VRL_OK


def test_split_and_slice_argument_errors(lib):
    f = lib.vrl_rowscore_split

    def call(n=4, splits=4, partials=P, lp=P, dtype=_lib.VRL_BF16):
        return f(P, dtype, n, 100000, 100000, P, None, lp, P, None, None, P, splits, partials, None)

    assert call(splits=0) == _lib.VRL_ERR_ARG
    assert call(splits=65) == _lib.VRL_ERR_ARG
    assert call(partials=None) == _lib.VRL_ERR_NULL
    assert call(partials=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(dtype=9) == _lib.VRL_ERR_DTYPE
    assert call(n=0, partials=None) == _lib.VRL_OK

    g = lib.vrl_rowscore_split_static

    def call_static(n=4, splits=4, lp=P, dtype=_lib.VRL_BF16):
        return g(P, dtype, n, 100000, 100000, P, None, lp, P, None, None, P, splits, None)

    assert call_static(splits=0) == _lib.VRL_ERR_ARG
    assert call_static(splits=65) == _lib.VRL_ERR_ARG
    assert call_static(dtype=9) == _lib.VRL_ERR_DTYPE
    assert call_static(lp=P + 2) == _lib.VRL_ERR_ALIGN
    assert call_static(n=0) == _lib.VRL_OK
    assert call_static(n=129, splits=64) == _lib.VRL_ERR_SCRATCH      # 8256 partials > VRL_STATIC_PARTIALS_MAX
    assert call_static(n=8193, splits=2) == _lib.VRL_ERR_SCRATCH
    m = re.search(r"#define VRL_STATIC_PARTIALS_MAX (\d+)", open(HEADER).read())
    assert int(m.group(1)) == _lib.STATIC_PARTIALS_MAX
    plan = lib.vrl_rowscore_split_plan
    assert plan(_lib.VRL_BF16, 8192, 151936) == 1          # enough rows: one workgroup per row
    assert plan(_lib.VRL_BF16, 2048, 151936) == 1
    assert plan(_lib.VRL_BF16, 256, 151936) == 1            # a 16-wavefront workgroup per row already fills a CU
    assert 2 <= plan(_lib.VRL_BF16, 64, 151936) <= 64
    assert plan(_lib.VRL_BF16, 1, 151936) >= 16
    assert plan(_lib.VRL_F32, 16, 1000) == 1                # rows too short to cut
    assert plan(7, 16, 151936) == 1 and plan(_lib.VRL_F32, 0, 10) == 1

    bw = lib.vrl_rowscore_backward

    def back(dtype=_lib.VRL_BF16, n=4, V=100, stride=100, dstride=100, labels=P, lse=P, ent=P, gl=P, gh=P, dx=P, x=P):
        return bw(x, dtype, n, V, stride, labels, None, lse, ent, gl, gh, dx, dstride, None)

    assert back(dtype=5) == _lib.VRL_ERR_DTYPE
    assert back(dstride=99) == _lib.VRL_ERR_SHAPE
    assert back(gl=None, gh=None) == _lib.VRL_ERR_ARG
    assert back(lse=None) == _lib.VRL_ERR_NULL
    assert back(labels=None) == _lib.VRL_ERR_NULL
    assert back(ent=None) == _lib.VRL_ERR_NULL
    assert back(dx=None) == _lib.VRL_ERR_NULL
    assert back(dx=P + 1) == _lib.VRL_ERR_ALIGN
    assert back(n=0, x=None, dx=None, lse=None) == _lib.VRL_OK

    g = lib.vrl_response_slice     # (values, row_bytes, cu, response_lens, B, n_tokens, T_out, out, err_flag, stream)
    assert g(P, 4, P, P, -1, 9, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, 4, P, P, 2, -1, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, 0, P, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_SHAPE       # a row holds at least one byte
    assert g(P, (1 << 30) + 1, P, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, 1 << 20, P, P, 2, 9, 1 << 20, P, P, None) == _lib.VRL_ERR_SHAPE   # a padded row block beyond the grid
    assert g(None, 4, P, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P, P, 2, 9, 4, P, None, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P + 4, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_ALIGN
    assert g(None, 4, None, None, 0, 0, 4, None, None, None) == _lib.VRL_OK


def test_label_logprob_argument_errors_and_flag_values(lib):
    f = lib.vrl_label_logprob     # (logits, dtype, n_rows, vocab, row_stride, labels, temperature, lse, out, err_flag, stream)
    assert f(P, 9, 4, 100, 100, P, None, P, P, P, None) == _lib.VRL_ERR_DTYPE
    assert f(P, _lib.VRL_BF16, -1, 100, 100, P, None, P, P, P, None) == _lib.VRL_ERR_SHAPE
    assert f(P, _lib.VRL_BF16, 4, 100, 99, P, None, P, P, P, None) == _lib.VRL_ERR_SHAPE
    for missing in (0, 5, 7, 8, 9):
        args = [P, _lib.VRL_BF16, 4, 100, 100, P, None, P, P, P, None]
        args[missing] = None
        assert f(*args) == _lib.VRL_ERR_NULL, missing
    assert f(P, _lib.VRL_F32, 4, 100, 100, P, None, P + 2, P, P, None) == _lib.VRL_ERR_ALIGN
    assert f(None, _lib.VRL_F32, 0, 100, 100, None, None, None, None, None, None) == _lib.VRL_OK
    text = open(HEADER).read()
    for name in ("VRL_FLAG_LABEL_OOB", "VRL_FLAG_SLICE_RANGE", "VRL_FLAG_SEQ_RANGE"):
        m = re.search(rf"#define {name} (\d+)", text)
        assert int(m.group(1)) == getattr(_lib, name), name


def test_score_responses_argument_errors(lib):
    f = lib.vrl_score_responses
    ok = dict(x=P, dt=_lib.VRL_BF16, n=8, V=100, stride=100, lab=None, ids=P, temp=None, cu=P, rl=P, B=2, T=4, tlp=None,
              th=None, rlp=P, rh=P, rlse=None, flag=P)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["x"], a["dt"], a["n"], a["V"], a["stride"], a["lab"], a["ids"], a["temp"], a["cu"], a["rl"], a["B"],
                 a["T"], a["tlp"], a["th"], a["rlp"], a["rh"], a["rlse"], a["flag"], None)

    assert call(dt=4) == _lib.VRL_ERR_DTYPE
    assert call(n=-1) == _lib.VRL_ERR_SHAPE
    assert call(stride=50) == _lib.VRL_ERR_SHAPE
    assert call(T=-1) == _lib.VRL_ERR_SHAPE
    assert call(n=2**31 - 1) == _lib.VRL_ERR_SHAPE                 # rows + sequences must fit one grid
    assert call(B=0) == _lib.VRL_ERR_SHAPE                         # rows that belong to no sequence
    assert call(rlp=None, rh=None) == _lib.VRL_ERR_ARG
    assert call(lab=P) == _lib.VRL_ERR_ARG                         # labels and input_ids together
    assert call(tlp=P, rlp=None) == _lib.VRL_ERR_ARG               # a per-token vector without its block
    assert call(th=P, rh=None) == _lib.VRL_ERR_ARG
    assert call(cu=None) == _lib.VRL_ERR_NULL
    assert call(rl=None) == _lib.VRL_ERR_NULL
    assert call(flag=None) == _lib.VRL_ERR_NULL
    assert call(x=None) == _lib.VRL_ERR_NULL
    assert call(ids=None) == _lib.VRL_ERR_NULL                     # log-probs asked for, no source of labels
    assert call(cu=P + 4) == _lib.VRL_ERR_ALIGN
    assert call(rh=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(rlse=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(n=0, B=0, x=None, cu=None, rl=None, flag=None) == _lib.VRL_OK


def test_score_responses_backward_argument_errors(lib):
    f = lib.vrl_score_responses_backward
    ok = dict(x=P, dt=_lib.VRL_BF16, n=8, V=100, stride=100, lab=None, ids=P, temp=None, cu=P, rl=P, B=2, T=4, lse=P,
              ent=P, gl=P, gh=P, out=P, ds=100)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["x"], a["dt"], a["n"], a["V"], a["stride"], a["lab"], a["ids"], a["temp"], a["cu"], a["rl"], a["B"],
                 a["T"], a["lse"], a["ent"], a["gl"], a["gh"], a["out"], a["ds"], None)

    assert call(dt=7) == _lib.VRL_ERR_DTYPE
    assert call(n=-1) == _lib.VRL_ERR_SHAPE
    assert call(stride=50) == _lib.VRL_ERR_SHAPE
    assert call(ds=50) == _lib.VRL_ERR_SHAPE
    assert call(T=-1) == _lib.VRL_ERR_SHAPE
    assert call(gl=None, gh=None) == _lib.VRL_ERR_ARG
    assert call(lab=P) == _lib.VRL_ERR_ARG                         # labels and input_ids together
    assert call(x=None) == _lib.VRL_ERR_NULL
    assert call(out=None) == _lib.VRL_ERR_NULL
    assert call(cu=None) == _lib.VRL_ERR_NULL
    assert call(lse=None) == _lib.VRL_ERR_NULL
    assert call(ids=None) == _lib.VRL_ERR_NULL                     # a log-prob gradient without a source of labels
    assert call(ent=None) == _lib.VRL_ERR_NULL                     # an entropy gradient without the entropies
    assert call(B=0) == _lib.VRL_ERR_SHAPE                         # rows that belong to no sequence
    assert call(out=P + 1) == _lib.VRL_ERR_ALIGN
    assert call(gl=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(n=0, x=None, out=None) == _lib.VRL_OK


def test_gemm_nt_argument_errors(lib):
    f = lib.vrl_gemm_nt
    ok = dict(x=P, y=P, dt=_lib.VRL_BF16, NX=512, NY=256, K=256, xs=256, ys=256, out=P, os=512, acc=0, parts=1, ws=None)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["x"], a["y"], a["dt"], a["NX"], a["NY"], a["K"], a["xs"], a["ys"], a["out"], a["os"], a["acc"],
                 a["parts"], a["ws"], None)

    assert call(dt=_lib.VRL_F32) == _lib.VRL_ERR_DTYPE
    assert call(NX=128) == _lib.VRL_ERR_SHAPE
    assert call(NY=255) == _lib.VRL_ERR_SHAPE
    assert call(NX=514, os=516) == _lib.VRL_ERR_SHAPE              # columns of out in quads
    assert call(K=96) == _lib.VRL_ERR_SHAPE
    assert call(K=64, xs=64, ys=64) == _lib.VRL_ERR_SHAPE          # the pipeline needs two steps
    assert call(xs=128) == _lib.VRL_ERR_SHAPE
    assert call(ys=260) == _lib.VRL_ERR_SHAPE
    assert call(os=510) == _lib.VRL_ERR_SHAPE
    assert call(parts=0) == _lib.VRL_ERR_ARG
    assert call(parts=17) == _lib.VRL_ERR_ARG
    assert call(parts=4) == _lib.VRL_ERR_ARG                        # ranges of fewer than two steps
    assert call(x=None) == _lib.VRL_ERR_NULL
    assert call(out=None) == _lib.VRL_ERR_NULL
    assert call(K=512, xs=512, ys=512, parts=2) == _lib.VRL_ERR_NULL   # ranges need the workspace
    assert call(x=P + 8) == _lib.VRL_ERR_ALIGN
    assert call(out=P + 4) == _lib.VRL_ERR_ALIGN
    need = ctypes.c_int64(-1)
    parts = lib.vrl_gemm_nt_plan(_lib.VRL_BF16, 3584, 4096, 152064, ctypes.addressof(need))
    assert 1 <= parts <= 16 and need.value == (parts * 3584 * 4096 if parts > 1 else 0)
    assert lib.vrl_gemm_nt_plan(_lib.VRL_F32, 3584, 4096, 152064, None) == _lib.VRL_ERR_DTYPE
    assert lib.vrl_gemm_nt_plan(_lib.VRL_BF16, 3584, 152064, 4096, ctypes.addressof(need)) == 1 and need.value == 0


def test_gemm_layout_argument_errors(lib):
    f = lib.vrl_gemm
    ok = dict(x=P, y=P, dt=_lib.VRL_BF16, NX=512, NY=256, K=256, xs=512, ys=256, xt=1, yt=0, out=P, os=512, acc=0, parts=1,
              ws=None)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["x"], a["y"], a["dt"], a["NX"], a["NY"], a["K"], a["xs"], a["ys"], a["xt"], a["yt"], a["out"], a["os"],
                 a["acc"], a["parts"], a["ws"], None)

    assert call(dt=_lib.VRL_F32) == _lib.VRL_ERR_DTYPE
    assert call(xs=256) == _lib.VRL_ERR_SHAPE                       # contraction-major x: stride counts its rows (512)
    assert call(NX=516, xs=520, os=516) == _lib.VRL_ERR_SHAPE      # ... which come in groups of 8
    assert call(yt=1, NY=260, ys=264) == _lib.VRL_ERR_SHAPE
    assert call(yt=1, NY=512, ys=256) == _lib.VRL_ERR_SHAPE
    assert call(xt=0, xs=128) == _lib.VRL_ERR_SHAPE                # row-major x: stride counts the contraction (256)
    assert call(K=96) == _lib.VRL_ERR_SHAPE
    assert call(xs=(1 << 28) + 8) == _lib.VRL_ERR_SHAPE            # lane offsets are 32-bit
    assert call(parts=0) == _lib.VRL_ERR_ARG
    assert call(y=None) == _lib.VRL_ERR_NULL
    assert call(x=P + 8) == _lib.VRL_ERR_ALIGN


def test_lmhead_dlogits_argument_errors(lib):
    f = lib.vrl_lmhead_dlogits
    ok = dict(h=P, w=P, dt=_lib.VRL_BF16, T=512, V=1024, K=128, hs=128, ws=128, lab=P, temp=None, lse=P, ent=P, gl=P, gh=P,
              S=2, out=P, ds=1024)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["h"], a["w"], a["dt"], a["T"], a["V"], a["K"], a["hs"], a["ws"], a["lab"], a["temp"], a["lse"], a["ent"],
                 a["gl"], a["gh"], a["S"], a["out"], a["ds"], None)

    assert call(dt=_lib.VRL_F32) == _lib.VRL_ERR_DTYPE
    assert call(T=100) == _lib.VRL_ERR_SHAPE
    assert call(K=96, hs=96, ws=96) == _lib.VRL_ERR_SHAPE
    assert call(V=1020, ds=1024) == _lib.VRL_ERR_SHAPE            # 8-byte stores need a vocabulary that is a multiple of 8
    assert call(ds=1016) == _lib.VRL_ERR_SHAPE
    assert call(ds=1028) == _lib.VRL_ERR_SHAPE
    assert call(S=0) == _lib.VRL_ERR_SHAPE
    assert call(gl=None, gh=None) == _lib.VRL_ERR_ARG
    assert call(lse=None) == _lib.VRL_ERR_NULL
    assert call(out=None) == _lib.VRL_ERR_NULL
    assert call(lab=None) == _lib.VRL_ERR_NULL
    assert call(ent=None) == _lib.VRL_ERR_NULL
    assert call(out=P + 8) == _lib.VRL_ERR_ALIGN
    assert call(lse=P + 2) == _lib.VRL_ERR_ALIGN


def test_response_pack_argument_errors(lib):
    g = lib.vrl_response_pack      # (values, row_bytes, cu, response_lens, out_offsets, B, n_tokens, out_total, out, err_flag, stream)
    assert g(P, 4, P, P, P, -1, 9, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, 4, P, P, P, 2, 9, -1, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, 4, P, P, P, 2, -9, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(P, -2, P, P, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_SHAPE
    assert g(None, 4, P, P, P, 2, 9, 4, P, P, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P, P, None, 2, 9, 4, P, P, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P, P, P, 2, 9, 4, None, P, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P, P, P, 2, 9, 4, P, None, None) == _lib.VRL_ERR_NULL
    assert g(P, 4, P, P, P + 4, 2, 9, 4, P, P, None) == _lib.VRL_ERR_ALIGN
    assert g(None, 4, None, None, None, 0, 0, 0, None, None, None) == _lib.VRL_OK


def test_lmhead_argument_errors(lib):
    f = lib.vrl_lmhead_score
    ok = dict(h=P, w=P, dt=_lib.VRL_BF16, T=512, V=1024, K=128, hs=128, ws=128, lab=P, temp=None, S=2, part=P, lp=P, ent=P,
              lse=None, flag=P, logits=None, ls=0, lr=0)

    def call(**kw):
        a = {**ok, **kw}
        return f(a["h"], a["w"], a["dt"], a["T"], a["V"], a["K"], a["hs"], a["ws"], a["lab"], a["temp"], a["S"], a["part"],
                 a["lp"], a["ent"], a["lse"], a["flag"], a["logits"], a["ls"], a["lr"], None)

    assert call(dt=_lib.VRL_F32) == _lib.VRL_ERR_DTYPE
    assert call(T=255) == _lib.VRL_ERR_SHAPE and call(V=100) == _lib.VRL_ERR_SHAPE
    assert call(K=96) == _lib.VRL_ERR_SHAPE and call(hs=64) == _lib.VRL_ERR_SHAPE and call(ws=132) == _lib.VRL_ERR_SHAPE
    assert call(S=0) == _lib.VRL_ERR_SHAPE and call(S=65) == _lib.VRL_ERR_SHAPE
    assert call(lp=None, ent=None) == _lib.VRL_ERR_ARG
    assert call(h=None) == _lib.VRL_ERR_NULL and call(part=None) == _lib.VRL_ERR_NULL
    assert call(lab=None) == _lib.VRL_ERR_NULL and call(flag=None) == _lib.VRL_ERR_NULL
    assert call(h=P + 8) == _lib.VRL_ERR_ALIGN and call(w=P + 2) == _lib.VRL_ERR_ALIGN
    # kept logits: a pitch that holds a row and keeps 8-byte groups aligned
    assert call(logits=P, ls=1000, lr=512) == _lib.VRL_ERR_SHAPE and call(logits=P, ls=1028, lr=512) == _lib.VRL_ERR_SHAPE
    assert call(logits=P, ls=1024, V=1020, lr=512) == _lib.VRL_ERR_SHAPE
    assert call(logits=P + 8, ls=1024, lr=512) == _lib.VRL_ERR_ALIGN
    assert call(lp=None, ent=None, logits=P, ls=1024, lr=256, h=None) == _lib.VRL_ERR_NULL   # the logits alone are a valid request
    # ... of the first logits_rows tokens, at least one and no more than there are
    assert call(logits=P, ls=1024, lr=0) == _lib.VRL_ERR_SHAPE and call(logits=P, ls=1024, lr=513) == _lib.VRL_ERR_SHAPE
    assert lib.vrl_lmhead_plan(8192, 152064) == 8 and lib.vrl_lmhead_plan(0, 5) == 1


def test_transpose_argument_errors(lib):
    t = lib.vrl_transpose
    Q = P + (1 << 20)                      # a second, disjoint address
    assert t(P, 1, 4, 4, 4, Q, 4, None) == _lib.VRL_ERR_DTYPE
    assert t(P, 8, 4, 4, 4, Q, 4, None) == _lib.VRL_ERR_DTYPE
    assert t(P, 2, -1, 4, 4, Q, 4, None) == _lib.VRL_ERR_SHAPE
    assert t(P, 2, 4, 4, 3, Q, 4, None) == _lib.VRL_ERR_SHAPE      # source pitch below the column count
    assert t(P, 2, 4, 4, 4, Q, 3, None) == _lib.VRL_ERR_SHAPE      # destination pitch below the row count
    assert t(None, 2, 4, 4, 4, Q, 4, None) == _lib.VRL_ERR_NULL
    assert t(P, 2, 4, 4, 4, None, 4, None) == _lib.VRL_ERR_NULL
    assert t(P + 1, 2, 4, 4, 4, Q, 4, None) == _lib.VRL_ERR_ALIGN
    assert t(P, 4, 4, 4, 4, Q + 2, 4, None) == _lib.VRL_ERR_ALIGN
    assert t(P, 4, 4, 4, 4, P, 4, None) == _lib.VRL_ERR_ARG        # in place
    assert t(P, 4, 4, 4, 4, P + 60, 4, None) == _lib.VRL_ERR_ARG   # last source word = first destination word
    assert t(None, 2, 0, 4, 4, None, 4, None) == _lib.VRL_OK       # nothing to move
    assert t(None, 4, 4, 0, 0, None, 4, None) == _lib.VRL_OK


def test_rollout_corr_argument_errors(lib):
    import ctypes

    f = lib.vrl_rollout_corr
    arr = (ctypes.c_float * 11)()
    host = ctypes.cast(arr, ctypes.c_void_p)

    def call(old=P, roll=P, B=2, T=8, is_mode=1, bits=1, lo=host, hi=host, w=P, keep=P, stats=P, sbits=P):
        return f(old, roll, None, B, T, is_mode, 0, 2.0, 0.0, 0.5, bits, lo, hi, w, keep, stats, sbits, None)

    assert call(B=-1) == _lib.VRL_ERR_SHAPE
    assert call(is_mode=3) == _lib.VRL_ERR_ARG
    assert call(bits=1 << 11) == _lib.VRL_ERR_ARG
    assert call(lo=None) == _lib.VRL_ERR_NULL
    assert call(stats=None) == _lib.VRL_ERR_NULL
    assert call(sbits=None) == _lib.VRL_ERR_NULL
    assert call(old=None) == _lib.VRL_ERR_NULL
    assert call(roll=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(B=0, old=None, roll=None, stats=None, sbits=None) == _lib.VRL_OK
    assert lib.vrl_rollout_corr_num_stats() == 40


def test_verify_argument_errors(lib):
    f = lib.vrl_spec_verify

    def call(ln=P, lo=P, lu=P, mask=None, cu=None, B=2, T=8, n=16, accept=P, first=P, prefix=P, near=P, ids=None,
             out_ids=None, out_mask=None, flag=None, work=None, work_bytes=0):
        return f(ln, lo, lu, mask, cu, B, T, n, 0.0, 1e-6, accept, first, prefix, near, ids, 0, out_ids, out_mask, flag,
                 work, work_bytes, None)

    assert call(n=15) == _lib.VRL_ERR_SHAPE                       # padded: the arrays hold exactly B*T tokens
    assert call(n=-1) == _lib.VRL_ERR_SHAPE
    assert call(cu=P, n=100) == _lib.VRL_ERR_NULL                 # packed: the offsets are checked on the device, which
    assert call(cu=P, n=100, flag=P + 2) == _lib.VRL_ERR_ALIGN    # needs somewhere to report to

    assert call(B=-1) == _lib.VRL_ERR_SHAPE
    assert call(T=-1) == _lib.VRL_ERR_SHAPE
    assert call(ln=None) == _lib.VRL_ERR_NULL
    assert call(lu=None) == _lib.VRL_ERR_NULL
    assert call(accept=None) == _lib.VRL_ERR_NULL
    assert call(first=None) == _lib.VRL_ERR_NULL
    assert call(ids=P) == _lib.VRL_ERR_ARG                      # draft without outputs
    assert call(ids=P, out_ids=P) == _lib.VRL_ERR_ARG
    assert call(lo=P + 2) == _lib.VRL_ERR_ALIGN
    assert call(cu=P + 4, flag=P) == _lib.VRL_ERR_ALIGN
    assert call(B=0, n=0, ln=None, lo=None, lu=None, accept=None, first=None, prefix=None, near=None) == _lib.VRL_OK
    # the scratch of the two-pass form: half a byte per token in whole tiles of 1024 tokens, plus 4 bytes per tile
    need = lib.vrl_spec_verify_workspace
    assert need(0) == 0 and need(1) == 16 * 4 * 8 + 4 and need(1024) == 516 and need(1025) == 2 * 516
    assert call(work=P, work_bytes=need(16) - 1) == _lib.VRL_ERR_SHAPE
    assert call(work=None, work_bytes=8) == _lib.VRL_ERR_ARG
    assert call(work=P, work_bytes=-1) == _lib.VRL_ERR_ARG
    assert call(work=P + 4, work_bytes=need(16)) == _lib.VRL_ERR_ALIGN
    plan = lib.vrl_spec_verify_plan
    assert plan(1, 512, 0, 1 << 20) == 1 and plan(1, 6, 0, 8192) == 0 and plan(1, 0, 0, 0) == 0
    assert plan(0, 16, 8192, 16 * 8192) == 1 and plan(0, 64, 1024, 65536) == 0 and plan(0, 4096, 256, 1 << 20) == 0


def test_truncate_and_fused_argument_errors(lib):
    t = lib.vrl_truncate_draft     # (ids, mask, cu, B, T, n_tokens, first_reject, pad_id, out_ids, out_mask, err_flag, stream)
    assert t(P, None, None, -1, 4, 8, P, 0, P, P, None, None) == _lib.VRL_ERR_SHAPE
    assert t(P, None, None, 2, 4, 7, P, 0, P, P, None, None) == _lib.VRL_ERR_SHAPE      # padded: n_tokens == B*T
    assert t(P, None, P, 2, 0, 7, P, 0, P, P, None, None) == _lib.VRL_ERR_NULL          # packed needs err_flag
    assert t(None, None, None, 2, 4, 8, P, 0, P, P, None, None) == _lib.VRL_ERR_NULL
    assert t(P, None, None, 2, 4, 8, None, 0, P, P, None, None) == _lib.VRL_ERR_NULL
    assert t(P + 4, None, None, 2, 4, 8, P, 0, P, P, None, None) == _lib.VRL_ERR_ALIGN
    assert t(None, None, None, 0, 4, 0, None, 0, None, None, None, None) == _lib.VRL_OK

    f = lib.vrl_fused_score_verify

    def call(n=16, B=2, T=8, lp=P, dtype=_lib.VRL_BF16, cu=None, lo=P):
        return f(P, dtype, n, 100, 100, P, None, lp, P, None, None, P, lo, P, None, cu, B, T, 0.0, 1e-6, P, P, P, P, None, 0, None, None, None)

    assert call(lp=None) == _lib.VRL_ERR_NULL                  # verify needs the log-probs
    assert call(dtype=3) == _lib.VRL_ERR_DTYPE
    assert call(n=15) == _lib.VRL_ERR_SHAPE                     # padded layout: n_rows must be B*T
    assert call(lo=None) == _lib.VRL_ERR_NULL
    assert call(B=-2) == _lib.VRL_ERR_SHAPE


def test_missing_library_is_a_loud_error(tmp_path):
    with pytest.raises(_lib.VrlLibraryError, match="does not exist"):
        _lib.load(str(tmp_path / "libvrl_hip.so"))
    bogus = tmp_path / "bogus.so"
    bogus.write_bytes(b"not an elf")
    with pytest.raises(_lib.VrlLibraryError, match="cannot load"):
        _lib.load(str(bogus))


def test_check_raises_with_text():
    with pytest.raises(_lib.VrlCallError, match="vocab") as ei:
        _lib.check("vrl_rowscore", _lib.VRL_ERR_SHAPE)
    assert ei.value.status == _lib.VRL_ERR_SHAPE
    _lib.check("vrl_rowscore", _lib.VRL_OK)


def test_header_is_plain_c(tmp_path):
    """include/vrl.h must be usable from C (no C++ in the signatures): gcc -std=c99 compiles a user of it."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "user.c"
    src.write_text('#include "vrl.h"\ntypedef int (*fn_t)(void);\nint main(void) { fn_t f = vrl_abi_version; (void)f; return VRL_OK; }\n')
    inc = os.path.dirname(HEADER)
    out = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-c", str(src), f"-I{inc}", "-o", str(tmp_path / "user.o")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert out.returncode == 0, out.stdout
