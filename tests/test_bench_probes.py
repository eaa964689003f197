"""The bench-side probe library: it is a library of its own (the scoring library neither exports nor declares the probes),
loads without a GPU and refuses bad arguments on the host."""

import ctypes
import os

from verl_amd import _lib

import bench_probes

P = 0x10000
HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "vrl.h")


def test_probes_are_not_part_of_the_scoring_library():
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in bench_probes.SIGNATURES:
        assert not hasattr(raw, name), name
        assert name not in _lib.SIGNATURES
        assert name not in open(HEADER).read()


def test_probe_argument_errors():
    lib = bench_probes.load()
    f = lib.vrl_mfma_probe
    assert f(-1, 10, 32, 1, P, None, None, None) == _lib.VRL_ERR_SHAPE
    assert f(4, -1, 16, 1, P, None, None, None) == _lib.VRL_ERR_SHAPE
    assert f(4, 10, 8, 1, P, None, None, None) == _lib.VRL_ERR_ARG
    assert f(4, bench_probes.MAX_ITERS + 1, 16, 1, P, None, None, None) == _lib.VRL_ERR_ARG   # no unbounded loops
    assert f(4, 10, 32, 1, None, None, None, None) == _lib.VRL_ERR_NULL
    assert f(4, 10, 16, 0, P + 2, None, None, None) == _lib.VRL_ERR_ALIGN
    assert f(4, 10, 32, 0, P, P + 4, None, None) == _lib.VRL_ERR_ALIGN
    assert f(0, 10, 16, 1, None, None, None, None) == _lib.VRL_OK
    g = lib.vrl_stream_probe
    assert g(P, None, 4, 64, 7, P, None) == _lib.VRL_ERR_ARG
    assert g(P, None, 4, 60, 0, P, None) == _lib.VRL_ERR_SHAPE
    assert g(None, None, 4, 64, 0, P, None) == _lib.VRL_ERR_NULL
    assert g(P, None, 4, 64, 1, None, None) == _lib.VRL_ERR_NULL
    assert g(P + 8, None, 4, 64, 0, P, None) == _lib.VRL_ERR_ALIGN
    assert g(P, None, 0, 64, 0, P, None) == _lib.VRL_OK
    m = int(open(os.path.join(os.path.dirname(bench_probes.__file__), "vrl_probe.h")).read().split("#define VRL_PROBE_MAX_ITERS")[1].split()[0])
    assert m == bench_probes.MAX_ITERS
