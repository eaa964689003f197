"""vrl_rowscore_split_static — the entry point that allocates nothing — against vrl_rowscore_split.

Both run the same kernels; only the home of the per-slice partials differs (a static device array inside the
library instead of caller-owned scratch), so every output must agree bit for bit. Two calls in a row share the
array: the second, smaller one must not see anything of the first.
"""

import numpy as np
import pytest
import torch

from verl_amd import _lib

pytestmark = pytest.mark.gpu


def _call_pair(lib, dev, n, V, dtype, splits, seed, with_temperature):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    x = (torch.randn((n, V), generator=g, device=dev, dtype=torch.float32) * 3.0).to(dtype)
    lab = torch.randint(0, V, (n,), generator=g, device=dev, dtype=torch.int64)
    temp = (0.5 + torch.rand(n, generator=g, device=dev, dtype=torch.float32)) if with_temperature else None
    code = {torch.float32: _lib.VRL_F32, torch.bfloat16: _lib.VRL_BF16, torch.float16: _lib.VRL_F16}[dtype]
    stream = _lib.stream_ptr(dev)
    tptr = None if temp is None else temp.data_ptr()

    def outs():
        return [torch.full((n,), float("nan"), dtype=torch.float32, device=dev) for _ in range(4)] + [
            torch.zeros(1, dtype=torch.int32, device=dev)]

    a = outs()
    partials = torch.empty(n * splits * 4, dtype=torch.float32, device=dev)
    st = lib.vrl_rowscore_split(x.data_ptr(), code, n, V, V, lab.data_ptr(), tptr, a[0].data_ptr(), a[1].data_ptr(),
                                a[2].data_ptr(), a[3].data_ptr(), a[4].data_ptr(), splits, partials.data_ptr(), stream)
    assert st == _lib.VRL_OK, lib.vrl_strerror(st)
    b = outs()
    st = lib.vrl_rowscore_split_static(x.data_ptr(), code, n, V, V, lab.data_ptr(), tptr, b[0].data_ptr(),
                                       b[1].data_ptr(), b[2].data_ptr(), b[3].data_ptr(), b[4].data_ptr(), splits, stream)
    assert st == _lib.VRL_OK, lib.vrl_strerror(st)
    torch.cuda.synchronize(dev)
    for name, ta, tb in zip(("logprob", "entropy", "sum_pi_sq", "lse", "flag"), a, b):
        na, nb = ta.cpu().numpy(), tb.cpu().numpy()
        assert not np.isnan(nb.astype(np.float64)).any(), name
        assert np.array_equal(na.view(np.uint32) if na.dtype == np.float32 else na,
                              nb.view(np.uint32) if nb.dtype == np.float32 else nb), name
    # and it is the right answer, not merely the same one
    ref = torch.log_softmax(x.float() / (1.0 if temp is None else temp[:, None]), -1)
    want = ref.gather(-1, lab[:, None]).squeeze(-1)
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    assert (b[0] - want).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_matches_caller_scratch_on_two_calls_in_a_row(dev, dtype):
    lib = _lib.load()
    print(f"[no_alloc] dtype={dtype} call 1: 96 rows x 50257, 32 splits; call 2: 5 rows x 151936, 64 splits", flush=True)
    with torch.cuda.device(dev):
        _call_pair(lib, dev, 96, 50257, dtype, 32, seed=11, with_temperature=True)     # 3072 partials
        _call_pair(lib, dev, 5, 151936, dtype, 64, seed=12, with_temperature=False)    # 320 partials, smaller
        _call_pair(lib, dev, 128, 32000, dtype, 64, seed=13, with_temperature=False)   # exactly the maximum


def test_static_scratch_limits(dev):
    lib = _lib.load()
    with torch.cuda.device(dev):
        n, V = 129, 4096
        x = torch.zeros((n, V), dtype=torch.bfloat16, device=dev)
        lab = torch.zeros(n, dtype=torch.int64, device=dev)
        out = torch.full((n,), 7.0, dtype=torch.float32, device=dev)
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        args = (x.data_ptr(), _lib.VRL_BF16, n, V, V, lab.data_ptr(), None, out.data_ptr(), None, None, None,
                flag.data_ptr())
        # 129 x 64 partials do not fit: refused before anything is launched
        assert lib.vrl_rowscore_split_static(*args, 64, _lib.stream_ptr(dev)) == _lib.VRL_ERR_SCRATCH
        torch.cuda.synchronize(dev)
        assert torch.all(out == 7.0)
        assert "VRL_STATIC_PARTIALS_MAX" in lib.vrl_strerror(_lib.VRL_ERR_SCRATCH).decode()
        # one workgroup per row needs no scratch and takes any number of rows
        assert lib.vrl_rowscore_split_static(*args, 1, _lib.stream_ptr(dev)) == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert torch.allclose(out, torch.full_like(out, -float(np.log(V))), atol=1e-5)
