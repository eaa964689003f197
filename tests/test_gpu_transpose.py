"""vrl_transpose on the GPU: bit-exact against the definition out[c, r] = x[r, c] (numpy's transpose of the raw
words), over aligned and ragged shapes, strided operands, both element sizes, and the argument checks."""

import pytest
import torch

from verl_amd import _lib, layout
from oracle import scoring

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (1, 700), (700, 1), (128, 128), (64, 64), (127, 129), (129, 127), (256, 384), (1000, 777),
          (513, 1031), (2048, 3584), (3, 152064), (4099, 260)]


def _words(x):
    return x.view(torch.int16 if x.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int32, torch.int16])
@pytest.mark.parametrize("shape", SHAPES)
def test_matches_definition_bit_for_bit(dev, dtype, shape):
    g = torch.Generator(device=dev).manual_seed(shape[0] * 131 + shape[1])
    bits = torch.randint(-2**31, 2**31 - 1, shape, generator=g, device=dev, dtype=torch.int64)
    # every bit pattern, NaNs and denormals included: the kernel moves words, it must not touch them
    x = bits.to(torch.int32).view(torch.int32)
    x = (x if dtype in (torch.float32, torch.int32) else x.to(torch.int16)).view(dtype)
    got = layout.transpose_2d(x)
    assert got.shape == (shape[1], shape[0]) and got.is_contiguous() and got.dtype == dtype
    assert torch.equal(_words(got).cpu(), _words(scoring.transpose_2d(x.cpu())))
    # an involution
    assert torch.equal(_words(layout.transpose_2d(got)), _words(x))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_strided_source_and_destination(dev, dtype):
    g = torch.Generator(device=dev).manual_seed(3)
    base = torch.randn(300, 1000, generator=g, device=dev).to(dtype)
    for r0, r1, c0, c1 in [(0, 300, 0, 1000), (5, 261, 8, 520), (1, 130, 3, 131), (0, 128, 16, 144)]:
        x = base[r0:r1, c0:c1]                       # row pitch 1000, start possibly off the 16-byte grid
        ref = scoring.transpose_2d(x.cpu().contiguous())
        assert torch.equal(_words(layout.transpose_2d(x)).cpu(), _words(ref))
        big = torch.zeros(c1 - c0 + 2, r1 - r0 + 24, dtype=dtype, device=dev)
        out = big[1:-1, 8:8 + (r1 - r0)]             # a window of a wider array
        layout.transpose_2d(x, out=out)
        assert torch.equal(_words(out.contiguous()).cpu(), _words(ref))
        big[1:-1, 8:8 + (r1 - r0)] = 0
        assert not big.any()                          # nothing written outside the window


def test_empty_and_argument_errors(dev):
    lib = _lib.load()
    s = torch.cuda.current_stream(dev).cuda_stream
    assert layout.transpose_2d(torch.empty(0, 5, device=dev)).shape == (5, 0)
    assert layout.transpose_2d(torch.empty(5, 0, device=dev)).shape == (0, 5)
    x = torch.arange(12, dtype=torch.float32, device=dev).view(3, 4)
    y = torch.empty(4, 3, dtype=torch.float32, device=dev)
    assert lib.vrl_transpose(x.data_ptr(), 1, 3, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_ERR_DTYPE
    assert lib.vrl_transpose(x.data_ptr(), 8, 3, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_ERR_DTYPE
    assert lib.vrl_transpose(x.data_ptr(), 4, -1, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_ERR_SHAPE
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 4, 3, y.data_ptr(), 3, s) == _lib.VRL_ERR_SHAPE   # src pitch < cols
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 4, 4, y.data_ptr(), 2, s) == _lib.VRL_ERR_SHAPE   # dst pitch < rows
    assert lib.vrl_transpose(None, 4, 3, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_ERR_NULL
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 4, 4, None, 3, s) == _lib.VRL_ERR_NULL
    assert lib.vrl_transpose(x.data_ptr() + 2, 4, 2, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_ERR_ALIGN
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 4, 4, x.data_ptr(), 3, s) == _lib.VRL_ERR_ARG     # in place
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 2, 4, x.data_ptr() + 8, 4, s) == _lib.VRL_ERR_ARG  # overlapping
    assert lib.vrl_transpose(x.data_ptr(), 4, 3, 4, 4, y.data_ptr(), 3, s) == _lib.VRL_OK
    assert torch.equal(y, x.t())
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        layout.transpose_2d(torch.zeros(2, 2))
    with pytest.raises(ValueError):
        layout.transpose_2d(torch.zeros(2, 2, 2, device=dev))
    with pytest.raises(TypeError):
        layout.transpose_2d(torch.zeros(2, 2, dtype=torch.float64, device=dev))
    with pytest.raises(ValueError):
        layout.transpose_2d(x, out=torch.empty(3, 4, device=dev))
