"""vrl_lmhead_score (LM head + scoring in one matrix-core kernel, no logits in memory) against torch.

The kernel keeps the logits in fp32, so the reference is the all-fp32 composition on the same bf16/fp16 operands
(products of 16-bit values are exact in fp32; only the summation order differs): 2e-5 absolute at these sizes.
Against the library-GEMM path (which rounds the logits to the operand type) the difference is that rounding."""

import pytest
import torch

from verl_amd import _lib
from verl_amd.fused_linear import fused_linear_for_ppo, lm_head_score_mfma

pytestmark = pytest.mark.gpu


def _reference(h, w, ids, temp):
    z = h.double() @ w.double().t()
    if temp is not None:
        z = z / (temp.double().clamp(min=1e-8)[:, None] if isinstance(temp, torch.Tensor) else float(temp))
    lse = torch.logsumexp(z, -1)
    lp = z.gather(-1, ids[:, None]).squeeze(-1) - lse
    ent = lse - (torch.softmax(z, -1) * z).sum(-1)
    return lp, ent


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,V,K,splits", [(256, 256, 64, 1), (256, 512, 128, 2), (512, 1024, 256, 3), (300, 700, 192, 2),
                                          (1000, 300, 64, 1), (257, 18992, 512, None), (2048, 4099, 320, None),
                                          (1024, 32000, 1024, 8)])
def test_matches_fp64_composition(dev, dtype, T, V, K, splits):
    g = torch.Generator(device=dev).manual_seed(T + V + K)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).to(dtype)
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    for t in (1.0, 0.7, temp):
        lp, ent = lm_head_score_mfma(h, w, ids, t, n_splits=splits)
        r_lp, r_ent = _reference(h, w, ids, None if t == 1.0 else t) if not isinstance(t, torch.Tensor) else _reference(h, w, ids, t)
        assert lp.dtype == torch.float32 and lp.shape == (T,)
        assert (lp.double() - r_lp).abs().max().item() <= 2e-5
        assert (ent.double() - r_ent).abs().max().item() <= 2e-5


def test_xcd_aware_workgroup_order_covers_every_token_block_and_split(dev):
    """32 token blocks x 8 splits takes the XCD-aware (token block, split) mapping of the workgroups (it needs the
    block count to divide by 8 and the split count by 4): every token of every block must come out right, which a
    wrong mapping (a block or split served twice, another never) would not."""
    T, V, K, splits = 8192, 8192, 256, 8
    g = torch.Generator(device=dev).manual_seed(99)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).bfloat16()
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    lp, ent = lm_head_score_mfma(h, w, ids, temp, n_splits=splits)
    r_lp, r_ent = _reference(h, w, ids, temp)
    assert (lp.double() - r_lp).abs().max().item() <= 2e-5
    assert (ent.double() - r_ent).abs().max().item() <= 2e-5


def test_benchmark_shape_against_the_chunked_fp64_composition(dev):
    """8192 tokens x 3584 -> 152064 bf16 (the shape bench.py --lm-head times; 594 vocabulary tiles over 8 splits,
    the last split shorter, XCD-aware order): all tokens against the fp64 composition, formed 256 tokens at a time."""
    T, K, V = 8192, 3584, 152064
    g = torch.Generator(device=dev).manual_seed(4000)
    h = torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = (torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g) * 0.05).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    lp, ent = lm_head_score_mfma(h, w, ids, 1.5)
    w64 = w.double()
    worst_lp = worst_ent = 0.0
    for lo in range(0, T, 256):
        r_lp, r_ent = _reference(h[lo:lo + 256], w64, ids[lo:lo + 256], 1.5)
        worst_lp = max(worst_lp, (lp[lo:lo + 256].double() - r_lp).abs().max().item())
        worst_ent = max(worst_ent, (ent[lo:lo + 256].double() - r_ent).abs().max().item())
    print(f"[lmhead 8192x3584->152064] max abs err vs fp64: log-prob {worst_lp:.2e}, entropy {worst_ent:.2e}", flush=True)
    assert worst_lp <= 2e-5 and worst_ent <= 2e-5


def test_close_to_the_library_path_and_3d_inputs(dev):
    g = torch.Generator(device=dev).manual_seed(4)
    B, S, K, V = 2, 260, 256, 5003
    h = torch.empty(B, S, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    ids = torch.randint(0, V, (B, S), generator=g, device=dev)
    lp, ent = lm_head_score_mfma(h, w, ids, 1.5)
    with torch.no_grad():
        lp2, ent2 = fused_linear_for_ppo(h, w, ids, 1.5)
    assert lp.shape == (B, S)
    # the other path rounds |logit| ~ 3 to bf16 (2^-8 relative) before the softmax
    assert (lp - lp2).abs().max().item() <= 3e-2 and (ent - ent2).abs().max().item() <= 3e-2


def test_special_values_and_errors(dev):
    g = torch.Generator(device=dev).manual_seed(6)
    T, V, K = 256, 512, 64
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).bfloat16()
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    bad = ids.clone()
    bad[7] = V
    with pytest.raises(IndexError):
        lm_head_score_mfma(h, w, bad)
    with pytest.raises(ValueError):
        lm_head_score_mfma(h[:100], w, ids[:100])                  # fewer than 256 tokens
    with pytest.raises(ValueError):
        lm_head_score_mfma(h[:, :32], w[:, :32], ids)              # hidden size not a multiple of 64
    with pytest.raises(TypeError):
        lm_head_score_mfma(h.float(), w.float(), ids)
    with pytest.raises(NotImplementedError):
        lm_head_score_mfma(h.clone().requires_grad_(), w, ids)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        lm_head_score_mfma(h.cpu(), w.cpu(), ids.cpu())
    # a token whose hidden state is zero: uniform distribution, log-prob -log V, entropy log V
    h0 = h.clone()
    h0[3] = 0
    lp, ent = lm_head_score_mfma(h0, w, ids)
    import math
    assert abs(lp[3].item() + math.log(V)) <= 1e-6 and abs(ent[3].item() - math.log(V)) <= 1e-6
    assert lib_plan_is_sane()


def lib_plan_is_sane():
    lib = _lib.load()
    return (lib.vrl_lmhead_plan(8192, 152064) == 8 and lib.vrl_lmhead_plan(256, 256) == 1
            and 1 <= lib.vrl_lmhead_plan(100000, 151936) <= 64 and lib.vrl_lmhead_plan(256, 151936) == 64)
