"""TEST INFRASTRUCTURE — CPU/any-device restatement of the reference's fused LM head + scoring step.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this. Nothing under verl_amd/ does.

The reference computes, per chunk of tokens (verl/utils/experimental/torch_functional.py:27-81):
  forward   logits = (hidden @ W^T) / temperature, in fp32;  entropy = logsumexp - sum(softmax * logits);
            log-prob = log_softmax(logits)[label]                                             (:27-51)
  backward  dlogits = g_lp * (onehot - p) - g_h * p * (log p + entropy), cast to the operands' type, / temperature;
            d hidden = dlogits @ W;  d W = dlogits^T @ hidden                                   (:54-81)
and its Triton-backed twin (verl/utils/kernel/linear_cross_entropy.py:38-119) is held to the same torch composition
by the reference's own test (tests/utils/test_linear_cross_entropy.py:97-118 run_torch_entropy, :211-224).

`forward` / `backward` below restate those lines with plain torch ops in a dtype the caller picks (float64 gives the
value of the formula on the given operands; float32 is what the reference runs); `dlogits` is the closed form alone.
The temperature may be one value per token as well as a float (the engine's per-token temperature), clamped at 1e-8
like the scoring path.

How they are pinned (tests/test_oracle_fused_linear.py), each by something a plausible mistake fails:
  forward   a one-hot hidden state makes a token's logits a column of W: equal to oracle.scoring.score_fp64 on that column
            (a transposed weight or a wrong contraction axis fails); zero hidden states give log-prob -log V and entropy
            log V; the temperature divides the logits, not the result (closed form on a two-entry vocabulary)
  dlogits   sums to zero over the vocabulary for a pure log-prob gradient and for a pure entropy gradient (a dropped
            term or a wrong sign does not); equals fp64 autograd of `forward` on tiny shapes, temperature included;
            a uniform row has zero entropy gradient
  backward  d hidden and d W against fp64 autograd through `forward`, also with one of the two incoming gradients
            absent (a transposed product or a swapped operand fails on the non-square shapes used)
"""

from __future__ import annotations

from typing import Optional, Union

import torch

MIN_TEMPERATURE = 1e-8

Temperature = Union[None, float, torch.Tensor]


def _scaled(z: torch.Tensor, temperature: Temperature) -> torch.Tensor:
    if temperature is None:
        return z
    if isinstance(temperature, torch.Tensor):
        return z / temperature.to(z.dtype).clamp(min=MIN_TEMPERATURE).reshape(-1, 1)
    return z / float(temperature)


def logits_of(hidden: torch.Tensor, weight: torch.Tensor, temperature: Temperature = None,
              dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """(hidden @ weight^T) / temperature, products and sums in `dtype`. verl/utils/experimental/torch_functional.py:33-35."""
    return _scaled(hidden.to(dtype) @ weight.to(dtype).t(), temperature)


def forward(hidden: torch.Tensor, weight: torch.Tensor, input_ids: torch.Tensor, temperature: Temperature = None,
            dtype: torch.dtype = torch.float64):
    """(log-probs, entropy, logsumexp) per token. verl/utils/experimental/torch_functional.py:27-51."""
    z = logits_of(hidden, weight, temperature, dtype)
    lse = torch.logsumexp(z, dim=-1)
    entropy = lse - torch.sum(torch.softmax(z, dim=-1) * z, dim=-1)
    logprob = torch.log_softmax(z, dim=-1).gather(-1, input_ids.reshape(-1, 1)).squeeze(-1)
    return logprob, entropy, lse


def dlogits(logits: torch.Tensor, input_ids: torch.Tensor, g_logprob: Optional[torch.Tensor],
            g_entropy: Optional[torch.Tensor], temperature: Temperature = None) -> torch.Tensor:
    """Gradient with respect to the UNSCALED logits (hidden @ W^T) given the scaled ones, `logits`:
    (g_lp * (onehot - p) - g_h * p * (log p + H)) / temperature. verl/utils/experimental/torch_functional.py:66-78."""
    p = torch.softmax(logits, dim=-1)
    d = torch.zeros_like(logits)
    if g_logprob is not None:
        onehot = torch.zeros_like(logits).scatter_(-1, input_ids.reshape(-1, 1), 1)
        d = d + g_logprob.to(logits.dtype).reshape(-1, 1) * (onehot - p)
    if g_entropy is not None:
        logp = torch.log_softmax(logits, dim=-1)
        entropy = torch.logsumexp(logits, dim=-1) - torch.sum(p * logits, dim=-1)
        d = d + p * (logp + entropy.reshape(-1, 1)) * (-g_entropy.to(logits.dtype).reshape(-1, 1))
    return _scaled(d, temperature)


def backward(hidden: torch.Tensor, weight: torch.Tensor, input_ids: torch.Tensor, g_logprob: Optional[torch.Tensor],
             g_entropy: Optional[torch.Tensor], temperature: Temperature = None, dtype: torch.dtype = torch.float64):
    """(d hidden, d weight) in `dtype`. verl/utils/experimental/torch_functional.py:54-81 (the reference rounds dlogits
    to the operands' type before the two products, :78; with `dtype` float64 nothing is rounded)."""
    z = logits_of(hidden, weight, temperature, dtype)
    d = dlogits(z, input_ids, g_logprob, g_entropy, temperature)
    return d @ weight.to(dtype), d.t() @ hidden.to(dtype)


def autograd_backward(hidden: torch.Tensor, weight: torch.Tensor, input_ids: torch.Tensor,
                      g_logprob: Optional[torch.Tensor], g_entropy: Optional[torch.Tensor],
                      temperature: Temperature = None, dtype: torch.dtype = torch.float64):
    """The same two gradients from torch autograd through `forward`: what pins `backward` and `dlogits`."""
    h = hidden.detach().to(dtype).requires_grad_(True)
    w = weight.detach().to(dtype).requires_grad_(True)
    lp, ent, _ = forward(h, w, input_ids, temperature, dtype)
    loss = torch.zeros((), dtype=dtype, device=h.device)
    if g_logprob is not None:
        loss = loss + (lp * g_logprob.to(dtype)).sum()
    if g_entropy is not None:
        loss = loss + (ent * g_entropy.to(dtype)).sum()
    return torch.autograd.grad(loss, (h, w))
