"""Seeded synthetic inputs for the five benchmark/parity workloads.

Everything is generated with torch generators on the device that is asked for
(CPU or GPU), in row chunks, so the 20 GB bf16 logits of the 64x1024x152064
workload never need an fp32 copy. The old log-probs are "new log-probs plus
drift"; the caller supplies the new ones (from whichever implementation it is
exercising), this module only adds the drift.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    B: int  # sequences
    T: int  # padded response length
    V: int  # vocabulary
    dtype: torch.dtype
    sigma: float  # logits ~ N(0, sigma)
    boost: float = 0.0  # added to the label logit ...
    boost_frac: float = 0.0  # ... on this fraction of tokens
    temperature: Optional[float] = None
    lengths: Tuple = ("full",)  # ("full",) | ("uniform", lo, hi) | ("loguniform", lo, hi)
    drift: Tuple = ("normal", 0.1)  # ("normal", std) | ("student_t", nu, scale)
    lenience: float = 1.0
    micro_batch_tokens: Optional[int] = None  # rows scored per launch when the logits cannot all be resident

    @property
    def n_tokens(self) -> int:
        return self.B * self.T

    def scaled(self, **kw) -> "Workload":
        """The same recipe at another size (parity tests run small copies)."""
        return replace(self, **kw)


WORKLOADS = {
    # 8 seqs x 512, vocab 32000, fp32 N(0,2), lengths U[64,512], drift N(0,0.1), lenience 1
    "c1": Workload("c1_plumbing_8x512_v32000_f32", 8, 512, 32000, torch.float32, 2.0,
                   lengths=("uniform", 64, 512), drift=("normal", 0.1), lenience=1.0),
    # 64 x 1024, vocab 152064, bf16 N(0,3), label logit +8 on 70 % of tokens, drift N(0,0.05)
    "c2": Workload("c2_qwen7b_64x1024_v152064_bf16", 64, 1024, 152064, torch.bfloat16, 3.0,
                   boost=8.0, boost_frac=0.7, drift=("normal", 0.05), lenience=1.0),
    # 128 prompts x 8 samples x 2048, vocab 151936 bf16, micro-batches of 8192 tokens, lengths U[256,2048]
    "c3": Workload("c3_grpo_1024x2048_v151936_bf16", 1024, 2048, 151936, torch.bfloat16, 3.0,
                   lengths=("uniform", 256, 2048), drift=("normal", 0.2), lenience=math.exp(0.5),
                   micro_batch_tokens=8192),
    # 16 x 8192, vocab 128256, fp32 N(0,2.5), temperature 0.7 in-kernel
    "c4": Workload("c4_llama3_16x8192_v128256_f32_T0.7", 16, 8192, 128256, torch.float32, 2.5,
                   temperature=0.7, drift=("normal", 0.1), lenience=1.0),
    # 512 seqs, lengths log-uniform [32,16384], vocab 151936 bf16, Student-t drift
    "c5": Workload("c5_imbalance_512_loguniform_v151936_bf16", 512, 16384, 151936, torch.bfloat16, 3.0,
                   lengths=("loguniform", 32, 16384), drift=("student_t", 3.0, 0.3), lenience=math.exp(0.5),
                   micro_batch_tokens=8192),
}


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def draw_lengths(w: Workload, seed: int) -> torch.Tensor:
    """int64 (B,) response lengths, drawn on the CPU so they are the same for every device."""
    g = _gen("cpu", seed)
    kind = w.lengths[0]
    if kind == "full":
        return torch.full((w.B,), w.T, dtype=torch.int64)
    lo, hi = int(w.lengths[1]), int(w.lengths[2])
    lo, hi = min(lo, w.T), min(hi, w.T)
    if kind == "uniform":
        return torch.randint(lo, hi + 1, (w.B,), generator=g, dtype=torch.int64)
    if kind == "loguniform":
        u = torch.rand(w.B, generator=g, dtype=torch.float64)
        L = torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))
        return L.round().to(torch.int64).clamp(lo, hi)
    raise ValueError(f"unknown length recipe {w.lengths}")


def right_pad_mask(lengths: torch.Tensor, T: int, device) -> torch.Tensor:
    """bool (B, T), True on the first lengths[b] positions (verl's response_mask convention)."""
    pos = torch.arange(T, device=device).unsqueeze(0)
    return pos < lengths.to(device).unsqueeze(1)


def make_logits(n_rows: int, V: int, dtype: torch.dtype, sigma: float, labels: torch.Tensor, device, seed: int,
                boost: float = 0.0, boost_frac: float = 0.0, chunk_rows: int = 2048) -> torch.Tensor:
    """(n_rows, V) logits ~ N(0, sigma); on a ``boost_frac`` share of rows the label logit gets ``+boost``."""
    g = _gen(device, seed)
    out = torch.empty((n_rows, V), dtype=dtype, device=device)
    pick = None
    if boost != 0.0 and boost_frac > 0.0:
        pick = torch.rand(n_rows, generator=g, device=device) < boost_frac
    for lo in range(0, n_rows, chunk_rows):
        hi = min(lo + chunk_rows, n_rows)
        blk = torch.randn((hi - lo, V), generator=g, device=device, dtype=torch.float32) * sigma
        if pick is not None:
            rows = torch.nonzero(pick[lo:hi], as_tuple=False).squeeze(1)
            if rows.numel():
                cols = labels[lo:hi][rows]
                blk[rows, cols] += boost
        out[lo:hi] = blk.to(dtype)
    return out


def make_tokens(w: Workload, device, seed: int):
    """Per-token inputs of the padded (B, T) layout: dict(lengths, mask, labels, log_u, temperature)."""
    g = _gen(device, seed + 1)
    lengths = draw_lengths(w, seed + 2)
    mask = right_pad_mask(lengths, w.T, device)
    labels = torch.randint(0, w.V, (w.B, w.T), generator=g, device=device, dtype=torch.int64)
    u = torch.rand((w.B, w.T), generator=g, device=device, dtype=torch.float32)
    temperature = None
    if w.temperature is not None:
        temperature = torch.full((w.B, w.T), float(w.temperature), dtype=torch.float32, device=device)
    return {"lengths": lengths, "mask": mask, "labels": labels, "log_u": torch.log(u), "temperature": temperature}


def make_padded(w: Workload, device, seed: int):
    """make_tokens plus the (B, T, V) logits, for workloads whose logits fit in memory at once."""
    tok = make_tokens(w, device, seed)
    logits = make_logits(w.n_tokens, w.V, w.dtype, w.sigma, tok["labels"].reshape(-1), device, seed + 3,
                         boost=w.boost, boost_frac=w.boost_frac)
    tok["logits"] = logits.view(w.B, w.T, w.V)
    return tok


def drift_old_logprobs(logp_new: torch.Tensor, w: Workload, seed: int) -> torch.Tensor:
    """old = new + drift (fp32), drift ~ N(0, std) or scale * Student-t(nu)."""
    dev = logp_new.device
    g = _gen(dev, seed + 4)
    shape = tuple(logp_new.shape)
    kind = w.drift[0]
    if kind == "normal":
        noise = torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * float(w.drift[1])
    elif kind == "student_t":
        nu, scale = float(w.drift[1]), float(w.drift[2])
        z = torch.randn(shape, generator=g, device=dev, dtype=torch.float32)
        # chi-square(nu) as a sum of nu squared normals (nu is a small integer here)
        k = int(round(nu))
        chi2 = torch.randn((k, *shape), generator=g, device=dev, dtype=torch.float32).pow(2).sum(0)
        noise = scale * z / torch.sqrt(chi2 / nu)
    else:
        raise ValueError(f"unknown drift recipe {w.drift}")
    return logp_new.float() + noise


def pack_by_lengths(lengths: torch.Tensor):
    """cu_seqlens (B+1,) int64 for sequences laid end to end."""
    cu = torch.zeros(lengths.numel() + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(lengths.to(torch.int64), 0)
    return cu
