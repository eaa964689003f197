"""TEST INFRASTRUCTURE — CPU restatement of the reference's per-token scoring path.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this. Nothing under verl_amd/ does.

Each function restates one reference function with plain torch ops (torch is
the reference's own dependency; the arithmetic of this path lives there) and
cites the lines it follows. Shapes follow the reference: logits (..., V),
labels (...).

How each function is pinned (tests/test_oracle_scoring.py):
  logprobs_*      closed forms (uniform row: -log V; the reference's peaked-row
                  construction, tests/utils/test_linear_cross_entropy.py:352-395),
                  sum_v exp(logp_v) = 1 by brute force over every label, shift
                  invariance, fp64 scipy.special.log_softmax, the independent C
                  restatement oracle/vrl_oracle.c
  entropy_*       uniform: log V, one-hot: 0, peaked closed form, fp64
                  scipy.stats.entropy(softmax), chunked == unchunked, C restatement
  apply_temperature   per-element IEEE division against numpy float32
  sum_pi_squared  the reference's own parametrisation and extreme-value case
                  (tests/utils/test_torch_functional.py:126-150)
  response_slice  the reference's fixture tests/models/test_fsdp_no_padding_on_gpu.py:180-201
"""

from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

MIN_TEMPERATURE = 1e-8


def gather_from_labels(data: torch.Tensor, label: torch.Tensor) -> torch.Tensor:
    """data[..., label] per leading position. verl/utils/torch_functional.py:50-70."""
    return data.gather(-1, label.unsqueeze(-1)).squeeze(-1)


def logprobs_from_logits_naive(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Full log-softmax, then pick the label. verl/utils/torch_functional.py:155-170."""
    return gather_from_labels(F.log_softmax(logits, dim=-1), labels)


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Row-at-a-time variant. verl/utils/torch_functional.py:173-207.

    fp32/fp64 (:194-198): label logit minus a logsumexp taken separately for each
    entry along dim 0. Other dtypes (:199-206): per entry along dim 0, log-softmax
    in the input dtype and pick the label; the result keeps the input dtype.
    """
    if logits.dtype in (torch.float32, torch.float64):
        picked = gather_from_labels(logits, labels)
        lse = torch.stack([torch.logsumexp(row, dim=-1) for row in logits])
        return picked - lse
    out = []
    for row_logits, row_labels in zip(logits, labels, strict=True):
        out.append(gather_from_labels(F.log_softmax(row_logits, dim=-1), row_labels))
    return torch.stack(out)


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """Dispatcher, verl/utils/torch_functional.py:73-107, on a host without flash-attn
    and without torch_npu (:95-106): the v2 branch."""
    del inplace_backward
    return logprobs_from_logits_v2(logits, labels)


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """logsumexp - sum(softmax * logits). verl/utils/torch_functional.py:231-245."""
    p = F.softmax(logits, dim=-1)
    return torch.logsumexp(logits, dim=-1) - (p * logits).sum(dim=-1)


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048) -> torch.Tensor:
    """Same per chunk of rows, upcast to fp32, fp32 result. verl/utils/torch_functional.py:248-270."""
    n = logits.shape[0]
    out = torch.zeros(n, device=logits.device)
    for lo in range(0, n, chunk_size):
        chunk = logits[lo : lo + chunk_size].float()
        p = F.softmax(chunk, dim=-1)
        out[lo : lo + chunk_size] = torch.logsumexp(chunk, dim=-1) - (p * chunk).sum(dim=-1)
    return out


def apply_temperature(logits: torch.Tensor, temperature: torch.Tensor) -> torch.Tensor:
    """logits / clamp(temperature, 1e-8) with the temperature cast to the logits dtype.
    verl/workers/engine/fsdp/transformer_impl.py:1357 (temperature: one fp32 value per token, :1149-1163)."""
    return logits / temperature.clamp(min=MIN_TEMPERATURE).unsqueeze(-1).to(logits.dtype)


def calculate_sum_pi_squared_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """exp(logsumexp(2x) - 2 logsumexp(x)). verl/utils/torch_functional.py:690-704."""
    return torch.exp(torch.logsumexp(2.0 * logits, dim=-1) - 2.0 * torch.logsumexp(logits, dim=-1))


# ---- the composition the engine runs, and the parity targets ---------------

def score_reference(logits: torch.Tensor, labels: torch.Tensor, temperature: torch.Tensor | None = None):
    """(log-probs, entropy) exactly as the engine composes them, in the logits' own dtype:
    divide (:1357), entropy_from_logits (:1364-1376), logprobs_from_logits (:1395-1399) of
    verl/workers/engine/fsdp/transformer_impl.py."""
    z = logits if temperature is None else apply_temperature(logits, temperature)
    return logprobs_from_logits(z, labels), entropy_from_logits(z)


def score_fp32(logits: torch.Tensor, labels: torch.Tensor, temperature: torch.Tensor | None = None):
    """The same composition evaluated on ``logits.float()``: the parity target for bf16 inputs
    (fp32 accumulation), and identical to score_reference for fp32 inputs. The upcast is what the
    reference itself does at verl/utils/torch_functional.py:266 and
    verl/utils/experimental/torch_functional.py:35."""
    return score_reference(logits.float(), labels, temperature)


def score_fp64(logits: torch.Tensor, labels: torch.Tensor, temperature: torch.Tensor | None = None):
    """Ground truth in fp64 of what score_fp32 rounds: z = RN_fp32(x / T) is kept (it is the
    reference's input to the reductions), everything after it is fp64."""
    z = logits.float()
    if temperature is not None:
        z = apply_temperature(z, temperature)
    z = z.double()
    lse = torch.logsumexp(z, dim=-1)
    lp = gather_from_labels(z, labels) - lse
    p = torch.softmax(z, dim=-1)
    # p * z with p == 0 and z == -inf is NaN in the reference as well; keep it
    h = lse - (p * z).sum(dim=-1)
    return lp, h


# ---- layout helpers either side of the path ---------------------------------

def roll_labels(input_ids_rmpad: torch.Tensor) -> torch.Tensor:
    """labels = ids rolled left by one over the PACKED token axis.
    verl/workers/engine/fsdp/transformer_impl.py:1177."""
    return torch.roll(input_ids_rmpad, shifts=-1, dims=-1)


def expand_as_nested_values(per_sequence: torch.Tensor, offsets) -> torch.Tensor:
    """The per-token values of the reference's ``expand_as_nested(tensor, nested)``: entry b repeated over the
    tokens of sequence b (``torch.repeat_interleave(tensor, offsets.diff())``). This is how the engine builds
    ``temperature_rmpad``. verl/utils/torch_functional.py:989-1011; caller fsdp/transformer_impl.py:1158-1162."""
    offsets = torch.as_tensor(offsets, dtype=torch.int64)
    assert per_sequence.dim() == 1, "The ndim of tensor must be 1"                      # :1003
    assert per_sequence.shape[0] == offsets.numel() - 1, "The batch shape must be the same"   # :1000-1002
    return torch.repeat_interleave(per_sequence, offsets.diff(), dim=0)


def response_slice(values: torch.Tensor, prompt_lens, response_lens, max_response_len: int | None = None) -> torch.Tensor:
    """Packed per-token values (total_nnz, ...) -> (B, max_response_len, ...): for each sequence the
    rows [end - resp_len - 1, end - 1) (model output is shifted left by one token), right-padded
    with zeros. verl/workers/utils/padding.py:97-141."""
    prompt_lens = [int(p) for p in prompt_lens]
    response_lens = [int(r) for r in response_lens]
    if any(p == 0 for p in prompt_lens):
        raise AssertionError("prompt_len must be > 0 for the left shift")  # padding.py:130
    if max_response_len is None or max_response_len < 0:
        max_response_len = max(response_lens)
    ends = np.cumsum([p + r for p, r in zip(prompt_lens, response_lens)])
    if int(ends[-1]) != values.shape[0]:
        raise AssertionError("sequence lengths do not add up to total_nnz")  # padding.py:129
    rows = []
    trailing = (0, 0) * (values.dim() - 1)
    for r, end in zip(response_lens, ends):
        piece = values[int(end) - r - 1 : int(end) - 1]
        rows.append(F.pad(piece, (*trailing, 0, max_response_len - r)))
    return torch.stack(rows, dim=0)


def response_from_nested(values: torch.Tensor, seq_offsets, response_lens):
    """Packed model output -> packed response part: for each sequence values[end - resp_len - 1 : end - 1], joined.
    Returns (values, offsets) as the jagged tensor of verl/workers/utils/padding.py:194-210 holds them;
    ``seq_offsets`` are that function's ``tensor.offsets()`` (B+1 entries)."""
    response_lens = [int(r) for r in response_lens]
    ends = [int(e) for e in seq_offsets][1:]
    pieces = [values[end - r - 1 : end - 1] for r, end in zip(response_lens, ends, strict=True)]
    offsets = np.concatenate([[0], np.cumsum(response_lens)]).astype(np.int64)
    return (torch.cat(pieces) if pieces else values[:0]), torch.from_numpy(offsets)


def transpose_2d(x: torch.Tensor) -> torch.Tensor:
    """Transposed contiguous copy, element bits untouched. The definition itself fixes the result
    (out[c, r] = x[r, c]); numpy does the move, on the raw 16- or 32-bit patterns so that NaN payloads and
    signed zeros cannot be normalised on the way."""
    import numpy as np

    words = x.contiguous().view(torch.int16 if x.element_size() == 2 else torch.int32).cpu().numpy()
    return torch.from_numpy(np.ascontiguousarray(words.T)).view(x.dtype)
