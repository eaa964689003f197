"""Writes tests/golden/*.npz: small seeded inputs with expected outputs.

The expected values come from this repository's own oracle (the fp64 C restatement for scores, the scalar
Python loops for verify), not from the reference package: it cannot be imported in the build container
(its torch_functional imports tensordict, which is absent) and every function on the path is pinned by
closed forms and library equivalence instead (tests/test_oracle_scoring.py, tests/test_oracle_verify.py).
Two fixtures restate data the reference's tests hold: the peaked row of
tests/utils/test_linear_cross_entropy.py:352-395 (closed form, computed here with math.*) and the
response-slice layout of tests/models/test_fsdp_no_padding_on_gpu.py:180-201.

Run from the repository root:  python tests/golden/make_golden.py
"""

import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import c_oracle, verify as ov  # noqa: E402


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.bfloat16().view(torch.int16).numpy().astype(np.uint16)


def scores():
    g = torch.Generator().manual_seed(20250101)
    n, V = 12, 2053  # odd vocab: rows are not 16-byte aligned
    x = torch.randn(n, V, generator=g) * 3
    lab = torch.randint(0, V, (n,), generator=g)
    temp = torch.rand(n, generator=g) * 1.2 + 0.4
    out = {"logits_f32": x.numpy(), "labels": lab.numpy(), "temperature": temp.numpy(), "logits_bf16_bits": bf16_bits(x)}
    for tag, xx in (("f32", x), ("bf16", x.bfloat16())):
        for ttag, t in (("", None), ("_T", temp)):
            lp, h = c_oracle.rowscore(xx, lab, t)
            out[f"logprob_{tag}{ttag}"] = lp
            out[f"entropy_{tag}{ttag}"] = h
    np.savez_compressed(os.path.join(HERE, "scores_12x2053.npz"), **out)


def peaked():
    # closed form for one logit a, the rest b (both exact in bf16)
    a, b = 3.0, -15.0
    rows = []
    for V in (152064, 149 * 1024):
        lse = math.log(math.exp(a) + (V - 1) * math.exp(b))
        ent = lse - (a * math.exp(a) + (V - 1) * b * math.exp(b)) / math.exp(lse)
        rows.append((V, a, b, a - lse, b - lse, ent))
    np.savez_compressed(os.path.join(HERE, "peaked_rows.npz"), rows=np.array(rows, dtype=np.float64))


def verify_cases():
    g = torch.Generator().manual_seed(77)
    B, T = 6, 150
    ln = -torch.rand(B, T, generator=g) * 5
    lo = ln + torch.randn(B, T, generator=g) * 0.3
    lu = torch.log(torch.rand(B, T, generator=g))
    lengths = torch.tensor([0, 1, 64, 65, 149, 150])
    mask = (torch.arange(T).unsqueeze(0) < lengths.unsqueeze(1))
    holes = mask & (torch.rand(B, T, generator=g) < 0.8)
    ids = torch.randint(0, 50000, (B, T), generator=g)
    out = {"logp_new": ln.numpy(), "logp_old": lo.numpy(), "log_u": lu.numpy(), "mask": mask.numpy().astype(np.uint8),
           "mask_holes": holes.numpy().astype(np.uint8), "draft_ids": ids.numpy()}
    for mtag, m in (("", mask), ("_holes", holes)):
        for otag, off in (("_m05", -0.5), ("_0", 0.0), ("_p05", 0.5)):
            r = ov.verify_loops(ln, lo, lu, m, off, draft_ids=ids, pad_id=-1)
            for k, v in r.items():
                out[f"{k}{mtag}{otag}"] = np.asarray(v)
    np.savez_compressed(os.path.join(HERE, "verify_6x150.npz"), **out)


if __name__ == "__main__":
    scores()
    peaked()
    verify_cases()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
