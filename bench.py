#!/usr/bin/env python3
"""Benchmark of the fused score + SPEC-RL verify path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c1|c5]
    python bench.py --backward [--workload ...]          (the row op's backward kernel)
    python bench.py --lm-head [--chunk N] [--keep-logits auto|yes|no]  (LM head + scoring, forward + backward)
    python bench.py --score-responses                     (packed logits -> (B, T) blocks in one launch, and its backward)
    python bench.py --ceilings                            (plain read / copy of the same buffers, matrix-core probe)

One step = one pass of vrl_fused_score_verify (row kernel + verify kernel, through
the C ABI, outputs preallocated) over the whole synthetic batch, logits resident
in HBM. Prints one JSON line: whole-job verified tokens/s, the HBM roofline of
the row kernel (algorithmic bytes / average kernel time: launches back to back
between one HIP event pair on the launch stream), and the same computation in torch on the host cores (bounded sample).
With no workload option the line also carries short records of every other workload under "workloads".
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import torch

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

import bench_probes  # noqa: E402  (measurement aids only: the read / copy / matrix-core ceilings)
from verl_amd import _lib, synthetic  # noqa: E402
from verl_amd import spec_rl as sv  # noqa: E402
from verl_amd import torch_functional as vf  # noqa: E402

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM bytes per row-kernel launch measured with rocprofv3 (--pmc FETCH_SIZE and --pmc WRITE_SIZE, one run each,
# both scaled by what the same counter reads for a plain 1 GiB device copy: x1.999956 and x1.0). The workload
# shapes are fixed, so the figure is a property of (kernel, shape); the counter summary is kept under profiles/.
MEASURED_TRAFFIC_BYTES = {"c1": 525600443, "c2": 19943644231, "c3": 2490946810, "c4": 67292547122}
METRIC = "verified tokens/sec + achieved HBM GB/s (% of peak), vocab 152k bf16, 1 GPU"


SPINUP_MS = 150.0
RING_MIN_BYTES = 2 << 30


def spin_up(fn, ms: float = SPINUP_MS):
    """Untimed: keep the GPU busy with the step itself until its clocks have left the idle state.
    The first ~20 ms of work after idle run ~12 % slower on this part (measured from C++ as well), which would
    otherwise land in the timed region of the short workloads (c1, c3, c5)."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def batch_time_ms(fn, launches: int, batches: int = 5):
    """Average time of one call of `fn` in ms: `launches` calls back to back between one pair of HIP events on the
    launch stream, the median over `batches` such batches. For kernels of a few microseconds an event pair per launch
    measures the events."""
    times = []
    for _ in range(batches):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(launches):
            fn()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) / launches)
    return statistics.median(times)


def algorithmic_bytes_per_token(V: int, esize: int, with_temperature: bool, with_verify: bool) -> int:
    """Logits once + label (8) + log-prob out (4) + entropy out (4) [+ temperature (4)];
    verify adds old log-prob (4), log u (4), mask (1), accept out (1)."""
    b = V * esize + 8 + 4 + 4 + (4 if with_temperature else 0)
    if with_verify:
        b += 4 + 4 + 1 + 1
    return b


class Step:
    """Preallocated buffers and the raw ABI calls for one workload.

    Workloads whose logits fit in HBM at once (c1, c2, c4) are one padded (B, T) batch. A workload with
    ``micro_batch_tokens`` (c3) is scored the way verl feeds it after padding removal: whole sequences packed
    end to end until the token budget is full (the last one cut to fit), so every row is a valid token.
    """

    def __init__(self, w: synthetic.Workload, dev, seed: int):
        self.dev = dev
        if w.micro_batch_tokens is None:
            d = synthetic.make_padded(w, dev, seed)
            self.logits = d["logits"].view(-1, w.V)
            self.labels = d["labels"].view(-1).contiguous()
            self.mask8 = d["mask"].contiguous().view(torch.uint8).view(-1)
            self.log_u = d["log_u"].contiguous().view(-1)
            self.temp = None if d["temperature"] is None else d["temperature"].view(-1).contiguous()
            self.B, self.T, self.cu = w.B, w.T, None
            self.layout = f"padded {w.B}x{w.T}"
        else:
            budget = int(w.micro_batch_tokens)
            lengths = synthetic.draw_lengths(w, seed + 2).tolist()
            picked, total = [], 0
            for L in lengths:
                take = min(L, budget - total)
                picked.append(take)
                total += take
                if total == budget:
                    break
            cu = synthetic.pack_by_lengths(torch.tensor(picked))
            g = torch.Generator(device=dev).manual_seed(seed + 1)
            self.labels = torch.randint(0, w.V, (total,), generator=g, device=dev, dtype=torch.int64)
            self.log_u = torch.log(torch.rand(total, generator=g, device=dev, dtype=torch.float32))
            self.logits = synthetic.make_logits(total, w.V, w.dtype, w.sigma, self.labels, dev, seed + 3,
                                                boost=w.boost, boost_frac=w.boost_frac)
            self.mask8 = torch.ones(total, dtype=torch.uint8, device=dev)
            self.temp = None if w.temperature is None else torch.full((total,), float(w.temperature), device=dev)
            self.B, self.T, self.cu = len(picked), 0, cu.to(dev)
            self.layout = f"packed {len(picked)} sequences, {total} tokens"
        self.w = w
        self.n = self.logits.shape[0]
        # A batch smaller than a few times the 256 MB last-level cache (c1: 524 MB) is timed over a ring of
        # distinct copies, so that no launch finds its rows still cached from the launch before.
        nbytes = self.logits.numel() * self.logits.element_size()
        copies = 1 if nbytes >= RING_MIN_BYTES else min(8, -(-RING_MIN_BYTES // nbytes))
        self.ring = [self.logits] + [self.logits.clone() for _ in range(copies - 1)]
        self.turn = 0
        self.n_valid = int(self.mask8.sum().item())
        self.off = sv.thresh_offset_from_lenience(w.lenience)
        f32 = dict(dtype=torch.float32, device=dev)
        self.lp = torch.empty(self.n, **f32)
        self.h = torch.empty(self.n, **f32)
        self.flag = torch.zeros(1, dtype=torch.int32, device=dev)
        self.accept = torch.empty(self.n, dtype=torch.uint8, device=dev)
        self.first = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.prefix = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.near = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.ids = self.labels
        self.out_ids = torch.empty_like(self.ids)
        self.out_mask = torch.empty(self.n, dtype=torch.uint8, device=dev)
        self.lib = _lib.load()
        self.dt = _lib.VRL_BF16 if w.dtype == torch.bfloat16 else _lib.VRL_F32
        self.stream = torch.cuda.current_stream(dev).cuda_stream
        # old log-probs = new (from the kernel) + drift
        self.score()
        torch.cuda.synchronize()
        self.lp_old = synthetic.drift_old_logprobs(self.lp, w, seed).contiguous()

    def _tp(self):
        return None if self.temp is None else self.temp.data_ptr()

    def score(self):
        logits = self.ring[self.turn]
        self.turn = (self.turn + 1) % len(self.ring)
        st = self.lib.vrl_rowscore(logits.data_ptr(), self.dt, self.n, self.w.V, self.logits.stride(0),
                                   self.labels.data_ptr(), self._tp(), self.lp.data_ptr(), self.h.data_ptr(), None,
                                   None, self.flag.data_ptr(), self.stream)
        _lib.check("vrl_rowscore", st)

    def fused(self):
        logits = self.ring[self.turn]
        self.turn = (self.turn + 1) % len(self.ring)
        st = self.lib.vrl_fused_score_verify(
            logits.data_ptr(), self.dt, self.n, self.w.V, self.logits.stride(0), self.labels.data_ptr(),
            self._tp(), self.lp.data_ptr(), self.h.data_ptr(), None, None, self.flag.data_ptr(),
            self.lp_old.data_ptr(), self.log_u.data_ptr(), self.mask8.data_ptr(),
            None if self.cu is None else self.cu.data_ptr(), self.B, self.T,
            self.off, 1e-6, self.accept.data_ptr(), self.first.data_ptr(), self.prefix.data_ptr(),
            self.near.data_ptr(), self.ids.data_ptr(), 0, self.out_ids.data_ptr(), self.out_mask.data_ptr(),
            self.stream)
        _lib.check("vrl_fused_score_verify", st)

    def check_against_torch(self, rows: int = 1024):
        """Guard, not timed: the first rows against torch on the GPU, in fp32 (what verl computes there) and in
        fp64 (the value of the same formula on the same fp32 inputs). Returns a record with the maximum
        distances and the number of rows whose distance from torch's fp32 result exceeds the plain bar
        (1e-5 for fp32 logits, 2e-3 for 16-bit ones): torch's own fp32 entropy is up to ~1.3e-5 from the fp64
        value at V ~ 128k, so a kernel that is closer to the fp64 value than torch can still sit outside 1e-5
        of torch on a few rows; the record shows how many."""
        z = self.logits[:rows].float()
        if self.temp is not None:
            z = z / self.temp[:rows].clamp(min=1e-8).unsqueeze(-1)
        lab = self.labels[:rows, None]
        lse = torch.logsumexp(z, -1)
        ref_lp = z.gather(-1, lab).squeeze(-1) - lse
        ref_h = lse - (torch.softmax(z, -1) * z).sum(-1)
        z64 = z.double()
        lse64 = torch.logsumexp(z64, -1)
        t_lp = z64.gather(-1, lab).squeeze(-1) - lse64
        t_h = lse64 - (torch.softmax(z64, -1) * z64).sum(-1)
        del z64
        lp, h = self.lp[:rows].double(), self.h[:rows].double()
        tol = 1e-5 if self.w.dtype == torch.float32 else 2e-3
        rec = {
            "rows": rows,
            "tolerance": tol,
            "max_abs_err_logprob": (lp - ref_lp).abs().max().item(),
            "max_abs_err_entropy": (h - ref_h).abs().max().item(),
            "max_abs_err_logprob_vs_fp64": (lp - t_lp).abs().max().item(),
            "max_abs_err_entropy_vs_fp64": (h - t_h).abs().max().item(),
            "torch_fp32_own_err_logprob": (ref_lp.double() - t_lp).abs().max().item(),
            "torch_fp32_own_err_entropy": (ref_h.double() - t_h).abs().max().item(),
            "rows_over_plain_tol_logprob": int(((lp - ref_lp).abs() > tol).sum().item()),
            "rows_over_plain_tol_entropy": int(((h - ref_h).abs() > tol).sum().item()),
        }
        # A coarse guard, not the parity test (tests/_parity.py is): 4e-6 of the fp64 value, and the bar widened
        # per row only by torch's own distance from the fp64 value.
        ok = (rec["max_abs_err_logprob_vs_fp64"] <= 4e-6 and rec["max_abs_err_entropy_vs_fp64"] <= 4e-6
              and bool(((lp - ref_lp).abs() <= tol + (ref_lp.double() - t_lp).abs()).all())
              and bool(((h - ref_h).abs() <= tol + (ref_h.double() - t_h).abs()).all()))
        if not ok:
            raise SystemExit(f"bench: kernel disagrees with torch: {rec}")
        if int(self.flag.item()) != 0:
            raise SystemExit("bench: an error flag is set after the guard run")
        return rec


# HBM bytes per launch of rowscore_backward_flat_kernel from rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE; same scaling as above).
MEASURED_BACKWARD_TRAFFIC_BYTES = {"c3": 4981856312}   # profiles/rowscore_backward_kernels_hbm_counters_c3.md
# profiles/score_responses_kernel_hbm_counters_c3_packed.md (forward, backward), for the packed micro-batch bench_score_responses builds
MEASURED_SCORE_RESPONSES_TRAFFIC_BYTES = (1676672404, 4167119102)


def bench_backward(args, dev, workload=None):
    """Throughput of vrl_rowscore_backward (gradient of log-prob and entropy with respect to the logits) on the
    workload's rows: reads the logits once, writes the gradient once (2 * V * sizeof + per-row scalars)."""
    workload = workload or args.workload
    w = synthetic.WORKLOADS[workload]
    step = Step(w, dev, seed=1000 * int(workload[1]))
    lse = torch.empty(step.n, dtype=torch.float32, device=dev)
    st = step.lib.vrl_rowscore(step.logits.data_ptr(), step.dt, step.n, w.V, step.logits.stride(0), step.labels.data_ptr(),
                               step._tp(), step.lp.data_ptr(), step.h.data_ptr(), None, lse.data_ptr(),
                               step.flag.data_ptr(), step.stream)
    _lib.check("vrl_rowscore", st)
    g = torch.Generator(device=dev).manual_seed(99)
    gl = torch.randn(step.n, generator=g, device=dev)
    gh = torch.randn(step.n, generator=g, device=dev) * 0.01
    dx = torch.empty_like(step.logits)

    def run():
        st = step.lib.vrl_rowscore_backward(step.logits.data_ptr(), step.dt, step.n, w.V, step.logits.stride(0),
                                            step.labels.data_ptr(), step._tp(), lse.data_ptr(), step.h.data_ptr(),
                                            gl.data_ptr(), gh.data_ptr(), dx.data_ptr(), dx.stride(0), step.stream)
        _lib.check("vrl_rowscore_backward", st)

    if args.copy_calibration:
        copy_calibration(dev)
    # guard: first rows against torch autograd in fp32
    run()
    rows = 256
    xr = step.logits[:rows].float().requires_grad_(True)
    z = xr if step.temp is None else xr / step.temp[:rows].clamp(min=1e-8).unsqueeze(-1)
    lsm = torch.log_softmax(z, -1)
    lpr = lsm.gather(-1, step.labels[:rows, None]).squeeze(-1)
    hr = -(lsm.exp() * lsm).sum(-1)
    ((lpr * gl[:rows]).sum() + (hr * gh[:rows]).sum()).backward()
    err = (dx[:rows].float() - xr.grad).abs()
    tol = xr.grad.abs() * (2.0 ** -7 if w.dtype == torch.bfloat16 else 0.0) + 2e-5
    if not bool((err <= tol).all()):
        raise SystemExit(f"bench: backward disagrees with torch autograd (max abs err {err.max().item()})")
    spin_up(run)
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    avg_ms = batch_time_ms(run, args.steps, 3)
    esize = 2 if w.dtype == torch.bfloat16 else 4
    bytes_launch = step.n * (2 * w.V * esize + 8 + 4 + 4 + 4 + 4 + (4 if step.temp is not None else 0))
    achieved = bytes_launch / (avg_ms * 1e-3) / 1e9
    return {
        "metric": "tokens/sec of the backward of the row op + achieved HBM GB/s", "value": step.n * args.steps / wall,
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3 / args.steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": w.name, "layout": step.layout, "rows_per_step": step.n, "vocab": w.V,
                   "step": "vrl_rowscore_backward through the C ABI (gradients of log-prob and entropy)"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_BACKWARD_TRAFFIC_BYTES.get(workload),
                     "kernel": "rowscore_backward_flat_kernel", "avg_kernel_ms": avg_ms,
                     "algorithmic_bytes_per_launch": bytes_launch},
    }


VERIFY_RING_BYTES = 3 * (256 << 20)   # three times the 256 MB last-level cache


class VerifyOnlyStep:
    """c5: 512 sequences with log-uniform lengths in [32, 16384], packed; only the verify kernel is timed
    (its logits would be 408 GB, scored in 8192-token micro-batches like c3). One set of per-token arrays is 30 bytes
    per token (44 MB), which the 256 MB last-level cache would hold from one launch to the next, so the launches walk a
    ring of identical sets that is three times that cache: every launch finds its inputs in HBM."""

    def __init__(self, w: synthetic.Workload, dev, seed: int, two_pass=None, lengths=None):
        self.w, self.dev = w, dev
        lengths = synthetic.draw_lengths(w, seed + 2) if lengths is None else torch.tensor(lengths)
        self.cu = synthetic.pack_by_lengths(lengths).to(dev)
        self.B = lengths.numel()
        self.n = int(lengths.sum())
        self.n_valid = self.n
        self.layout = f"packed {self.B} sequences, {self.n} tokens (verify only)"
        g = torch.Generator(device=dev).manual_seed(seed + 1)
        lp = -torch.rand(self.n, generator=g, device=dev) * 6
        lp_old = synthetic.drift_old_logprobs(lp, w, seed).contiguous()
        log_u = torch.log(torch.rand(self.n, generator=g, device=dev))
        ids = torch.randint(0, w.V, (self.n,), generator=g, device=dev)
        self.off = sv.thresh_offset_from_lenience(w.lenience)
        self.bytes_per_set = self.n * (4 + 4 + 4 + 8 + 1 + 8 + 1)
        copies = min(32, max(2, -(-VERIFY_RING_BYTES // self.bytes_per_set)))
        self.ring = []
        for i in range(copies):
            # (copies made by an elementwise kernel: a device-to-device memcpy does not survive counter collection)
            src = (lp, lp_old, log_u, ids) if i == 0 else tuple(t.add(0) for t in (lp, lp_old, log_u, ids))
            self.ring.append(src + (torch.empty(self.n, dtype=torch.uint8, device=dev), torch.empty_like(ids),
                                    torch.empty(self.n, dtype=torch.uint8, device=dev)))
        self.lp, self.lp_old, self.log_u, self.ids, self.accept, self.out_ids, self.out_mask = self.ring[0]
        self.turn = 0
        self.first = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.prefix = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.near = torch.empty(self.B, dtype=torch.int32, device=dev)
        self.flag = torch.zeros(1, dtype=torch.int32, device=dev)
        self.lib = _lib.load()
        self.stream = torch.cuda.current_stream(dev).cuda_stream
        # the form the library plans for this shape: two flat passes with half a byte per token of scratch
        self.two_pass = bool(self.lib.vrl_spec_verify_plan(1, self.B, 0, self.n)) if two_pass is None else bool(two_pass)
        self.work = (torch.empty(int(self.lib.vrl_spec_verify_workspace(self.n)), dtype=torch.uint8, device=dev)
                     if self.two_pass else None)

    def verify(self):
        lp, lp_old, log_u, ids, accept, out_ids, out_mask = self.ring[self.turn]
        self.turn = (self.turn + 1) % len(self.ring)
        st = self.lib.vrl_spec_verify(
            lp.data_ptr(), lp_old.data_ptr(), log_u.data_ptr(), None, self.cu.data_ptr(), self.B, 0,
            self.n, self.off, 1e-6, accept.data_ptr(), self.first.data_ptr(), self.prefix.data_ptr(),
            self.near.data_ptr(), ids.data_ptr(), 0, out_ids.data_ptr(), out_mask.data_ptr(),
            self.flag.data_ptr(), None if self.work is None else self.work.data_ptr(),
            0 if self.work is None else self.work.numel(), self.stream)
        _lib.check("vrl_spec_verify", st)


# HBM bytes per call of the two verify kernels at c5 from rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE; same scaling as above),
# profiles/verify_two_pass_kernels_c5_trace_and_hbm_counters.md: 17.63 + 2.23 MB (verify_tokens_kernel) and 1.24 + 13.13 MB
# (verify_finish_kernel); the 0.73 MB of ballot words are written once and read once on top of the algorithmic bytes.
MEASURED_VERIFY_TRAFFIC_BYTES = {"two-pass": 34229825}


def bench_verify_only(args, dev, with_cpu_baseline=True):
    """tokens/s of vrl_spec_verify alone on the c5 workload. Algorithmic bytes per token: 4+4+4 in (new and old
    log-probs, log u), 1 out (accept), and for the truncated draft 8+1 out = 22 B/token, plus 8 in for every token
    before its sequence's cut (a draft id is only read where it is kept) and 20 B per sequence."""
    w = synthetic.WORKLOADS["c5"]
    def note(msg):
        print(f"[bench c5] {msg}", file=sys.stderr, flush=True)

    step = VerifyOnlyStep(w, dev, seed=5000, two_pass={"auto": None, "two-pass": True, "per-sequence": False}[args.verify_form])
    note(f"{len(step.ring)} array sets built")
    # guard: the first set's results against the vectorised statement of the rule, bit for bit
    step.verify()
    torch.cuda.synchronize()
    from oracle import verify as overify  # checker / baseline only

    if not args.no_guard:
        ref = overify.verify(step.lp.cpu(), step.lp_old.cpu(), step.log_u.cpu(), None, step.off, cu_seqlens=step.cu.cpu(),
                             draft_ids=step.ids.cpu())
        same = (torch.equal(step.accept.cpu(), ref["accept"].to(torch.uint8)) and
                torch.equal(step.first.cpu(), ref["first_reject"].to(torch.int32)) and
                torch.equal(step.prefix.cpu(), ref["prefix_len"].to(torch.int32)) and
                torch.equal(step.out_ids.cpu(), ref["out_ids"]) and
                torch.equal(step.out_mask.cpu(), ref["out_mask"].to(torch.uint8)))
        if not same or int(step.flag.item()) != 0:
            raise SystemExit("bench: vrl_spec_verify disagrees with the oracle on c5")
    note("guard done")
    spin_up(step.verify)
    for _ in range(args.warmup):
        step.verify()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step.verify()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    launches = max(args.steps, len(step.ring) * 4)
    avg_ms = batch_time_ms(step.verify, launches)
    note("timed")
    if args.copy_calibration:
        copy_calibration(dev)
        note("copy calibration done")
    # what the same call costs when it moves next to nothing (8 packed sequences of 512 tokens): the launches themselves
    tiny = VerifyOnlyStep(w.scaled(name="c5_tiny", B=8, T=512), dev, seed=5100, two_pass=step.two_pass, lengths=[512] * 8)
    spin_up(tiny.verify, 30.0)
    floor_ms = batch_time_ms(tiny.verify, launches)
    kept = int(step.first.sum().item())   # no mask here: the tokens before a sequence's first rejection are the kept ones
    bytes_launch = step.n * (4 + 4 + 4 + 1 + 8 + 1) + kept * 8 + step.B * (12 + 8)
    achieved = bytes_launch / (avg_ms * 1e-3) / 1e9
    out = {
        "metric": METRIC, "value": step.n * args.steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall * 1e3 / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w.name, "layout": step.layout, "launches_per_step": 1, "tokens_per_step": step.n,
                   "lenience": w.lenience, "array_sets_rotated": len(step.ring),
                   "launches_per_call": 2 if step.two_pass else 1,
                   "step": "vrl_spec_verify with truncated draft, through the C ABI"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MEASURED_VERIFY_TRAFFIC_BYTES.get("two-pass" if step.two_pass else "per-sequence"),
                     "kernel": "verify_tokens_kernel + verify_finish_kernel" if step.two_pass else "spec_verify_kernel",
                     "avg_kernel_ms": avg_ms, "algorithmic_bytes_per_launch": bytes_launch,
                     "timing": f"{launches} launches back to back between one HIP event pair, median of 5 batches",
                     "launch_floor_ms": floor_ms,
                     "achieved_net_of_launch_floor": bytes_launch / max((avg_ms - floor_ms) * 1e-3, 1e-9) / 1e9,
                     "launch_floor": "the same call on 8 packed sequences of 512 tokens (0.1 MB): what the launches cost "
                                     "before any byte moves"},
        "parity_guard": "skipped (--no-guard)" if args.no_guard else
                        "accept, first_reject, prefix_len and the truncated draft equal to the oracle, bit for bit",
    }
    if with_cpu_baseline:
        ln, lo, lu, ids, cu = step.lp.cpu(), step.lp_old.cpu(), step.log_u.cpu(), step.ids.cpu(), step.cu.cpu()
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            overify.verify(ln, lo, lu, None, step.off, cu_seqlens=cu, draft_ids=ids)
            times.append(time.perf_counter() - t0)
        out["cpu_baseline"] = {"value": step.n / statistics.median(times), "unit": "tokens/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the whole workload ({step.n} tokens), median of 3 runs of the vectorised torch statement of the rule"}
    return out


def bench_lm_head(args, dev):
    """LM head + scoring without the full logits (verl_amd.fused_linear) at c3's micro-batch: 8192 tokens, hidden
    3584 (Qwen2.5-7B), vocab 152064 bf16, temperature 1.5; forward and forward + backward. The step is bound by the
    library GEMMs, so the roofline object is the bf16 matrix peak over the algorithmic flops (2*T*D*V forward,
    4*T*D*V backward; the second projection of the backward is not algorithmic)."""
    from verl_amd.fused_linear import fused_linear_for_ppo
    from verl_amd.layout import transpose_2d

    T, D, V = 8192, 3584, 152064
    g = torch.Generator(device=dev).manual_seed(4000)
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = (torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g) * 0.05).bfloat16().requires_grad_()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    g_lp = torch.randn(T, generator=g, device=dev)
    g_h = torch.randn(T, generator=g, device=dev) * 0.01
    temperature, chunk = 1.5, args.chunk
    keep = {"auto": None, "yes": True, "no": False}[args.keep_logits]

    def fwd():
        with torch.no_grad():
            return fused_linear_for_ppo(hidden, weight, ids, temperature, chunk)

    def fwd_library():
        with torch.no_grad():
            return fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, False, "library")

    def fwd_bwd():
        lp, h = fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, keep)
        return torch.autograd.grad((lp, h), (hidden, weight), (g_lp, g_h))

    if args.own_only:
        # for a kernel trace of the default call alone: nothing but the package's own path runs
        spin_up(fwd_bwd, 300.0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fwd_bwd()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        return {"metric": "tokens/sec of LM head + scoring, forward + backward", "value": T / ms * 1e3, "unit": "tokens/s",
                "ms_per_step": ms, "steps": args.steps, "dtype": "bf16",
                "config": {"workload": "lm_head_8192x3584_v152064_bf16", "keep_logits": args.keep_logits,
                           "chunk_tokens": chunk, "step": "fused_linear_for_ppo forward + backward, default kernels only"}}

    # guard: first tokens of the library forward against torch in fp32 on the bf16 logits the same GEMM produces
    lp, h = fwd_library()
    z = torch.matmul(hidden[:256].detach(), weight.detach().t()).float() / temperature
    e1 = (lp[:256] - torch.log_softmax(z, -1).gather(-1, ids[:256, None]).squeeze(-1)).abs().max().item()
    e2 = (h[:256] - (torch.logsumexp(z, -1) - (torch.softmax(z, -1) * z).sum(-1))).abs().max().item()
    if not (e1 <= 2e-3 and e2 <= 2e-3):
        raise SystemExit(f"bench: LM-head scores disagree with torch (logprob {e1}, entropy {e2})")

    def timed(fn):
        spin_up(fn, 300.0)
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps

    from verl_amd.fused_linear import lm_head_score_mfma

    def fwd_mfma():
        return lm_head_score_mfma(hidden.detach(), weight.detach(), ids, temperature)

    lp_m, h_m = fwd_mfma()
    # guard: 8 tokens out of every 256-token block (every workgroup's tile) against the fp32 composition
    pick = (torch.arange(0, T, 256, device=dev)[:, None] + torch.tensor([0, 37, 64, 101, 128, 190, 222, 255], device=dev)).reshape(-1)
    zz = (hidden.detach()[pick].float() @ weight.detach().float().t()) / temperature
    e3 = (lp_m[pick] - torch.log_softmax(zz, -1).gather(-1, ids[pick, None]).squeeze(-1)).abs().max().item()
    e4 = (h_m[pick] - (torch.logsumexp(zz, -1) - (torch.softmax(zz, -1) * zz).sum(-1))).abs().max().item()
    del zz
    if not (e3 <= 1e-4 and e4 <= 1e-4):   # fp32 sums of exact products on both sides; only the order differs
        raise SystemExit(f"bench: matrix-core LM-head scores disagree with torch (log-prob {e3}, entropy {e4})")
    def fwd_bwd_recompute():
        lp, h = fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, False, "auto")
        return torch.autograd.grad((lp, h), (hidden, weight), (g_lp, g_h))

    def fwd_bwd_kept():
        lp, h = fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, True, "auto")
        return torch.autograd.grad((lp, h), (hidden, weight), (g_lp, g_h))

    def fwd_bwd_library():
        lp, h = fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, False, "library")
        return torch.autograd.grad((lp, h), (hidden, weight), (g_lp, g_h))

    def fwd_bwd_library_kept():
        lp, h = fused_linear_for_ppo(hidden, weight, ids, temperature, chunk, True, "library")
        return torch.autograd.grad((lp, h), (hidden, weight), (g_lp, g_h))

    # guard: the paths with this package's matrix-core kernels against the all-library one
    ga = fwd_bwd_library()
    for gb, which in ((fwd_bwd_recompute(), "recomputing"), (fwd_bwd_kept(), "kept-logits")):
        for x, y, what in ((ga[0], gb[0], "d hidden"), (ga[1], gb[1], "d weight")):
            err = (x.float() - y.float()).abs().max().item()
            if not err <= 3e-2 * max(x.float().abs().max().item(), 1e-6):
                raise SystemExit(f"bench: the {which} backward disagrees with the library path on {what} ({err})")
        del gb
    del ga
    # The part is power-managed and drifts by a few per cent within seconds: the paths that are compared are timed
    # alternately, twice, and each keeps its better time.
    def timed_pairwise(*fns):
        best = [float("inf")] * len(fns)
        for _ in range(2):
            for i, fn in enumerate(fns):
                best[i] = min(best[i], timed(fn))
        return best

    t_f, t_f_lib, t_m = timed_pairwise(fwd, fwd_library, fwd_mfma)
    t_fb_rec, t_fb_lib, t_fb_kept, t_fb_lib_kept = timed_pairwise(fwd_bwd_recompute, fwd_bwd_library, fwd_bwd_kept,
                                                                  fwd_bwd_library_kept)
    from verl_amd import fused_linear as _fl
    kept_by_default = keep is True or (keep is None and T * V * 2 <= _fl.DEFAULT_KEEP_LOGITS_BYTES)
    t_fb = t_fb_kept if kept_by_default else t_fb_rec
    wt = torch.empty(D, V, dtype=weight.dtype, device=dev)
    t_tr = timed(lambda: transpose_2d(weight.detach(), wt))
    # Kernel by kernel: `launches` calls back to back between one HIP event pair; the library's products beside the
    # package's own on operands laid out as the library likes them best (transposed copies made beforehand, not timed).
    from verl_amd import fused_linear as own_fl
    from verl_amd import gemm as own_gemm

    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    n_c = min(chunk, T)
    flops_c, flops_all = 2.0 * n_c * D * V, 2.0 * T * D * V

    def rec(kernel, what, ms, flops, library_ms=None):
        r = {"kernel": kernel, "what": what, "avg_kernel_ms": ms, "flops": flops, "tflops": flops / ms / 1e9,
             "frac": flops / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS}
        if library_ms is not None:
            r["library_ms"] = library_ms
        return r

    def per_launch(fn, n=10):
        spin_up(fn, 200.0)
        return batch_time_ms(fn, n, 3)

    with torch.no_grad():
        G = (torch.randn(n_c, V, generator=g, device=dev) * 0.01).bfloat16()
        Hd, Wd = hidden.detach(), weight.detach()
        Hc = Hd[:n_c]
        Ht = transpose_2d(Hc)
        d_h = torch.empty(n_c, D, dtype=torch.bfloat16, device=dev)
        d_w = torch.zeros(V, D, dtype=torch.bfloat16, device=dev)
        lp_f, ent_f, lse_f, _ = own_fl._own_forward(Hd, Wd, ids, torch.full((T,), temperature, device=dev), None, "bench")
        temp_c = torch.full((n_c,), temperature, device=dev)
        splits_c = lib.vrl_lmhead_plan(n_c, V)

        def dlogits():
            st = lib.vrl_lmhead_dlogits(Hc.data_ptr(), Wd.data_ptr(), _lib.VRL_BF16, n_c, V, D, D, D, ids.data_ptr(),
                                        temp_c.data_ptr(), lse_f.data_ptr(), ent_f.data_ptr(), g_lp.data_ptr(),
                                        g_h.data_ptr(), splits_c, G.data_ptr(), V, stream)
            _lib.check("vrl_lmhead_dlogits", st)

        kernels = [
            rec("lmhead_partial_kernel<bf16, false> + lmhead_finish_kernel", f"forward, {T} tokens", t_m * 1e3, flops_all),
            rec("lmhead_partial_kernel<bf16, true> + lmhead_finish_kernel", f"forward that also writes the logits, {T} tokens",
                per_launch(lambda: own_fl._own_forward(Hd, Wd, ids, None, None, "bench", keep_rows=T), 5), flops_all),
            rec("lmhead_dlogits_kernel<bf16>", f"logits formed again, their gradient written, {n_c} tokens", per_launch(dlogits),
                flops_c),
        ]
        G.copy_((torch.randn(n_c, V, generator=g, device=dev) * 0.01).bfloat16())
        kernels += [
            rec("lm_gemm_kernel<bf16, W contraction-major> (+ lm_gemm_reduce_kernel when the contraction is cut)", f"d hidden = G . W, {n_c} tokens",
                per_launch(lambda: own_gemm.gemm(Wd, G, x_t=True, out=d_h)), flops_c,
                per_launch(lambda: torch.matmul(G, wt.t(), out=d_h))),
            rec("lm_gemm_kernel<bf16, stored, both contraction-major>", f"d W = G^T . H stored, {n_c} tokens",
                per_launch(lambda: own_gemm.gemm(Hc, G, x_t=True, y_t=True, out=d_w)), flops_c,
                per_launch(lambda: torch.matmul(G.t(), Ht.t(), out=d_w))),
            rec("lm_gemm_kernel<bf16, accumulated, both contraction-major>", f"d W += G^T . H accumulated, {n_c} tokens",
                per_launch(lambda: own_gemm.gemm(Hc, G, x_t=True, y_t=True, out=d_w, accumulate=True)), flops_c,
                per_launch(lambda: d_w.addmm_(G.t(), Ht.t()))),
        ]
        del G, Ht
        if T > n_c:
            G8 = (torch.randn(T, V, generator=g, device=dev) * 0.01).bfloat16()
            H8t = transpose_2d(Hd)
            d_h8 = torch.empty(T, D, dtype=torch.bfloat16, device=dev)
            kernels += [
                rec("lm_gemm_kernel<bf16, W contraction-major> (+ lm_gemm_reduce_kernel when the contraction is cut)", f"d hidden = G . W, {T} tokens (kept logits)",
                    per_launch(lambda: own_gemm.gemm(Wd, G8, x_t=True, out=d_h8), 5), flops_all,
                    per_launch(lambda: torch.matmul(G8, wt.t(), out=d_h8), 5)),
                rec("lm_gemm_kernel<bf16, stored, both contraction-major>", f"d W = G^T . H stored, {T} tokens (kept logits)",
                    per_launch(lambda: own_gemm.gemm(Hd, G8, x_t=True, y_t=True, out=d_w), 5), flops_all,
                    per_launch(lambda: torch.matmul(G8.t(), H8t.t(), out=d_w), 5)),
            ]
            del G8, H8t, d_h8
        del d_h, d_w
    flops_f = 2.0 * T * D * V
    executed = (3 if kept_by_default else 4) * flops_f
    ceiling = mfma_ceiling(dev, args.steps)
    return {
        "metric": "tokens/sec of LM head + scoring, forward + backward",
        "value": T / t_fb, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": t_fb * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "lm_head_8192x3584_v152064_bf16", "chunk_tokens": chunk, "keep_logits": args.keep_logits,
                   "logits_kept": kept_by_default, "temperature": temperature,
                   "step": "verl_amd.fused_linear_for_ppo forward + torch.autograd.grad for hidden and weight with the "
                           "package's own kernels throughout (no library GEMM): " +
                           ("forward that also writes the logits, vrl_rowscore_backward over them in place, one vrl_gemm each "
                            "for d hidden and d W" if kept_by_default else
                            "vrl_lmhead_score forward; per chunk vrl_lmhead_dlogits and vrl_gemm for d hidden and d W")},
        "forward_ms": t_f * 1e3,
        "forward_tokens_per_s": T / t_f,
        "roofline": {"bound": "mfma", "achieved": 3 * flops_f / t_fb / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": 3 * flops_f / t_fb / 1e12 / MFMA_BF16_PEAK_TFLOPS, "traffic": None,
                     "flops": "algorithmic: 2*T*D*V forward + 4*T*D*V backward",
                     "executed_flops_frac": executed / t_fb / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "kernel": "whole step; the kernels one by one are under `kernels`",
                     "forward_tflops": flops_f / t_f / 1e12},
        "kernels": kernels,
        "paths_forward_backward_ms": {
            "own kernels, logits kept (default when they fit DEFAULT_KEEP_LOGITS_BYTES)": t_fb_kept * 1e3,
            "own kernels, logits formed again per chunk (keep_logits=False)": t_fb_rec * 1e3,
            "library products, logits kept": t_fb_lib_kept * 1e3,
            "library products, logits formed again per chunk": t_fb_lib * 1e3},
        "single_kernel_forward": {"ms": t_m * 1e3, "tflops": flops_f / t_m / 1e12, "frac_of_mfma_peak": flops_f / t_m / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                                  "kernel": "lmhead_partial_kernel<bf16> + lmhead_finish_kernel (vrl_lmhead_score)",
                                  "parity_guard": {"rows": int(pick.numel()), "max_abs_err_logprob": e3, "max_abs_err_entropy": e4},
                                  "frac_of_sustained_mfma_rate": flops_f / t_m / 1e12 / ceiling["tflops"],
                                  "note": "hand-written MFMA kernel, logits never written"},
        "matrix_core_ceiling": ceiling,
        "all_library": {"forward_ms": t_f_lib * 1e3, "forward_backward_ms": t_fb_lib * 1e3,
                        "forward_backward_kept_ms": t_fb_lib_kept * 1e3,
                        "kernel": "torch.matmul for every product (kernels=\"library\")"},
        "weight_transpose": {"ms": t_tr * 1e3, "gbps": 2.0 * V * D * 2 / t_tr / 1e9, "kernel": "transpose_kernel<2>",
                             "note": "the copy the all-library backward makes once per call; the package's own path needs none"},
        "parity_guard": {"rows": 256, "max_abs_err_logprob": e1, "max_abs_err_entropy": e2},
    }


def cpu_baseline(step: Step, budget_s: float = 12.0, runs: int = 4):
    """The torch restatement of the reference composition on the host cores, on a slice of the same batch.
    A pilot on 1024 rows sizes the slice so that `runs` timed runs take about `budget_s` seconds together."""
    from oracle import scoring, verify as overify  # checker/baseline only

    w = step.w

    def make(rows):
        x = step.logits[:rows].cpu()
        lab = step.labels[:rows].cpu()
        temp = None if step.temp is None else step.temp[:rows].cpu()
        old = step.lp_old[:rows].cpu().view(1, rows)
        lu = step.log_u[:rows].cpu().view(1, rows)
        mk = step.mask8[:rows].cpu().view(1, rows)

        def once():
            t0 = time.perf_counter()
            lp, h = scoring.score_reference(x, lab, temp)
            overify.verify(lp.float().view(1, rows), old, lu, mk, step.off)
            return time.perf_counter() - t0

        return once

    pilot_rows = min(step.n, 1024)
    pilot = make(pilot_rows)
    pilot()                                   # first touch: thread pool, allocator
    per_row = pilot() / pilot_rows
    rows = int(budget_s / runs / max(per_row, 1e-9))
    rows = max(pilot_rows, min(step.n, 32768, rows // 1024 * 1024))
    once = make(rows)
    times = [once() for _ in range(runs)]
    best = statistics.median(times)
    return {
        "value": rows / best,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{rows} rows of the same batch (V={w.V}, {str(w.dtype).replace('torch.', '')}), "
                  f"median of {len(times)} runs ({sum(times):.1f} s of CPU work), torch {torch.__version__} on "
                  f"{os.cpu_count()} logical CPUs",
    }


def copy_calibration(dev):
    """A plain copy kernel of known size: reads 1 GiB, writes 1 GiB. Whatever FETCH_SIZE / WRITE_SIZE report for it
    is the scale that converts the same counters of the row kernels into bytes."""
    src = torch.empty(1 << 29, dtype=torch.int16, device=dev).fill_(3)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def bench_ceilings(args, dev):
    """The memory system's own ceilings for the row kernels' access pattern (vrl_stream_probe): a non-temporal read
    of c3's rows (forward kernel) and a non-temporal copy of them (backward kernel), plus torch's device copy."""
    lib = bench_probes.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    out = {"metric": "HBM GB/s delivered to the row kernels' access pattern without arithmetic", "unit": "GB/s",
           "peak": HBM_PEAK_GBPS, "probes": []}
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    for name, rows, row_bytes in (("c3 micro-batch, 8192 x 151936 bf16", 8192, 151936 * 2),
                                  ("c2, 65536 x 152064 bf16", 65536, 152064 * 2),
                                  ("c1, 4096 x 32000 f32", 4096, 32000 * 4)):
        src = torch.empty(rows * row_bytes // 2, dtype=torch.int16, device=dev).fill_(5)
        small = rows * row_bytes < (1 << 30)
        modes = ((3, "non-temporal read, 32-bit row shape", 1),) if small else (
            (0, "non-temporal read", 1), (4, "non-temporal read, 1024 workgroups walking the whole buffer", 1),
            (1, "non-temporal copy", 2),
            (2, "non-temporal copy, 512 workgroups walking the whole buffer", 2))
        for mode, what, factor in modes:
            if mode in (1, 2) and rows * row_bytes > (8 << 30):
                continue
            dst = torch.empty_like(src) if mode in (1, 2) else None

            def run():
                st = lib.vrl_stream_probe(src.data_ptr(), None if dst is None else dst.data_ptr(), rows, row_bytes, mode,
                                          sink.data_ptr(), stream)
                _lib.check("vrl_stream_probe", st)

            spin_up(run)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
            for a, b in evs:
                a.record()
                run()
                b.record()
            torch.cuda.synchronize()
            ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
            if dst is not None and not torch.equal(dst, src):
                raise SystemExit("bench: the copy probe did not copy")
            out["probes"].append({"buffer": name, "probe": what, "kernel": "stream_probe_kernel", "avg_kernel_ms": ms,
                                  "bytes_per_launch": factor * rows * row_bytes,
                                  "gbps": factor * rows * row_bytes / (ms * 1e-3) / 1e9,
                                  "frac_of_peak": factor * rows * row_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS})
            del dst
        del src
        torch.cuda.empty_cache()
    out["matrix_cores"] = mfma_ceiling(dev, args.steps)
    print(json.dumps(out), flush=True)


def mfma_ceiling(dev, steps):
    """What the part sustains on bf16 matrix instructions alone (vrl_mfma_probe: one workgroup of 8 wavefronts per CU,
    register operands, no memory traffic), with the shader clock it ran at: on pseudo-random operands with the
    instruction of the LM-head kernels (16x16x32; what their matrix time is measured against: the part holds a lower
    clock when the operand bits toggle), the same with 32x32x16, and on small constants (the nominal rate). Returns the
    first record with the others inside."""
    lib = bench_probes.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    n_wg = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 20000   # 64 x 128 x 16 wavefront tiles: about as many as the LM-head kernel forms per wavefront at 8192 tokens
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    khz = ctypes.c_int64(0)
    records = []
    for instruction, random_operands in ((16, 1), (32, 1), (32, 0)):
        def run():
            st = lib.vrl_mfma_probe(n_wg, iters, instruction, random_operands, sink.data_ptr(), clocks.data_ptr(),
                                    ctypes.addressof(khz), stream)
            _lib.check("vrl_mfma_probe", st)

        spin_up(run)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in evs:
            a.record()
            run()
            b.record()
        torch.cuda.synchronize()
        ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
        flops = n_wg * 8 * iters * 2.0 * 64 * 128 * 16
        cyc, ticks = clocks.tolist()
        records.append({"instruction": "v_mfma_f32_16x16x32_bf16" if instruction == 16 else "v_mfma_f32_32x32x16_bf16",
                        "operands": "pseudo-random bf16 in (-1, 1)" if random_operands else "small constants",
                        "avg_kernel_ms": ms, "tflops": flops / (ms * 1e-3) / 1e12,
                        "frac_of_peak": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                        "shader_clock_ghz": (cyc / ticks) * khz.value * 1e-6 if ticks else None})
    out = {"probe": "bf16 matrix instructions on register operands, 8 wavefronts per CU, nothing else",
           "kernel": "mfma_probe_kernel", "workgroups": n_wg}
    out.update(records[0])
    out["same_operands_32x32x16"] = records[1]
    out["with_constant_operands"] = records[2]
    return out


def bench_forward(args, dev, workload, steps, warmup, with_cpu_baseline):
    """The fused score + verify step on one workload; returns the JSON record."""
    w = synthetic.WORKLOADS[workload]
    if args.vocab or args.seqs or args.dtype:
        # the workload's recipe at another vocabulary / batch / element type (e.g. 32000, 128256, 129280, 262144)
        kw = {"name": w.name + "_resized"}
        if args.vocab:
            kw["V"] = args.vocab
        if args.seqs:
            kw["B"] = args.seqs
        if args.dtype:
            kw["dtype"] = {"bf16": torch.bfloat16, "f32": torch.float32}[args.dtype]
        w = w.scaled(**kw)
    step = Step(w, dev, seed=1000 * int(workload[1]))
    guard = step.check_against_torch()

    if args.copy_calibration:
        copy_calibration(dev)

    spin_up(step.fused)
    for _ in range(warmup):
        step.fused()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step.fused()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    tokens_per_s = step.n_valid * steps / wall

    # Row kernel alone: `steps` launches back to back between one HIP event pair on the launch stream, median of 3 batches.
    avg_kern_ms = batch_time_ms(step.score, steps, 3)
    esize = 2 if w.dtype == torch.bfloat16 else 4
    bytes_score = algorithmic_bytes_per_token(w.V, esize, step.temp is not None, False) * step.n
    achieved = bytes_score / (avg_kern_ms * 1e-3) / 1e9
    bytes_fused = algorithmic_bytes_per_token(w.V, esize, step.temp is not None, True) * step.n
    resized = bool(args.vocab or args.seqs or args.dtype)

    out = {
        "metric": METRIC,
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "spinup_ms": SPINUP_MS,
        "config": {
            "workload": step.w.name,
            "layout": step.layout,
            "logits_buffers_rotated": len(step.ring),
            "launches_per_step": 2,
            "rows_per_step": step.n,
            "valid_tokens_per_step": step.n_valid,
            "vocab": w.V,
            "lenience": w.lenience,
            "temperature": w.temperature,
            "step": "vrl_fused_score_verify through the C ABI, logits resident in HBM",
        },
        "hbm_gbps_fused_step": bytes_fused / (ms_per_step * 1e-3) / 1e9,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": None if resized else MEASURED_TRAFFIC_BYTES.get(workload),
            "traffic_source": None if resized or workload not in MEASURED_TRAFFIC_BYTES else
            "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel at this shape, profiles/rowscore_kernel_hbm_counters_" +
            ("c1.md" if workload == "c1" else "c2_c3_c4.md"),
            "kernel": "rowscore_kernel",
            "avg_kernel_ms": avg_kern_ms,
            "algorithmic_bytes_per_launch": bytes_score,
        },
        "parity_guard": guard,
    }
    if with_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(step)
    return out


def bench_score_responses(args, dev, steps, warmup):
    """c3's packed micro-batch through vrl_score_responses: label roll, scoring and the (B, T) response slicing in
    one launch; only rows inside a response window are read. Sequences are prompt + response with the response
    lengths of the workload and prompts of a quarter of that."""
    w = synthetic.WORKLOADS["c3"]
    budget = int(w.micro_batch_tokens)
    resp_all = synthetic.draw_lengths(w, 3002).tolist()
    seqs, total = [], 0
    for r in resp_all:
        p = max(1, r // 4)
        if total + p + r > budget:
            break
        seqs.append((p, r))
        total += p + r
    seqs[-1] = (seqs[-1][0] + budget - total, seqs[-1][1])   # the last prompt takes up the rest of the budget
    n = budget
    cu = torch.zeros(len(seqs) + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(torch.tensor([p + r for p, r in seqs]), 0)
    resp = torch.tensor([r for _, r in seqs], dtype=torch.int64)
    g = torch.Generator(device=dev).manual_seed(3001)
    ids = torch.randint(0, w.V, (n,), generator=g, device=dev, dtype=torch.int64)
    logits = synthetic.make_logits(n, w.V, w.dtype, w.sigma, torch.roll(ids, -1), dev, 3003, boost=w.boost,
                                   boost_frac=w.boost_frac)
    B, T = len(seqs), w.T
    cu_d, resp_d = cu.to(dev), resp.to(dev)
    r_lp = torch.empty((B, T), dtype=torch.float32, device=dev)
    r_h = torch.empty_like(r_lp)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream

    def run():
        st = lib.vrl_score_responses(logits.data_ptr(), _lib.VRL_BF16, n, w.V, logits.stride(0), None, ids.data_ptr(),
                                     None, cu_d.data_ptr(), resp_d.data_ptr(), B, T, None, None, r_lp.data_ptr(),
                                     r_h.data_ptr(), None, flag.data_ptr(), stream)
        _lib.check("vrl_score_responses", st)

    run()
    # guard: equal to the separate entry points
    lp, h = vf.fused_logprob_entropy(logits, torch.roll(ids, -1))
    from verl_amd import layout
    if not (torch.equal(r_lp, layout.response_slice(lp, cu_d, resp_d, T)) and torch.equal(r_h, layout.response_slice(h, cu_d, resp_d, T))):
        raise SystemExit("bench: vrl_score_responses disagrees with vrl_rowscore + vrl_response_slice")
    if int(flag.item()) != 0:
        raise SystemExit("bench: vrl_score_responses set an error flag")
    spin_up(run)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    avg_ms = batch_time_ms(run, steps, 3)
    n_resp = int(resp.sum())
    bytes_launch = n_resp * (w.V * 2 + 8 + 4 + 4) + (B + 1) * 8 + B * 8 + B * T * 8 - n_resp * 8
    achieved = bytes_launch / (avg_ms * 1e-3) / 1e9

    # The gradient of the same blocks (vrl_score_responses_backward): response rows are read once and their gradient
    # written, every other row of the gradient is written as zeros without being read.
    r_lse = torch.empty_like(r_lp)
    st = lib.vrl_score_responses(logits.data_ptr(), _lib.VRL_BF16, n, w.V, logits.stride(0), None, ids.data_ptr(),
                                 None, cu_d.data_ptr(), resp_d.data_ptr(), B, T, None, None, r_lp.data_ptr(),
                                 r_h.data_ptr(), r_lse.data_ptr(), flag.data_ptr(), stream)
    _lib.check("vrl_score_responses", st)
    gg = torch.Generator(device=dev).manual_seed(3004)
    g_lp = torch.randn((B, T), generator=gg, device=dev)
    g_h = torch.randn((B, T), generator=gg, device=dev)
    dlogits = torch.empty_like(logits)

    def run_backward():
        st = lib.vrl_score_responses_backward(
            logits.data_ptr(), _lib.VRL_BF16, n, w.V, logits.stride(0), None, ids.data_ptr(), None, cu_d.data_ptr(),
            resp_d.data_ptr(), B, T, r_lse.data_ptr(), r_h.data_ptr(), g_lp.data_ptr(), g_h.data_ptr(),
            dlogits.data_ptr(), dlogits.stride(0), stream)
        _lib.check("vrl_score_responses_backward", st)

    run_backward()
    # guard: equal to the row op's backward fed with the per-token gradients (zero outside the response windows)
    tok_lp = torch.zeros(n, device=dev)
    tok_h = torch.zeros(n, device=dev)
    for b in range(B):
        end, r = int(cu[b + 1]), int(resp[b])
        tok_lp[end - r - 1:end - 1] = g_lp[b, :r]
        tok_h[end - r - 1:end - 1] = g_h[b, :r]
    x = logits.detach().clone().requires_grad_(True)
    lp2, h2 = vf.fused_logprob_entropy(x, torch.roll(ids, -1))
    torch.autograd.backward([lp2, h2], [tok_lp, tok_h])
    if not torch.equal(x.grad, dlogits):
        raise SystemExit("bench: vrl_score_responses_backward disagrees with vrl_rowscore_backward")
    del x, lp2, h2
    for _ in range(warmup):
        run_backward()
    torch.cuda.synchronize()
    bwd_ms = batch_time_ms(run_backward, steps, 3)
    bwd_bytes = n_resp * (w.V * 2 + 8 + 16) + n * w.V * 2 + (B + 1) * 8 + B * 8
    # the counters were read at this very micro-batch (5515 response rows of 8192); another one has no measured traffic
    measured = MEASURED_SCORE_RESPONSES_TRAFFIC_BYTES if (n, n_resp, B) == (8192, 5515, 4) else (None, None)
    backward = {"avg_kernel_ms": bwd_ms, "kernel": "score_responses_backward_flat_kernel",
                "algorithmic_bytes_per_launch": bwd_bytes, "achieved_gbps": bwd_bytes / (bwd_ms * 1e-3) / 1e9,
                "traffic": measured[1],
                "all_rows_backward_bytes": n * (w.V * 4 + 8 + 16),
                "parity_guard": "bit-equal to vrl_rowscore_backward with per-token gradients"}
    return {
        "metric": "response tokens/sec from packed logits to padded (B, T) log-probs and entropies, one launch",
        "value": n_resp * steps / wall, "unit": "tokens/s", "ms_per_step": wall * 1e3 / steps, "dtype": "bf16",
        "config": {"workload": "c3_grpo_packed_prompt_plus_response_v151936_bf16", "rows_per_step": n,
                   "response_rows_per_step": n_resp, "sequences": B, "padded_response_len": T,
                   "step": "vrl_score_responses through the C ABI (labels rolled in-kernel, prompt rows not read)"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": measured[0],
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel at this micro-batch, "
                                       "profiles/score_responses_kernel_hbm_counters_c3_packed.md",
                     "kernel": "score_responses_kernel",
                     "avg_kernel_ms": avg_ms, "algorithmic_bytes_per_launch": bytes_launch},
        "all_rows_equivalent_tokens_per_s": n * steps / wall,
        "backward": backward,
    }


def compact(rec: dict) -> dict:
    """The fields of a workload record that the headline line carries for every other workload."""
    keep = ("value", "unit", "ms_per_step", "dtype", "hbm_gbps_fused_step", "parity_guard")
    out = {"workload": rec["config"]["workload"], "step": rec["config"]["step"]}
    out.update({k: rec[k] for k in keep if k in rec})
    r = rec["roofline"]
    out["roofline"] = {k: r[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "avg_kernel_ms",
                                         "algorithmic_bytes_per_launch", "timing", "launch_floor_ms",
                                         "achieved_net_of_launch_floor", "flops", "executed_flops_frac") if k in r}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=["c1", "c2", "c3", "c4", "c5"],
                    help="time this workload only (c5 times the verify kernel alone: its logits do not fit, they are "
                         "scored like c3). Default: c2 as the headline plus a short record of every other workload")
    ap.add_argument("--vocab", type=int, default=0, help="run the workload's recipe at another vocabulary size")
    ap.add_argument("--seqs", type=int, default=0, help="... with another number of sequences")
    ap.add_argument("--dtype", choices=["bf16", "f32"], default=None, help="... with another logits element type")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-lm-head", action="store_true",
                    help="default run: leave out the short LM-head record (its library path launches the row kernels too, "
                         "which mixes their averages in a kernel trace)")
    ap.add_argument("--backward", action="store_true",
                    help="time vrl_rowscore_backward on the workload instead of the fused forward step")
    ap.add_argument("--score-responses", action="store_true",
                    help="time vrl_score_responses (packed logits -> padded response blocks, one launch) on c3")
    ap.add_argument("--lm-head", action="store_true",
                    help="time the LM head + scoring step (verl_amd.fused_linear) instead of the fused forward step")
    ap.add_argument("--chunk", type=int, default=4096, help="--lm-head: tokens projected at a time")
    ap.add_argument("--keep-logits", choices=["auto", "yes", "no"], default="auto",
                    help="--lm-head: keep the logits for the backward (auto: when they fit the package's default budget)")
    ap.add_argument("--own-only", action="store_true",
                    help="--lm-head: run the default call (the package's own kernels) alone, without the library paths it "
                         "is compared with (for a kernel trace)")
    ap.add_argument("--ceilings", action="store_true",
                    help="time plain non-temporal read / copy probes with the row kernels' access pattern")
    ap.add_argument("--verify-form", choices=["auto", "two-pass", "per-sequence"], default="auto",
                    help="--workload c5: which form of vrl_spec_verify to time (auto: what vrl_spec_verify_plan says)")
    ap.add_argument("--no-guard", action="store_true",
                    help="--workload c5: leave out the comparison with the oracle on the host (a counter-collecting "
                         "profiler does not survive the large device-to-host copies it needs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain device copy of known size (for scaling rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.lm_head:
        if args.copy_calibration:
            copy_calibration(dev)
        print(json.dumps(bench_lm_head(args, dev)), flush=True)
        return
    if args.ceilings:
        bench_ceilings(args, dev)
        return
    if args.score_responses:
        if args.copy_calibration:
            copy_calibration(dev)
        print(json.dumps(bench_score_responses(args, dev, args.steps, args.warmup)), flush=True)
        return
    if args.backward:
        args.workload = args.workload or "c2"
        print(json.dumps(bench_backward(args, dev)), flush=True)
        return
    if args.workload == "c5":
        print(json.dumps(bench_verify_only(args, dev, not args.no_cpu_baseline)), flush=True)
        return
    if args.workload is not None or args.vocab or args.seqs or args.dtype:
        rec = bench_forward(args, dev, args.workload or "c2", args.steps, args.warmup, not args.no_cpu_baseline)
        print(json.dumps(rec), flush=True)
        return

    # Default: the headline workload (c2, the configuration the metric is quoted on) in full, then every other
    # workload with fewer steps and without a CPU leg, as short records under "workloads".
    out = bench_forward(args, dev, "c2", args.steps, args.warmup, not args.no_cpu_baseline)
    few = argparse.Namespace(**vars(args))
    few.steps, few.warmup = min(args.steps, 10), min(args.warmup, 3)
    others = []
    for name in ("c3", "c4", "c1"):
        torch.cuda.empty_cache()
        others.append(compact(bench_forward(few, dev, name, few.steps, few.warmup, False)))
    torch.cuda.empty_cache()
    others.append(compact(bench_verify_only(few, dev, False)))
    torch.cuda.empty_cache()
    others.append(compact(bench_backward(few, dev, "c3")))
    torch.cuda.empty_cache()
    others.append(compact(bench_score_responses(few, dev, few.steps, few.warmup)))
    # the LM head fused with the scoring (matrix-core bound, its own roofline): the short form of `--lm-head`
    if not args.no_lm_head:
        torch.cuda.empty_cache()
        lm = argparse.Namespace(**vars(args))
        lm.steps, lm.warmup = min(args.steps, 5), min(args.warmup, 2)
        rec = bench_lm_head(lm, dev)
        short = compact(rec)
        short.update({k: rec[k] for k in ("forward_ms", "all_library", "kernels", "paths_forward_backward_ms")})
        short["single_kernel_forward"] = {k: rec["single_kernel_forward"][k] for k in ("ms", "tflops", "frac_of_mfma_peak",
                                                                                     "frac_of_sustained_mfma_rate")}
        others.append(short)
    out["workloads"] = others
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
