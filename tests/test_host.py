"""Host-side logic that needs no GPU: input validation of the wrappers, install()/uninstall() on a stand-in
``verl`` package, the synthetic workload recipes."""

import math
import sys
import types

import pytest
import torch

import verl_amd
from verl_amd import hook as inst
from verl_amd import spec_rl, synthetic
from verl_amd import torch_functional as vf


# ---- wrappers refuse what they cannot do, loudly -----------------------------

def test_cpu_tensors_are_refused_not_computed():
    x, lab = torch.randn(2, 10), torch.zeros(2, dtype=torch.long)
    for call in (
        lambda: vf.logprobs_from_logits(x, lab),
        lambda: vf.logprobs_from_logits_v2(x, lab),
        lambda: vf.logprobs_from_logits_naive(x, lab),
        lambda: vf.entropy_from_logits(x),
        lambda: vf.entropy_from_logits_with_chunking(x),
        lambda: vf.fused_logprob_entropy(x, lab, 0.7),
        lambda: spec_rl.spec_verify(x, x, None, seed=0),
        lambda: spec_rl.fused_score_verify(x, lab, torch.zeros(2), seed=0),
        lambda: spec_rl.truncate_draft(lab.view(1, 2), None, torch.zeros(1, dtype=torch.int32)),
    ):
        with pytest.raises(RuntimeError, match="no CPU implementation"):
            call()


def test_chunk_size_is_validated():
    with pytest.raises(ValueError):
        vf.entropy_from_logits_with_chunking(torch.randn(2, 4), chunk_size=0)


def test_lenience_offset():
    assert spec_rl.thresh_offset_from_lenience(1.0) == 0.0
    assert spec_rl.thresh_offset_from_lenience(math.exp(0.5)) == 0.5
    assert spec_rl.thresh_offset_from_lenience(math.exp(0.5), "relax") == -0.5
    assert spec_rl.thresh_offset_from_lenience(math.e) == 1.0
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(ValueError):
            spec_rl.thresh_offset_from_lenience(bad)
    with pytest.raises(ValueError):
        spec_rl.thresh_offset_from_lenience(2.0, "other")


def test_package_surface():
    for name in ("logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking",
                 "fused_logprob_entropy", "spec_verify", "fused_score_verify", "truncate_draft", "install", "uninstall",
                 "score_responses", "response_slice", "response_from_packed", "expand_per_sequence"):
        assert callable(getattr(verl_amd, name)), name


# ---- install() on a stand-in verl -------------------------------------------------

@pytest.fixture
def fake_verl():
    calls = []

    def make(name):
        def original(logits, *a, **k):
            calls.append(name)
            return ("verl", name)
        original.__name__ = name
        return original

    mods = {}
    for mod_name in ("verl", "verl.utils", "verl.utils.torch_functional", "verl.workers", "verl.workers.engine_impl"):
        mods[mod_name] = types.ModuleType(mod_name)
    tf = mods["verl.utils.torch_functional"]
    for name in inst.PATCHED_NAMES:
        setattr(tf, name, make(name))
    tf.masked_mean = lambda *a: "untouched"
    # an engine module that bound the names at import, like `from verl.utils.torch_functional import logprobs_from_logits`
    eng = mods["verl.workers.engine_impl"]
    eng.logprobs_from_logits = tf.logprobs_from_logits
    eng.verl_F = tf
    saved = {k: sys.modules.get(k) for k in mods}
    sys.modules.update(mods)
    try:
        yield mods, calls
    finally:
        inst.uninstall()
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_install_patches_module_and_bound_names(fake_verl):
    mods, calls = fake_verl
    tf, eng = mods["verl.utils.torch_functional"], mods["verl.workers.engine_impl"]
    orig = tf.logprobs_from_logits
    replaced = inst.install()
    assert "verl.utils.torch_functional.logprobs_from_logits" in replaced
    assert "verl.workers.engine_impl.logprobs_from_logits" in replaced
    assert tf.logprobs_from_logits is not orig and eng.logprobs_from_logits is tf.logprobs_from_logits
    assert eng.verl_F.entropy_from_logits is tf.entropy_from_logits
    assert tf.masked_mean() == "untouched"
    assert tf.logprobs_from_logits.__verl_amd_original__ is orig
    assert inst.install() == []  # second call is a no-op

    # CPU tensors and unsupported dtypes go to verl's own function
    x = torch.randn(2, 5)
    assert tf.logprobs_from_logits(x, torch.zeros(2, dtype=torch.long)) == ("verl", "logprobs_from_logits")
    assert eng.logprobs_from_logits(x, torch.zeros(2, dtype=torch.long), inplace_backward=False) == ("verl", "logprobs_from_logits")
    assert tf.entropy_from_logits(x.double()) == ("verl", "entropy_from_logits")
    assert tf.entropy_from_logits_with_chunking(x, chunk_size=3) == ("verl", "entropy_from_logits_with_chunking")
    assert {k: inst.stats()[k] for k in ("hip_calls", "passed_to_verl", "memo_hits")} == {"hip_calls": 0, "passed_to_verl": 4, "memo_hits": 0}

    class Wrapped(torch.Tensor):        # stands for DTensor and other tensor subclasses
        pass

    assert not inst._eligible(torch.randn(2, 5).as_subclass(Wrapped))

    inst.uninstall()
    assert tf.logprobs_from_logits is orig and eng.logprobs_from_logits is orig
    assert {k: inst.stats()[k] for k in ("hip_calls", "passed_to_verl", "memo_hits")} == {"hip_calls": 0, "passed_to_verl": 0, "memo_hits": 0}


def test_install_patches_the_fused_linear_entry_points_when_present(fake_verl):
    mods, _ = fake_verl

    class RefModule:
        def __init__(self, chunk_size=512):
            self.chunk_size = chunk_size

        def forward(self, hidden_states, vocab_weights, input_ids, temperature=1.0):
            return ("verl", "FusedLinearForPPO", self.chunk_size)

    def ref_lce(hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None):
        return ("verl", "linear_cross_entropy", reduction)

    extra = {n: types.ModuleType(n) for n in ("verl.utils.experimental", "verl.utils.experimental.torch_functional",
                                                "verl.utils.kernel", "verl.utils.kernel.linear_cross_entropy")}
    extra["verl.utils.experimental.torch_functional"].FusedLinearForPPO = RefModule
    extra["verl.utils.kernel.linear_cross_entropy"].linear_cross_entropy = ref_lce
    sys.modules.update(extra)
    try:
        replaced = inst.install()
        assert "verl.utils.experimental.torch_functional.FusedLinearForPPO" in replaced
        assert "verl.utils.kernel.linear_cross_entropy.linear_cross_entropy" in replaced
        cls = extra["verl.utils.experimental.torch_functional"].FusedLinearForPPO
        assert cls is not RefModule and cls.__verl_amd_original__ is RefModule
        h, w, ids = torch.randn(3, 8), torch.randn(16, 8), torch.zeros(3, dtype=torch.long)
        # CPU tensors: the reference's own module and function serve the call, constructed as the caller asked
        assert cls().forward(hidden_states=h, vocab_weights=w, input_ids=ids, temperature=1.0) == ("verl", "FusedLinearForPPO", 512)
        assert cls(64).forward(h, w, ids) == ("verl", "FusedLinearForPPO", 64)
        lce = extra["verl.utils.kernel.linear_cross_entropy"].linear_cross_entropy
        assert lce(h, w, ids, 1.0, "mean") == ("verl", "linear_cross_entropy", "mean")
        assert inst.stats()["passed_to_verl"] == 3
        inst.uninstall()
        assert extra["verl.utils.experimental.torch_functional"].FusedLinearForPPO is RefModule
        assert extra["verl.utils.kernel.linear_cross_entropy"].linear_cross_entropy is ref_lce
    finally:
        for n in extra:
            sys.modules.pop(n, None)


def test_plugin_module_installs_on_import(fake_verl):
    mods, _ = fake_verl
    tf = mods["verl.utils.torch_functional"]
    orig = tf.entropy_from_logits
    sys.modules.pop("verl_amd.plugin", None)
    import importlib

    importlib.import_module("verl_amd.plugin")   # what VERL_USE_EXTERNAL_MODULES=verl_amd.plugin triggers
    assert tf.entropy_from_logits is not orig
    sys.modules.pop("verl_amd.plugin", None)


# ---- synthetic workloads ------------------------------------------------------------

def test_workload_recipes_match_the_five_configs():
    w = synthetic.WORKLOADS
    assert (w["c1"].B, w["c1"].T, w["c1"].V, w["c1"].dtype) == (8, 512, 32000, torch.float32)
    assert (w["c2"].B, w["c2"].T, w["c2"].V, w["c2"].dtype) == (64, 1024, 152064, torch.bfloat16)
    assert (w["c3"].B, w["c3"].T, w["c3"].V, w["c3"].micro_batch_tokens) == (1024, 2048, 151936, 8192)
    assert (w["c4"].B, w["c4"].T, w["c4"].V, w["c4"].temperature) == (16, 8192, 128256, 0.7)
    assert (w["c5"].B, w["c5"].V) == (512, 151936) and w["c5"].drift[0] == "student_t"
    assert abs(math.log(w["c3"].lenience) - 0.5) < 1e-12 and w["c1"].lenience == 1.0


def test_generators_are_seeded_and_shaped():
    w = synthetic.WORKLOADS["c2"].scaled(B=3, T=20, V=501)
    a, b = synthetic.make_padded(w, "cpu", 5), synthetic.make_padded(w, "cpu", 5)
    c = synthetic.make_padded(w, "cpu", 6)
    assert a["logits"].shape == (3, 20, 501) and a["logits"].dtype == torch.bfloat16
    assert torch.equal(a["logits"], b["logits"]) and torch.equal(a["log_u"], b["log_u"]) and not torch.equal(a["logits"], c["logits"])
    assert a["mask"].all() and a["temperature"] is None and (a["log_u"] <= 0).all()
    # boosted labels: +8 on ~70 % of tokens, so the label logits average ~5.6 instead of 0
    picked = a["logits"].float().gather(-1, a["labels"].unsqueeze(-1)).mean().item()
    assert 3.5 < picked < 7.5

    w1 = synthetic.WORKLOADS["c1"].scaled(V=100)
    d = synthetic.make_padded(w1, "cpu", 1)
    L = d["lengths"]
    assert L.min() >= 64 and L.max() <= 512 and torch.equal(d["mask"].sum(1), L)
    assert torch.equal(d["mask"], synthetic.right_pad_mask(L, 512, "cpu"))
    assert abs(d["logits"].std().item() - 2.0) < 0.05

    L5 = synthetic.draw_lengths(synthetic.WORKLOADS["c5"], 7)
    assert L5.min() >= 32 and L5.max() <= 16384 and 1500 < L5.float().mean().item() < 4000
    cu = synthetic.pack_by_lengths(L5)
    assert cu[0] == 0 and cu[-1] == L5.sum() and cu.numel() == 513

    w4 = synthetic.WORKLOADS["c4"].scaled(B=2, T=4, V=50)
    assert torch.all(synthetic.make_tokens(w4, "cpu", 0)["temperature"] == 0.7)


def test_drift_recipes():
    base = torch.zeros(200, 200)
    n = synthetic.drift_old_logprobs(base, synthetic.WORKLOADS["c3"], 3)
    assert abs(n.std().item() - 0.2) < 0.01
    t = synthetic.drift_old_logprobs(base, synthetic.WORKLOADS["c5"], 3)
    # Student-t(3) * 0.3: heavy tails, median absolute deviation 0.3 * 0.765
    assert abs(t.abs().median().item() - 0.3 * 0.7649) < 0.02 and t.abs().max().item() > 3.0


def test_deprecated_label_check_switch_still_switches():
    """Setting verl_amd.torch_functional.LABEL_CHECK (the switch of earlier versions) maps onto verl_amd.errors."""
    import warnings

    from verl_amd import errors, torch_functional as vf

    before = errors.DEFAULT_MODE
    try:
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            vf.LABEL_CHECK = False
        assert errors.DEFAULT_MODE == "off" and errors.mode() == "off" and vf.LABEL_CHECK is False
        assert any(issubclass(w.category, DeprecationWarning) for w in caught)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            vf.LABEL_CHECK = True
        assert errors.DEFAULT_MODE == "sync" and vf.LABEL_CHECK is True
    finally:
        errors.DEFAULT_MODE = before


def test_gemm_takes_refuses_what_vrl_gemm_would_refuse():
    """Operands vrl_gemm rejects (storage that starts off the 16-byte grid, a row stride below the row) must be refused
    by gemm_takes too, so that callers send them to the library product instead of into an error in mid-backward."""
    import torch

    from verl_amd import gemm

    x = torch.zeros(512 * 128 + 8, dtype=torch.bfloat16)
    y = torch.zeros(256 * 128 + 8, dtype=torch.bfloat16)
    aligned_x, aligned_y = x[:512 * 128].view(512, 128), y[:256 * 128].view(256, 128)
    assert gemm.gemm_takes(aligned_x, aligned_y)
    off_x = x[1:512 * 128 + 1].view(512, 128)            # starts 2 bytes into the allocation
    assert off_x.data_ptr() % 16 != 0 and not gemm.gemm_takes(off_x, aligned_y)
    assert not gemm.gemm_takes(aligned_x, y[4:256 * 128 + 4].view(256, 128))
    assert not gemm.gemm_takes(aligned_x.float(), aligned_y.float())
