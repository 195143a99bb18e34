"""Committed fixtures of tests/golden: the CPU checker must reproduce them, and the GPU engine must match
them (tolerances of the target: relative L2 <= 1e-2 on logits and gradients)."""
import ctypes as C
import json
from pathlib import Path

import numpy as np
import pytest

GOLDEN = Path(__file__).resolve().parent / "golden"
KNOWN = json.loads((GOLDEN / "known_answers.json").read_text())


def tiny():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_vectors", GOLDEN / "make_vectors.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def rel(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def test_known_answers_hold_for_the_checker_and_the_library(orc):
    from turbogpt_amd import bridge
    for seed, want in KNOWN["hash_u64"].items():
        assert orc.hash_u64(int(seed)) == int(want, 16)
    lib = bridge.library()
    for step, (multiplier, momentum) in KNOWN["onecycle_total20"].items():
        got = orc.onecycle_point(20, int(step))
        assert got == pytest.approx((multiplier, momentum), rel=2e-6)
        rates = bridge.StepRates()
        assert lib.tg_onecycle_point(C.byref(bridge.OneCycle(20)), int(step), C.byref(rates)) == 0
        assert (rates.multiplier, rates.momentum) == got
    for bits, want in KNOWN["bf16_round_to_nearest_even"].items():
        value = np.array([int(bits, 16)], np.uint32).view(np.float32)
        assert orc.bf16_round(value).view(np.uint32)[0] >> 16 == int(want, 16)
    for bits, want in KNOWN["bf16_truncate"].items():
        value = np.array([int(bits, 16)], np.uint32).view(np.float32)
        assert orc.bf16_trunc(value).view(np.uint32)[0] >> 16 == int(want, 16)


def test_checker_reproduces_the_tiny_model_fixture(orc):
    fixture = np.load(GOLDEN / "tiny_model.npz")
    cfg, w, x, y = tiny().tiny_inputs(orc)
    logits, grad, losses = orc.model_batch(cfg, w, x, y)
    assert grad.size == int(fixture["parameter_count"])
    np.testing.assert_allclose(logits.reshape(-1, 256), fixture["logits"], rtol=0, atol=2e-5)
    np.testing.assert_allclose(losses, fixture["losses"], rtol=0, atol=2e-5)
    np.testing.assert_allclose(grad[fixture["gradient_index"]], fixture["gradient_value"], rtol=1e-4, atol=1e-7)


@pytest.mark.gpu
def test_engine_matches_the_tiny_model_fixture(orc):
    from turbogpt_amd.bridge import ModelConfig, Native
    fixture = np.load(GOLDEN / "tiny_model.npz")
    module = tiny()
    cfg, w, x, y = module.tiny_inputs(orc)
    with Native(ModelConfig(**module.TINY)) as engine:
        assert engine.count == int(fixture["parameter_count"])
        engine.set_weights(w)
        logits, grad, losses = engine.batch(x, y)
    assert rel(logits.reshape(-1, 256), fixture["logits"]) < 1e-2
    assert abs(float(losses.mean()) - float(fixture["losses"].mean())) < 3e-3
    assert rel(grad[fixture["gradient_index"]], fixture["gradient_value"]) < 1e-2
    layout = orc.Layout(cfg)
    for (name, off, shape), want in zip(layout.entries, fixture["gradient_norms"]):
        got = np.linalg.norm(grad[off:off + int(np.prod(shape))].astype(np.float64))
        assert abs(got - want) <= 2e-2 * want + 1e-9, name
