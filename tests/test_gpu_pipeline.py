"""Batches in flight (Config.inflight > 1): versioned weights, stale gradients, ordered updates.
The procedure of the reference's tests/pipeline.py: train in chunks, read the version each step used
(tg_training_versions), check the staleness bound, then replay the run serially - the gradient of every step
from a synchronous engine holding the recorded version, the update from a second synchronous engine - and
compare the final weights.  Here the schedule of versions is fixed on the host, so the replay must agree
to the last bit (the reference allows 0.002 of the update because its embedding atomics are unordered).
Every replayed step is also checked against the CPU checker, as tests/pipeline.py:79-121 checks it against
the independent PyTorch model: logits 0.005, gradient 0.02 as a whole and per parameter tensor, and the
checker's own optimizer fed with the engine's gradients ends within 0.01 of the total update."""
import ctypes as C

import numpy as np
import pytest

from oracle import width16 as w16
from turbogpt_amd import bridge
from test_gpu_width16 import reference_style_weights

pytestmark = pytest.mark.gpu


def relative(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


class Width16Checker:
    """The independent model and optimizer pair for an engine made from the plain Config (oracle/width16.py)."""

    def __init__(self, base, total):
        self.model = w16.Width16(base.depth, base.context, base.batch)
        self.optimizer = w16.Optimizer(base.depth, learning_rate=base.learning_rate, muon_lr=base.muon_lr, beta1=base.beta1,
                                       beta2=base.beta2, momentum=base.momentum, weight_decay=base.weight_decay,
                                       epsilon=base.epsilon, clip=base.clip, ns_steps=base.ns_steps)
        self.tensors = [(name, offset, int(np.prod(shape))) for name, (offset, shape) in self.model.entries.items()]
        self.total = total

    def batch(self, weights, x, y):
        logits, gradient, _ = self.model.batch(weights, x, y)
        return logits, gradient

    def update(self, orc, weights, gradient, step):
        return self.optimizer.update(weights, gradient, orc.onecycle_point(self.total, step))


class WideChecker:
    """The same for the softmax / LayerNorm / GELU model (oracle/tg_oracle.c): AdamW on every parameter."""

    def __init__(self, orc, cfg, total):
        base = cfg.base
        self.orc, self.base, self.total = orc, base, total
        self.cfg = orc.model(base.depth, base.context, base.batch, cfg.d_model, cfg.heads, cfg.vocab, cfg.ffn, cfg.ln_eps,
                             emulate=True)
        self.tensors = [(name, offset, int(np.prod(shape))) for name, offset, shape in orc.Layout(self.cfg).entries]
        self.mask = orc.decay_mask(self.cfg)
        self.m = self.v = None

    def batch(self, weights, x, y):
        logits, gradient, _ = self.orc.model_batch(self.cfg, weights, x, y)
        return logits, gradient

    def update(self, orc, weights, gradient, step):
        if self.m is None:
            self.m, self.v = np.zeros_like(weights), np.zeros_like(weights)
        multiplier, momentum = orc.onecycle_point(self.total, step)
        b = self.base
        scale = orc.clip_scale(gradient, b.clip) if b.clip > 0 else 1.0
        weights, self.m, self.v = orc.adamw(weights, self.m, self.v, gradient, self.mask,
                                            np.float32(b.learning_rate) * np.float32(multiplier), momentum, b.beta2, b.epsilon,
                                            b.weight_decay, scale, step)
        return weights


def run_and_replay(make_config, initial, orc, inflight):
    cfg = make_config(inflight)
    base = cfg if isinstance(cfg, bridge.Config) else cfg.base
    data = np.random.default_rng(718).integers(0, 256, 8192, dtype=np.uint8)
    chunks = [max(11, inflight + 5), max(9, inflight + 3)]  # slot reuse, launch boundaries, a partial tail
    total = sum(chunks)
    versions, history = [], []
    with bridge.Native(cfg) as engine:
        engine.set_weights(initial)
        engine.set_data(data)
        engine.set_onecycle(total)
        for count in chunks:
            engine.train(count)
            trace = np.empty(count, np.int32)
            engine.check(engine.lib.tg_training_versions(engine.handle, trace.ctypes.data, count))
            versions.extend(trace.tolist())
            history.append(engine.training_losses(count))
        actual = engine.weights()
        mean, maximum = C.c_double(), C.c_int()
        engine.check(engine.lib.tg_pipeline_stats(engine.handle, C.byref(mean), C.byref(maximum)))
        if inflight > 1:  # cuda/runtime.cu:357-358
            grad = np.zeros(engine.count, np.float32)
            assert engine.lib.tg_optimizer_test(engine.handle, grad.ctypes.data, 1) < 0
            assert b"synchronous" in engine.lib.tg_error()
    history = np.concatenate(history)
    for step, version in enumerate(versions):  # tests/pipeline.py:71
        assert max(0, step - inflight + 1) <= version <= step, (step, version, versions)
    assert maximum.value == max(s - v for s, v in enumerate(versions))
    assert mean.value == pytest.approx(np.mean([s - v for s, v in enumerate(versions)]))
    serial = make_config(1)
    checker = Width16Checker(base, total) if isinstance(cfg, bridge.Config) else WideChecker(orc, cfg, total)
    live = initial.copy()  # the checker's own optimizer, fed with the engine's gradients (tests/pipeline.py:107-118)
    worst_logits = worst_gradient = 0.0
    with bridge.Native(serial) as model_engine, bridge.Native(serial) as optimizer_engine:
        optimizer_engine.set_weights(initial)
        optimizer_engine.set_onecycle(total)
        snapshots = [initial]
        for step, version in enumerate(versions):
            x, y = orc.sample_batch(data, base.seed, step, base.batch, base.context)
            model_engine.set_weights(snapshots[version])
            logits, gradient, losses = model_engine.batch(x, y)
            np.testing.assert_allclose(history[step], losses, rtol=1e-6, atol=1e-6)
            # the same step on the independent model holding the recorded version: tests/pipeline.py:79-105
            want_logits, want_gradient = checker.batch(snapshots[version], x, y)
            logit_error, gradient_error = relative(logits, want_logits), relative(gradient, want_gradient)
            worst_logits, worst_gradient = max(worst_logits, logit_error), max(worst_gradient, gradient_error)
            assert logit_error < .005, (step, logit_error)
            assert gradient_error < .02, (step, gradient_error)
            for name, offset, count in checker.tensors:
                part = relative(gradient[offset:offset + count], want_gradient[offset:offset + count])
                assert part < .02, (step, name, part)
            optimizer_engine.optimizer_test(gradient)
            live = checker.update(orc, live, gradient, step)
            snapshots.append(optimizer_engine.weights())
    expected = snapshots[-1]
    error = np.linalg.norm(actual - expected) / np.linalg.norm(expected - initial)
    optimizer_error = np.linalg.norm(expected - live) / np.linalg.norm(expected - initial)
    print(f"inflight={inflight} versions={versions}; serial replay error={error:.3g}; checker logits={worst_logits:.3g}, "
          f"gradient={worst_gradient:.3g}, optimizer={optimizer_error:.3g}", flush=True)
    assert optimizer_error < .01, optimizer_error  # tests/pipeline.py:128
    return actual, expected, versions


@pytest.mark.parametrize("inflight,context,depth,batch", [(1, 4, 4, 16), (2, 4, 4, 16), (4, 4, 4, 16), (8, 4, 4, 16),
                                                          (16, 4, 4, 16), (4, 8, 8, 16), (2, 4, 4, 2560)])
def test_width16_pipeline_replays_serially(inflight, context, depth, batch, orc):
    initial = reference_style_weights(depth, scale=0.05)
    actual, expected, versions = run_and_replay(
        lambda k: bridge.Config(inflight=k, context=context, depth=depth, batch=batch), initial, orc, inflight)
    np.testing.assert_array_equal(actual, expected)
    if inflight > 1:
        assert versions[inflight:] == list(range(1, len(versions) - inflight + 1))  # the fixed schedule


@pytest.mark.parametrize("inflight", [2, 3])
def test_wide_model_pipeline_replays_serially(inflight, orc):
    make = lambda k: bridge.ModelConfig(d_model=256, depth=2, context=128, batch=4, inflight=k)
    count = orc.parameter_count(orc.model(2, 128, 4, 256, 4))
    initial = (np.random.default_rng(5).standard_normal(count) * 0.02).astype(np.float32)
    actual, expected, _ = run_and_replay(make, initial, orc, inflight)
    np.testing.assert_array_equal(actual, expected)


def test_pipeline_state_survives_resume(orc):
    """tg_set_optimizer_state moves the weights to the ring place of the resumed step: a run split by a
    get / set round trip through a fresh engine equals the unsplit one."""
    cfg = lambda: bridge.Config(inflight=3, context=8, depth=4, batch=16)
    initial = reference_style_weights(4, scale=0.05)
    data = np.random.default_rng(9).integers(0, 256, 4096, dtype=np.uint8)
    with bridge.Native(cfg()) as whole:
        whole.set_weights(initial)
        whole.set_data(data)
        whole.train(10)
        expected = whole.weights()
    with bridge.Native(cfg()) as first:
        first.set_weights(initial)
        first.set_data(data)
        first.train(4)
        weights, (m, v, step) = first.weights(), first.optimizer_state()
    assert step == 4
    with bridge.Native(cfg()) as second:
        second.set_weights(weights)
        second.set_optimizer_state(m, v, step)
        second.set_data(data)
        second.train(6)
        resumed = second.weights()
        trace = np.empty(6, np.int32)
        second.check(second.lib.tg_training_versions(second.handle, trace.ctypes.data, 6))
    # after a resume the first batches can only read the resumed version, so the split run is its own
    # schedule: bounded staleness, and a deterministic result
    assert trace.tolist() == [4, 4, 4, 5, 6, 7]
    assert np.isfinite(resumed).all() and np.abs(resumed - expected).max() < 0.05
