"""The reference's own width-16 network behind the plain Config, through the tg_* C ABI, checked with
the procedure and tolerances of the reference's tests/verify.py against the CPU checker
(oracle/width16.py) in the place of its PyTorch model: logits 0.005, gradients 0.01 (0.02 per tensor),
per-position losses atol 0.003, AdamW-owned weights atol 2e-6, Muon part 0.04; bit-exact causality,
batch independence and launch-size independence."""
import ctypes as C

import numpy as np
import pytest

from oracle import width16 as w16
from turbogpt_amd import bridge

pytestmark = pytest.mark.gpu


def relative(a, b):
    return float(np.linalg.norm(np.asarray(a, np.float64) - b) / max(np.linalg.norm(b), 1e-12))


def reference_style_weights(depth, seed=42, scale=0.08):
    """The initialisation shape of tests/reference.py:27-38: unit scales, N(0, scale) matrices, the two
    residual projections divided by sqrt(2 depth)."""
    rng = np.random.default_rng(seed)
    entries, count = w16.layout(depth)
    flat = np.zeros(count, np.float32)
    for name, (offset, shape) in entries.items():
        n = int(np.prod(shape))
        if w16.is_scale(name):
            flat[offset:offset + n] = 1.0
        else:
            value = rng.standard_normal(n) * scale
            if name.endswith(("attention", "down")):
                value /= np.sqrt(2 * depth)
            flat[offset:offset + n] = value
    return flat


# tests/verify.py:204-208
@pytest.mark.parametrize("depth,context,batch", [(4, 4, 16), (4, 8, 16), (8, 4, 16), (8, 8, 16), (4, 4, 4),
                                                 (4, 4, 12), (8, 8, 12), (4, 8, 2560)])
def test_model_against_the_checker(depth, context, batch):
    cfg = bridge.Config(depth=depth, context=context, batch=batch)
    flat = reference_style_weights(depth)
    checker = w16.Width16(depth, context, batch)
    with bridge.Native(cfg) as engine:
        assert engine.count == w16.parameter_count(depth)
        engine.set_weights(flat)
        rng = np.random.default_rng(71)
        x = rng.integers(0, 256, (batch, context), dtype=np.uint8)
        y = rng.integers(0, 256, x.shape, dtype=np.uint8)
        logits, gradients, losses = engine.batch(x, y)
        target, expected_grad, expected_losses = checker.batch(flat, x, y)
        print(f"depth={depth} ctx={context} batch={batch}: logits rel={relative(logits, target):.3g}; "
              f"grad rel={relative(gradients, expected_grad):.3g}", flush=True)
        np.testing.assert_allclose(losses, expected_losses, atol=.003, rtol=.001)
        assert relative(logits, target) < .005
        assert relative(gradients, expected_grad) < .01
        for name, (offset, shape) in checker.entries.items():
            n = int(np.prod(shape))
            part = relative(gradients[offset:offset + n], expected_grad[offset:offset + n])
            assert part < .02, (name, part)
        if batch > 64:
            return
        # every prefix, and cross-example independence (tests/verify.py:43-50)
        for pos in range(context - 1):
            changed = x.copy()
            changed[:, pos + 1:] = rng.integers(0, 256, changed[:, pos + 1:].shape, dtype=np.uint8)
            later = engine.batch(changed, y, False)[0]
            np.testing.assert_array_equal(logits[:, :pos + 1], later[:, :pos + 1])
        changed = x.copy()
        changed[1:] = rng.integers(0, 256, changed[1:].shape, dtype=np.uint8)
        np.testing.assert_array_equal(logits[0], engine.batch(changed, y, False)[0][0])
        # a second identical call reproduces the gradient bit for bit (fixed-order folds, no atomics)
        np.testing.assert_array_equal(gradients, engine.batch(x, y)[1])


def adam_mask(depth):
    entries, _ = w16.layout(depth)
    return np.concatenate([np.full(int(np.prod(shape)), not w16.is_hidden_matrix(name)) for name, (_, shape) in entries.items()])


# tests/verify.py:63-105
@pytest.mark.parametrize("scheduled", [False, True])
def test_optimizer_pair(scheduled, orc):
    cfg = bridge.Config(batch=4, clip=0)
    initial = reference_style_weights(4, scale=0.02)
    checker = w16.Optimizer(4, clip=0)
    with bridge.Native(cfg) as engine:
        engine.set_weights(initial)
        if scheduled:
            engine.set_onecycle(20)
        rng = np.random.default_rng(192)
        w = initial.copy()
        for step in range(20):
            grad = (rng.standard_normal(engine.count) * .01).astype(np.float32)
            engine.check(engine.lib.tg_optimizer_test(engine.handle, grad.ctypes.data, 1))
            w = checker.update(w, grad, orc.onecycle_point(20, step) if scheduled else None)
        actual = engine.weights()
        if scheduled:  # the schedule is exhausted (tests/verify.py:147)
            assert engine.lib.tg_optimizer_test(engine.handle, grad.ctypes.data, 1) < 0
    a = adam_mask(4)
    error = relative(actual - initial, w - initial)
    adam_error = relative(actual[a] - initial[a], w[a] - initial[a])
    print(f"{'OneCycle ' if scheduled else ''}update rel={error:.3g}, AdamW part rel={adam_error:.3g}, "
          f"max abs={np.max(abs(actual - w)):.3g}", flush=True)
    assert error < .04
    assert adam_error < .0001
    np.testing.assert_allclose(actual[a], w[a], atol=2e-6, rtol=2e-5)


def test_optimizer_pair_with_clipping(orc):
    cfg = bridge.Config(batch=4, clip=0.05)
    initial = reference_style_weights(4, scale=0.02)
    checker = w16.Optimizer(4, clip=0.05)
    with bridge.Native(cfg) as engine:
        engine.set_weights(initial)
        rng = np.random.default_rng(7)
        w = initial.copy()
        for _ in range(5):
            grad = (rng.standard_normal(engine.count) * .01).astype(np.float32)  # norm about 1.5: clipped
            engine.check(engine.lib.tg_optimizer_test(engine.handle, grad.ctypes.data, 1))
            w = checker.update(w, grad)
        actual = engine.weights()
    a = adam_mask(4)
    assert relative(actual[a] - initial[a], w[a] - initial[a]) < .0005
    assert relative(actual - initial, w - initial) < .04


# tests/verify.py:108-127
def test_small_updates_are_retained():
    cfg = bridge.Config(batch=4, learning_rate=1e-5, weight_decay=0, clip=0)
    with bridge.Native(cfg) as engine:
        w = np.full(engine.count, .5, np.float32)
        g = np.full(engine.count, .01, np.float32)
        engine.set_weights(w)
        engine.check(engine.lib.tg_optimizer_test(engine.handle, g.ctypes.data, 64))
        actual = engine.weights()
    checker = w16.Optimizer(4, learning_rate=1e-5, weight_decay=0, clip=0)
    expected = w.copy()
    for _ in range(64):
        expected = checker.update(expected, g)
    a = adam_mask(4)
    np.testing.assert_allclose(actual[a], expected[a], atol=2e-6, rtol=0)
    assert np.max(abs(actual[a] - .5)) > .0005  # 64 sub-ulp steps moved a weight whose bf16 ulp is 2^-9


# tests/verify.py:130-148
@pytest.mark.parametrize("scheduled", [False, True])
def test_persistence(scheduled):
    cfg = bridge.Config(batch=32)
    flat = reference_style_weights(4, scale=0.02)
    data = np.random.default_rng(4).integers(0, 256, 4096, dtype=np.uint8)
    engines = [bridge.Native(cfg), bridge.Native(cfg)]
    try:
        for e in engines:
            e.set_weights(flat)
            e.set_data(data)
            if scheduled:
                e.set_onecycle(8)
        engines[0].train(8)
        for _ in range(8):
            engines[1].train(1)
        np.testing.assert_array_equal(engines[0].weights(), engines[1].weights())
        assert np.abs(engines[0].weights() - flat).max() > 1e-4
        if scheduled:
            assert engines[0].lib.tg_train(engines[0].handle, 1) < 0
            assert b"OneCycle" in engines[0].lib.tg_error()
    finally:
        for e in engines:
            e.close()


# tests/verify.py:151-176
@pytest.mark.parametrize("context", [4, 8])
def test_stream_evaluation(context):
    depth, batch = 8, 24
    if batch * context % 16:
        batch = 32
    cfg = bridge.Config(context=context, depth=depth, batch=batch, blocks=1)
    flat = reference_style_weights(depth, scale=0.02)
    data = np.random.default_rng(314).integers(0, 256, 4096, dtype=np.uint8)
    endpoints = np.array([8 + 17 * i for i in range(batch)], dtype=np.int64)
    x = np.stack([data[e - context:e] for e in endpoints])
    y = np.stack([data[e - context + 1:e + 1] for e in endpoints])
    checker = w16.Width16(depth, context, batch)
    expected = checker.token_losses(checker.forward(flat, x), y).mean(0)
    with bridge.Native(cfg) as engine:
        engine.set_weights(flat)
        engine.set_data(data)
        for _ in range(3):
            loss = engine.batch(x, y, False)[2]
            np.testing.assert_allclose(loss, expected, rtol=1e-6, atol=1e-6)


def test_training_follows_the_checker(orc):
    """Three optimizer steps of tg_train against the checker run on the same hash-sampled batches
    (cuda/dataset.cuh:13-27), and the recorded per-position losses (cuda/trainer.cuh:79-100)."""
    depth, context, batch = 4, 8, 32
    cfg = bridge.Config(depth=depth, context=context, batch=batch)
    flat = reference_style_weights(depth, scale=0.05)
    data = np.random.default_rng(11).integers(0, 256, 8192, dtype=np.uint8)
    checker = w16.Width16(depth, context, batch)
    optimizer = w16.Optimizer(depth)
    w, history = flat.copy(), []
    for step in range(3):
        x, y = orc.sample_batch(data, 3407, step, batch, context)
        _, grad, losses = checker.batch(w, x, y)
        history.append(losses)
        w = optimizer.update(w, grad)
    with bridge.Native(cfg) as engine:
        engine.set_weights(flat)
        engine.set_data(data)
        engine.train(3)
        recorded = engine.training_losses(3)
        actual = engine.weights()
        versions = np.empty(3, np.int32)
        engine.check(engine.lib.tg_training_versions(engine.handle, versions.ctypes.data, 3))
    np.testing.assert_array_equal(versions, [0, 1, 2])
    np.testing.assert_allclose(recorded, np.array(history), atol=.003, rtol=.001)
    assert relative(actual - flat, w - flat) < .05


def test_predict_is_the_last_position_of_a_batch():
    cfg = bridge.Config(depth=4, context=8, batch=16)
    flat = reference_style_weights(4)
    context = np.random.default_rng(2).integers(0, 256, 8, dtype=np.uint8)
    with bridge.Native(cfg) as engine:
        engine.set_weights(flat)
        predicted = engine.predict(context)
        x = np.tile(context, (16, 1))
        logits = engine.batch(x, np.zeros_like(x), False)[0]
    np.testing.assert_array_equal(predicted, logits[3, -1])
    expected = w16.Width16(4, 8, 1).forward(flat, context[None])[0, -1]
    assert relative(predicted, expected) < .005
