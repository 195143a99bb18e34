"""Batches in flight (Config.inflight > 1): versioned weights, stale gradients, ordered updates.
The procedure of the reference's tests/pipeline.py: train in chunks, read the version each step used
(tg_training_versions), check the staleness bound, then replay the run serially - the gradient of every step
from a synchronous engine holding the recorded version, the update from a second synchronous engine - and
compare the final weights.  Here the schedule of versions is fixed on the host, so the replay must agree
to the last bit (the reference allows 0.002 of the update because its embedding atomics are unordered)."""
import ctypes as C

import numpy as np
import pytest

from turbogpt_amd import bridge
from test_gpu_width16 import reference_style_weights

pytestmark = pytest.mark.gpu


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
    with bridge.Native(serial) as model_engine, bridge.Native(serial) as optimizer_engine:
        optimizer_engine.set_weights(initial)
        optimizer_engine.set_onecycle(total)
        snapshots = [initial]
        for step, version in enumerate(versions):
            x, y = orc.sample_batch(data, base.seed, step, base.batch, base.context)
            model_engine.set_weights(snapshots[version])
            _, gradient, losses = model_engine.batch(x, y)
            np.testing.assert_allclose(history[step], losses, rtol=1e-6, atol=1e-6)
            optimizer_engine.optimizer_test(gradient)
            snapshots.append(optimizer_engine.weights())
    expected = snapshots[-1]
    error = np.linalg.norm(actual - expected) / np.linalg.norm(expected - initial)
    print(f"inflight={inflight} versions={versions}; serial replay error={error:.3g}", flush=True)
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
