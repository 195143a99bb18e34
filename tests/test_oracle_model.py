"""Pins the CPU checker's full model (forward, backward, training step) against a GPT assembled
from torch library ops in fp64, with the acceptance rules of tests/verify.py:14-52."""
import numpy as np
import pytest

from torch_gpt import forward_backward


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


@pytest.fixture(scope="module")
def small(orc):
    cfg = orc.model(depth=2, context=16, batch=3, d_model=32, heads=2)
    rng = np.random.default_rng(71)
    w = orc.init_weights(cfg, seed=42, scale=0.08)  # larger scale makes errors visible (verify.py:16)
    lay = orc.Layout(cfg)
    for name, off, shape in lay.entries:  # make norm scales/biases non-trivial
        if name.endswith(("_g", "_b")):
            w[off:off + shape[0]] += rng.standard_normal(shape[0]).astype(np.float32) * 0.1
    x = rng.integers(0, 256, (cfg.batch, cfg.context), dtype=np.uint8)
    y = rng.integers(0, 256, x.shape, dtype=np.uint8)
    return cfg, lay, w, x, y


def test_layout_and_decay_mask(orc, small):
    cfg, lay, w, _, _ = small
    assert orc.parameter_count(cfg) == lay.count == w.size
    mask = orc.decay_mask(cfg)
    for name, off, shape in lay.entries:
        n = int(np.prod(shape))
        decays = len(shape) == 2 and name not in ("embedding", "positions")  # cuda/optim.cuh:5-15
        assert mask[off:off + n].all() == decays and mask[off:off + n].any() == decays, name


def test_model_matches_torch_fp64(orc, small):
    cfg, lay, w, x, y = small
    logits, grad, loss = orc.model_batch(cfg, w, x, y)
    want_logits, want_grad, want_loss = forward_backward(lay, w, x, y, cfg.heads)
    assert rel(logits, want_logits) < 1e-5
    np.testing.assert_allclose(loss, want_loss, rtol=1e-4, atol=1e-5)
    assert rel(grad, want_grad) < 1e-4
    for name, off, shape in lay.entries:  # every tensor on its own (verify.py:35-42)
        n = int(np.prod(shape))
        assert rel(grad[off:off + n], want_grad[off:off + n]) < 2e-4, name


def test_bf16_emulation_stays_within_the_device_tolerances(orc, small):
    cfg, lay, w, x, y = small
    emu = orc.model(cfg.depth, cfg.context, cfg.batch, cfg.d_model, cfg.heads, emulate=True)
    logits, grad, loss = orc.model_batch(emu, w, x, y)
    want_logits, want_grad, want_loss = orc.model_batch(cfg, w, x, y)
    # rounding at the device's store points moves results, but stays inside the 1e-2 budget that
    # the device path is held to against the fp32 checker
    assert 1e-5 < rel(logits, want_logits) < 1e-2
    assert rel(grad, want_grad) < 1e-2
    np.testing.assert_allclose(loss.mean(0), want_loss.mean(0), atol=3e-3, rtol=1e-3)


def test_model_is_causal_and_batch_independent(orc, small):
    cfg, _, w, x, y = small
    rng = np.random.default_rng(9)
    logits = orc.model_batch(cfg, w, x, y, backward=False)[0]
    for pos in (0, 5, 14):
        changed = x.copy()
        changed[:, pos + 1:] = rng.integers(0, 256, changed[:, pos + 1:].shape, dtype=np.uint8)
        later = orc.model_batch(cfg, w, changed, y, backward=False)[0]
        np.testing.assert_array_equal(logits[:, :pos + 1], later[:, :pos + 1])
    changed = x.copy()
    changed[1:] = rng.integers(0, 256, changed[1:].shape, dtype=np.uint8)
    np.testing.assert_array_equal(logits[0], orc.model_batch(cfg, w, changed, y, backward=False)[0][0])


def test_training_reduces_loss_and_chunks_compose(orc, small):
    cfg, _, w, _, _ = small
    data = orc.fill_zipf_bytes(4096, 71)
    z = np.zeros_like(w)
    args = dict(lr=3e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, clip=1.0)
    w8, m8, v8, l8 = orc.train(cfg, w, z, z, data, 3407, 0, 8, **args)
    assert l8[-1].mean() < l8[0].mean() - 0.2
    assert abs(l8[0].mean() - np.log(256)) < 0.5
    # 8 steps in one call == 8 calls of one step (verify.py:130-148)
    wa, ma, va = w, z, z
    for s in range(8):
        wa, ma, va, l1 = orc.train(cfg, wa, ma, va, data, 3407, s, 1, **args)
        np.testing.assert_array_equal(l1[0], l8[s])
    np.testing.assert_array_equal(wa, w8)
