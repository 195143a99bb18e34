"""BASELINE configs[3] (d768 L12 T1024 B16) and configs[4] (d1024 L24 H16 T4096 B4) at full size
through the tg_* C ABI, checked by properties that do not need the CPU checker at that size:
bit-exact causality (tests/verify.py:43-50), run-to-run determinism of training, a first loss near
ln 256 for N(0, 0.02) weights that falls under AdamW, and the flat-gradient identity
<grad, w> for the scale-free final LayerNorm."""
import numpy as np
import pytest

from turbogpt_amd.bridge import ModelConfig, Native

pytestmark = pytest.mark.gpu

CONFIGS = {
    "configs[3]": dict(d_model=768, depth=12, context=1024, batch=16, heads=12),
    "configs[4]": dict(d_model=1024, depth=24, context=4096, batch=4, heads=16),
}


def weights(count, cfg, seed):
    """N(0, 0.02) matrices, gamma = 1, beta = 0, in the flat order of include/tg_model.h."""
    d, L, T, F = cfg["d_model"], cfg["depth"], cfg["context"], 4 * cfg["d_model"]
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal(count, dtype=np.float32) * 0.02).astype(np.float32)
    at = 256 * d + T * d
    for _ in range(L):
        w[at:at + d], w[at + d:at + 2 * d] = 1.0, 0.0
        at += 2 * d + 3 * d * d + d * d
        w[at:at + d], w[at + d:at + 2 * d] = 1.0, 0.0
        at += 2 * d + 2 * F * d
    w[at:at + d], w[at + d:at + 2 * d] = 1.0, 0.0
    assert at + 2 * d + 256 * d == count
    return w


def zipf_bytes(n, seed, s=1.1):
    p = np.arange(1, 257, dtype=np.float64) ** -s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, np.random.default_rng(seed).random(n)), 255).astype(np.uint8)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_causality_and_gradient_identity_at_full_size(name):
    cfg = CONFIGS[name]
    B, T, d = cfg["batch"], cfg["context"], cfg["d_model"]
    with Native(ModelConfig(**cfg)) as engine:
        w = weights(engine.count, cfg, 3407)
        engine.set_weights(w)
        x = zipf_bytes(B * T, 71).reshape(B, T)
        y = np.roll(x, -1, axis=1)
        logits, grad, losses = engine.batch(x, y)
        assert np.isfinite(logits).all() and np.isfinite(grad).all()
        assert abs(float(losses.mean()) - np.log(256)) < 0.6  # ln 256 + half the logit variance
        # the final LayerNorm output does not change when its input is scaled, so the loss does not depend
        # on a common scale of (gamma_f, beta_f) only through the head: d loss / d log-scale of the head's
        # input equals <grad_head, W_head> = <grad_gamma_f, gamma_f> + <grad_beta_f, beta_f>
        head = slice(engine.count - 256 * d, engine.count)
        lnf = slice(engine.count - 256 * d - 2 * d, engine.count - 256 * d)
        lhs = float(np.dot(grad[head].astype(np.float64), w[head].astype(np.float64)))
        rhs = float(np.dot(grad[lnf].astype(np.float64), w[lnf].astype(np.float64)))
        assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs), 1e-3)
        # causality, bit for bit: changing the last token of every sequence leaves every earlier position alone
        x2 = x.copy()
        x2[:, -1] ^= 0x55
        logits2, _, _ = engine.batch(x2, y, backward=False)
        a = logits.reshape(B, T, 256)[:, :-1]
        b = logits2.reshape(B, T, 256)[:, :-1]
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
        assert not np.array_equal(logits.reshape(B, T, 256)[:, -1], logits2.reshape(B, T, 256)[:, -1])


@pytest.mark.parametrize("name", list(CONFIGS))
def test_training_is_deterministic_and_learns_at_full_size(name):
    cfg = CONFIGS[name]
    steps = 6
    data = zipf_bytes(1 << 22, 71)
    runs = []
    for _ in range(2):
        with Native(ModelConfig(learning_rate=3e-4, beta1=0.9, beta2=0.95, weight_decay=0.1, clip=1.0, seed=3407,
                                **cfg)) as engine:
            engine.set_weights(weights(engine.count, cfg, 3407))
            engine.set_data(data)
            engine.train(steps)
            runs.append(engine.training_losses(steps).copy())
    np.testing.assert_array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))
    per_step = runs[0].mean(1)
    assert np.isfinite(per_step).all()
    assert abs(per_step[0] - np.log(256)) < 0.6
    assert per_step[-1] < per_step[0] - 0.02  # six AdamW steps already lower the loss


def against_the_checker(orc, cfg, seed):
    """tg_batch of one sequence against the CPU checker on the same weights and tokens.  Returns the relative errors
    (logits, flat gradient, worst parameter tensor, mean loss) of the device against the fp32 checker, and the
    errors of the checker's own rounding variant (bf16 at the device's store points) against its fp32 self: the size
    of the rounding noise this depth and width produce, measured rather than assumed."""
    T, d = cfg["context"], cfg["d_model"]
    oc = orc.model(cfg["depth"], T, 1, d, cfg["heads"])
    with Native(ModelConfig(**cfg)) as engine:
        assert engine.count == orc.parameter_count(oc)
        w = weights(engine.count, cfg, seed)
        rng = np.random.default_rng(5)
        for name, offset, shape in orc.Layout(oc).entries:  # norm parameters off their defaults
            if name.endswith(("_g", "_b")):
                w[offset:offset + shape[0]] += rng.standard_normal(shape[0]).astype(np.float32) * 0.1
        engine.set_weights(w)
        x = zipf_bytes(T, 71).reshape(1, T)
        y = np.roll(x, -1, axis=1)
        logits, grad, losses = engine.batch(x, y)

    def rel(a, b):
        a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
        return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))

    def worst(g, want):
        return max((rel(g[o:o + int(np.prod(s))], want[o:o + int(np.prod(s))]), name)
                   for name, o, s in orc.Layout(oc).entries)

    want_logits, want_grad, want_loss = orc.model_batch(oc, w, x, y)
    rounding = orc.model(cfg["depth"], T, 1, d, cfg["heads"], emulate=True)
    noisy_logits, noisy_grad, _ = orc.model_batch(rounding, w, x, y)
    device = (rel(logits, want_logits), rel(grad, want_grad), worst(grad, want_grad),
              abs(float(losses.mean()) - float(want_loss.mean())))
    noise = (rel(noisy_logits, want_logits), rel(noisy_grad, want_grad), worst(noisy_grad, want_grad))
    return device, noise


def test_long_context_shape_against_the_checker(orc):
    """Two blocks of the long-context model (d1024 H16 T4096: the widths, tile shapes and attention loop of
    configs[4]; depth 2 and one sequence keep the CPU checker at a minute) through tg_batch against the checker:
    logits and the flat gradient to 1e-2, every parameter tensor's gradient to 2e-2, mean loss to 3e-3; and no
    further from the fp32 checker than bf16 rounding at the device's store points takes the checker itself."""
    cfg = dict(CONFIGS["configs[4]"], depth=2, batch=1)
    (logits, grad, worst, loss), noise = against_the_checker(orc, cfg, 99)
    print(f"long-context shape: logits {logits:.3g}, gradient {grad:.3g}, worst tensor {worst}; rounding noise of the "
          f"checker itself: logits {noise[0]:.3g}, gradient {noise[1]:.3g}, worst {noise[2]}", flush=True)
    assert logits < 1e-2 and grad < 1e-2 and worst[0] < 2e-2 and loss < 3e-3
    assert logits < 1.3 * noise[0] + 5e-4 and grad < 1.3 * noise[1] + 5e-4


def test_headline_shape_against_the_rounding_checker(orc):
    """The headline shape (d768 L12 H12 T1024, one sequence).  Twelve blocks of bf16 stores put the logits close to
    the 1e-2 bar against the fp32 checker; how much of that is rounding is measured, not assumed: the checker's own
    variant that rounds at the device's store points lands as far from its fp32 self.  (The two rounded computations
    cannot be held to each other more tightly - a different summation order flips bf16 ties and they drift apart like
    independent samples - so the bound is on the size of the error, not on the difference.)  An error on top of
    rounding shows as a device error beyond 1.3 x that noise."""
    cfg = dict(CONFIGS["configs[3]"], batch=1)
    (logits, grad, worst, loss), noise = against_the_checker(orc, cfg, 3407)
    print(f"headline shape: logits {logits:.3g}, gradient {grad:.3g}, worst tensor {worst}; rounding noise of the "
          f"checker itself: logits {noise[0]:.3g}, gradient {noise[1]:.3g}, worst {noise[2]}", flush=True)
    assert logits < 1.3 * noise[0] + 5e-4 and grad < 1.3 * noise[1] + 5e-4 and worst[0] < 1.3 * noise[2][0] + 1e-3


def test_headline_shape_against_the_checker(orc):
    """One sequence of the headline model (d768 L12 H12 T1024, the shape bench.py times at batch 16) through
    tg_batch against the CPU checker on the same weights and tokens: logits and the flat gradient to 1e-2,
    every parameter tensor's gradient to 2e-2, mean loss to 3e-3 (tests/verify.py:31-42 of the reference)."""
    cfg = dict(CONFIGS["configs[3]"], batch=1)
    T, d = cfg["context"], cfg["d_model"]
    oc = orc.model(cfg["depth"], T, 1, d, cfg["heads"])
    with Native(ModelConfig(**cfg)) as engine:
        assert engine.count == orc.parameter_count(oc)
        w = weights(engine.count, cfg, 3407)
        rng = np.random.default_rng(5)
        for name, offset, shape in orc.Layout(oc).entries:  # norm parameters off their defaults
            if name.endswith(("_g", "_b")):
                w[offset:offset + shape[0]] += rng.standard_normal(shape[0]).astype(np.float32) * 0.1
        engine.set_weights(w)
        x = zipf_bytes(T, 71).reshape(1, T)
        y = np.roll(x, -1, axis=1)
        logits, grad, losses = engine.batch(x, y)
    want_logits, want_grad, want_loss = orc.model_batch(oc, w, x, y)

    def rel(a, b):
        a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
        return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))

    assert rel(logits, want_logits) < 1e-2
    assert abs(float(losses.mean()) - float(want_loss.mean())) < 3e-3
    assert rel(grad, want_grad) < 1e-2
    worst = max((rel(grad[o:o + int(np.prod(s))], want_grad[o:o + int(np.prod(s))]), name)
                for name, o, s in orc.Layout(oc).entries)
    print(f"headline shape: logits {rel(logits, want_logits):.3g}, gradient {rel(grad, want_grad):.3g}, worst tensor {worst}",
          flush=True)
    assert worst[0] < 2e-2, worst
