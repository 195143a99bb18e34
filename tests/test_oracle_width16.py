"""Pins the CPU checker of the reference's width-16 network (oracle/width16.py) without importing
anything from the reference: finite differences, closed forms, the constants and known answers the
reference's sources hold, and library optimizers (torch.optim.AdamW / Muon, as tests/verify.py:52-105
uses them)."""
import math

import numpy as np
import pytest

from oracle import width16 as w16


def random_weights(depth, seed, scale=0.08):
    rng = np.random.default_rng(seed)
    entries, count = w16.layout(depth)
    flat = np.zeros(count, np.float32)
    for name, (offset, shape) in entries.items():
        n = int(np.prod(shape))
        if w16.is_scale(name):
            flat[offset:offset + n] = 1.0 + 0.1 * rng.standard_normal(n)
        else:
            flat[offset:offset + n] = scale * rng.standard_normal(n)
    return flat


def relative(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def test_layout_matches_the_reference_counts():
    # model.h:12-37: 21,648 parameters at depth 4 and 35,088 at depth 8
    assert w16.parameter_count(4) == 21648 and w16.parameter_count(8) == 35088
    entries, _ = w16.layout(4)
    assert entries["0.attention_norm"][0] == 4096 and entries["0.qkv"][0] == 4112
    assert entries["0.up"][0] == entries["0.gate"][0] + 768  # adjacent: one packed projection
    assert entries["head"][0] + 4096 == 21648


def test_rope_table_is_the_reference_constant_table():
    # cuda/attention.cuh:7-14
    cos_ref = [1.0, 0.5403022766113281, -0.416146844625473, -0.9899924993515015, -0.6536436080932617,
               0.28366219997406006, 0.9601702690124512, 0.7539022564888]
    sin_ref = [0.0, 0.8414709568023682, 0.9092974066734314, 0.14112000167369843, -0.756802499294281,
               -0.9589242935180664, -0.279415488243103, 0.6569865942001343]
    cos, sin = w16.rope_table(8)
    assert cos.dtype == np.float32
    np.testing.assert_array_equal(cos, np.array(cos_ref, dtype=np.float32))
    np.testing.assert_array_equal(sin, np.array(sin_ref, dtype=np.float32))


@pytest.mark.parametrize("depth,context,batch,seed", [(4, 8, 6, 11), (8, 4, 5, 12), (4, 4, 16, 13)])
def test_float64_model_equals_a_model_of_torch_library_ops(depth, context, batch, seed):
    """The float64 variant of the checker against the same network assembled only from torch library ops
    (tests/torch_width16.py) and differentiated by autograd: logits to 1e-9, every parameter tensor's
    gradient to 1e-6, per-position losses to 1e-9.  A wrong RoPE pairing, a wrong gate (gelu of the winning
    score), SiLU in the place of the up projection or a wrong head layout fails here; the rounded variant is
    tied to this one by test_rounded_model_tracks_the_exact_one."""
    import torch_width16
    rng = np.random.default_rng(seed)
    flat = random_weights(depth, seed).astype(np.float64)
    x = rng.integers(0, 256, (batch, context), dtype=np.uint8)
    y = rng.integers(0, 256, (batch, context), dtype=np.uint8)
    model = w16.Width16(depth, context, batch, exact=True)
    logits, grad, position_losses = model.batch(flat, x, y)
    want_logits, want_grad, want_losses = torch_width16.forward_backward(model.entries, flat, x, y, depth)
    assert relative(logits, want_logits) < 1e-9
    np.testing.assert_allclose(position_losses, want_losses.mean(0), rtol=0, atol=1e-9)
    for name, (offset, shape) in model.entries.items():
        n = int(np.prod(shape))
        assert relative(grad[offset:offset + n], want_grad[offset:offset + n]) < 1e-6, name


def test_rounding_helpers():
    x = np.array([1.0, 1.00390625, 1.005859375, 3.14159265, -2.71828], np.float32)
    # 1 + 2^-8 is a tie between 1.0 and 1 + 2^-7: nearest even keeps 1.0; 1 + 3*2^-9 rounds up
    np.testing.assert_array_equal(w16.rn(x)[:3], np.array([1.0, 1.0, 1.0078125], np.float32))
    assert w16.truncate(np.array([3.14159265], np.float32))[0] == np.float32(3.140625)
    import torch
    big = np.random.default_rng(0).standard_normal(4096).astype(np.float32) * 37
    np.testing.assert_array_equal(w16.rn(big), torch.tensor(big).bfloat16().float().numpy())


@pytest.mark.parametrize("depth,context", [(4, 4), (8, 8)])
def test_backward_against_finite_differences(depth, context):
    model = w16.Width16(depth, context, batch=4, exact=True)
    rng = np.random.default_rng(5 + depth)
    flat = random_weights(depth, seed=depth).astype(np.float64)
    x = rng.integers(0, 256, (4, context), dtype=np.uint8)
    y = rng.integers(0, 256, (4, context), dtype=np.uint8)
    _, grad, _ = model.batch(flat, x, y)
    checked = 0
    for name, (offset, shape) in model.entries.items():
        n = int(np.prod(shape))
        if name == "embedding":  # only rows that occur carry a gradient
            picks = [offset + int(x[0, 0]) * 16 + 3, offset + int(x[2, 1]) * 16 + 11]
        else:
            picks = offset + rng.choice(n, size=2, replace=False)
        for i in picks:
            eps = 1e-6
            hi, lo = flat.copy(), flat.copy()
            hi[i] += eps
            lo[i] -= eps
            numeric = (model.mean_loss(hi, x, y) - model.mean_loss(lo, x, y)) / (2 * eps)
            assert numeric == pytest.approx(grad[i], rel=2e-5, abs=1e-9), (name, i)
            checked += 1
    assert checked >= 2 * len(model.entries)


def test_rounded_model_tracks_the_exact_one():
    depth, context, batch = 4, 8, 16
    flat = random_weights(depth, seed=42)
    rng = np.random.default_rng(71)
    x = rng.integers(0, 256, (batch, context), dtype=np.uint8)
    y = rng.integers(0, 256, (batch, context), dtype=np.uint8)
    rounded = w16.Width16(depth, context, batch)
    exact = w16.Width16(depth, context, batch, exact=True)
    # the exact model sees the same truncated matrices, so the difference is activation rounding alone
    entries, _ = w16.layout(depth)
    seen = flat.copy()
    for name, (offset, shape) in entries.items():
        if not w16.is_scale(name):
            n = int(np.prod(shape))
            seen[offset:offset + n] = w16.truncate(flat[offset:offset + n])
    # a rounding error can flip an arg-max between two nearly tied keys, which changes the graph: compare
    # the sequences whose selections agree in every layer (most of them)
    _, (_, saved, _, _) = rounded.forward(flat, x, keep=True)
    _, (_, saved64, _, _) = exact.forward(seen.astype(np.float64), x, keep=True)
    same = np.ones(batch, bool)
    for a, b in zip(saved, saved64):
        same &= (a["selected"] == b["selected"]).all(axis=(1, 2))
    assert same.sum() >= batch // 2
    logits, grad, losses = rounded.batch(flat, x[same], y[same])
    logits64, grad64, losses64 = exact.batch(seen.astype(np.float64), x[same], y[same])
    assert relative(logits, logits64) < 0.01
    assert relative(grad, grad64) < 0.02
    np.testing.assert_allclose(losses, losses64, atol=0.01)
    assert logits.dtype == np.float32 and np.array_equal(logits, w16.rn(logits))  # bf16-valued logits


def test_first_key_wins_ties_and_the_graph_is_causal():
    depth, context, batch = 4, 8, 4
    model = w16.Width16(depth, context, batch)
    flat = random_weights(depth, seed=9)
    entries, _ = w16.layout(depth)
    tied = flat.copy()
    off, shape = entries["0.qkv"]
    tied[off:off + 48 * 16] = 0  # all scores of layer 0 are 0: every query must pick the first key
    x = np.random.default_rng(3).integers(0, 256, (batch, context), dtype=np.uint8)
    _, (_, saved, _, _) = model.forward(tied, x, keep=True)
    assert not saved[0]["selected"].any()
    logits = model.forward(flat, x)
    rng = np.random.default_rng(4)
    for pos in range(context - 1):
        changed = x.copy()
        changed[:, pos + 1:] = rng.integers(0, 256, changed[:, pos + 1:].shape, dtype=np.uint8)
        np.testing.assert_array_equal(logits[:, :pos + 1], model.forward(flat, changed)[:, :pos + 1])


def torch_optimizers(flat, depth, **cfg):
    import torch
    entries, _ = w16.layout(depth)
    params, groups, matrices = {}, [], []
    for name, (offset, shape) in entries.items():
        p = torch.nn.Parameter(torch.tensor(flat[offset:offset + int(np.prod(shape))].reshape(shape)))
        params[name] = p
        if w16.is_hidden_matrix(name):
            matrices.append(p)
        else:
            groups.append({"params": [p], "weight_decay": cfg["weight_decay"] if name == "head" else 0})
    adam = torch.optim.AdamW(groups, lr=cfg["learning_rate"], betas=(cfg["beta1"], cfg["beta2"]), eps=cfg["epsilon"],
                             foreach=False, fused=False)
    muon = torch.optim.Muon(matrices, lr=cfg["muon_lr"], momentum=cfg["momentum"], weight_decay=cfg["weight_decay"],
                            ns_steps=cfg["ns_steps"])
    return params, adam, muon


def test_optimizer_pair_against_torch_adamw_and_muon():
    """The procedure of tests/verify.py:63-105 with the checker in the engine's place."""
    import torch
    depth = 4
    cfg = dict(learning_rate=0.0006, muon_lr=0.02, beta1=0.9, beta2=0.95, momentum=0.95, weight_decay=0.1,
               epsilon=1e-8, ns_steps=5)
    entries, count = w16.layout(depth)
    initial = random_weights(depth, seed=42, scale=0.02)
    params, adam, muon = torch_optimizers(initial, depth, **cfg)
    ours = w16.Optimizer(depth, clip=0, **cfg)
    w = initial.copy()
    rng = np.random.default_rng(192)
    for _ in range(20):
        grad = (rng.standard_normal(count) * 0.01).astype(np.float32)
        w = ours.update(w, grad)
        for name, (offset, shape) in entries.items():
            params[name].grad = torch.tensor(grad[offset:offset + int(np.prod(shape))].reshape(shape))
        adam.step()
        muon.step()
    expected = np.concatenate([params[name].detach().numpy().reshape(-1) for name in entries])
    mask = np.concatenate([np.full(int(np.prod(shape)), not w16.is_hidden_matrix(name)) for name, (_, shape) in entries.items()])
    assert relative(w[mask] - initial[mask], expected[mask] - initial[mask]) < 1e-4
    np.testing.assert_allclose(w[mask], expected[mask], atol=2e-6, rtol=2e-5)
    assert relative(w - initial, expected - initial) < 0.04  # bf16 Newton-Schulz against torch's


def test_newton_schulz_orthogonalises():
    rng = np.random.default_rng(1)
    for shape in ((48, 16), (16, 16), (16, 48)):
        o = w16.newton_schulz(rng.standard_normal(shape).astype(np.float32), 5).astype(np.float64)
        singular = np.linalg.svd(o, compute_uv=False)
        assert singular.min() > 0.3 and singular.max() < 1.3  # the quintic's plateau, as in Muon
        assert o.shape == shape


def test_small_updates_known_answer():
    # tests/verify.py:108-127: w = 0.5, g = 0.01, lr = 1e-5, no decay, no clip: 64 steps move the AdamW-owned
    # weights by about 64 * lr although one bf16 ulp at 0.5 is 2^-9
    depth = 4
    entries, count = w16.layout(depth)
    opt = w16.Optimizer(depth, learning_rate=1e-5, weight_decay=0, clip=0)
    w = np.full(count, 0.5, np.float32)
    g = np.full(count, 0.01, np.float32)
    for _ in range(64):
        w = opt.update(w, g)
    off, shape = entries["embedding"]
    moved = 0.5 - w[off:off + 16]
    assert np.all(moved > 5e-4) and np.allclose(moved, 64e-5, rtol=0.02)
