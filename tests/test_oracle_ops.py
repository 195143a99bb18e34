"""Pins the CPU checker's operators against independent library routines (numpy fp64 matmul,
torch CPU fp64 ops + autograd, scipy) and against closed-form special cases.  The reference holds
no stored vectors for these; its tests compare live against PyTorch the same way
(tests/verify.py:14-52)."""
import numpy as np
import pytest
import torch
from torch.nn import functional as F


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def test_gemm_family_matches_fp64_and_adjoint_identities(orc):
    rng = np.random.default_rng(1)
    M, N, K = 48, 40, 72
    x, w, dy = rng.standard_normal((M, K)), rng.standard_normal((N, K)), rng.standard_normal((M, N))
    r = rng.standard_normal((M, N))
    y = orc.gemm_fwd(x, w)
    assert rel(y, x @ w.T) < 1e-6
    assert rel(orc.gemm_fwd(x, w, residual=r), x @ w.T + r) < 1e-6
    dx = orc.gemm_dgrad(dy, w)
    assert rel(dx, dy @ w) < 1e-6
    dw = orc.gemm_wgrad(dy, x)
    assert rel(dw, dy.T @ x) < 1e-6
    # <dY, X W^T> = <dY W, X> = <dY^T X, W>
    a = float(np.sum(dy * y.astype(np.float64)))
    assert abs(a - np.sum(dx.astype(np.float64) * x)) < 1e-3 * abs(a)
    assert abs(a - np.sum(dw.astype(np.float64) * w)) < 1e-3 * abs(a)
    # accumulate flag (cuda/ops.cuh:100-105)
    assert rel(orc.gemm_wgrad(dy, x, into=dw), 2 * (dy.T @ x)) < 1e-6
    # identity weight is a copy; one-hot row picks a column
    np.testing.assert_array_equal(orc.gemm_fwd(x, np.eye(K)), x.astype(np.float32))


def test_gemm_emulation_rounds_store_then_residual(orc):
    rng = np.random.default_rng(2)
    x = orc.bf16_round(rng.standard_normal((16, 32)))
    w = orc.bf16_round(rng.standard_normal((8, 32)))
    r = orc.bf16_round(rng.standard_normal((16, 8)))
    exact = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
    want = torch.from_numpy(exact).bfloat16() + torch.from_numpy(r).bfloat16()  # bf16 add, cuda/mma.cuh:96-97
    got = orc.gemm_fwd(x, w, residual=r, emulate=True)
    assert np.mean(got == want.float().numpy()) > 0.98  # fp32 vs fp64 accumulation can flip a tie


def torch_attention(qkv, B, H, T, hd, scale):
    d = H * hd
    q, k, v = [t.reshape(B, T, H, hd).transpose(1, 2) for t in qkv.reshape(B, T, 3 * d).split(d, -1)]
    s = (q @ k.transpose(-1, -2)) * scale
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(s, -1)
    o = torch.softmax(s, -1) @ v
    return o.transpose(1, 2).reshape(B * T, d), lse


@pytest.mark.parametrize("B,H,T,hd", [(2, 3, 17, 8), (1, 2, 64, 64)])
def test_attention_forward_backward_match_torch_fp64(orc, B, H, T, hd):
    rng = np.random.default_rng(3)
    d = H * hd
    qkv = rng.standard_normal((B * T, 3 * d))
    dout = rng.standard_normal((B * T, d))
    scale = 1 / np.sqrt(hd)
    tq = torch.tensor(qkv, dtype=torch.float64, requires_grad=True)
    o, lse = torch_attention(tq, B, H, T, hd, scale)
    (o * torch.tensor(dout)).sum().backward()
    got_o, got_lse = orc.attn_fwd(qkv, B, H, T, hd, scale)
    assert rel(got_o, o.detach().numpy()) < 1e-5
    np.testing.assert_allclose(got_lse, lse.detach().numpy(), rtol=1e-5, atol=1e-5)
    # library cross-check of the kernel itself
    q, k, v = [t.reshape(B, T, H, hd).transpose(1, 2) for t in tq.detach().reshape(B, T, 3 * d).split(d, -1)]
    sdpa = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)
    assert rel(got_o, sdpa.transpose(1, 2).reshape(B * T, d).numpy()) < 1e-5
    got_d = orc.attn_bwd(qkv, got_o, got_lse, dout, B, H, T, hd, scale)
    want = tq.grad.numpy()
    for part, name in enumerate("qkv"):
        assert rel(got_d[:, part * d:(part + 1) * d], want[:, part * d:(part + 1) * d]) < 2e-5, name


def test_attention_special_cases(orc):
    rng = np.random.default_rng(4)
    B, H, T, hd = 2, 2, 9, 4
    d = H * hd
    qkv = rng.standard_normal((B * T, 3 * d)).astype(np.float32)
    o, lse = orc.attn_fwd(qkv, B, H, T, hd, 0.5)
    # the first position attends to itself only: O = V, lse = its own score
    for b in range(B):
        np.testing.assert_allclose(o[b * T], qkv[b * T, 2 * d:], rtol=1e-6)
        for h in range(H):
            s = 0.5 * np.dot(qkv[b * T, h * hd:(h + 1) * hd], qkv[b * T, d + h * hd:d + (h + 1) * hd])
            assert lse[b, h, 0] == pytest.approx(s, rel=1e-5, abs=1e-6)
    # causality is exact: changing later tokens leaves earlier rows bit-identical (verify.py:43-50)
    changed = qkv.copy().reshape(B, T, 3 * d)
    changed[:, 5:] = rng.standard_normal(changed[:, 5:].shape)
    o2, lse2 = orc.attn_fwd(changed.reshape(B * T, 3 * d), B, H, T, hd, 0.5)
    np.testing.assert_array_equal(o.reshape(B, T, d)[:, :5], o2.reshape(B, T, d)[:, :5])
    np.testing.assert_array_equal(lse[:, :, :5], lse2[:, :, :5])
    # zero queries: uniform attention over the causal window = running mean of V
    flat = qkv.copy()
    flat[:, :d] = 0
    o3, lse3 = orc.attn_fwd(flat, B, H, T, hd, 0.5)
    v = flat[:, 2 * d:].reshape(B, T, d)
    want = np.cumsum(v, 1) / np.arange(1, T + 1)[None, :, None]
    np.testing.assert_allclose(o3.reshape(B, T, d), want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(lse3[0, 0], np.log(np.arange(1, T + 1)), rtol=1e-6, atol=1e-6)


def test_layernorm_matches_torch_fp64(orc):
    rng = np.random.default_rng(5)
    M, D = 37, 48
    x, dy = rng.standard_normal((M, D)) * 2 + 0.3, rng.standard_normal((M, D))
    g, b = rng.standard_normal(D), rng.standard_normal(D)
    tx = torch.tensor(x, requires_grad=True)
    tg, tb = torch.tensor(g, requires_grad=True), torch.tensor(b, requires_grad=True)
    y = F.layer_norm(tx, (D,), tg, tb, eps=1e-5)
    (y * torch.tensor(dy)).sum().backward()
    assert rel(orc.layernorm_fwd(x, g, b), y.detach().numpy()) < 1e-6
    dx, dg, db = orc.layernorm_bwd(x, dy, g)
    assert rel(dx, tx.grad.numpy()) < 1e-5
    assert rel(dg, tg.grad.numpy()) < 1e-5
    assert rel(db, tb.grad.numpy()) < 1e-5
    prior = rng.standard_normal((M, D))
    dx2, _, _ = orc.layernorm_bwd(x, dy, g, dx_in=prior)
    assert rel(dx2, tx.grad.numpy() + prior) < 1e-5


def test_gelu_matches_torch_and_scipy(orc):
    from scipy.special import erf
    u = np.linspace(-6, 6, 2001)
    da = np.random.default_rng(6).standard_normal(u.size)
    assert rel(orc.gelu_fwd(u), 0.5 * u * (1 + erf(u / np.sqrt(2)))) < 1e-6
    tu = torch.tensor(u, requires_grad=True)
    (F.gelu(tu) * torch.tensor(da)).sum().backward()
    assert rel(orc.gelu_bwd(u, da), tu.grad.numpy()) < 1e-6


def test_cross_entropy_matches_torch(orc):
    rng = np.random.default_rng(7)
    M, V = 50, 256
    logits = rng.standard_normal((M, V)) * 3
    y = rng.integers(0, V, M, dtype=np.uint8)
    tl = torch.tensor(logits, requires_grad=True)
    per = F.cross_entropy(tl, torch.tensor(y).long(), reduction="none")
    per.mean().backward()
    loss, dl = orc.cross_entropy(logits, y)
    np.testing.assert_allclose(loss, per.detach().numpy(), rtol=1e-5, atol=1e-5)
    assert rel(dl, tl.grad.numpy()) < 1e-5
    # uniform logits: loss = ln V
    loss, _ = orc.cross_entropy(np.zeros((3, V)), y[:3])
    np.testing.assert_allclose(loss, np.log(V), rtol=1e-6)


def test_adamw_matches_torch_and_keeps_small_updates(orc):
    # tests/verify.py:64-105 (AdamW part): 20 steps, N(0, 0.01) gradients, rng 192
    rng = np.random.default_rng(192)
    n = 4096
    w0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    decay = (np.arange(n) % 2).astype(np.uint8)
    pa = torch.nn.Parameter(torch.tensor(w0[decay == 0]))
    pb = torch.nn.Parameter(torch.tensor(w0[decay == 1]))
    opt = torch.optim.AdamW([{"params": [pa], "weight_decay": 0.0}, {"params": [pb], "weight_decay": 0.1}],
                            lr=6e-4, betas=(0.9, 0.95), eps=1e-8, foreach=False, fused=False)
    w, m, v = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(20):
        g = (rng.standard_normal(n) * 0.01).astype(np.float32)
        w, m, v = orc.adamw(w, m, v, g, decay, 6e-4, 0.9, 0.95, 1e-8, 0.1, 1.0, step)
        pa.grad, pb.grad = torch.tensor(g[decay == 0]), torch.tensor(g[decay == 1])
        opt.step()
    want = w0.copy()
    want[decay == 0], want[decay == 1] = pa.detach().numpy(), pb.detach().numpy()
    assert rel(w - w0, want - w0) < 1e-4
    np.testing.assert_allclose(w, want, atol=2e-6, rtol=2e-5)
    # tests/verify.py:108-127: w=.5, g=.01, lr=1e-5, 64 steps => moved by about 64*lr
    w, m, v = np.full(8, 0.5, np.float32), np.zeros(8, np.float32), np.zeros(8, np.float32)
    for step in range(64):
        w, m, v = orc.adamw(w, m, v, np.full(8, 0.01, np.float32), np.zeros(8, np.uint8), 1e-5, 0.9, 0.95, 1e-8,
                            0.0, 1.0, step)
    assert np.all(np.abs(w - 0.5) > 5e-4) and np.allclose(0.5 - w, 64e-5, rtol=0.02)


def test_clip_scale(orc):
    g = np.full(100, 0.5, np.float32)  # norm 5
    assert orc.clip_scale(g, 1.0) == pytest.approx(1.0 / (5 + 1e-6), rel=1e-6)
    assert orc.clip_scale(g, 10.0) == 1.0
    assert orc.clip_scale(g, 0.0) == 1.0
