"""GPU parity of the HBM-bound operators (embedding, LayerNorm, cross-entropy, AdamW on hi/lo
weights, sampling, loss means) against the CPU checker, through the C ABI.  bf16 outputs are held
to relative L2 <= 1e-2 (and to agreement with the checker's bf16-rounding mode); fp32 outputs to
1e-5; integer/byte results bit-exactly."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import check, host, library, rel, stream, sync, to_bf16_device

pytestmark = pytest.mark.gpu


def dev(a, dtype=None):
    return torch.from_numpy(np.ascontiguousarray(a if dtype is None else a.astype(dtype))).cuda()


def hilo(orc, w):
    hi, lo = orc.split_hilo(w)
    return dev(hi.view(np.int16)), dev(lo.view(np.int16))


@pytest.mark.parametrize("B,T,D", [(2, 128, 256), (3, 64, 768), (9, 256, 128), (2, 50, 64), (5, 1000, 320)])
def test_embedding_forward_and_backward(orc, B, T, D):
    lib = library()
    rng = np.random.default_rng(B + T + D)
    table, th = to_bf16_device(rng.standard_normal((256, D)))
    pos, ph = to_bf16_device(rng.standard_normal((T, D)))
    x = orc.fill_zipf_bytes(B * T, 71)  # repeated symbols exercise the gather-sum
    xd = dev(x)
    out = torch.empty(B * T, D, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_embed_fwd(stream(), B * T, T, D, xd.data_ptr(), table.data_ptr(), pos.data_ptr(), out.data_ptr()))
    sync()
    want = orc.bf16_round(th[x] + np.tile(ph, (B, 1)))
    np.testing.assert_array_equal(host(out), want)
    dh, dhh = to_bf16_device(rng.standard_normal((B * T, D)))
    dt = torch.full((256, D), 1.0, dtype=torch.float32, device="cuda")
    dp = torch.full((T, D), 1.0, dtype=torch.float32, device="cuda")
    need = lib.tgk_embed_bwd_workspace(B * T, D)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    check(lib.tgk_embed_bwd(stream(), B, T, D, 256, xd.data_ptr(), dh.data_ptr(), dt.data_ptr(), dp.data_ptr(), 0,
                            ws.data_ptr(), need))
    sync()
    want_t = np.zeros((256, D), np.float64)
    np.add.at(want_t, x, dhh.astype(np.float64))
    assert rel(host(dt), want_t) < 1e-6
    assert rel(host(dp), dhh.reshape(B, T, D).astype(np.float64).sum(0)) < 1e-6
    check(lib.tgk_embed_bwd(stream(), B, T, D, 256, xd.data_ptr(), dh.data_ptr(), dt.data_ptr(), dp.data_ptr(), 1,
                            ws.data_ptr(), need))
    sync()
    assert rel(host(dt), 2 * want_t) < 1e-6
    # the two-part form: the exact one-hot matrix (its product with dh is the table gradient) and the same positions
    onehot = torch.full((B * T, 256), 7.0, dtype=torch.bfloat16, device="cuda")
    dp2 = torch.full((T, D), 1.0, dtype=torch.float32, device="cuda")
    check(lib.tgk_embed_bwd_onehot(stream(), B, T, D, xd.data_ptr(), dh.data_ptr(), onehot.data_ptr(), dp2.data_ptr(), 0))
    sync()
    want_hot = np.zeros((B * T, 256), np.float32)
    want_hot[np.arange(B * T), x] = 1.0
    np.testing.assert_array_equal(onehot.float().cpu().numpy(), want_hot)
    check(lib.tgk_embed_bwd(stream(), B, T, D, 256, xd.data_ptr(), dh.data_ptr(), dt.data_ptr(), dp.data_ptr(), 0,
                            ws.data_ptr(), need))
    sync()
    assert torch.equal(dp2, dp)


@pytest.mark.parametrize("M,D", [(64, 256), (333, 768), (128, 1024), (16, 2048)])
def test_layernorm_forward_backward(orc, M, D):
    lib = library()
    rng = np.random.default_rng(M + D)
    x, xh = to_bf16_device(rng.standard_normal((M, D)) * 2 + 0.5)
    dy, dyh = to_bf16_device(rng.standard_normal((M, D)))
    gamma = (1 + 0.2 * rng.standard_normal(D)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(D)).astype(np.float32)
    gh, gl = hilo(orc, gamma)
    bh, bl = hilo(orc, beta)
    y = torch.empty(M, D, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_layernorm_fwd(stream(), M, D, x.data_ptr(), gh.data_ptr(), gl.data_ptr(), bh.data_ptr(),
                                bl.data_ptr(), y.data_ptr(), 1e-5))
    sync()
    assert rel(host(y), orc.layernorm_fwd(xh, gamma, beta)) < 1e-2
    assert np.mean(host(y) == orc.layernorm_fwd(xh, gamma, beta, emulate=True)) > 0.98
    need = lib.tgk_layernorm_bwd_workspace(M, D)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    for residual in (0, 1):
        prior, ph = to_bf16_device(rng.standard_normal((M, D)))
        dx = prior.clone()
        dg = torch.full((D,), 2.0, dtype=torch.float32, device="cuda")
        db = torch.full((D,), 2.0, dtype=torch.float32, device="cuda")
        check(lib.tgk_layernorm_bwd(stream(), M, D, x.data_ptr(), dy.data_ptr(), gh.data_ptr(), gl.data_ptr(),
                                    dx.data_ptr(), dg.data_ptr(), db.data_ptr(), 1e-5, residual, residual,
                                    ws.data_ptr(), need))
        sync()
        want_dx, want_dg, want_db = orc.layernorm_bwd(xh, dyh, gamma, dx_in=ph if residual else None)
        assert rel(host(dx), want_dx) < 1e-2
        base = 2.0 if residual else 0.0  # accumulate flag follows residual in this test
        assert rel(host(dg) - base, want_dg) < 1e-4
        assert rel(host(db) - base, want_db) < 1e-4
        # the same with the residual gradient read from a buffer of its own, which stays untouched
        apart = torch.empty_like(dx)
        check(lib.tgk_layernorm_bwd_add(stream(), M, D, x.data_ptr(), dy.data_ptr(), gh.data_ptr(), gl.data_ptr(),
                                        prior.data_ptr() if residual else None, apart.data_ptr(), dg.data_ptr(),
                                        db.data_ptr(), 1e-5, 0, ws.data_ptr(), need))
        sync()
        assert torch.equal(apart, dx)
        assert np.array_equal(host(prior), ph)


def test_layernorm_backward_in_two_halves_equals_the_single_call(orc):
    """tgk_layernorm_bwd_rows for three LayerNorms, then ONE tgk_layernorm_bwd_fold: dx and the parameter gradients
    equal three tgk_layernorm_bwd_add calls bit for bit (same partial sums, same order of additions)."""
    lib = library()
    M, D, jobs = 333, 768, 3
    rng = np.random.default_rng(12)
    stride = lib.tgk_layernorm_bwd_workspace(M, D)
    partials = torch.empty(jobs * stride, dtype=torch.uint8, device="cuda")
    ws = torch.empty(stride, dtype=torch.uint8, device="cuda")
    got = torch.full((jobs, 2, D), 7.0, dtype=torch.float32, device="cuda")
    want = torch.full((jobs, 2, D), 7.0, dtype=torch.float32, device="cuda")
    table = torch.tensor([[got[j, 0].data_ptr(), got[j, 1].data_ptr()] for j in range(jobs)], dtype=torch.int64,
                         device="cuda")
    keep = []
    for j in range(jobs):
        x, _ = to_bf16_device(rng.standard_normal((M, D)) * (1 + j))
        dy, _ = to_bf16_device(rng.standard_normal((M, D)))
        residual, _ = to_bf16_device(rng.standard_normal((M, D)))
        gh, gl = hilo(orc, (1 + 0.2 * rng.standard_normal(D)).astype(np.float32))
        dx_a, dx_b = torch.empty_like(x), torch.empty_like(x)
        with_residual = residual.data_ptr() if j != 1 else None
        check(lib.tgk_layernorm_bwd_rows(stream(), M, D, x.data_ptr(), dy.data_ptr(), gh.data_ptr(), gl.data_ptr(),
                                         with_residual, dx_a.data_ptr(), 1e-5, partials.data_ptr() + j * stride, stride))
        check(lib.tgk_layernorm_bwd_add(stream(), M, D, x.data_ptr(), dy.data_ptr(), gh.data_ptr(), gl.data_ptr(),
                                        with_residual, dx_b.data_ptr(), want[j, 0].data_ptr(), want[j, 1].data_ptr(), 1e-5, 0,
                                        ws.data_ptr(), stride))
        keep.append((x, dy, residual, gh, gl, dx_a, dx_b))
    check(lib.tgk_layernorm_bwd_fold(stream(), M, D, jobs, partials.data_ptr(), stride, table.data_ptr(), 0))
    sync()
    for _, _, _, _, _, dx_a, dx_b in keep:
        assert torch.equal(dx_a, dx_b)
    assert torch.equal(got, want) and float(got.abs().sum()) > 0 and not bool((got == 7.0).any())
    # accumulate adds to what is there
    check(lib.tgk_layernorm_bwd_fold(stream(), M, D, jobs, partials.data_ptr(), stride, table.data_ptr(), 1))
    sync()
    assert torch.equal(got, want + want)
    # a job stride below one LayerNorm's partial block is refused on the host
    assert lib.tgk_layernorm_bwd_fold(stream(), M, D, jobs, partials.data_ptr(), stride - 16, table.data_ptr(), 0) == -1


def test_cross_entropy_loss_logits_and_gradient(orc):
    lib = library()
    rng = np.random.default_rng(17)
    M = 1000
    logits, lh = to_bf16_device(rng.standard_normal((M, 256)) * 3)
    y = rng.integers(0, 256, M, dtype=np.uint8)
    yd = dev(y)
    loss = torch.empty(M, dtype=torch.float32, device="cuda")
    f32 = torch.empty(M, 256, dtype=torch.float32, device="cuda")
    work = logits.clone()
    check(lib.tgk_cross_entropy(stream(), M, 256, work.data_ptr(), yd.data_ptr(), loss.data_ptr(), f32.data_ptr(),
                                1.0 / M, 0))
    sync()
    want_loss, want_grad = orc.cross_entropy(lh, y)
    np.testing.assert_allclose(host(loss), want_loss, rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(host(f32), lh)
    assert torch.equal(work, logits)  # evaluation mode leaves the logits alone
    check(lib.tgk_cross_entropy(stream(), M, 256, work.data_ptr(), yd.data_ptr(), loss.data_ptr(), None, 1.0 / M, 1))
    sync()
    assert rel(host(work), want_grad) < 1e-2
    assert rel(host(work), orc.cross_entropy(lh, y, emulate=True)[1]) < 1e-3


def run_adamw(orc, w, m, v, g, bounds, flags, steps, clip, lr=6e-4, wd=0.1):
    lib = library()
    n = w.size
    hi, lo = hilo(orc, w)
    md, vd = dev(m), dev(v)
    bd, fd = dev(np.asarray(bounds, np.int64)), dev(np.asarray(flags, np.uint8))
    parts = torch.empty(1024, dtype=torch.float32, device="cuda")
    for step, grad in enumerate(g[:steps]):
        gd = dev(grad)
        check(lib.tgk_sumsq_partials(stream(), gd.data_ptr(), n, parts.data_ptr(), 1024))
        check(lib.tgk_adamw(stream(), n, hi.data_ptr(), lo.data_ptr(), md.data_ptr(), vd.data_ptr(), gd.data_ptr(),
                            parts.data_ptr(), 1024, bd.data_ptr(), fd.data_ptr(), len(bounds), lr, 0.9, 0.95, 1e-8,
                            wd, clip, step))
        sync()
    out = orc.join_hilo(hi.cpu().numpy().view(np.uint16), lo.cpu().numpy().view(np.uint16))
    return out, md.cpu().numpy(), vd.cpu().numpy()


def test_sums_of_squares_over_a_list_of_ranges():
    """tgk_sumsq_segments: one partial per range, equal to numpy's sum over that range; ranges of every length class
    (shorter than a block's stride, not a multiple of it, many strides long), NaN outside the ranges."""
    lib = library()
    rng = np.random.default_rng(11)
    g = rng.standard_normal(200_000).astype(np.float32)
    ranges = [(0, 4), (8, 1536), (4096, 8192), (20_000, 8188), (100_000, 65_536)]
    masked = np.full_like(g, np.nan)
    for start, length in ranges:
        masked[start:start + length] = g[start:start + length]
    gd = dev(masked)
    rd = dev(np.asarray(ranges, np.int64))
    parts = torch.full((len(ranges),), float("nan"), dtype=torch.float32, device="cuda")
    check(lib.tgk_sumsq_segments(stream(), gd.data_ptr(), rd.data_ptr(), len(ranges), parts.data_ptr()))
    sync()
    want = [float((g[a:a + n].astype(np.float64) ** 2).sum()) for a, n in ranges]
    np.testing.assert_allclose(parts.cpu().numpy(), want, rtol=2e-6)
    assert lib.tgk_sumsq_segments(stream(), gd.data_ptr(), None, 1, parts.data_ptr()) == -1
    assert lib.tgk_sumsq_segments(stream(), gd.data_ptr(), rd.data_ptr(), 0, parts.data_ptr()) == -1


@pytest.mark.parametrize("clip", [0.0, 1.0])
def test_adamw_matches_the_checker_over_20_steps(orc, clip):
    # tests/verify.py:64-105 (AdamW part): N(0, 0.01) gradients from default_rng(192)
    rng = np.random.default_rng(192)
    n = 40960
    bounds, flags = [0, 4096, 8192, 30000], [0, 1, 0, 1]
    decay = np.zeros(n, np.uint8)
    decay[4096:8192] = 1
    decay[30000:] = 1
    w0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    grads = [(rng.standard_normal(n) * (0.01 if clip == 0 else 0.05)).astype(np.float32) for _ in range(20)]
    got, gm, gv = run_adamw(orc, w0, np.zeros(n, np.float32), np.zeros(n, np.float32), grads, bounds, flags, 20, clip)
    w, m, v = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step, g in enumerate(grads):
        w, m, v = orc.adamw(w, m, v, g, decay, 6e-4, 0.9, 0.95, 1e-8, 0.1, orc.clip_scale(g, clip), step)
    assert rel(got - w0, w - w0) < 1e-4              # verify.py:101
    np.testing.assert_allclose(got, w, atol=2e-6, rtol=2e-5)  # verify.py:103
    np.testing.assert_allclose(gm, m, rtol=1e-4, atol=1e-9)
    np.testing.assert_allclose(gv, v, rtol=1e-4, atol=1e-12)


def test_adamw_keeps_updates_below_one_bf16_ulp(orc):
    # tests/verify.py:108-127: w=.5, g=.01, lr=1e-5, 64 steps; plain bf16 would stall at .5
    n = 4096
    grads = [np.full(n, 0.01, np.float32)] * 64
    got, _, _ = run_adamw(orc, np.full(n, 0.5, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32),
                          grads, [0], [0], 64, 0.0, lr=1e-5, wd=0.0)
    assert np.max(np.abs(got - 0.5)) > 5e-4
    np.testing.assert_allclose(0.5 - got, 64e-5, rtol=0.02)
    plain = torch.tensor(0.5, dtype=torch.bfloat16)
    for _ in range(64):
        plain -= 1e-5
    assert plain.item() == 0.5


def test_sampling_and_position_means_are_exact(orc):
    lib = library()
    data = orc.fill_zipf_bytes(100000, 71)
    dd = dev(data)
    for batch, context, step in [(16, 4, 0), (12, 8, 5), (16, 1024, 3)]:
        x = torch.empty(batch, context, dtype=torch.uint8, device="cuda")
        y = torch.empty_like(x)
        check(lib.tgk_sample_batch(stream(), dd.data_ptr(), data.size, 3407, step, batch, context, x.data_ptr(),
                                   y.data_ptr()))
        sync()
        wx, wy = orc.sample_batch(data, 3407, step, batch, context)
        np.testing.assert_array_equal(x.cpu().numpy(), wx)
        np.testing.assert_array_equal(y.cpu().numpy(), wy)
    tl = np.random.default_rng(3).random((24, 256)).astype(np.float32)
    out = torch.empty(256, dtype=torch.float32, device="cuda")
    check(lib.tgk_position_means(stream(), dev(tl).data_ptr(), 24, 256, out.data_ptr()))
    sync()
    np.testing.assert_array_equal(host(out), (tl.astype(np.float64).sum(0) / 24).astype(np.float32))
