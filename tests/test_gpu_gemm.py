"""GPU parity of the bf16 MFMA GEMM family against the CPU checker, through the C ABI.
Tolerance: relative L2 error <= 1e-2 for bf16 outputs (the target's bar); fp32 wgrad is held to
1e-4.  Metric and thresholds follow tests/verify.py:10-11,32-33 of the reference."""
import numpy as np
import pytest
import torch

from gpu_util import check, host, library, rel, stream, sync, to_bf16_device

pytestmark = pytest.mark.gpu

SHAPES = [(128, 128, 64), (256, 256, 128), (256, 192, 192), (512, 384, 320), (384, 768, 64)]


def run_fwd(x, w, residual=None, gelu=False):
    lib = library()
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    g = torch.empty(M, N, dtype=torch.bfloat16, device="cuda") if gelu else None
    check(lib.tgk_gemm_fwd(stream(), M, N, K, x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
                           y.data_ptr(), y.stride(0), residual.data_ptr() if residual is not None else None,
                           residual.stride(0) if residual is not None else 0,
                           g.data_ptr() if gelu else None, N if gelu else 0))
    sync()
    return y, g


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_forward_plain_residual_gelu(orc, M, N, K):
    rng = np.random.default_rng(M + N + K)
    x, xh = to_bf16_device(rng.standard_normal((M, K)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)))
    r, rh = to_bf16_device(rng.standard_normal((M, N)) * 4)
    y, _ = run_fwd(x, w)
    assert rel(host(y), orc.gemm_fwd(xh, wh)) < 1e-2
    want = orc.gemm_fwd(xh, wh, emulate=True)
    assert np.mean(host(y) == want) > 0.99  # same bf16 values up to accumulation-order ties
    y, _ = run_fwd(x, w, residual=r)
    assert rel(host(y), orc.gemm_fwd(xh, wh, residual=rh)) < 1e-2
    assert np.mean(host(y) == orc.gemm_fwd(xh, wh, residual=rh, emulate=True)) > 0.99
    small, sh = to_bf16_device(rng.standard_normal((N, K)) / np.sqrt(K))
    y, g = run_fwd(x, small, gelu=True)
    pre = orc.gemm_fwd(xh, sh)
    assert rel(host(y), pre) < 1e-2
    assert rel(host(g), orc.gelu_fwd(pre)) < 1e-2
    np.testing.assert_allclose(host(g), orc.gelu_fwd(host(y), emulate=True), rtol=1e-2, atol=1e-6)


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_forward_with_transposed_weights(orc, M, N, K):
    """tgk_gemm_fwd_t (Wt[K][N]) against the checker and against tgk_gemm_fwd; the batched transpose
    that produces Wt is exact."""
    lib = library()
    rng = np.random.default_rng(M * 5 + N + K)
    x, xh = to_bf16_device(rng.standard_normal((M, K)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)))
    r, rh = to_bf16_device(rng.standard_normal((M, N)) * 4)
    # two matrices in one buffer, transposed by one launch
    other, oh = to_bf16_device(rng.standard_normal((64, 128)))
    flat = torch.cat([w.flatten(), other.flatten()])
    out = torch.zeros_like(flat)
    jobs = np.zeros(2, dtype=[("offset", np.int64), ("rows", np.int32), ("cols", np.int32),
                              ("first_tile", np.int32), ("pad", np.int32)])
    jobs[0] = (0, N, K, 0, 0)
    jobs[1] = (N * K, 64, 128, (N // 64) * (K // 64), 0)
    jd = torch.from_numpy(jobs.view(np.uint8)).cuda()
    check(lib.tgk_transpose_batch(stream(), flat.data_ptr(), out.data_ptr(), jd.data_ptr(), 2,
                                  (N // 64) * (K // 64) + 2))
    sync()
    wt = out[:N * K].view(K, N)
    assert torch.equal(wt, w.t().contiguous())
    assert torch.equal(out[N * K:].view(128, 64), other.t().contiguous())
    y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    g = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_gemm_fwd_t(stream(), M, N, K, x.data_ptr(), K, wt.data_ptr(), N, y.data_ptr(), N, None, 0, None, 0))
    sync()
    assert rel(host(y), orc.gemm_fwd(xh, wh)) < 1e-2
    assert torch.equal(y, run_fwd(x, w)[0])  # same products, same summation order
    check(lib.tgk_gemm_fwd_t(stream(), M, N, K, x.data_ptr(), K, wt.data_ptr(), N, y.data_ptr(), N, r.data_ptr(), N,
                             None, 0))
    sync()
    assert rel(host(y), orc.gemm_fwd(xh, wh, residual=rh)) < 1e-2
    check(lib.tgk_gemm_fwd_t(stream(), M, N, K, x.data_ptr(), K, wt.data_ptr(), N, y.data_ptr(), N, None, 0,
                             g.data_ptr(), N))
    sync()
    assert rel(host(g), orc.gelu_fwd(orc.gemm_fwd(xh, wh))) < 1e-2


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_dgrad_and_fused_gelu_backward(orc, M, N, K):
    # dX[M][K] = dY[M][N] W[N][K]; here the tiled output dims are (M, K), the reduced one is N
    M, K, N = M, N, K
    lib = library()
    rng = np.random.default_rng(M * 3 + N + K)
    dy, dyh = to_bf16_device(rng.standard_normal((M, N)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)))
    u, uh = to_bf16_device(rng.standard_normal((M, K)))
    dx = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_gemm_dgrad(stream(), M, N, K, dy.data_ptr(), N, w.data_ptr(), K, dx.data_ptr(), K, None, 0))
    sync()
    want = orc.gemm_dgrad(dyh, wh)
    assert rel(host(dx), want) < 1e-2
    check(lib.tgk_gemm_dgrad(stream(), M, N, K, dy.data_ptr(), N, w.data_ptr(), K, dx.data_ptr(), K,
                             u.data_ptr(), K))
    sync()
    assert rel(host(dx), orc.gelu_bwd(uh, want)) < 1e-2
    # the same two products from the transposed weight (Wt[K][N]): same values, same summation order
    wt = w.t().contiguous()
    dxt = torch.empty_like(dx)
    check(lib.tgk_gemm_dgrad_t(stream(), M, N, K, dy.data_ptr(), N, wt.data_ptr(), N, dxt.data_ptr(), K,
                               u.data_ptr(), K))
    sync()
    assert torch.equal(dxt, dx)
    check(lib.tgk_gemm_dgrad_t(stream(), M, N, K, dy.data_ptr(), N, wt.data_ptr(), N, dxt.data_ptr(), K, None, 0))
    sync()
    assert rel(host(dxt), want) < 1e-2
    assert np.mean(host(dxt) == orc.gemm_dgrad(dyh, wh, emulate=True)) > 0.99


@pytest.mark.parametrize("M,N,K", [(64, 128, 128), (256, 256, 192), (1024, 384, 256), (4096, 256, 128),
                                   (2048, 768, 768)])
def test_wgrad_split_k_and_accumulate(orc, M, N, K):
    lib = library()
    rng = np.random.default_rng(M + 7 * N + K)
    dy, dyh = to_bf16_device(rng.standard_normal((M, N)))
    x, xh = to_bf16_device(rng.standard_normal((M, K)))
    need = lib.tgk_gemm_wgrad_workspace(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    dw = torch.full((N, K), 3.0, dtype=torch.float32, device="cuda")
    args = (stream(), M, N, K, dy.data_ptr(), N, x.data_ptr(), K, dw.data_ptr(), K)
    check(lib.tgk_gemm_wgrad(*args, 0, ws.data_ptr(), need))
    sync()
    want = orc.gemm_wgrad(dyh, xh)
    assert rel(host(dw), want) < 1e-4
    first = host(dw).copy()
    check(lib.tgk_gemm_wgrad(*args, 1, ws.data_ptr(), need))
    sync()
    np.testing.assert_allclose(host(dw), 2 * first, rtol=1e-6)
    # fixed reduction order: a second run is bit-identical
    dw2 = torch.empty_like(dw)
    check(lib.tgk_gemm_wgrad(stream(), M, N, K, dy.data_ptr(), N, x.data_ptr(), K, dw2.data_ptr(), K, 0,
                             ws.data_ptr(), need))
    sync()
    np.testing.assert_array_equal(host(dw2), first)


def run_wgrad_batch(M, shapes, rng, accumulate=0, start=0.0):
    """One tgk_gemm_wgrad_batch over `shapes` (N, K); returns (gradients, inputs)."""
    import ctypes as C
    from turbogpt_amd.bridge import WgradJob
    lib = library()
    jobs = (WgradJob * len(shapes))()
    keep, inputs = [], []
    for j, (N, K) in enumerate(shapes):
        dy, dyh = to_bf16_device(rng.standard_normal((M, N)))
        x, xh = to_bf16_device(rng.standard_normal((M, K)))
        dw = torch.full((N, K), start, dtype=torch.float32, device="cuda")
        keep.append((dy, x, dw))
        inputs.append((dyh, xh))
        jobs[j] = WgradJob(N, K, dy.data_ptr(), N, x.data_ptr(), K, dw.data_ptr(), K)
    need = lib.tgk_gemm_wgrad_batch_workspace(M, len(shapes), C.addressof(jobs))
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    check(lib.tgk_gemm_wgrad_batch(stream(), M, len(shapes), C.addressof(jobs), accumulate, ws.data_ptr(), need))
    sync()
    return keep, inputs, (jobs, ws, need)


@pytest.mark.parametrize("M,shapes", [(64, [(128, 192)]), (256, [(128, 192), (256, 384)]),
                                      (2048, [(768, 768), (256, 192), (128, 576), (384, 192)]),
                                      (4096, [(128, 192), (128, 192), (128, 192)]),
                                      (128, [(2560, 1920), (2560, 1920), (2560, 1920)])])  # more tiles than blocks
def test_wgrad_batch_against_the_checker(orc, M, shapes):
    """Several weight gradients in one launch: every job against the checker, accumulate, and a second run
    bit-identical (runs and pieces are summed in a fixed order)."""
    lib = library()
    keep, inputs, (jobs, ws, need) = run_wgrad_batch(M, shapes, np.random.default_rng(M + len(shapes)), start=3.0)
    firsts = []
    for (dy, x, dw), (dyh, xh) in zip(keep, inputs):
        assert rel(host(dw), orc.gemm_wgrad(dyh, xh)) < 1e-4
        firsts.append(host(dw).copy())
    import ctypes as C
    check(lib.tgk_gemm_wgrad_batch(stream(), M, len(shapes), C.addressof(jobs), 1, ws.data_ptr(), need))
    sync()
    for (dy, x, dw), first in zip(keep, firsts):
        np.testing.assert_allclose(host(dw), 2 * first, rtol=1e-6)
    check(lib.tgk_gemm_wgrad_batch(stream(), M, len(shapes), C.addressof(jobs), 0, ws.data_ptr(), need))
    sync()
    for (dy, x, dw), first in zip(keep, firsts):
        np.testing.assert_array_equal(host(dw), first)


def test_wgrad_batch_of_a_block_at_full_size(orc):
    """The four weight gradients of one transformer block at M = 16384 in one launch, against one
    tgk_gemm_wgrad per matrix (fp32 sums in a different order: 1e-5) and the checker on sampled rows."""
    lib = library()
    M = 16384
    shapes = [(768, 3072), (3072, 768), (768, 768), (2304, 768)]
    rng = np.random.default_rng(99)
    keep, inputs, _ = run_wgrad_batch(M, shapes, rng)
    for (dy, x, dw), (dyh, xh), (N, K) in zip(keep, inputs, shapes):
        need = lib.tgk_gemm_wgrad_workspace(M, N, K)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        single = torch.empty(N, K, dtype=torch.float32, device="cuda")
        check(lib.tgk_gemm_wgrad(stream(), M, N, K, dy.data_ptr(), N, x.data_ptr(), K, single.data_ptr(), K, 0,
                                 ws.data_ptr(), need))
        sync()
        assert rel(host(dw), host(single)) < 1e-5
        cols = np.sort(rng.choice(N, 24, replace=False))
        assert rel(host(dw)[cols], orc.gemm_wgrad(np.ascontiguousarray(dyh[:, cols]), xh)) < 1e-4


def test_wgrad_batch_rejects_bad_jobs():
    import ctypes as C
    from turbogpt_amd.bridge import WgradJob
    lib = library()
    t = torch.zeros(256 * 256, dtype=torch.bfloat16, device="cuda")
    f = torch.zeros(256 * 256, dtype=torch.float32, device="cuda")
    jobs = (WgradJob * 1)(WgradJob(128, 128, t.data_ptr(), 128, t.data_ptr(), 128, f.data_ptr(), 128))
    assert lib.tgk_gemm_wgrad_batch_workspace(64, 1, C.addressof(jobs)) == 0
    assert lib.tgk_gemm_wgrad_batch(stream(), 64, 1, C.addressof(jobs), 0, t.data_ptr(), 1 << 20) == -1
    assert b"every K of 192" in lib.tgk_error()
    jobs[0].K = jobs[0].ldx = jobs[0].lddw = 192
    assert lib.tgk_gemm_wgrad_batch(stream(), 60, 1, C.addressof(jobs), 0, t.data_ptr(), 1 << 20) == -1
    assert lib.tgk_gemm_wgrad_batch(stream(), 64, 5, C.addressof(jobs), 0, t.data_ptr(), 1 << 20) == -1
    assert lib.tgk_gemm_wgrad_batch(stream(), 64, 1, C.addressof(jobs), 0, None, 0) == -1
    assert b"workspace" in lib.tgk_error()
    sync()


def run_wgrad_list(M, shapes, rng, strides=None):
    """One tgk_gemm_wgrad_list over `shapes` (N, K); dW starts as NaN so an unwritten element shows."""
    import ctypes as C
    from turbogpt_amd.bridge import WgradJob
    lib = library()
    jobs = (WgradJob * len(shapes))()
    keep, inputs = [], []
    for j, (N, K) in enumerate(shapes):
        extra = 0 if strides is None else strides[j]
        dy, dyh = to_bf16_device(rng.standard_normal((M, N + extra)))
        x, xh = to_bf16_device(rng.standard_normal((M, K + extra)))
        dw = torch.full((N, K + extra), float("nan"), dtype=torch.float32, device="cuda")
        keep.append((dy, x, dw))
        inputs.append((np.ascontiguousarray(dyh[:, :N]), np.ascontiguousarray(xh[:, :K])))
        jobs[j] = WgradJob(N, K, dy.data_ptr(), N + extra, x.data_ptr(), K + extra, dw.data_ptr(), K + extra)
    table_bytes = lib.tgk_gemm_wgrad_list_table_bytes(M, len(shapes), C.addressof(jobs))
    assert table_bytes > 0
    table = torch.empty(table_bytes, dtype=torch.uint8, device="cuda")
    need = lib.tgk_gemm_wgrad_list_workspace(M, len(shapes), C.addressof(jobs))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    check(lib.tgk_gemm_wgrad_list_prepare(M, len(shapes), C.addressof(jobs), table.data_ptr(), table_bytes))
    # the sums of squares of what the call writes come with it: their total is ||dW||^2 over all jobs
    count = lib.tgk_gemm_wgrad_list_sumsq_count(M, len(shapes), C.addressof(jobs))
    assert 0 < count <= 4096
    squares = torch.full((count,), float("nan"), dtype=torch.float32, device="cuda")
    call = lambda: check(lib.tgk_gemm_wgrad_list(stream(), M, len(shapes), C.addressof(jobs), table.data_ptr(), 0,
                                                 ws.data_ptr(), need, squares.data_ptr()))
    call()
    sync()
    written = sum(float((dw.double()[:, :K] ** 2).sum()) for (dy, x, dw), (N, K) in zip(keep, shapes))
    assert abs(float(squares.double().sum()) - written) <= 1e-5 * written
    first = squares.clone()
    call()
    sync()
    assert torch.equal(first, squares)  # fixed order: bit-reproducible
    return keep, inputs, (jobs, table, ws, call)


@pytest.mark.parametrize("M,shapes", [(128, [(256, 256)]),                      # one tile, one quad
                                      (512, [(768, 768)]),                      # fewer tiles than blocks: all split
                                      (1024, [(256, 768), (768, 256), (512, 512)]),
                                      (512, [(3072, 3072), (3072, 3072), (256, 768)]),  # whole tiles and split ones
                                      (256, [(3072, 3072)] * 4),                # two whole tiles per block, then halves
                                      (8192, [(768, 768)]),                     # long token ranges
                                      (256, [(2304, 768), (768, 768), (3072, 768), (768, 3072)] * 3),
                                      (384, [(1024, 4096), (4096, 1024), (1024, 1024), (3072, 1024), (256, 1024)])])
def test_wgrad_list_against_the_checker(orc, M, shapes):
    """All weight gradients of a step in one launch: every job against the checker, every element written, and a
    second run bit-identical (whole tiles are summed in token order by one block, pieces in token-range order)."""
    keep, inputs, (jobs, table, ws, call) = run_wgrad_list(M, shapes, np.random.default_rng(M + len(shapes)))
    firsts = []
    for (dy, x, dw), (dyh, xh) in zip(keep, inputs):
        got = host(dw)
        assert np.isfinite(got).all()
        assert rel(got, orc.gemm_wgrad(dyh, xh)) < 1e-4
        firsts.append(got.copy())
        dw.fill_(float("nan"))
    call()
    sync()
    for (dy, x, dw), first in zip(keep, firsts):
        np.testing.assert_array_equal(host(dw), first)


def test_wgrad_list_with_leading_dimensions(orc):
    # operands and gradients that are column slices of wider buffers
    shapes = [(512, 256), (256, 768)]
    keep, inputs, _ = run_wgrad_list(256, shapes, np.random.default_rng(12), strides=[64, 8])
    for (dy, x, dw), (dyh, xh), (N, K) in zip(keep, inputs, shapes):
        got = host(dw)
        assert rel(got[:, :K], orc.gemm_wgrad(dyh, xh)) < 1e-4
        assert np.isnan(got[:, K:]).all()  # nothing written beside the gradient


def test_wgrad_list_of_a_step_at_full_size(orc):
    """A block's four weight gradients at M = 16384 (config 2's shapes), three blocks' worth plus the head's, in one
    launch: against one tgk_gemm_wgrad per matrix (fp32 sums in a different order: 1e-5) and the checker on sampled
    rows of every matrix."""
    lib = library()
    M = 16384
    shapes = [(768, 3072), (3072, 768), (768, 768), (2304, 768)] * 3 + [(256, 768)]
    rng = np.random.default_rng(77)
    keep, inputs, _ = run_wgrad_list(M, shapes, rng)
    for (dy, x, dw), (dyh, xh), (N, K) in zip(keep, inputs, shapes):
        need = lib.tgk_gemm_wgrad_workspace(M, N, K)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        single = torch.empty(N, K, dtype=torch.float32, device="cuda")
        check(lib.tgk_gemm_wgrad(stream(), M, N, K, dy.data_ptr(), N, x.data_ptr(), K, single.data_ptr(), K, 0,
                                 ws.data_ptr(), need))
        sync()
        assert rel(host(dw), host(single)) < 1e-5
        cols = np.sort(rng.choice(N, 8, replace=False))
        assert rel(host(dw)[cols], orc.gemm_wgrad(np.ascontiguousarray(dyh[:, cols]), xh)) < 1e-4


def test_wgrad_list_rejects_bad_jobs():
    import ctypes as C
    from turbogpt_amd.bridge import WgradJob
    lib = library()
    t = torch.zeros(256 * 256, dtype=torch.bfloat16, device="cuda")
    f = torch.zeros(256 * 256, dtype=torch.float32, device="cuda")
    jobs = (WgradJob * 1)(WgradJob(256, 192, t.data_ptr(), 256, t.data_ptr(), 192, f.data_ptr(), 192))
    assert lib.tgk_gemm_wgrad_list_table_bytes(128, 1, C.addressof(jobs)) == 0
    assert lib.tgk_gemm_wgrad_list_prepare(128, 1, C.addressof(jobs), f.data_ptr(), 1 << 16) == -1
    assert b"multiple of 256" in lib.tgk_error()
    jobs[0].K = jobs[0].ldx = jobs[0].lddw = 256
    bytes_needed = lib.tgk_gemm_wgrad_list_table_bytes(128, 1, C.addressof(jobs))
    assert bytes_needed > 0
    assert lib.tgk_gemm_wgrad_list_table_bytes(64, 1, C.addressof(jobs)) == 0  # M % 128
    assert lib.tgk_gemm_wgrad_list_prepare(128, 1, C.addressof(jobs), f.data_ptr(), bytes_needed - 1) == -1
    assert b"table too small" in lib.tgk_error()
    check(lib.tgk_gemm_wgrad_list_prepare(128, 1, C.addressof(jobs), f.data_ptr(), 1 << 16))
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    assert lib.tgk_gemm_wgrad_list(stream(), 128, 1, C.addressof(jobs), f.data_ptr(), 1, ws.data_ptr(), 1 << 20, None) == -1
    assert b"accumulate" in lib.tgk_error()
    assert lib.tgk_gemm_wgrad_list(stream(), 128, 1, C.addressof(jobs), None, 0, ws.data_ptr(), 1 << 20, None) == -1
    assert lib.tgk_gemm_wgrad_list(stream(), 128, 0, C.addressof(jobs), f.data_ptr(), 0, ws.data_ptr(), 1 << 20, None) == -1
    sync()


def test_strided_views_of_a_packed_buffer(orc):
    # the engine hands out column slices of wider buffers: leading dimensions differ from widths
    lib = library()
    rng = np.random.default_rng(5)
    M, N, K = 256, 128, 128
    xw, xwh = to_bf16_device(rng.standard_normal((M, 3 * K)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)))
    yw = torch.zeros(M, 2 * N, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_gemm_fwd(stream(), M, N, K, xw.data_ptr() + 2 * K, 3 * K, w.data_ptr(), K,
                           yw.data_ptr() + 2 * N, 2 * N, None, 0, None, 0))
    sync()
    assert rel(host(yw)[:, N:], orc.gemm_fwd(xwh[:, K:2 * K], wh)) < 1e-2
    assert not host(yw)[:, :N].any()


def test_rejects_bad_shapes_without_launching():
    lib = library()
    t = torch.zeros(256 * 256, dtype=torch.bfloat16, device="cuda")
    p = t.data_ptr()
    assert lib.tgk_gemm_fwd(stream(), 100, 128, 64, p, 64, p, 64, p, 128, None, 0, None, 0) == -1
    assert b"multiple of 128" in lib.tgk_error()
    assert lib.tgk_gemm_fwd(stream(), 128, 128, 60, p, 64, p, 64, p, 128, None, 0, None, 0) == -1
    assert lib.tgk_gemm_fwd(stream(), 128, 128, 64, p + 2, 64, p, 64, p, 128, None, 0, None, 0) == -1
    assert lib.tgk_gemm_fwd(stream(), 128, 128, 64, None, 64, p, 64, p, 128, None, 0, None, 0) == -1
    assert lib.tgk_gemm_wgrad(stream(), 4096, 256, 128, p, 256, p, 128, p, 128, 0, None, 0) == -1
    assert b"workspace" in lib.tgk_error()
    sync()


@pytest.mark.parametrize("M,N,K,residual", [(16384, 1024, 256, False), (16384, 1024, 512, True), (8192, 2048, 1024, False),
                                          (16384, 3072, 1024, True), (16384, 1024, 4096, False)])
def test_256x128_tiles_rows_sampled(orc, M, N, K, residual):
    """The widths of configs[4] (multiples of 128 and 256 that 192 does not divide) run on 256 x 128 tiles whose
    epilogue buffers lie in a ring slot: forward with every epilogue and the input gradient on the transposed weight,
    plain and times GELU', one to six tiles per block and one to sixteen periods per tile, against the checker on sampled rows and bit
    for bit against the kernels for k-strided weights, which sum in the same order."""
    lib = library()
    rng = np.random.default_rng(M + N + K)
    x, xh = to_bf16_device(rng.standard_normal((M, K)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)) / np.sqrt(K))
    r, rh = to_bf16_device(rng.standard_normal((M, N)))
    rows = np.sort(rng.choice(M, 64, replace=False))
    y, _ = run_fwd(x, w, residual=r if residual else None)
    want = orc.gemm_fwd(xh[rows], wh, residual=rh[rows] if residual else None)
    assert rel(host(y)[rows], want) < 1e-2
    assert np.mean(host(y)[rows] == orc.gemm_fwd(xh[rows], wh, residual=rh[rows] if residual else None, emulate=True)) > 0.99
    yt = torch.empty_like(y)
    wt = w.t().contiguous()
    check(lib.tgk_gemm_fwd_t(stream(), M, N, K, x.data_ptr(), K, wt.data_ptr(), N, yt.data_ptr(), N,
                             r.data_ptr() if residual else None, N if residual else 0, None, 0))
    sync()
    assert torch.equal(yt, y)  # 32-k stages on the k-strided weight: same products, same summation order
    # the GELU epilogue (two outputs) on the same tiles
    y2, g2 = run_fwd(x, w, gelu=True)
    pre = orc.gemm_fwd(xh[rows], wh)
    assert rel(host(y2)[rows], pre) < 1e-2
    assert rel(host(g2)[rows], orc.gelu_fwd(pre)) < 1e-2
    gt = torch.empty_like(y)
    check(lib.tgk_gemm_fwd_t(stream(), M, N, K, x.data_ptr(), K, wt.data_ptr(), N, yt.data_ptr(), N, None, 0,
                             gt.data_ptr(), N))
    sync()
    assert torch.equal(yt, y2) and torch.equal(gt, g2)
    # input gradient: dX[M][K] = dY[M][N] W[N][K], tiled over (M, K) and reduced over N
    dy, dyh = to_bf16_device(rng.standard_normal((M, N)))
    w2, w2h = to_bf16_device(rng.standard_normal((N, K)) / np.sqrt(N))
    dx = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    dxt = torch.empty_like(dx)
    w2t = w2.t().contiguous()
    check(lib.tgk_gemm_dgrad_t(stream(), M, N, K, dy.data_ptr(), N, w2t.data_ptr(), N, dxt.data_ptr(), K, None, 0))
    check(lib.tgk_gemm_dgrad(stream(), M, N, K, dy.data_ptr(), N, w2.data_ptr(), K, dx.data_ptr(), K, None, 0))
    sync()
    want = orc.gemm_dgrad(dyh[rows], w2h)
    assert rel(host(dxt)[rows], want) < 1e-2
    assert torch.equal(dxt, dx)
    # ... and times GELU' of a saved pre-activation
    u, uh = to_bf16_device(rng.standard_normal((M, K)))
    check(lib.tgk_gemm_dgrad_t(stream(), M, N, K, dy.data_ptr(), N, w2t.data_ptr(), N, dxt.data_ptr(), K, u.data_ptr(), K))
    check(lib.tgk_gemm_dgrad(stream(), M, N, K, dy.data_ptr(), N, w2.data_ptr(), K, dx.data_ptr(), K, u.data_ptr(), K))
    sync()
    assert rel(host(dxt)[rows], orc.gelu_bwd(uh[rows], want)) < 1e-2
    assert torch.equal(dxt, dx)


@pytest.mark.parametrize("N,K", [(2304, 768), (768, 768), (3072, 768), (768, 3072)])
def test_full_size_sweep_rows_sampled(orc, N, K):
    """BASELINE config 2 at M = 16384: the checker covers a sample of output rows/columns."""
    lib = library()
    M = 16384
    rng = np.random.default_rng(N + K)
    x, xh = to_bf16_device(rng.standard_normal((M, K)))
    w, wh = to_bf16_device(rng.standard_normal((N, K)))
    dy, dyh = to_bf16_device(rng.standard_normal((M, N)))
    rows = np.sort(rng.choice(M, 96, replace=False))
    y, _ = run_fwd(x, w)
    assert rel(host(y)[rows], orc.gemm_fwd(xh[rows], wh)) < 1e-2
    dx = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    check(lib.tgk_gemm_dgrad(stream(), M, N, K, dy.data_ptr(), N, w.data_ptr(), K, dx.data_ptr(), K, None, 0))
    sync()
    assert rel(host(dx)[rows], orc.gemm_dgrad(dyh[rows], wh)) < 1e-2
    dxt = torch.empty_like(dx)
    wt = w.t().contiguous()
    check(lib.tgk_gemm_dgrad_t(stream(), M, N, K, dy.data_ptr(), N, wt.data_ptr(), N, dxt.data_ptr(), K, None, 0))
    sync()
    assert torch.equal(dxt, dx)  # the engine's path: 64-k stages on the transposed weight
    need = lib.tgk_gemm_wgrad_workspace(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    dw = torch.empty(N, K, dtype=torch.float32, device="cuda")
    check(lib.tgk_gemm_wgrad(stream(), M, N, K, dy.data_ptr(), N, x.data_ptr(), K, dw.data_ptr(), K, 0,
                             ws.data_ptr(), need))
    sync()
    cols = np.sort(rng.choice(N, 48, replace=False))
    assert rel(host(dw)[cols], orc.gemm_wgrad(np.ascontiguousarray(dyh[:, cols]), xh)) < 1e-4
    # adjoint identity over the whole problem: <dY, X W^T> = <dY W, X> = <dY^T X, W>
    a = float((dy.float() * y.float()).sum())
    b = float((dx.float() * x.float()).sum())
    c = float((dw * w.float()).sum())
    assert abs(a - b) < 2e-2 * abs(a) + 1e3 and abs(a - c) < 2e-2 * abs(a) + 1e3
