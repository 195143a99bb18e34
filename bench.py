#!/usr/bin/env python3
"""Headline benchmark: training tokens/sec of the byte-level GPT d768 L12 H12 T1024 B16
(the fourth benchmark configuration, configs[3]) on one MI355X, through the tg_* C ABI.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--kernels] [--config 3|4]

--config 4 runs the long-context configuration (configs[4]: d1024 L24 H16 T4096 B4) through the same code and prints
the same JSON shape; the default is the configuration the metric is quoted on.

Prints ONE JSON line.  A step = sample a batch on the GPU, forward, backward, gradient norm, AdamW
(nothing skipped; inputs are resident in HBM before the timed region).  After the timed region the
same step is run with a HIP event pair around every operator launch (tg_profile_step) to attribute
time per operator class; `roofline` describes the dominant MFMA kernel class from those live
measurements.  `cpu_baseline` times the CPU checker (oracle/, a port - the reference has no CPU
path) on the host cores for a bounded sample of the same workload.  With --kernels, further JSON
lines for the isolated GEMM sweep (configs[1]) and attention (configs[2]) go to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
V = 256
CONFIGS = {3: dict(D=768, L=12, H=12, T=1024, B=16), 4: dict(D=1024, L=24, H=16, T=4096, B=4)}
D, L, H, T, B = (CONFIGS[3][k] for k in "DLHTB")
F = 4 * D
M = B * T
TRAFFIC_PROFILE = "profiles/gemm256_plain_residual_hbm_traffic.md"


def select_config(index):
    global D, L, H, T, B, F, M
    D, L, H, T, B = (CONFIGS[index][k] for k in "DLHTB")
    F, M = 4 * D, B * T


def algorithmic_bytes_per_launch():
    """Mean over the dominant kernel's six launches per layer of 2 * (M*K + N*K + M*N [+ M*N residual]) bytes: operands
    read once, the result written once."""
    launches = [(3 * D, D, 0), (D, D, 1), (D, F, 1), (D, F, 0), (D, D, 0), (D, 3 * D, 0)]  # (N, K, residual read)
    return sum(2 * (M * k + n * k + M * n * (1 + r)) for n, k, r in launches) / len(launches)


def hbm_traffic_per_launch():
    """HBM bytes per launch of the dominant kernel and the kernel build they were measured on, as the committed
    rocprofv3 FETCH_SIZE / WRITE_SIZE summary of `--traffic-probe` states them ("... = 151.0 MB, against ..." and a
    "kernel source: ..." line): figures of that profile (configs[3] shapes), not of this run."""
    import re
    text = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_PROFILE)).read()
    found = re.search(r"=\s*([0-9.]+)\s*MB,\s*against", text)
    source = re.search(r"kernel source:\s*(.+)", text)
    if not found or not source:
        sys.exit(f"bench.py: {TRAFFIC_PROFILE} no longer states the traffic per launch ('= X MB, against') or the "
                 "kernel build it was measured on ('kernel source: ...')")
    return float(found.group(1)) * 1e6, source.group(1).strip()


def gemm_flops():
    """Algorithmic FLOPs of one launch of each block projection (2*M*N*K), per layer."""
    shapes = [(3 * D, D), (D, D), (F, D), (D, F)]  # (N, K): qkv, attention-out, mlp-up, mlp-down
    return [2.0 * M * n * k for n, k in shapes]


def class_work():
    """Algorithmic work per training step for every operator class: ('flop'|'byte', amount)."""
    per_layer = sum(gemm_flops())
    attn_fwd = 4.0 * B * H * T * T * 64 / 2  # causal-counted
    act, wide = M * D * 2, M * F * 2
    params = V * D * 2 + T * D + L * (4 * D + 4 * D * D + 2 * F * D) + 2 * D
    qkv, out, up, down = gemm_flops()
    # widths that 256 divides: one launch computes every weight gradient, the head's and the token table's included
    listed = 2 if D % 256 == 0 else 0
    return {
        "gemm_fwd": ("flop", L * (qkv + out + down)),     # plain / residual epilogues
        "gemm_fwd_gelu": ("flop", L * up),                # MLP-up: pre-activation and GELU written
        "gemm_dgrad": ("flop", L * (qkv + out + up)),     # plain epilogue
        "gemm_dgrad_gelu": ("flop", L * down),            # MLP-down dgrad times GELU'
        "gemm_wgrad": ("flop", L * per_layer + listed * 2.0 * M * V * D),
        "attn_fwd": ("flop", L * attn_fwd),
        "attn_bwd": ("flop", L * attn_fwd * 2.5),
        "head": ("flop", (3 - listed // 2) * 2.0 * M * V * D),
        "layernorm_fwd": ("byte", (2 * L + 1) * 2 * act),
        "layernorm_bwd": ("byte", (2 * L + 1) * 3 * act + 2 * L * act),  # x, dy, dx (+ residual read)
        "optimizer": ("byte", params * 28.0 + params * 4.0),            # AdamW 28 B/param + norm pass
        "other": ("byte", 4 * act + 3 * M * V * 2),
    }, params


def synthetic_weights(layout_count, rng):
    """N(0, 0.02) matrices, residual-writing ones scaled by 1/sqrt(2L), gamma = 1, beta = 0."""
    w = np.empty(layout_count, np.float32)
    n = 0

    def take(size, scale=None, fill=None):
        nonlocal n
        if fill is None:
            w[n:n + size] = rng.standard_normal(size, dtype=np.float32) * scale
        else:
            w[n:n + size] = fill
        n += size

    inner = 0.02 / np.sqrt(2 * L)
    take(V * D, 0.02)
    take(T * D, 0.02)
    for _ in range(L):
        take(D, fill=1.0), take(D, fill=0.0)
        take(3 * D * D, 0.02), take(D * D, inner)
        take(D, fill=1.0), take(D, fill=0.0)
        take(F * D, 0.02), take(D * F, inner)
    take(D, fill=1.0), take(D, fill=0.0)
    take(V * D, 0.02)
    assert n == layout_count
    return w


def zipf_bytes(n, rng, s=1.1):
    p = np.arange(1, 257, dtype=np.float64) ** -s
    cdf = np.cumsum(p / p.sum())
    return np.minimum(np.searchsorted(cdf, rng.random(n)), 255).astype(np.uint8)


def cpu_baseline(sequences=8):
    """The CPU checker on some of the step's sequences (same model, smaller batch): forward, backward, AdamW."""
    import oracle
    cfg = oracle.model(depth=L, context=T, batch=sequences, d_model=D, heads=H)
    w = oracle.init_weights(cfg)
    z = np.zeros_like(w)
    data = oracle.fill_zipf_bytes(1 << 16, 71)
    start = time.perf_counter()
    oracle.train(cfg, w, z, z, data, 3407, 0, 1, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1.0)
    seconds = time.perf_counter() - start
    return {"value": sequences * T / seconds, "unit": "tokens/s", "cores": oracle.threads(), "kind": "port",
            "sample": f"one training step of the same model on {sequences} of the {B} sequences "
                      f"(B={sequences}, T={T}): {seconds:.1f} s of the fp32 OpenMP checker (oracle/tg_oracle.c)"}


def kernel_sweeps(out):
    """configs[1] (GEMM sweep, M=16384) and configs[2] (attention B16 H12 T1024) through tgk_*."""
    import torch
    from turbogpt_amd.bridge import check, library
    lib = library()
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn, iters=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    for k, n in [(D, 3 * D), (D, D), (D, F), (F, D)]:
        x = torch.randn(M, k, device="cuda").bfloat16()
        w = torch.randn(n, k, device="cuda").bfloat16()
        dy = torch.randn(M, n, device="cuda").bfloat16()
        y = torch.empty(M, n, device="cuda", dtype=torch.bfloat16)
        dx = torch.empty(M, k, device="cuda", dtype=torch.bfloat16)
        dw = torch.empty(n, k, device="cuda")
        wt = w.t().contiguous()
        need = lib.tgk_gemm_wgrad_workspace(M, n, k)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        flop = 2.0 * M * n * k
        runs = {
            "fwd": lambda: check(lib.tgk_gemm_fwd(stream, M, n, k, x.data_ptr(), k, w.data_ptr(), k, y.data_ptr(), n,
                                                  None, 0, None, 0)),
            "fwd_t": lambda: check(lib.tgk_gemm_fwd_t(stream, M, n, k, x.data_ptr(), k, wt.data_ptr(), n,
                                                      y.data_ptr(), n, None, 0, None, 0)),
            "dgrad": lambda: check(lib.tgk_gemm_dgrad(stream, M, n, k, dy.data_ptr(), n, w.data_ptr(), k,
                                                      dx.data_ptr(), k, None, 0)),
            "dgrad_t": lambda: check(lib.tgk_gemm_dgrad_t(stream, M, n, k, dy.data_ptr(), n, wt.data_ptr(), n,
                                                          dx.data_ptr(), k, None, 0)),
            "wgrad": lambda: check(lib.tgk_gemm_wgrad(stream, M, n, k, dy.data_ptr(), n, x.data_ptr(), k,
                                                      dw.data_ptr(), k, 0, ws.data_ptr(), need)),
        }
        # comparator only, never in the product: the vendor library (hipBLASLt behind torch.matmul) on the same
        # operands - forward X W^T, dgrad dY W, wgrad dY^T X (bf16 out where ours is fp32)
        library_runs = {"fwd": lambda: torch.matmul(x, w.t(), out=y), "dgrad": lambda: torch.matmul(dy, w, out=dx),
                        "wgrad": lambda: torch.matmul(dy.t(), x)}
        library_ms = {name: timed(fn) for name, fn in library_runs.items()}
        for name, fn in runs.items():
            ms = timed(fn)
            versus = library_ms.get(name.replace("_t", ""))
            print(json.dumps({"kernel": f"gemm_{name}", "M": M, "K": k, "N": n, "ms": round(ms, 4),
                              "tflops": round(flop / ms / 1e9, 1),
                              "frac_of_bf16_peak": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                              "vendor_library_tflops": round(flop / versus / 1e9, 1)}), file=out)
    # the four weight gradients of one block in one launch, as the engine runs them
    import ctypes
    from turbogpt_amd.bridge import WgradJob
    shapes = [(D, F), (F, D), (D, D), (3 * D, D)]
    keep, jobs = [], (WgradJob * 4)()
    for j, (n, k) in enumerate(shapes):
        dy = torch.randn(M, n, device="cuda").bfloat16()
        x = torch.randn(M, k, device="cuda").bfloat16()
        dw = torch.empty(n, k, device="cuda")
        keep.append((dy, x, dw))
        jobs[j] = WgradJob(n, k, dy.data_ptr(), n, x.data_ptr(), k, dw.data_ptr(), k)
    need = lib.tgk_gemm_wgrad_batch_workspace(M, 4, ctypes.addressof(jobs))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    if need:  # widths that are multiples of 192 only
        ms = timed(lambda: check(lib.tgk_gemm_wgrad_batch(stream, M, 4, ctypes.addressof(jobs), 0, ws.data_ptr(), need)))
        flop = sum(2.0 * M * n * k for n, k in shapes)
        print(json.dumps({"kernel": "gemm_wgrad_batch", "M": M, "shapes_N_K": shapes, "ms": round(ms, 4),
                          "tflops": round(flop / ms / 1e9, 1),
                          "frac_of_bf16_peak": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}), file=out)
    del keep, ws
    # every weight gradient of the step in one launch, as the engine runs them (each layer with operands of its own)
    shapes = [(D, F), (F, D), (D, D), (3 * D, D)] * L + [(V, D)]
    keep, jobs = [], (WgradJob * len(shapes))()
    for j, (n, k) in enumerate(shapes):
        dy = torch.randn(M, n, device="cuda").bfloat16()
        x = torch.randn(M, k, device="cuda").bfloat16()
        dw = torch.empty(n, k, device="cuda")
        keep.append((dy, x, dw))
        jobs[j] = WgradJob(n, k, dy.data_ptr(), n, x.data_ptr(), k, dw.data_ptr(), k)
    table_bytes = lib.tgk_gemm_wgrad_list_table_bytes(M, len(shapes), ctypes.addressof(jobs))
    if table_bytes:
        table = torch.empty(table_bytes, dtype=torch.uint8, device="cuda")
        need = lib.tgk_gemm_wgrad_list_workspace(M, len(shapes), ctypes.addressof(jobs))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        check(lib.tgk_gemm_wgrad_list_prepare(M, len(shapes), ctypes.addressof(jobs), table.data_ptr(), table_bytes))
        ms = timed(lambda: check(lib.tgk_gemm_wgrad_list(stream, M, len(shapes), ctypes.addressof(jobs), table.data_ptr(),
                                                         0, ws.data_ptr(), need, None)), iters=5)
        flop = sum(2.0 * M * n * k for n, k in shapes)
        print(json.dumps({"kernel": "gemm_wgrad_list", "M": M, "jobs": len(shapes), "ms": round(ms, 4),
                          "tflops": round(flop / ms / 1e9, 1),
                          "frac_of_bf16_peak": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                          "operands": "N(0,1), cold (4.8 GB at configs[3])"}), file=out)
        del table, ws
    # comparators with a long reduction, the vendor library beside this library's kernel for the same layout:
    # 8192^3 with both operands strided along the reduction (the weight-gradient layout), and one weight gradient of
    # the step's largest shape both ways round
    for rows, cols, reduced in [(8192, 8192, 8192), (F, D, M), (D, F, M)]:
        a = torch.randn(reduced, rows, device="cuda").bfloat16()
        b = torch.randn(reduced, cols, device="cuda").bfloat16()
        c = torch.empty(rows, cols, device="cuda")
        one = (WgradJob * 1)(WgradJob(rows, cols, a.data_ptr(), rows, b.data_ptr(), cols, c.data_ptr(), cols))
        table_bytes = lib.tgk_gemm_wgrad_list_table_bytes(reduced, 1, ctypes.addressof(one))
        table = torch.empty(max(table_bytes, 16), dtype=torch.uint8, device="cuda")
        need = lib.tgk_gemm_wgrad_list_workspace(reduced, 1, ctypes.addressof(one))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        flop = 2.0 * rows * cols * reduced
        line = {"kernel": "long_reduction", "C": [rows, cols], "reduced": reduced, "layout": "A^T B, both [reduced][n]"}
        if table_bytes:
            check(lib.tgk_gemm_wgrad_list_prepare(reduced, 1, ctypes.addressof(one), table.data_ptr(), table_bytes))
            ms = timed(lambda: check(lib.tgk_gemm_wgrad_list(stream, reduced, 1, ctypes.addressof(one), table.data_ptr(), 0,
                                                             ws.data_ptr(), need, None)), iters=10)
            line["tflops"] = round(flop / ms / 1e9, 1)
        ms = timed(lambda: torch.matmul(a.t(), b), iters=10)
        line["vendor_library_tflops"] = round(flop / ms / 1e9, 1)
        if rows == cols:  # the library's best layout for the same product, for scale
            ms = timed(lambda: torch.matmul(a, b.t()), iters=10)
            line["vendor_library_tflops_both_contiguous"] = round(flop / ms / 1e9, 1)
        print(json.dumps(line), file=out)
        del a, b, c, table, ws
    del keep
    d = H * 64
    qkv = torch.randn(M, 3 * d, device="cuda").bfloat16()
    do = torch.randn(M, d, device="cuda").bfloat16()
    o = torch.empty(M, d, device="cuda", dtype=torch.bfloat16)
    lse = torch.empty(B, H, T, device="cuda")
    dqkv = torch.empty_like(qkv)
    need = lib.tgk_attn_bwd_workspace(B, H, T)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    p, g = qkv.data_ptr(), dqkv.data_ptr()
    flop = 4.0 * B * H * T * T * 64 / 2
    ms = timed(lambda: check(lib.tgk_attn_fwd(stream, B, H, T, 64, p, p + 2 * d, p + 4 * d, 3 * d, o.data_ptr(), d,
                                              lse.data_ptr(), 0.125)))
    print(json.dumps({"kernel": "attn_fwd", "B": B, "H": H, "T": T, "ms": round(ms, 4),
                      "tflops_causal_counted": round(flop / ms / 1e9, 1),
                      "frac_of_bf16_peak": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}), file=out)
    ms = timed(lambda: check(lib.tgk_attn_bwd(stream, B, H, T, 64, p, p + 2 * d, p + 4 * d, 3 * d, o.data_ptr(), d,
                                              lse.data_ptr(), do.data_ptr(), d, g, g + 2 * d, g + 4 * d, 3 * d, 0.125,
                                              ws.data_ptr(), need)))
    print(json.dumps({"kernel": "attn_bwd", "B": B, "H": H, "T": T, "ms": round(ms, 4),
                      "tflops_causal_counted": round(2.5 * flop / ms / 1e9, 1),
                      "frac_of_bf16_peak": round(2.5 * flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}), file=out)


def traffic_probe():
    """For `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: one plain copy of known size (256 MiB in,
    256 MiB out: the calibration dispatch) followed by the six launches per layer of the kernel that
    `roofline` describes, through the entries the engine uses: QKV, attention-out (+ residual) and MLP-down
    (+ residual) forward on the weights, then MLP-up, attention-out and QKV dgrad on the transposed copies."""
    import torch
    from turbogpt_amd.bridge import check, library
    lib = library()
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.ones(1 << 27, dtype=torch.bfloat16, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    bf16 = torch.bfloat16
    forward = [(D, 3 * D, False), (D, D, True), (F, D, True)]  # (K, N, residual)
    for k, n, residual in forward:
        x = torch.randn(M, k, device="cuda").to(bf16)
        w = (torch.randn(n, k, device="cuda") * 0.02).to(bf16)
        r = torch.randn(M, n, device="cuda").to(bf16) if residual else None
        y = torch.empty(M, n, device="cuda", dtype=bf16)
        torch.cuda.synchronize()
        check(lib.tgk_gemm_fwd(stream, M, n, k, x.data_ptr(), k, w.data_ptr(), k, y.data_ptr(), n,
                               r.data_ptr() if residual else None, n if residual else 0, None, 0))
        torch.cuda.synchronize()
    dgrad = [(D, F), (D, D), (D, 3 * D)]  # (K = width of dx, N = width of dy)
    for k, n in dgrad:
        dy = torch.randn(M, n, device="cuda").to(bf16)
        wt = (torch.randn(k, n, device="cuda") * 0.02).to(bf16)
        dx = torch.empty(M, k, device="cuda", dtype=bf16)
        torch.cuda.synchronize()
        check(lib.tgk_gemm_dgrad_t(stream, M, n, k, dy.data_ptr(), n, wt.data_ptr(), n, dx.data_ptr(), k, None, 0))
        torch.cuda.synchronize()
    print(json.dumps({"probe": "traffic", "copy_bytes_each_way": 1 << 28,
                      "order": "forward (K, N, residual) x 3, then dgrad (K, N) x 3",
                      "forward": forward, "dgrad": dgrad,
                      "algorithmic_bytes_per_launch":
                          [2 * (M * k + n * k + M * n * (2 if r else 1)) for k, n, r in forward] +
                          [2 * (M * n + n * k + M * k) for k, n in dgrad]}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--kernels", action="store_true", help="also print the isolated kernel sweeps to stderr")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="run only the copy and the six dominant GEMM dispatches used to read HBM traffic counters")
    ap.add_argument("--config", type=int, default=3, choices=sorted(CONFIGS),
                    help="3: d768 L12 T1024 B16 (the metric's configuration); 4: d1024 L24 T4096 B4")
    args = ap.parse_args()
    select_config(args.config)
    if args.traffic_probe:
        return traffic_probe()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures one GPU (the engine is single-device); run with --gpus 1")
    if not 1 <= args.steps <= 4096 or not 0 <= args.warmup <= 4096:
        sys.exit("bench.py: steps must be 1..4096 and warmup 0..4096 (one tg_train call each)")

    if args.kernels:
        # torch ships its own HIP runtime: it has to be the first one loaded in this process
        import torch
        torch.cuda.init()
    from turbogpt_amd.bridge import ModelConfig, Native
    cfg = ModelConfig(d_model=D, depth=L, context=T, batch=B, heads=H, ffn=F, learning_rate=3e-4, beta1=0.9,
                      beta2=0.95, weight_decay=0.1, clip=1.0, seed=3407)
    rng = np.random.default_rng(3407)
    with Native(cfg) as engine:
        engine.set_weights(synthetic_weights(engine.count, rng))
        engine.set_data(zipf_bytes(1 << 24, np.random.default_rng(71)))
        if args.warmup:
            engine.train(args.warmup)
        engine.synchronize()
        start = time.perf_counter()
        engine.train(args.steps)
        engine.synchronize()
        seconds = time.perf_counter() - start
        losses = engine.training_losses(args.steps).mean(1)

        work, params = class_work()
        profile = {}
        for _ in range(3):
            for name, (ms, launches) in engine.profile_step().items():
                total, count = profile.get(name, (0.0, 0))
                profile[name] = (total + ms, count + launches)
    classes = {}
    for name, (ms, launches) in profile.items():
        kind, amount = work[name]
        per_step_ms = ms / 3
        rate = amount / (per_step_ms * 1e-3) / 1e12 if per_step_ms > 0 else 0.0
        classes[name] = {"ms_per_step": round(per_step_ms, 4), "launches_per_step": launches // 3,
                         ("tflops" if kind == "flop" else "tb_per_s"): round(rate, 2)}
    traffic, traffic_source = hbm_traffic_per_launch() if args.config == 3 else (None, "not measured for this configuration")
    # Dominant MFMA kernel: the forward block projections and input gradients with a plain or residual epilogue, six
    # launches per layer - QKV, attention-out and MLP-down forward (on the weights), MLP-up, attention-out and QKV dgrad
    # (on the transposed copies).  Widths that 192 and 384 divide run them on gemm256_kernel<192,3,...> (256 x 192
    # tiles), widths that 128 and 256 divide on gemm256_kernel<128,4,...> (256 x 128), others on gemm64_kernel.
    fwd_ms, fwd_launches = profile["gemm_fwd"]
    dgrad_ms, dgrad_launches = profile["gemm_dgrad"]
    launch_ms = (fwd_ms + dgrad_ms) / (fwd_launches + dgrad_launches)
    qkv, out, up, down = gemm_flops()
    flops_per_launch = (2 * qkv + 2 * out + up + down) / 6
    achieved = flops_per_launch / (launch_ms * 1e-3) / 1e12
    kernel = ("gemm256_kernel<192,3,EpilogueBf16As<0|1>> (256x192 tiles, one wave per SIMD)" if D % 384 == 0 else
              "gemm256_kernel<128,4,EpilogueBf16As<0|1>> (256x128 tiles, one wave per SIMD)" if D % 256 == 0 else
              "gemm64_kernel<128,128|192,true,true,EpilogueBf16As<0|1>>")
    ms_per_step = seconds / args.steps * 1e3
    result = {
        "metric": f"train tokens/sec at d{D} L{L} T{T} (1 GPU)",
        "value": round(args.steps * M / seconds, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"configs[{args.config}]: full training step, byte-level GPT d_model={D} L={L} H={H} "
                               f"T={T} B={B} ffn={F} vocab=256, bf16 weights with fp32 masters, AdamW lr 3e-4 betas "
                               "0.9/0.95 wd 0.1 clip 1.0, Zipf(1.1) bytes sampled on the GPU",
                   "global_batch": B, "seq_len": T, "parameters": params, "parallelism": "single GPU"},
        "roofline": {"bound": "mfma",
                     "kernel": kernel + ", plain and residual epilogues together: QKV, attention-out, MLP-down "
                               "forward and MLP-up, attention-out, QKV dgrad (six launches per layer)",
                     "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                     "traffic_unit": "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE of --traffic-probe, "
                                     "calibrated on a copy of known size)",
                     "traffic_source": (TRAFFIC_PROFILE + " (read from that committed profile, not measured in this "
                                        "run; taken on: " + traffic_source + ")") if traffic else traffic_source,
                     "algorithmic_bytes_per_launch": algorithmic_bytes_per_launch(),
                     "flops_per_launch": flops_per_launch, "avg_launch_ms": round(launch_ms, 5)},
        "classes": classes,
        # algorithmic work per step (9.45 TFLOP at configs[3]; attention causal-counted, backward = 2.5 x forward)
        "model_tflops": round((3 * L * sum(gemm_flops()) + 3 * 2.0 * M * V * D +
                               L * 3.5 * 4.0 * B * H * T * T * 64 / 2) / (ms_per_step * 1e-3) / 1e12, 1),
        "loss_first_last": [round(float(losses[0]), 4), round(float(losses[-1]), 4)],
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(8 if args.config == 3 else 1)
    if args.kernels:
        kernel_sweeps(sys.stderr)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
