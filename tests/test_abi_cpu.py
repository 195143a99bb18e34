"""Host-only checks of the C-ABI library (no GPU needed): it loads, exports every symbol the
headers declare, keeps the reference's POD layouts, and its pure-host entry points behave like the
reference's (tests/verify.py:177-200 for OneCycle; cuda/runtime.cu:65-78 for rejected configs)."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

from turbogpt_amd import bridge

ROOT = Path(__file__).resolve().parents[1]


def declared(header, marker):
    text = (ROOT / "include" / header).read_text()
    return re.findall(marker + r"\s+[\w\s\*]+?\b(tgk?_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    lib = bridge.library()
    kernel = declared("tgk_kernels.h", "TGK_API")
    engine = declared("tg_runtime.h", "TG_API")
    checkpoint = declared("tg_checkpoint.h", "TG_API")
    events = declared("tg_events.h", "TG_API")
    assert len(kernel) >= 23 and len(engine) >= 23 and len(checkpoint) == 4 and len(events) == 7
    for name in kernel + engine + checkpoint + events:
        assert hasattr(lib, name), name
    assert set(events) == set(bridge.EVENTS_ABI)
    assert set(kernel) == set(bridge.KERNEL_ABI)
    assert set(engine) == set(bridge.ENGINE_ABI)
    assert set(checkpoint) == set(bridge.CHECKPOINT_ABI)


def test_pod_layouts_match_the_reference():
    # config.h:5-13 (72 bytes, seed at 56, inflight at 64), optim.h:6-16
    assert C.sizeof(bridge.Config) == 72
    assert bridge.Config.seed.offset == 56 and bridge.Config.inflight.offset == 64
    assert C.sizeof(bridge.OneCycle) == 48 and C.sizeof(bridge.StepRates) == 8
    assert C.sizeof(bridge.ModelConfig) == 104 and bridge.ModelConfig.d_model.offset == 72
    cfg = bridge.Config()
    assert (cfg.depth, cfg.context, cfg.seed, cfg.inflight) == (4, 4, 3407, 1)
    assert cfg.beta2 == pytest.approx(0.95) and cfg.weight_decay == pytest.approx(0.1)


def point(total, step):
    lib = bridge.library()
    rates = bridge.StepRates()
    status = lib.tg_onecycle_point(C.byref(bridge.OneCycle(total)), step, C.byref(rates))
    return status, rates.multiplier, rates.momentum


def test_onecycle_point_known_answers_and_checker(orc):
    assert point(20, 0)[1:] == pytest.approx((0.04, 0.95), rel=1e-7)
    assert point(20, 5)[1:] == pytest.approx((1.0, 0.85), rel=1e-7)
    assert point(20, 19)[1:] == pytest.approx((4e-6, 0.95), rel=1e-6)
    for total in (1, 8, 20, 37, 48829, 488282):  # the totals of tests/verify.py:181
        for step in sorted(set([0, min(1, total - 1), total // 3, int(0.3 * total), total // 2, total - 1])):
            status, mult, mom = point(total, step)
            assert status == 0
            assert (mult, mom) == orc.onecycle_point(total, step)  # same double arithmetic: bit equal
    lib = bridge.library()
    assert point(20, 20)[0] == -1 and b"Invalid OneCycle" in lib.tg_error()
    assert point(0, 0)[0] == -1


def test_create_rejects_bad_configurations_before_touching_a_device():
    lib = bridge.library()
    # the plain Config builds the reference's width-16 network, with the reference's limits (cuda/runtime.cu:65-78)
    for kwargs, needle in [(dict(batch=16, context=5), b"depth 4/8, context 4/8"), (dict(batch=16, depth=3), b"depth 4/8"),
                           (dict(batch=2), b"batch at least 4"), (dict(batch=6), b"divisible by 16"),
                           (dict(batch=16, inflight=0), b"inflight must be 1..16"),
                           (dict(batch=16, inflight=17), b"inflight must be 1..16"),
                           (dict(batch=16, inflight=2, blocks=4), b"synchronous training only"),
                           (dict(batch=16, ns_steps=0), b"ns_steps")]:
        assert lib.tg_create(C.byref(bridge.Config(**kwargs))) is None
        assert needle in lib.tg_error(), (kwargs, lib.tg_error())
    assert lib.tg_create(None) is None
    cases = [(dict(d_model=100), b"d_model"), (dict(d_model=256, heads=3), b"head_dim"),
             (dict(d_model=256, vocab=100), b"vocabulary"), (dict(d_model=256, depth=0), b"depth"),
             (dict(d_model=256, depth=2, context=100), b"context"),
             (dict(d_model=256, depth=2, context=128, inflight=17), b"inflight must be 1..16"),
             (dict(d_model=256, depth=2, context=128, batch=0), b"batch"),
             (dict(d_model=256, ffn=1000, depth=2, context=128), b"ffn")]
    for kwargs, needle in cases:
        assert lib.tg_create_ex(C.byref(bridge.ModelConfig(**kwargs))) is None
        assert needle in lib.tg_error(), (kwargs, lib.tg_error())
    assert lib.tg_create_ex(None) is None


def test_kernel_entry_points_validate_arguments_on_the_host():
    lib = bridge.library()
    assert lib.tgk_gemm_fwd(None, 100, 128, 64, None, 64, None, 64, None, 128, None, 0, None, 0) == -1
    assert lib.tgk_attn_fwd(None, 1, 1, 100, 64, None, None, None, 192, None, 64, None, 0.125) == -1
    assert lib.tgk_gemm_wgrad_workspace(64, 100, 128) == 0
    assert lib.tgk_attn_bwd_workspace(2, 3, 128) == 2 * (2 * 3 * 128 * 4)
    assert lib.tgk_layernorm_bwd_workspace(16384, 768) == 768 * 2 * 768 * 4  # one partial row pair per block
    assert lib.tgk_w16_parameter_count(4) == 21648 and lib.tgk_w16_parameter_count(8) == 35088  # model.h:12-37
    assert lib.tgk_w16_workspace(4, 16, 8) % 256 == 0 and lib.tgk_w16_workspace(4, 16, 9) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(bridge, "_LIB", None)
    monkeypatch.setenv("TURBOGPT_LIBRARY", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        bridge.library()


def test_headers_are_plain_c_and_the_host_program_links(tmp_path):
    """The boundary is a C ABI: every header under include/ compiles as C99 (-pedantic) and as C++17 on its
    own, and the host program (turbogpt_amd/host/train_bytes.cpp) builds with plain g++ against the
    library and refuses to run without arguments."""
    import subprocess
    from turbogpt_amd import build as native
    for header in sorted((ROOT / "include").glob("*.h")):
        for compiler, std, lang in (("gcc", "-std=c99", "c"), ("g++", "-std=c++17", "c++")):
            done = subprocess.run([compiler, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", lang,
                                   str(header)], capture_output=True, text=True)
            assert done.returncode == 0, f"{header.name} as {lang}: {done.stderr}"
    program = native.build_host()
    done = subprocess.run([str(program)], capture_output=True, text=True)
    assert done.returncode == 1 and "usage: train_bytes --data FILE" in done.stderr
