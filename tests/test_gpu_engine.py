"""Engine-level parity through the tg_* C ABI, written after the reference's own checks
(tests/verify.py): check_model (logits / flat gradient / every parameter tensor / per-position
loss vs the checker, bit-exact causality and batch independence), check_optimizers,
check_small_updates, check_persistence, stream evaluation, and the 50-step loss parity the
target names.  Tolerances are the reference's where both sides round to bf16 alike (the checker in
emulation mode) and the target's 1e-2 against the all-fp32 checker."""
import ctypes as C

import numpy as np
import pytest

from turbogpt_amd.bridge import ModelConfig, Native, OneCycle, library

pytestmark = pytest.mark.gpu


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def checker_config(orc, cfg, emulate=False):
    b = cfg.base
    return orc.model(b.depth, b.context, b.batch, cfg.d_model, cfg.heads, cfg.vocab, cfg.ffn, cfg.ln_eps, emulate)


def test_parameter_layout_matches_the_checker(orc):
    cfg = ModelConfig(d_model=256, depth=4, context=256, batch=8)
    with Native(cfg) as engine:
        assert engine.count == orc.parameter_count(checker_config(orc, cfg))
        assert engine.count == orc.Layout(checker_config(orc, cfg)).count
        used = C.c_double()
        engine.check(engine.lib.tg_memory(engine.handle, C.byref(used)))
        assert 0.01 < used.value < 4
        assert engine.lib.tg_blocks(engine.handle) == 256
        w = orc.init_weights(checker_config(orc, cfg))
        engine.set_weights(w)
        np.testing.assert_array_equal(engine.weights().view(np.uint32), w.view(np.uint32))  # exact fp32 round trip


@pytest.mark.parametrize("depth,context,batch,d_model", [(2, 128, 2, 128), (4, 256, 8, 256), (1, 128, 3, 384)])
def test_model_against_the_checker(orc, depth, context, batch, d_model):
    """check_model of tests/verify.py:14-52; (4, 256, 8, 256) is BASELINE config 1."""
    cfg = ModelConfig(d_model=d_model, depth=depth, context=context, batch=batch)
    oc, oe = checker_config(orc, cfg), checker_config(orc, cfg, emulate=True)
    lay = orc.Layout(oc)
    rng = np.random.default_rng(71)
    # verify.py:16 inflates the init scale to 0.08 at width 16 (0.08*sqrt(16) = 0.32) to make errors
    # visible; the same activation scale at width d is 0.32/sqrt(d), inflated once more by 1.4 here
    w = orc.init_weights(oc, seed=42, scale=0.45 / np.sqrt(d_model))
    for name, off, shape in lay.entries:
        if name.endswith(("_g", "_b")):
            w[off:off + shape[0]] += rng.standard_normal(shape[0]).astype(np.float32) * 0.1
    x = rng.integers(0, 256, (batch, context), dtype=np.uint8)
    y = rng.integers(0, 256, x.shape, dtype=np.uint8)
    with Native(cfg) as engine:
        engine.set_weights(w)
        logits, grad, losses = engine.batch(x, y)
        # Per-position losses average only `batch` samples here, so bf16 rounding of the logits shows
        # directly; the reference's atol .003 (verify.py:31) applies to the mean over positions.
        for mode, cfgc, logit_tol, grad_tol, part_tol, loss_tol in [("fp32", oc, 1e-2, 1e-2, 2e-2, 3e-2),
                                                                    ("bf16", oe, 8e-3, 1e-2, 2e-2, 2e-2)]:
            want_logits, want_grad, want_loss = orc.model_batch(cfgc, w, x, y)
            print(f"d={d_model} L={depth} T={context} B={batch} vs {mode} checker: logits rel="
                  f"{rel(logits, want_logits):.3g} grad rel={rel(grad, want_grad):.3g} per-position loss max diff="
                  f"{np.abs(losses - want_loss.mean(0)).max():.3g} mean loss diff="
                  f"{abs(losses.mean() - want_loss.mean()):.3g}", flush=True)
            np.testing.assert_allclose(losses, want_loss.mean(0), atol=loss_tol, rtol=1e-3)
            assert abs(losses.mean() - want_loss.mean()) < 3e-3
            assert rel(logits, want_logits) < logit_tol                                     # verify.py:32
            assert rel(grad, want_grad) < grad_tol                                          # verify.py:33
            for name, off, shape in lay.entries:                                            # verify.py:35-42
                n = int(np.prod(shape))
                assert rel(grad[off:off + n], want_grad[off:off + n]) < part_tol, (mode, name)
        # verify.py:43-50: later tokens cannot change any earlier logit; examples are independent
        for pos in (0, 63, 64, context - 2):
            changed = x.copy()
            changed[:, pos + 1:] = rng.integers(0, 256, changed[:, pos + 1:].shape, dtype=np.uint8)
            later = engine.batch(changed, y, False)[0]
            np.testing.assert_array_equal(logits[:, :pos + 1], later[:, :pos + 1])
        if batch > 1:
            changed = x.copy()
            changed[1:] = rng.integers(0, 256, changed[1:].shape, dtype=np.uint8)
            np.testing.assert_array_equal(logits[0], engine.batch(changed, y, False)[0][0])
        # evaluation repeats exactly and leaves no state behind (verify.py:151-174)
        for _ in range(2):
            again = engine.batch(x, y, False)
            np.testing.assert_array_equal(again[0], logits)
            np.testing.assert_array_equal(again[2], losses)
        # tg_predict returns the last position of the replicated context (cuda/runtime.cu:322-351)
        np.testing.assert_array_equal(engine.predict(x[0]), logits[0, -1])


@pytest.mark.parametrize("scheduled", [False, True])
def test_optimizer_against_the_checker(orc, scheduled):
    """check_optimizers of tests/verify.py:64-105, AdamW on every parameter."""
    cfg = ModelConfig(d_model=128, depth=2, context=128, batch=1, clip=0)
    oc = checker_config(orc, cfg)
    with Native(cfg) as engine:
        w0 = orc.init_weights(oc)
        engine.set_weights(w0)
        if scheduled:
            engine.set_onecycle(20)
        mask = orc.decay_mask(oc)
        rng = np.random.default_rng(192)
        w, m, v = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
        for step in range(20):
            grad = (rng.standard_normal(engine.count) * 0.01).astype(np.float32)
            engine.optimizer_test(grad, 1)
            mult, mom = orc.onecycle_point(20, step) if scheduled else (1.0, 0.9)
            w, m, v = orc.adamw(w, m, v, grad, mask, np.float32(6e-4) * np.float32(mult), mom, 0.95, 1e-8, 0.1, 1.0,
                                step)
        got = engine.weights()
        assert rel(got - w0, w - w0) < 1e-4                       # verify.py:101
        np.testing.assert_allclose(got, w, atol=2e-6, rtol=2e-5)  # verify.py:103
        gm, gv, gstep = engine.optimizer_state()
        assert gstep == 20
        np.testing.assert_allclose(gm, m, rtol=1e-4, atol=1e-9)
        if scheduled:  # the schedule is exhausted: verify.py:145-146
            assert engine.lib.tg_optimizer_test(engine.handle, grad.ctypes.data, 1) < 0
            assert b"OneCycle" in engine.lib.tg_error()


def test_small_updates_survive(orc):
    """check_small_updates of tests/verify.py:108-127."""
    cfg = ModelConfig(d_model=128, depth=1, context=128, batch=1, learning_rate=1e-5, weight_decay=0, clip=0)
    with Native(cfg) as engine:
        w = np.full(engine.count, 0.5, np.float32)
        engine.set_weights(w)
        engine.optimizer_test(np.full(engine.count, 0.01, np.float32), 64)
        got = engine.weights()
        assert np.max(np.abs(got - w)) > 5e-4
        np.testing.assert_allclose(0.5 - got, 64e-5, rtol=0.02)


def make_engine(orc, cfg, data, scheduled_steps=0):
    engine = Native(cfg)
    engine.set_weights(orc.init_weights(checker_config(orc, cfg)))
    engine.set_data(data)
    if scheduled_steps:
        engine.set_onecycle(scheduled_steps)
    return engine


@pytest.mark.parametrize("scheduled", [False, True])
def test_one_launch_of_eight_steps_equals_eight_launches(orc, scheduled):
    """check_persistence of tests/verify.py:130-148; every kernel here has a fixed summation order,
    so the match is exact rather than within 2e-6."""
    cfg = ModelConfig(d_model=128, depth=2, context=128, batch=4)
    data = orc.fill_zipf_bytes(8192, 4)
    a, b = make_engine(orc, cfg, data, 8 if scheduled else 0), make_engine(orc, cfg, data, 8 if scheduled else 0)
    try:
        a.train(8)
        la = a.training_losses(8)
        lb = []
        for _ in range(8):
            b.train(1)
            lb.append(b.training_losses(1)[0])
        np.testing.assert_array_equal(a.weights(), b.weights())
        np.testing.assert_array_equal(la, np.stack(lb))
        assert a.optimizer_state()[2] == 8
        versions = np.empty(8, np.int32)
        a.check(a.lib.tg_training_versions(a.handle, versions.ctypes.data, 8))
        np.testing.assert_array_equal(versions, np.arange(8))
        if scheduled:
            assert a.lib.tg_train(a.handle, 1) < 0
        # resume: state moved into a fresh engine continues identically (cuda/engine_state.cu:94-130)
        c = make_engine(orc, cfg, data)
        c.set_weights(a.weights())
        m, v, step = a.optimizer_state()
        c.set_optimizer_state(m, v, step)
        if not scheduled:
            a.train(2)
            c.train(2)
            np.testing.assert_array_equal(a.training_losses(2), c.training_losses(2))
            np.testing.assert_array_equal(a.weights(), c.weights())
        c.close()
    finally:
        a.close()
        b.close()


def test_resume_from_a_checkpoint_file(orc, tmp_path):
    """trainer.cpp:76-80 / checkpoint.cpp:506-579: weights and optimizer state written to a .pt file and
    read into a fresh engine continue bit-identically to the uninterrupted run."""
    from turbogpt_amd.bridge import read_checkpoint, write_checkpoint
    cfg = ModelConfig(d_model=128, depth=2, context=128, batch=4)
    data = orc.fill_zipf_bytes(8192, 4)
    a, b = make_engine(orc, cfg, data), make_engine(orc, cfg, data)
    try:
        a.train(5)
        m, v, step = a.optimizer_state()
        path = tmp_path / "run.pt"
        write_checkpoint(path, cfg, a.weights(), m, v, step, train_seconds=1.0)
        state = read_checkpoint(path, expect=cfg)
        assert state["step"] == 5
        b.set_weights(state["weights"])
        b.set_optimizer_state(state["momentum"], state["variance"], state["step"])
        a.train(3)
        b.train(3)
        np.testing.assert_array_equal(a.training_losses(3), b.training_losses(3))
        np.testing.assert_array_equal(a.weights().view(np.uint32), b.weights().view(np.uint32))
    finally:
        a.close()
        b.close()


# the keys of the reference's JSON lines, in its order: report.cpp:46-59, :61-80, :82-117
CONFIG_KEYS = ["architecture", "depth", "ctx", "batch", "inflight", "chunk", "optimizer", "parameters", "blocks",
               "shared_bytes", "steps", "dataset_bytes", "schedule", "warmup_fraction", "initial_lr_fraction",
               "final_lr_fraction", "low_momentum", "high_momentum"]
STEP_KEYS = ["step", "tokens", "last_bpb", "position_bpb", "adam_lr", "muon_lr", "momentum", "train_seconds",
             "tokens_per_second"]
SUMMARY_KEYS = ["architecture", "depth", "ctx", "batch", "inflight", "chunk", "seed", "optimizer", "learning_rate", "muon_lr",
                "schedule", "schedule_steps", "warmup_fraction", "initial_lr_fraction", "final_lr_fraction", "low_momentum",
                "high_momentum", "requested_tokens", "tokens", "final_loss", "final_bpb", "position_bpb", "sample",
                "initialization_seconds", "mean_staleness", "max_staleness", "dataset_load_seconds", "training_seconds",
                "sample_seconds", "process_seconds", "tokens_per_second", "sample_temperature"]


def host_program_lines(stdout):
    """-> (config object, step objects, summary object); asserts the reference's keys lead every object in order."""
    import json
    lines = [json.loads(line) for line in stdout.splitlines()]
    config, steps, summary = lines[0]["config"], lines[1:-1], lines[-1]["summary"]
    assert list(config)[:len(CONFIG_KEYS)] == CONFIG_KEYS
    for step in steps:
        assert list(step)[:len(STEP_KEYS)] == STEP_KEYS
    assert list(summary)[:len(SUMMARY_KEYS)] == SUMMARY_KEYS
    return config, steps, summary


def test_host_program_trains_and_resumes(orc, tmp_path):
    """turbogpt_amd/host/train_bytes (plain g++ over the C ABI): the loss falls; 12 steps in one run equal
    6 steps + checkpoint + 6 resumed steps, to the last printed digit (trainer.cpp:51-80,105-121)."""
    import json
    import subprocess
    from turbogpt_amd import build as native
    program = native.HOST_PROGRAM
    assert program.exists(), "build it with python -m turbogpt_amd.build"
    data = tmp_path / "bytes.bin"
    data.write_bytes(orc.fill_zipf_bytes(1 << 16, 4).tobytes())
    common = [str(program), "--data", str(data), "--depth", "2", "--context", "128", "--batch", "4", "--d_model", "128",
              "--chunk", "3", "--tokens", str(12 * 4 * 128)]

    def run(*extra):
        done = subprocess.run(common + list(extra), capture_output=True, text=True, timeout=120)
        assert done.returncode == 0, done.stderr
        return host_program_lines(done.stdout)

    config, chunks, whole = run("--save", str(tmp_path / "whole.pt"))
    assert config["architecture"] == "gelu-layernorm-softmax" and config["optimizer"] == "adamw" and config["steps"] == 12
    assert config["d_model"] == 128 and config["ctx"] == 128 and config["dataset_bytes"] == 1 << 16
    assert [r["step"] for r in chunks] == [3, 6, 9, 12] and whole["steps"] == 12
    assert [r["tokens"] for r in chunks] == [n * 4 * 128 for n in (3, 6, 9, 12)]
    assert all(len(r["position_bpb"]) == 128 and r["last_bpb"] == r["position_bpb"][-1] for r in chunks)
    assert chunks[-1]["loss"] < chunks[0]["loss"] - 0.05 and len(whole["sample"]) == 68
    assert whole["tokens_per_second"] > 0 and whole["sample_temperature"] == 1.0
    # a run cut after six steps: same schedule (--tokens), fewer steps trained
    first = subprocess.run(common + ["--save", str(tmp_path / "half.pt"), "--chunk", "6"], capture_output=True, text=True,
                           timeout=120, env={"TRAIN_BYTES_STOP_AFTER": "6", **__import__("os").environ})
    assert first.returncode == 0, first.stderr
    _, _, resumed = run("--load", str(tmp_path / "half.pt"), "--save", str(tmp_path / "resumed.pt"))
    assert resumed["steps"] == 12 and resumed["final_loss"] == whole["final_loss"] and resumed["last_loss"] == whole["last_loss"]
    assert resumed["position_bpb"] == whole["position_bpb"]
    from turbogpt_amd.bridge import read_checkpoint
    a, b = read_checkpoint(tmp_path / "whole.pt"), read_checkpoint(tmp_path / "resumed.pt")
    np.testing.assert_array_equal(a["weights"].view(np.uint32), b["weights"].view(np.uint32))
    assert a["step"] == b["step"] == 12


def test_host_program_logs_a_run(orc, tmp_path):
    """--log-to: TensorBoard events whose framing and payloads parse (the parser of tests/test_events.py) and a
    report.json with the loss averaged over the last 1 % of the steps (loss_summary.cpp:5-29), for the
    reference's own width-16 network (--width16 1, through tg_create) with four batches in flight."""
    import json
    import struct
    import subprocess
    from test_events import fields, one, records
    from turbogpt_amd import build as native
    data = tmp_path / "bytes.bin"
    data.write_bytes(orc.fill_zipf_bytes(1 << 16, 9).tobytes())
    run_dir = tmp_path / "runs" / "w16"
    steps, batch, context = 300, 64, 8
    done = subprocess.run([str(native.HOST_PROGRAM), "--data", str(data), "--width16", "1", "--depth", "4", "--context",
                           str(context), "--batch", str(batch), "--chunk", "50", "--tokens", str(steps * batch * context),
                           "--inflight", "4", "--log-to", str(run_dir), "--save", str(tmp_path / "w16.pt")],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr
    config, lines, summary = host_program_lines(done.stdout)
    assert config["architecture"] == "swiglu48-rmsnorm-rope" and config["optimizer"] == "muon" and config["parameters"] == 21648
    assert [r["step"] for r in lines] == [50, 100, 150, 200, 250, 300]
    assert lines[-1]["loss"] < lines[0]["loss"] - 0.3  # it learns the Zipf byte frequencies
    assert lines[-1]["muon_lr"] < lines[1]["muon_lr"] and lines[-1]["adam_lr"] < lines[1]["adam_lr"]  # OneCycle descends
    report = json.loads((run_dir / "report.json").read_text())
    assert report == summary and list(report)[:len(SUMMARY_KEYS)] == SUMMARY_KEYS  # the file holds the summary object
    assert report["tokens_per_second"] > 0  # also with --save and --log-to together
    assert report["architecture"] == "swiglu48-rmsnorm-rope" and report["optimizer"] == "muon"
    assert report["parameters"] == 21648 and report["steps"] == steps and report["tokens"] == steps * batch * context
    assert report["final_loss_batches"] == 3 and len(report["position_bpb"]) == context  # last ceil(300 / 100) steps
    assert report["final_bpb"] == pytest.approx(report["final_loss"] / np.log(2), rel=1e-6)
    assert abs(report["final_loss"] * context - sum(report["position_bpb"]) * np.log(2) * 1.0) < 50  # finite numbers
    assert report["max_staleness"] == 3 and 2.9 < report["mean_staleness"] <= 3.0
    (event_file,) = list(run_dir.glob("events.out.tfevents.*"))
    payloads = records(event_file)
    scalars = {}
    for payload in payloads[1:]:
        event = fields(payload)
        value = fields(one(fields(one(event, 5)), 1))
        tensor = fields(one(value, 8))
        if one(tensor, 1) == 1:
            scalars.setdefault(one(value, 1).decode(), []).append((one(event, 2), struct.unpack("<f", one(tensor, 5))[0]))
    assert [step for step, _ in scalars["loss"]] == [n * batch * context for n in (50, 100, 150, 200, 250, 300)]
    assert scalars["loss"][-1][1] == pytest.approx(lines[-1]["loss"], abs=1e-5)
    assert scalars["bits-per-byte"][-1][1] == pytest.approx(scalars["last_loss"][-1][1] / np.log(2), rel=1e-6)
    assert scalars["model_bytes"] == [(0, 21648 * 4.0)] and scalars["lr"][-1][1] < scalars["lr"][1][1]
    from turbogpt_amd.bridge import read_checkpoint
    saved = read_checkpoint(tmp_path / "w16.pt")
    assert saved["step"] == steps and saved["weights"].size == 21648 and saved["final_loss_batches"] == 3


def test_engine_error_paths(orc):
    cfg = ModelConfig(d_model=128, depth=1, context=128, batch=1)
    with Native(cfg) as engine:
        lib = engine.lib
        assert lib.tg_train(engine.handle, 1) < 0 and b"Load data first" in lib.tg_error()
        small = np.zeros(100, np.uint8)
        assert lib.tg_set_data(engine.handle, small.ctypes.data, small.size) < 0  # shorter than one window
        data = orc.fill_zipf_bytes(4096, 1)
        engine.set_data(data)
        assert lib.tg_set_data(engine.handle, data.ctypes.data, data.size) < 0 and b"already" in lib.tg_error()
        assert lib.tg_train(engine.handle, 0) < 0 and lib.tg_train(engine.handle, 4097) < 0
        assert lib.tg_get_training_losses(engine.handle, None, 1) < 0
        engine.set_onecycle(4)
        assert lib.tg_set_onecycle(engine.handle, C.byref(OneCycle(4))) < 0 and b"once" in lib.tg_error()
        assert lib.tg_optimizer_test(engine.handle, np.zeros(engine.count, np.float32).ctypes.data, 65) < 0


def test_fifty_training_steps_track_the_checker(orc):
    """BASELINE config 1 (d256 L4 H4 T256 B8), AdamW lr 3e-4 betas (0.9, 0.95) wd 0.1 on a Zipf(1.1)
    byte stream: the mean training loss after 50 steps must agree with the fp32 checker."""
    cfg = ModelConfig(d_model=256, depth=4, context=256, batch=8, learning_rate=3e-4, beta1=0.9, beta2=0.95,
                      weight_decay=0.1, clip=1.0)
    oc = checker_config(orc, cfg)
    data = orc.fill_zipf_bytes(1 << 16, 71)
    w0 = orc.init_weights(oc)
    with make_engine(orc, cfg, data) as engine:
        engine.train(50)
        got = engine.training_losses(50).mean(1)
    z = np.zeros_like(w0)
    _, _, _, want = orc.train(oc, w0, z, z, data, 3407, 0, 50, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1.0)
    want = want.mean(1)
    print("loss step0 gpu/cpu", got[0], want[0], "step49", got[-1], want[-1], "max diff", np.abs(got - want).max(),
          flush=True)
    assert want[-1] < want[0] - 0.5  # it trains
    assert abs(got[-1] - want[-1]) < 1e-3
    assert np.abs(got - want).max() < 3e-3
