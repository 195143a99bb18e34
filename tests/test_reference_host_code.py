"""The library's host-side formats against the reference's OWN host code, compiled from the reference tree by
oracle/Makefile (checkpoint.cpp, loss_summary.cpp, tensorboard.cpp behind oracle/ref_host_io_shim.cpp; no GPU):
  - a width-16 checkpoint written by tg_checkpoint_write loads through the reference's load_training_state with
    identical arrays, and one written by save_training_state reads through tg_checkpoint_read;
  - an event file written through tg_events_* and one written by the reference's TensorBoardLogger parse to the
    same records (the independent parser of tests/test_events.py; wall times and the writer's name aside);
  - tg_final_loss_add keeps the sums and counts of FinalLossAverage, resumed in the middle of a run.
Skipped where oracle/_ref was never built (the reference tree is not mounted and no prebuilt copy travelled)."""
import ctypes as C
import struct

import numpy as np
import pytest

import oracle
from oracle import width16 as w16
from test_events import fields, one, records
from turbogpt_amd import bridge

ref = oracle.ref_io()
pytestmark = pytest.mark.skipif(ref is None, reason="oracle/_ref/libtgref_io.so was not built")

DEPTH, CONTEXT = 4, 8
COUNT = w16.parameter_count(DEPTH)


def state(seed):
    rng = np.random.default_rng(seed)
    arrays = [rng.standard_normal(COUNT).astype(np.float32) for _ in range(3)]
    arrays[2] = np.abs(arrays[2])
    sums = rng.random(CONTEXT) * 7
    return arrays, sums


def pointer(a):
    return a.ctypes.data_as(C.c_void_p)


def reference_load(path):
    arrays = [np.empty(COUNT, np.float32) for _ in range(3)]
    scalars, reals, sums = np.zeros(3, np.int64), np.zeros(6, np.float64), np.zeros(CONTEXT, np.float64)
    status = ref.tgref_checkpoint_load(str(path).encode(), DEPTH, CONTEXT, C.c_int64(COUNT), *map(pointer, arrays),
                                       pointer(scalars), pointer(reals), pointer(sums))
    assert status == 0, ref.tgref_io_error()
    return arrays, scalars, reals, sums


def test_the_reference_loads_a_checkpoint_the_library_wrote(tmp_path):
    (weights, momentum, variance), sums = state(1)
    scheduler = bridge.OneCycle(1000)
    path = tmp_path / "ours.pt"
    bridge.write_checkpoint(path, bridge.ModelConfig(d_model=16, heads=4, ffn=48, depth=DEPTH, context=CONTEXT), weights,
                            momentum, variance, step=997, scheduler=scheduler, train_seconds=12.5, final_loss_sums=sums,
                            final_loss_batches=7)
    arrays, scalars, reals, got_sums = reference_load(path)
    for got, want in zip(arrays, (weights, momentum, variance)):
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    assert scalars.tolist() == [997, 1000, 7]
    assert reals.tolist() == [0.3, 0.04, 0.000004, 0.85, 0.95, 12.5]
    np.testing.assert_array_equal(got_sums, sums)
    # the reference refuses what it should: another depth, and a file without its serialization id would not get here
    status = ref.tgref_checkpoint_load(str(path).encode(), 8, CONTEXT, C.c_int64(w16.parameter_count(8)), None, None, None,
                                       None, None, None)
    assert status == -1 and b"architecture mismatch" in ref.tgref_io_error()


def test_the_library_reads_a_checkpoint_the_reference_wrote(tmp_path):
    (weights, momentum, variance), sums = state(2)
    # step 64 of 64: the final-loss window is the last max(1, ceil(64 / 100)) = 1 step, and it has run: one batch
    # with live sums (a state outside the window, such as step 40 with one batch, the reference refuses to save)
    scalars = np.array([64, 64, 1], np.int64)
    reals = np.array([0.3, 0.04, 0.000004, 0.85, 0.95, 3.25])
    path = tmp_path / "reference.pt"
    status = ref.tgref_checkpoint_save(str(path).encode(), DEPTH, CONTEXT, C.c_int64(COUNT), pointer(weights),
                                       pointer(momentum), pointer(variance), pointer(scalars), pointer(reals), pointer(sums))
    assert status == 0, ref.tgref_io_error()
    early = np.array([40, 64, 1], np.int64)
    assert ref.tgref_checkpoint_save(str(tmp_path / "early.pt").encode(), DEPTH, CONTEXT, C.c_int64(COUNT), pointer(weights),
                                     pointer(momentum), pointer(variance), pointer(early), pointer(reals),
                                     pointer(sums)) != 0
    assert b"final loss" in ref.tgref_io_error()
    got = bridge.read_checkpoint(path)
    for name, want in (("weights", weights), ("momentum", momentum), ("variance", variance)):
        np.testing.assert_array_equal(got[name].view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(got["final_loss_sums"], sums)
    assert got["step"] == 64 and got["train_seconds"] == 3.25 and got["final_loss_batches"] == 1
    assert got["scheduler"] == dict(total_steps=64, warmup_fraction=0.3, initial_lr_fraction=0.04,
                                    final_lr_fraction=0.000004, low_momentum=0.85, high_momentum=0.95)
    # no width fields in the file: it reads as the reference's own network
    c = bridge.Checkpoint()
    bridge.check(bridge.library().tg_checkpoint_inspect(str(path).encode(), C.byref(c)))
    assert (c.model.d_model, c.model.heads, c.model.vocab, c.model.ffn) == (16, 4, 256, 48)
    assert (c.model.base.depth, c.model.base.context, c.parameter_count) == (DEPTH, CONTEXT, COUNT)
    # and torch reads both writers' files to the same dictionary
    import torch
    ours = tmp_path / "ours.pt"
    bridge.write_checkpoint(ours, bridge.ModelConfig(d_model=16, heads=4, ffn=48, depth=DEPTH, context=CONTEXT), weights,
                            momentum, variance, step=64, scheduler=bridge.OneCycle(64), train_seconds=3.25,
                            final_loss_sums=sums, final_loss_batches=1)
    a, b = torch.load(path, weights_only=True), torch.load(ours, weights_only=True)
    assert set(a) == set(b) == {"model", "opt", "lr_scheduler", "trainer"}
    for section in a:
        for key, value in a[section].items():
            assert torch.equal(value, b[section][key]), (section, key)


def test_the_library_refuses_width16_states_the_reference_would_refuse(tmp_path):
    """A width-16 file is promised to load through the reference's reader, so the writer applies the reference's own
    conditions (checkpoint.cpp:535-550) and writes nothing when they fail; the reference's writer refuses the same."""
    (weights, momentum, variance), sums = state(3)
    model = bridge.ModelConfig(d_model=16, heads=4, ffn=48, depth=DEPTH, context=CONTEXT)
    good = dict(step=64, scheduler=bridge.OneCycle(64), train_seconds=1.0, final_loss_sums=sums, final_loss_batches=1)
    bridge.write_checkpoint(tmp_path / "good.pt", model, weights, momentum, variance, **good)
    cases = {
        "window": dict(good, step=40),                          # one batch before the window has begun
        "steps": dict(good, scheduler=bridge.OneCycle(0), step=0, final_loss_batches=0),
        "past": dict(good, step=65),
        "sums": dict(good, final_loss_sums=None, final_loss_batches=0),
        "schedule": dict(good, scheduler=bridge.OneCycle(64, warmup_fraction=1.5)),
    }
    for name, fields_ in cases.items():
        path = tmp_path / (name + ".pt")
        with pytest.raises(RuntimeError):
            bridge.write_checkpoint(path, model, weights, momentum, variance, **fields_)
        assert not path.exists(), name
    # the reference's writer on the first of them
    early = np.array([40, 64, 1], np.int64)
    reals = np.array([0.3, 0.04, 0.000004, 0.85, 0.95, 1.0])
    assert ref.tgref_checkpoint_save(str(tmp_path / "ref.pt").encode(), DEPTH, CONTEXT, C.c_int64(COUNT), pointer(weights),
                                     pointer(momentum), pointer(variance), pointer(early), pointer(reals),
                                     pointer(sums)) != 0


def summaries(path):
    """[(step, tag, plugin, kind, value)] of an event file, wall times dropped."""
    out = []
    for payload in records(path)[1:]:
        event = fields(payload)
        value = fields(one(fields(one(event, 5)), 1))
        tensor = fields(one(value, 8))
        metadata = fields(one(value, 9))
        plugin = one(fields(one(metadata, 1)), 1).decode()
        if one(tensor, 1) == 1:  # DT_FLOAT
            content = struct.unpack("<f", one(tensor, 5))[0]
        else:
            content = one(tensor, 8).decode()
        out.append((one(event, 2) if any(n == 2 for n, _, _ in event) else 0, one(value, 1).decode(), plugin,
                    one(tensor, 1), one(metadata, 2).decode(), one(metadata, 4), content))
    return out


def test_event_files_of_both_writers_parse_to_the_same_records(tmp_path):
    lib = bridge.library()
    script = [("scalar", "loss", 5.5, 1024), ("scalar", "lr", 0.0006, 1024), ("text", "description", "```\nd=16\n```", 0),
              ("scalar", "loss", 4.25, 2048), ("text", "sample", "The quick \"brown\" föx", 2048),
              ("scalar", "tokens_per_second", 2.5e7, 2048)]
    ours = lib.tg_events_open(str(tmp_path / "ours").encode(), b"unit-test")
    theirs = ref.tgref_events_open(str(tmp_path / "theirs").encode())
    assert ours and theirs
    for kind, tag, value, step in script:
        if kind == "scalar":
            bridge.check(lib.tg_events_scalar(ours, tag.encode(), value, step))
            assert ref.tgref_events_scalar(theirs, tag.encode(), value, step) == 0
        else:
            bridge.check(lib.tg_events_text(ours, tag.encode(), value.encode(), step))
            assert ref.tgref_events_text(theirs, tag.encode(), value.encode(), step) == 0
    bridge.check(lib.tg_events_close(ours))
    assert ref.tgref_events_close(theirs) == 0
    (a,) = (tmp_path / "ours").glob("events.out.tfevents.*")
    (b,) = (tmp_path / "theirs").glob("events.out.tfevents.*")
    got, want = summaries(a), summaries(b)
    assert got == want and len(got) == len(script)
    # the first record of both: file version "brain.Event:2"
    for path in (a, b):
        assert one(fields(records(path)[0]), 3) == b"brain.Event:2"


def test_final_loss_summary_equals_the_reference_class():
    lib = bridge.library()
    rng = np.random.default_rng(3)
    for total in (1, 7, 100, 101, 250, 1000):
        positions = 8
        losses = rng.random((total, positions)).astype(np.float32) * 6
        # in one go, and resumed from a checkpoint in the middle of the window
        for cut in (0, max(0, total - 2)):
            sums, batches = np.zeros(positions), C.c_uint64(0)
            for step in range(1, total + 1):
                if step == cut + 1 and cut:  # what a checkpoint carries: sums and count
                    sums, batches = sums.copy(), C.c_uint64(batches.value)
                bridge.check(lib.tg_final_loss_add(total, positions, step, pointer(losses[step - 1]), pointer(sums),
                                                   C.byref(batches)))
            want_sums, want_batches, average = np.zeros(positions), C.c_uint64(0), np.zeros(positions, np.float32)
            assert ref.tgref_final_loss(total, positions, 1, total, pointer(losses), pointer(want_sums),
                                        C.byref(want_batches), pointer(average)) == 0
            assert batches.value == want_batches.value == max(1, (total + 99) // 100)
            np.testing.assert_array_equal(sums, want_sums)
            np.testing.assert_array_equal((sums / batches.value).astype(np.float32), average)
