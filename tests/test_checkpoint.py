"""The .pt checkpoint writer / reader (include/tg_checkpoint.h), host only.  What pins it: PyTorch's own
loader reads the file (torch.load, weights_only=True) and returns the dictionary of the reference's
checkpoints (checkpoint.cpp:155-197) with bit-identical tensors; Python's zipfile agrees with every
CRC; the library's reader round-trips it and rejects damaged or mismatching files the way
load_training_state does (checkpoint.cpp:373-551)."""
import ctypes as C
import zipfile

import numpy as np
import pytest
import torch

from turbogpt_amd import bridge


def small_model():
    return bridge.ModelConfig(d_model=128, depth=2, context=128, batch=2)


def parameter_count(m):
    d, f = m.d_model, m.ffn
    return 2 * m.vocab * d + m.base.context * d + m.base.depth * (4 * d + 4 * d * d + 2 * f * d) + 2 * d


def make_state(seed=5):
    m = small_model()
    rng = np.random.default_rng(seed)
    n = parameter_count(m)
    state = dict(weights=rng.standard_normal(n).astype(np.float32),
                 momentum=rng.standard_normal(n).astype(np.float32) * 1e-3,
                 variance=rng.random(n).astype(np.float32) * 1e-6, step=1234567,
                 scheduler=bridge.OneCycle(48829), train_seconds=321.125,
                 final_loss_sums=rng.random(m.base.context) * 7, final_loss_batches=99)
    return m, state


def test_torch_loads_the_file_with_identical_contents(tmp_path):
    m, s = make_state()
    path = tmp_path / "state.pt"
    bridge.write_checkpoint(path, m, **s)
    assert not (tmp_path / "state.pt.tmp").exists()
    loaded = torch.load(path, weights_only=True)
    assert list(loaded) == ["model", "opt", "lr_scheduler", "trainer"]
    assert list(loaded["model"]) == ["depth", "context", "weights", "d_model", "heads", "vocab", "ffn"]
    assert [int(loaded["model"][k]) for k in ("depth", "context", "d_model", "heads", "vocab", "ffn")] == \
        [2, 128, 128, 2, 256, 512]
    for group, key, want in (("model", "weights", s["weights"]), ("opt", "momentum", s["momentum"]),
                             ("opt", "variance", s["variance"])):
        got = loaded[group][key]
        assert got.dtype == torch.float32 and got.shape == (want.size,)
        np.testing.assert_array_equal(got.numpy().view(np.uint32), want.view(np.uint32))
    assert int(loaded["opt"]["step"]) == int(loaded["lr_scheduler"]["step"]) == 1234567
    sched = loaded["lr_scheduler"]
    assert int(sched["total_steps"]) == 48829
    assert [float(sched[k]) for k in ("warmup_fraction", "initial_lr_fraction", "final_lr_fraction", "low_momentum",
                                      "high_momentum")] == [.3, .04, .000004, .85, .95]
    trainer = loaded["trainer"]
    assert float(trainer["train_seconds"]) == 321.125 and int(trainer["final_loss_batches"]) == 99
    assert trainer["final_loss_sums"].dtype == torch.float64
    np.testing.assert_array_equal(trainer["final_loss_sums"].numpy(), s["final_loss_sums"])


def test_container_is_a_valid_aligned_zip(tmp_path):
    m, s = make_state()
    path = tmp_path / "state.pt"
    bridge.write_checkpoint(path, m, **s)
    with zipfile.ZipFile(path) as z:
        assert z.testzip() is None  # every CRC-32 agrees with zlib's
        names = z.namelist()
        assert names[0] == "archive/data.pkl" and "archive/version" in names and "archive/byteorder" in names
        assert {f"archive/data/{i}" for i in range(19)} <= set(names)
        assert z.read("archive/data/2") == s["weights"].tobytes()  # the reference's numbering: 2 = weights
        assert z.read("archive/data/0") == np.int64(2).tobytes()
        raw = path.read_bytes()
        for info in z.infolist():
            assert info.compress_type == zipfile.ZIP_STORED
            name_len, extra_len = np.frombuffer(raw, "<u2", 2, info.header_offset + 26)
            assert (info.header_offset + 30 + int(name_len) + int(extra_len)) % 64 == 0


def test_round_trip_through_the_library(tmp_path):
    m, s = make_state(seed=9)
    path = tmp_path / "state.pt"
    bridge.write_checkpoint(path, m, **s)
    back = bridge.read_checkpoint(path, expect=m)
    for key in ("weights", "momentum", "variance"):
        np.testing.assert_array_equal(back[key].view(np.uint32), s[key].view(np.uint32))
    np.testing.assert_array_equal(back["final_loss_sums"], s["final_loss_sums"])
    assert (back["step"], back["train_seconds"], back["final_loss_batches"]) == (1234567, 321.125, 99)
    assert back["scheduler"]["total_steps"] == 48829 and back["scheduler"]["low_momentum"] == .85
    assert back["model"] == dict(depth=2, context=128, d_model=128, heads=2, vocab=256, ffn=512)
    # no schedule, no loss window: the optional parts may be absent
    bridge.write_checkpoint(path, m, s["weights"], s["momentum"], s["variance"], step=0)
    back = bridge.read_checkpoint(path)
    assert back["scheduler"]["total_steps"] == 0 and back["final_loss_sums"].size == 0 and back["step"] == 0
    assert torch.load(path, weights_only=True)["trainer"]["final_loss_sums"].numel() == 0


def test_files_with_another_storage_numbering_are_rejected(tmp_path):
    """The reader goes by record names (storage numbers), as checkpoint.cpp:432-448 does, not by the
    pickle.  torch.save numbers storages in pickling order, which puts d_model at 3 where this layout
    keeps the momentum: such a file must be refused with a reason, not misread."""
    m, s = make_state(seed=11)
    t = lambda v, dt: torch.tensor([v], dtype=dt)
    step = t(77, torch.int64)
    state = {
        "model": {"depth": t(2, torch.int64), "context": t(128, torch.int64), "weights": torch.from_numpy(s["weights"]),
                  "d_model": t(128, torch.int64), "heads": t(2, torch.int64), "vocab": t(256, torch.int64),
                  "ffn": t(512, torch.int64)},
        "opt": {"momentum": torch.from_numpy(s["momentum"]), "variance": torch.from_numpy(s["variance"]), "step": step},
        "lr_scheduler": {"total_steps": t(20, torch.int64), "step": step, "warmup_fraction": t(.3, torch.float64),
                         "initial_lr_fraction": t(.04, torch.float64), "final_lr_fraction": t(4e-6, torch.float64),
                         "low_momentum": t(.85, torch.float64), "high_momentum": t(.95, torch.float64)},
        "trainer": {"train_seconds": t(1.5, torch.float64), "final_loss_sums": torch.from_numpy(s["final_loss_sums"]),
                    "final_loss_batches": t(3, torch.int64)},
    }
    path = tmp_path / "from_torch.pt"
    torch.save(state, path)
    with pytest.raises(RuntimeError, match="checkpoint"):
        bridge.read_checkpoint(path)


def test_damaged_and_mismatching_files_are_rejected(tmp_path):
    m, s = make_state()
    path = tmp_path / "state.pt"
    bridge.write_checkpoint(path, m, **s)
    raw = bytearray(path.read_bytes())
    with zipfile.ZipFile(path) as z:
        info = z.getinfo("archive/data/3")
    name_len, extra_len = np.frombuffer(bytes(raw), "<u2", 2, info.header_offset + 26)
    payload = info.header_offset + 30 + int(name_len) + int(extra_len)

    def expect(data, message, **kwargs):
        bad = tmp_path / "bad.pt"
        bad.write_bytes(bytes(data))
        with pytest.raises(RuntimeError, match=message):
            bridge.read_checkpoint(bad, **kwargs)

    flipped = bytearray(raw)
    flipped[payload + 1000] ^= 0x10
    expect(flipped, "CRC mismatch in record archive/data/3")
    expect(raw[:len(raw) // 2], "checkpoint")                      # truncated: no end record
    expect(raw[:-30] + bytes(30), "checkpoint")                    # end record destroyed
    expect(b"not a zip file at all, just text" * 4, "no ZIP end record")
    other = bridge.ModelConfig(d_model=128, depth=3, context=128, batch=2)
    with pytest.raises(RuntimeError, match="architecture mismatch"):
        bridge.read_checkpoint(path, expect=other)
    with pytest.raises(RuntimeError, match="cannot open"):
        bridge.read_checkpoint(tmp_path / "missing.pt")
    # writer-side validation
    with pytest.raises(RuntimeError, match="does not match the model"):
        bridge.write_checkpoint(path, m, s["weights"][:-1], s["momentum"][:-1], s["variance"][:-1], step=0)
    with pytest.raises(RuntimeError, match="final_loss_positions"):
        bridge.write_checkpoint(path, m, s["weights"], s["momentum"], s["variance"], step=0,
                                final_loss_sums=np.zeros(5))
    with pytest.raises(RuntimeError, match="cannot create"):
        bridge.write_checkpoint(tmp_path / "no_such_dir" / "x.pt", m, s["weights"], s["momentum"], s["variance"], 0)


def test_record_checksums_equal_zlib(tmp_path):
    """Every CRC-32 in the central directory equals zlib.crc32 of the record (check value of the
    polynomial: crc32("123456789") = 0xcbf43926)."""
    import zlib
    assert zlib.crc32(b"123456789") == 0xcbf43926
    m, s = make_state()
    path = tmp_path / "state.pt"
    bridge.write_checkpoint(path, m, **s)
    with zipfile.ZipFile(path) as z:
        for info in z.infolist():
            assert info.CRC == zlib.crc32(z.read(info.filename)), info.filename
