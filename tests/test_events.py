"""TensorBoard event files written through include/tg_events.h (host only, no GPU): CRC-32C against the
published check values, TFRecord framing and the protobuf payloads read back with an independent parser
written here (the format the reference's tensorboard.cpp:72-110,198-246 produces)."""
import re
import struct

import pytest

from turbogpt_amd import bridge


def crc32c_bitwise(data):
    crc = 0xFFFFFFFF
    for byte in data:
        crc ^= byte
        for _ in range(8):
            crc = (crc >> 1) ^ (0x82F63B78 if crc & 1 else 0)
    return crc ^ 0xFFFFFFFF


def masked(crc):
    return (((crc >> 15) | (crc << 17)) + 0xA282EAD8) & 0xFFFFFFFF


def fields(buf):
    """protobuf wire format -> list of (field number, wire type, value)."""
    out, i = [], 0
    while i < len(buf):
        key, shift = 0, 0
        while True:
            b = buf[i]
            i += 1
            key |= (b & 127) << shift
            shift += 7
            if b < 128:
                break
        number, kind = key >> 3, key & 7
        if kind == 0:
            value, shift = 0, 0
            while True:
                b = buf[i]
                i += 1
                value |= (b & 127) << shift
                shift += 7
                if b < 128:
                    break
        elif kind == 1:
            value = buf[i:i + 8]
            i += 8
        elif kind == 5:
            value = buf[i:i + 4]
            i += 4
        elif kind == 2:
            size, shift = 0, 0
            while True:
                b = buf[i]
                i += 1
                size |= (b & 127) << shift
                shift += 7
                if b < 128:
                    break
            value = buf[i:i + size]
            i += size
        else:
            raise AssertionError(f"unexpected wire type {kind}")
        out.append((number, kind, value))
    assert i == len(buf)
    return out


def one(parsed, number):
    hits = [v for n, _, v in parsed if n == number]
    assert len(hits) == 1, (number, parsed)
    return hits[0]


def records(path):
    data = open(path, "rb").read()
    at, out = 0, []
    while at < len(data):
        (length,) = struct.unpack_from("<Q", data, at)
        (head_crc,) = struct.unpack_from("<I", data, at + 8)
        assert head_crc == masked(crc32c_bitwise(data[at:at + 8]))
        payload = data[at + 12:at + 12 + length]
        (body_crc,) = struct.unpack_from("<I", data, at + 12 + length)
        assert body_crc == masked(crc32c_bitwise(payload))
        out.append(payload)
        at += 16 + length
    assert at == len(data)
    return out


def test_crc32c_known_answers():
    lib = bridge.library()
    # RFC 3720 B.4 and the common check value
    for data, want in [(b"123456789", 0xE3069283), (bytes(32), 0x8A9136AA), (b"\xff" * 32, 0x62A8AB43),
                       (bytes(range(32)), 0x46DD794E), (bytes(range(31, -1, -1)), 0x113FDB5C), (b"", 0)]:
        assert lib.tg_crc32c(data, len(data)) == want
        assert crc32c_bitwise(data) == want
    blob = bytes((i * 131 + 7) & 255 for i in range(1027))  # every tail length of the 4-byte loop
    for n in (1, 2, 3, 4, 5, 63, 64, 1027):
        assert lib.tg_crc32c(blob[:n], n) == crc32c_bitwise(blob[:n])


def test_event_file_reads_back(tmp_path):
    lib = bridge.library()
    log = lib.tg_events_open(str(tmp_path / "run" / "nested").encode(), b"unit-test")
    assert log, lib.tg_error()
    path = lib.tg_events_path(log).decode()
    assert re.fullmatch(r".*/events\.out\.tfevents\.\d+\..+\.\d+\.0", path)
    points = [("loss", 5.545, 0), ("loss", 2.25, 16384), ("bits-per-byte", 3.2462, 16384), ("lr", 6e-4, 2**40)]
    for tag, value, step in points:
        assert lib.tg_events_scalar(log, tag.encode(), value, step) == 0
    assert lib.tg_events_text(log, b"description", "```\nd768 L12 é\n```".encode(), 7) == 0
    assert lib.tg_events_flush(log) == 0
    assert lib.tg_events_close(log) == 0
    payloads = records(path)
    assert len(payloads) == 1 + len(points) + 1
    first = fields(payloads[0])
    assert one(first, 3) == b"brain.Event:2" and one(fields(one(first, 10)), 1) == b"unit-test"
    assert 1.6e9 < struct.unpack("<d", one(first, 1))[0] < 4e9
    for payload, (tag, value, step) in zip(payloads[1:], points):
        event = fields(payload)
        assert one(event, 2) == step
        value_message = fields(one(fields(one(event, 5)), 1))
        assert one(value_message, 1) == tag.encode()
        tensor = fields(one(value_message, 8))
        assert one(tensor, 1) == 1 and one(tensor, 2) == b""  # DT_FLOAT, scalar shape
        assert struct.unpack("<f", one(tensor, 5))[0] == pytest.approx(value, rel=1e-6)
        metadata = fields(one(value_message, 9))
        assert one(fields(one(metadata, 1)), 1) == b"scalars" and one(metadata, 4) == 1
    text = fields(one(fields(one(fields(payloads[-1]), 5)), 1))
    assert one(text, 1) == b"description/text_summary"
    tensor = fields(one(text, 8))
    assert one(tensor, 1) == 7 and one(tensor, 8).decode() == "```\nd768 L12 é\n```"
    assert one(fields(one(fields(one(tensor, 2)), 2)), 1) == 1  # shape [1]
    assert one(fields(one(fields(one(text, 9)), 1)), 1) == b"text"


def test_event_errors_are_reported(tmp_path):
    lib = bridge.library()
    assert lib.tg_events_open(None, None) is None and b"directory" in lib.tg_error()
    blocker = tmp_path / "file"
    blocker.write_text("x")
    assert lib.tg_events_open(str(blocker / "below").encode(), None) is None
    assert lib.tg_events_scalar(None, b"x", 1.0, 0) == -1
    assert lib.tg_events_close(None) == 0
