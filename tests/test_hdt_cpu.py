"""The .hdt container (crates/hodu_core/src/format/hdt.rs) against byte strings assembled by hand from postcard's
published rules (struct = fields in order, Vec / String = varint length + items, usize = unsigned LEB128, u8 = one
byte) and the little-endian element encodings of tensor/bytes.rs.  The reference ships no .hdt file and its own tests
only round-trip, so this pins the reader / writer to the wire format's definition, not to a reference artefact."""
import struct

import numpy as np
import pytest

from hodu_amd import hdt


def test_single_tensor_bytes():
    # the tensor of the reference's round-trip test (format/hdt.rs:127-139): f32 [[1, 2], [3, 4]]
    data = struct.pack("<4f", 1.0, 2.0, 3.0, 4.0)
    want = bytes([2, 2, 2, 5, 16]) + data  # shape len 2, dims 2 2, dtype id 5 (f32), 16 data bytes
    assert hdt.encode_tensor_data([2, 2], "f32", data) == want
    assert hdt.decode_tensor_data(want) == ([2, 2], "f32", data, len(want))
    # a scalar has an empty shape; bf16 is id 3
    assert hdt.encode_tensor_data([], "bf16", b"\x80\x3f") == bytes([0, 3, 2, 0x80, 0x3F])


def test_varints_cross_byte_boundaries():
    n = 300 * 200
    data = bytes(n)  # u8 zeros
    enc = hdt.encode_tensor_data([300, 200], "u8", data)
    # 300 = 0b10_0101100 -> AC 02; 200 -> C8 01; 60000 = 0xEA60 -> E0 D4 03
    assert enc[:10] == bytes([2, 0xAC, 0x02, 0xC8, 0x01, 7, 0xE0, 0xD4, 0x03, 0])
    assert hdt.decode_tensor_data(enc)[:2] == ([300, 200], "u8")


def test_named_collection_bytes():
    a = struct.pack("<2i", -1, 7)
    items = [("w", [2], "i32", a), ("bias.0", [1, 1], "f16", b"\x00\x3c")]
    want = (bytes([2]) + bytes([1]) + b"w" + bytes([1, 2, 13, 8]) + a
            + bytes([6]) + b"bias.0" + bytes([2, 1, 1, 4, 2, 0x00, 0x3C]))
    assert hdt.serialize_many_bytes(items) == want
    assert hdt.deserialize_many_bytes(want) == items


def test_malformed_input_is_rejected():
    good = hdt.encode_tensor_data([2, 2], "f32", bytes(16))
    for bad in (good[:-1], good[:3], bytes([2, 2, 2, 99, 16]) + bytes(16), bytes([2, 2, 2, 5, 15]) + bytes(15), bytes([0x80] * 11)):
        with pytest.raises(hdt.HdtError):
            hdt.decode_tensor_data(bad)
    with pytest.raises(hdt.HdtError):
        hdt.deserialize_many_bytes(bytes([1, 1]) + b"w" + good + b"\x00")
    with pytest.raises(ValueError):
        hdt.encode_tensor_data([3], "f32", bytes(8))
