"""Reader / writer of hodu's tensor container (.hdt), straight onto the device.

crates/hodu_core/src/format/hdt.rs:11-23 defines the payload -- `TensorData { shape: Vec<usize>, dtype: DType,
data: Vec<u8> }`, or `TensorCollection { tensors: Vec<(String, TensorData)> }` for named tensors -- and serialises
it with the `postcard` crate (workspace dependency, version 1.1.3; not vendored in the reference tree).  postcard's
published wire format is what is implemented here: a struct is its fields in order; a sequence or string is its
length as a varint followed by the items; `usize` is a varint (unsigned LEB128: seven bits per byte, low bits
first, high bit = more follows); `u8` is one byte.  `DType` derives `serde_repr` over `repr(u8)`
(crates/hodu_core/src/types/dtype.rs:3-28), so it is the single byte of its id.  `data` is the row-major elements in
little-endian order (crates/hodu_core/src/tensor/bytes.rs:90-180), which is the device's own element encoding: the
bytes go to the GPU unchanged.

The reference holds no .hdt file and its tests only round-trip (format/hdt.rs:127-139), so against the reference this
container is parity unpinned; tests/test_hdt_cpu.py holds it to byte strings assembled by hand from the rules above.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import numpy as np

from .ffi import DTYPE_ID, DTYPE_SIZE

DTYPE_NAME = {v: k for k, v in DTYPE_ID.items()}
_BITS = {1: np.uint8, 2: np.dtype("<u2"), 4: np.dtype("<u4"), 8: np.dtype("<u8")}


class HdtError(ValueError):
    """HoduError::DeserializationFailed"""


def _varint(n: int) -> bytes:
    out = bytearray()
    while True:
        b = n & 0x7F
        n >>= 7
        out.append(b | (0x80 if n else 0))
        if not n:
            return bytes(out)


def _read_varint(buf: bytes, pos: int) -> Tuple[int, int]:
    value = shift = 0
    while True:
        if pos >= len(buf):
            raise HdtError("truncated varint")
        b = buf[pos]
        pos += 1
        value |= (b & 0x7F) << shift
        if not b & 0x80:
            return value, pos
        shift += 7
        if shift > 63:
            raise HdtError("varint longer than 64 bits")


def encode_tensor_data(shape, dtype: str, data: bytes) -> bytes:
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    if len(data) != n * DTYPE_SIZE[dtype]:
        raise ValueError(f"{len(data)} bytes do not fill shape {list(shape)} of {dtype}")
    return (_varint(len(shape)) + b"".join(_varint(int(d)) for d in shape) + bytes([DTYPE_ID[dtype]])
            + _varint(len(data)) + bytes(data))


def decode_tensor_data(buf: bytes, pos: int = 0):
    """-> (shape, dtype name, data bytes, next position)"""
    nd, pos = _read_varint(buf, pos)
    if nd > 64:
        raise HdtError(f"{nd} dimensions")
    shape = []
    for _ in range(nd):
        d, pos = _read_varint(buf, pos)
        shape.append(d)
    if pos >= len(buf):
        raise HdtError("truncated before the dtype")
    if buf[pos] not in DTYPE_NAME:
        raise HdtError(f"unknown dtype id {buf[pos]}")
    dtype = DTYPE_NAME[buf[pos]]
    pos += 1
    n, pos = _read_varint(buf, pos)
    if pos + n > len(buf):
        raise HdtError("truncated data")
    want = (int(np.prod(shape, dtype=np.int64)) if shape else 1) * DTYPE_SIZE[dtype]
    if n != want:
        raise HdtError(f"{n} data bytes for shape {shape} of {dtype} (expected {want})")
    return shape, dtype, bytes(buf[pos:pos + n]), pos + n


def serialize_many_bytes(items: List[Tuple[str, list, str, bytes]]) -> bytes:
    out = bytearray(_varint(len(items)))
    for name, shape, dtype, data in items:
        raw = name.encode("utf-8")
        out += _varint(len(raw)) + raw + encode_tensor_data(shape, dtype, data)
    return bytes(out)


def deserialize_many_bytes(buf: bytes) -> List[Tuple[str, list, str, bytes]]:
    count, pos = _read_varint(buf, 0)
    items = []
    for _ in range(count):
        n, pos = _read_varint(buf, pos)
        if pos + n > len(buf):
            raise HdtError("truncated name")
        name = bytes(buf[pos:pos + n]).decode("utf-8")
        pos += n
        shape, dtype, data, pos = decode_tensor_data(buf, pos)
        items.append((name, shape, dtype, data))
    if pos != len(buf):
        raise HdtError(f"{len(buf) - pos} trailing bytes")
    return items


# ---- tensors on the device (format/hdt.rs:25-52: load, save, load_many, save_many) -----------------------
def _to_device(shape, dtype, data, device):
    from .tensor import Tensor
    bits = np.frombuffer(data, dtype=_BITS[DTYPE_SIZE[dtype]]).astype(_BITS[DTYPE_SIZE[dtype]].newbyteorder("=") if DTYPE_SIZE[dtype] > 1 else np.uint8)
    return Tensor.from_bits(bits, dtype, shape, device)


def _from_device(t) -> Tuple[list, str, bytes]:
    bits = t.to_bits()
    return t.shape, t.dtype, bits.astype(bits.dtype.newbyteorder("<")).tobytes()


def deserialize(buf: bytes, device: int = 0):
    shape, dtype, data, pos = decode_tensor_data(buf, 0)
    if pos != len(buf):
        raise HdtError(f"{len(buf) - pos} trailing bytes")
    return _to_device(shape, dtype, data, device)


def serialize(t) -> bytes:
    return encode_tensor_data(*_from_device(t))


def load(path, device: int = 0):
    with open(path, "rb") as f:
        return deserialize(f.read(), device)


def save(t, path) -> None:
    with open(path, "wb") as f:
        f.write(serialize(t))


def load_many(path, device: int = 0) -> Dict[str, object]:
    with open(path, "rb") as f:
        return {name: _to_device(shape, dtype, data, device) for name, shape, dtype, data in deserialize_many_bytes(f.read())}


def save_many(tensors: Dict[str, object], path) -> None:
    with open(path, "wb") as f:
        f.write(serialize_many_bytes([(name,) + _from_device(t) for name, t in tensors.items()]))
