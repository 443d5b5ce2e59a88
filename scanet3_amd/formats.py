"""Byte formats on either side of the training step, host side only (no device work, no third-party library):

* TensorBoard event files as the reference writes them for loss and accuracy curves
  (core/TensorBoard.scala:25-38,57-67 over native/TfRecord.scala:10-32 and native/Hashing.scala:10-49);
* the layout the reference's Kryo `TensorSerializer` gives a tensor on the wire between Spark executors
  (optimizers/KryoSerializers.scala:27-62).
"""
from __future__ import annotations

import os
import socket
import struct
import time
import zlib
from typing import Iterable, List, Optional, Sequence, Tuple

import numpy as np

# --------------------------------------------------------------------------- hashing (native/Hashing.scala)
_CRC_MASK = 0xA282EAD8
_M32 = 0xFFFFFFFF


def _crc32c_table() -> List[int]:
    table = []
    for n in range(256):
        c = n
        for _ in range(8):
            c = (c >> 1) ^ 0x82F63B78 if c & 1 else c >> 1      # Castagnoli polynomial, reflected
        table.append(c)
    return table


_TABLE = _crc32c_table()


def crc32c(data: bytes) -> int:
    """CRC-32C of `data` as an unsigned 32-bit value (Hashing.crc32c, :37-39)."""
    c = _M32
    for b in data:
        c = _TABLE[(c ^ b) & 0xFF] ^ (c >> 8)
    return c ^ _M32


def crc32(data: bytes) -> int:
    """Hashing.crc32 (:31-35): the zlib polynomial."""
    return zlib.crc32(data) & _M32


def mask(value: int) -> int:
    """Hashing.mask (:15-19): rotate right by 15 and add a constant, modulo 2^32."""
    v = value & _M32
    return (((v >> 15) | (v << 17)) + _CRC_MASK) & _M32


def unmask(value: int) -> int:
    """Hashing.unmask (:21-25)."""
    v = ((value & _M32) - _CRC_MASK) & _M32
    return ((v >> 17) | (v << 15)) & _M32


def crc32c_masked(data: bytes) -> int:
    return mask(crc32c(data))


def as_int32(value: int) -> int:
    """The JVM's view of an unsigned 32-bit value (the reference's tests quote signed ints)."""
    value &= _M32
    return value - (1 << 32) if value & 0x80000000 else value


# --------------------------------------------------------------------------- TFRecord framing (native/TfRecord.scala:10-32)
def tf_record(payload: bytes) -> bytes:
    """uint64 length, masked crc32c of those 8 bytes, payload, masked crc32c of the payload; little endian."""
    length = struct.pack("<Q", len(payload))
    return length + struct.pack("<I", crc32c_masked(length)) + payload + struct.pack("<I", crc32c_masked(payload))


def read_tf_records(blob: bytes) -> List[bytes]:
    """Inverse of `tf_record` over a whole file; raises ValueError on a checksum mismatch."""
    out, pos = [], 0
    while pos < len(blob):
        (length,) = struct.unpack_from("<Q", blob, pos)
        (lcrc,) = struct.unpack_from("<I", blob, pos + 8)
        if lcrc != crc32c_masked(blob[pos:pos + 8]):
            raise ValueError(f"length checksum mismatch at byte {pos}")
        payload = blob[pos + 12:pos + 12 + length]
        (pcrc,) = struct.unpack_from("<I", blob, pos + 12 + length)
        if len(payload) != length or pcrc != crc32c_masked(payload):
            raise ValueError(f"payload checksum mismatch at byte {pos}")
        out.append(payload)
        pos += 16 + length
    return out


# --------------------------------------------------------------------------- the two protobuf messages, hand encoded
def _varint(n: int) -> bytes:
    out = bytearray()
    while True:
        b = n & 0x7F
        n >>= 7
        out.append(b | (0x80 if n else 0))
        if not n:
            return bytes(out)


def _field_bytes(number: int, data: bytes) -> bytes:
    return _varint((number << 3) | 2) + _varint(len(data)) + data


def event_file_version(version: str = "brain.Event:2") -> bytes:
    """tensorflow.Event with file_version (field 3) set (TensorBoard.scala:58)."""
    return _field_bytes(3, version.encode())


def event_scalar(tag: str, value: float, step: int, wall_time: float) -> bytes:
    """tensorflow.Event{wall_time = 1 (double), step = 2 (int64), summary = 5{value = 1{tag = 1, simple_value = 2 (float)}}}
    as `addScalar` builds it (TensorBoard.scala:25-38).  Zero-valued scalar fields are left out, as proto3 does."""
    val = _field_bytes(1, tag.encode())
    if np.float32(value).tobytes() != b"\x00\x00\x00\x00":
        val += _varint((2 << 3) | 5) + struct.pack("<f", float(value))
    summary = _field_bytes(1, val)
    out = b""
    if wall_time != 0.0:
        out += _varint((1 << 3) | 1) + struct.pack("<d", wall_time)
    if step != 0:
        out += _varint((2 << 3) | 0) + _varint(step & 0xFFFFFFFFFFFFFFFF)
    return out + _field_bytes(5, summary)


class TensorBoard:
    """`TensorBoard(dir)` (core/TensorBoard.scala:15-67): every call writes one new events file holding the version
    record and the new events."""

    def __init__(self, directory: str = ""):
        self.dir = directory or "."
        os.makedirs(self.dir, exist_ok=True)
        self._seq = 0

    def write_events(self, events: Iterable[bytes], subpath: Optional[str] = None) -> str:
        root = os.path.join(self.dir, subpath) if subpath else self.dir
        os.makedirs(root, exist_ok=True)
        # the reference names files by the millisecond; a counter keeps two files of one millisecond apart
        self._seq += 1
        name = f"events.out.tfevents.{int(time.time() * 1000)}.{socket.gethostname()}.{self._seq}"
        path = os.path.join(root, name)
        with open(path, "wb") as f:
            for e in [event_file_version()] + list(events):
                f.write(tf_record(e))
        return path

    def add_scalar(self, tag: str, value: float, step: int, path: Optional[str] = None) -> str:
        return self.write_events([event_scalar(tag, float(value), int(step), time.time())], path)


# --------------------------------------------------------------------------- Kryo tensor layout (KryoSerializers.scala:27-62)
# TensorFlow DataType codes of the numeric types the reference supports (core/TensorType.scala): the `code` the
# serializer writes first.
_DT = {np.dtype(np.float32): 1, np.dtype(np.float64): 2, np.dtype(np.int32): 3, np.dtype(np.uint8): 4, np.dtype(np.int8): 6,
       np.dtype(np.int64): 9, np.dtype(np.bool_): 10}
_DT_INV = {v: k for k, v in _DT.items()}


def kryo_tensor_bytes(tensor: np.ndarray) -> bytes:
    """What `TensorSerializer.write` puts on the wire for a numeric tensor: Kryo's fixed-width big-endian
    `writeInt(type code)`, `writeInt(rank)`, `writeLongs(dims)`, `writeInt(byte count)`, then the tensor's bytes as
    they sit in memory (little endian, row major)."""
    t = np.asarray(tensor, order="C")      # (ascontiguousarray would turn a scalar into a vector)
    if t.dtype not in _DT:
        raise ValueError(f"no TensorFlow type code for {t.dtype}")
    data = t.astype(t.dtype.newbyteorder("<"), copy=False).tobytes()
    return (struct.pack(">ii", _DT[t.dtype], t.ndim) + b"".join(struct.pack(">q", d) for d in t.shape) +
            struct.pack(">i", len(data)) + data)


def kryo_tensor_read(blob: bytes, offset: int = 0) -> Tuple[np.ndarray, int]:
    """Inverse of `kryo_tensor_bytes`; returns (tensor, offset after it)."""
    code, rank = struct.unpack_from(">ii", blob, offset)
    if code not in _DT_INV:
        raise ValueError(f"unknown tensor type code {code}")
    if rank < 0 or rank > 64:
        raise ValueError(f"implausible rank {rank}")
    dims = struct.unpack_from(f">{rank}q", blob, offset + 8) if rank else ()
    pos = offset + 8 + 8 * rank
    (nbytes,) = struct.unpack_from(">i", blob, pos)
    dt = _DT_INV[code]
    count = int(np.prod(dims)) if rank else 1
    if nbytes != count * dt.itemsize:
        raise ValueError(f"{nbytes} bytes do not hold a {dt} tensor of shape {tuple(dims)}")
    data = np.frombuffer(blob, dtype=dt.newbyteorder("<"), count=count, offset=pos + 4)
    return data.astype(dt).reshape(dims), pos + 4 + nbytes
