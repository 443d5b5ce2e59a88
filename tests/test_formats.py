"""Host-side byte formats (scanet3_amd/formats.py): checksums against the reference's known answers, the TFRecord
framing, the two protobuf messages against the protobuf library as an independent decoder, the Kryo tensor layout."""
import os
import struct

import numpy as np
import pytest

from scanet3_amd import formats as F


def test_hashing_known_answers():
    """native/HashingSpec.scala:9-29 (the JVM's signed view of the 32-bit values)."""
    assert F.as_int32(F.mask(123)) == -1552356648
    assert F.unmask(F.mask(123)) == 123
    assert F.as_int32(F.crc32(b"c")) == 112844655
    assert F.as_int32(F.crc32c(b"c")) == 552285127
    assert F.as_int32(F.crc32c_masked(bytes([24, 0, 0, 0, 0, 0, 0, 0]))) == 575373219
    # the CRC-32C check value of RFC 3720 (B.4), which the table construction must reproduce
    assert F.crc32c(b"123456789") == 0xE3069283
    assert F.crc32c(bytes(32)) == 0x8A9136AA
    for v in (0, 1, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 0xA282EAD8):
        assert F.unmask(F.mask(v)) == v


def test_tf_record_framing_round_trip_and_corruption():
    payloads = [b"", b"x", bytes(range(256)) * 3]
    blob = b"".join(F.tf_record(p) for p in payloads)
    assert len(blob) == sum(16 + len(p) for p in payloads)
    assert blob[:8] == struct.pack("<Q", 0)
    # native/TfRecord.scala:20-28 with the reference's own known answer for the length field of a 24-byte message
    rec = F.tf_record(bytes(24))
    assert F.as_int32(struct.unpack_from("<I", rec, 8)[0]) == 575373219
    assert F.read_tf_records(blob) == payloads
    bad = bytearray(blob)
    bad[-7] ^= 1
    with pytest.raises(ValueError):
        F.read_tf_records(bytes(bad))


def _event_classes():
    """tensorflow.Event / Summary restricted to the fields the writer uses, built as dynamic descriptors so that the
    protobuf library, not this repository's encoder, decodes the bytes."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    fd = descriptor_pb2.FileDescriptorProto(name="scanet_events_test.proto", package="tensorflow", syntax="proto3")
    T = descriptor_pb2.FieldDescriptorProto
    value = fd.message_type.add(name="SummaryValue")
    value.field.add(name="tag", number=1, type=T.TYPE_STRING, label=T.LABEL_OPTIONAL)
    value.field.add(name="simple_value", number=2, type=T.TYPE_FLOAT, label=T.LABEL_OPTIONAL)
    summary = fd.message_type.add(name="Summary")
    summary.field.add(name="value", number=1, type=T.TYPE_MESSAGE, label=T.LABEL_REPEATED, type_name=".tensorflow.SummaryValue")
    event = fd.message_type.add(name="Event")
    event.field.add(name="wall_time", number=1, type=T.TYPE_DOUBLE, label=T.LABEL_OPTIONAL)
    event.field.add(name="step", number=2, type=T.TYPE_INT64, label=T.LABEL_OPTIONAL)
    event.field.add(name="file_version", number=3, type=T.TYPE_STRING, label=T.LABEL_OPTIONAL)
    event.field.add(name="summary", number=5, type=T.TYPE_MESSAGE, label=T.LABEL_OPTIONAL, type_name=".tensorflow.Summary")
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    desc = pool.FindMessageTypeByName("tensorflow.Event")
    get = getattr(message_factory, "GetMessageClass", None)
    return get(desc) if get else message_factory.MessageFactory(pool).GetPrototype(desc)


@pytest.mark.parametrize("tag,value,step,wall", [("loss", 0.25, 7, 1700000000.5), ("accuracy", 0.0, 0, 0.0),
                                                 ("loss", -3.5e-7, 2 ** 40 + 3, 12.0), ("läss", 1e30, 300, 1.0)])
def test_event_encoding_is_what_protobuf_decodes(tag, value, step, wall):
    Event = _event_classes()
    e = Event()
    e.ParseFromString(F.event_scalar(tag, value, step, wall))
    assert e.wall_time == wall and e.step == step and len(e.summary.value) == 1
    assert e.summary.value[0].tag == tag and e.summary.value[0].simple_value == np.float32(value)
    # and byte for byte what the library itself serializes for the same message
    ref = Event(wall_time=wall, step=step)
    v = ref.summary.value.add()
    v.tag, v.simple_value = tag, value
    assert F.event_scalar(tag, value, step, wall) == ref.SerializeToString()
    ver = Event()
    ver.ParseFromString(F.event_file_version())
    assert ver.file_version == "brain.Event:2"


def test_tensorboard_writes_version_then_events(tmp_path):
    """core/TensorBoard.scala:57-67: every call is one file: the version record, then the events."""
    Event = _event_classes()
    board = F.TensorBoard(str(tmp_path / "board"))
    p1 = board.add_scalar("loss", 1.5, 10)
    p2 = board.add_scalar("loss", 1.25, 20, path="run2")
    assert p1 != p2 and os.path.basename(p1).startswith("events.out.tfevents.") and "run2" in p2
    for path, val, step in ((p1, 1.5, 10), (p2, 1.25, 20)):
        records = F.read_tf_records(open(path, "rb").read())
        assert len(records) == 2
        first, second = Event(), Event()
        first.ParseFromString(records[0])
        second.ParseFromString(records[1])
        assert first.file_version == "brain.Event:2"
        assert second.step == step and second.summary.value[0].simple_value == val and second.wall_time > 1.6e9


def test_kryo_tensor_layout():
    """optimizers/KryoSerializers.scala:32-47 for `Tensor.vector(1f, 2f, 3f)` (KryoSerializersSpec.scala:14-16 round-trips
    it; no reference test holds the bytes, so the expected bytes below follow the writer's calls one by one)."""
    t = np.array([1, 2, 3], np.float32)
    blob = F.kryo_tensor_bytes(t)
    assert blob == (bytes([0, 0, 0, 1]) +                       # writeInt(DT_FLOAT = 1), big endian
                    bytes([0, 0, 0, 1]) +                       # writeInt(rank)
                    bytes([0, 0, 0, 0, 0, 0, 0, 3]) +           # writeLongs(dims)
                    bytes([0, 0, 0, 12]) +                      # writeInt(bytes.length)
                    t.tobytes())                                # the tensor's native (little endian) bytes
    back, end = F.kryo_tensor_read(blob)
    assert end == len(blob) and back.dtype == np.float32 and np.array_equal(back, t)
    rng = np.random.default_rng(3)
    parts = [rng.standard_normal((2, 3, 4)).astype(np.float32), np.arange(5, dtype=np.int64), np.float64(2.5) * np.ones(()),
             rng.integers(0, 255, (4, 1)).astype(np.uint8), np.zeros((0, 3), np.int32)]
    stream = b"".join(F.kryo_tensor_bytes(p) for p in parts)
    pos = 0
    for p in parts:
        got, pos = F.kryo_tensor_read(stream, pos)
        assert got.dtype == p.dtype and got.shape == p.shape and np.array_equal(got, p)
    assert pos == len(stream)
    with pytest.raises(ValueError):
        F.kryo_tensor_read(bytes([0, 0, 0, 99]) + blob[4:])
    with pytest.raises(ValueError):
        F.kryo_tensor_read(blob[:19] + bytes([13]) + blob[20:])
    with pytest.raises(ValueError):
        F.kryo_tensor_bytes(np.array(["a"]))


# --------------------------------------------------------------------------- batching of records (optimizers/IteratorsSpec.scala)
def _records(n):
    return [([3 * i + 1, 3 * i + 2], [3 * i + 3]) for i in range(n)]


def test_tensor_iterator_known_answers():
    """The four cases of IteratorsSpec.scala:11-78, plus the default (`Skip`) the optimizer relies on."""
    from scanet3_amd import dsl as S
    it = S.TensorIterator(_records(2), ((2,), (1,)), 2)
    assert it.has_next()
    x, y = next(it)
    np.testing.assert_array_equal(x, [[1, 2], [4, 5]])
    np.testing.assert_array_equal(y, [[3], [6]])
    assert not it.has_next()
    batches = list(S.TensorIterator(_records(4), ((2,), (1,)), 2))
    assert len(batches) == 2
    np.testing.assert_array_equal(batches[1][0], [[7, 8], [10, 11]])
    np.testing.assert_array_equal(batches[1][1], [[9], [12]])
    (x, y), = list(S.TensorIterator(_records(2), ((2,), (1,)), 3, remaining=S.PadZeros))
    np.testing.assert_array_equal(x, [[1, 2], [4, 5], [0, 0]])
    np.testing.assert_array_equal(y, [[3], [6], [0]])
    (x, y), = list(S.TensorIterator(_records(2), ((2,), (1,)), 3, remaining=S.Partial))
    np.testing.assert_array_equal(x, [[1, 2], [4, 5]])
    np.testing.assert_array_equal(y, [[3], [6]])
    assert list(S.TensorIterator(_records(2), ((2,), (1,)), 3)) == []          # Skip: a short batch is dropped
    assert len(list(S.TensorIterator(_records(7), ((2,), (1,)), 3))) == 2
    assert [b[0].shape[0] for b in S.TensorIterator(_records(7), ((2,), (1,)), 3, remaining=S.Partial)] == [3, 3, 1]
    assert x.dtype == np.float32
    with pytest.raises(ValueError):
        S.TensorIterator(_records(1), ((2,), (1,)), 1, remaining="Wrap")
