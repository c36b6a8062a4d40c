"""Tensor-bundle checkpoint files: checksum known answers, table layout, and
the reader against the writer.  No file written by TensorFlow exists here, so
reading TensorFlow's own files stays unpinned; these tests pin the checksum
(RFC 3720 vectors), the table's published constants and the two directions
against each other."""

import os
import struct

import numpy as np
import pytest

from mesh_amd import tensor_bundle as tb


def _crc32c_bitwise(data):
  crc = 0xffffffff
  for byte in data:
    crc ^= byte
    for _ in range(8):
      crc = (crc >> 1) ^ (0x82f63b78 if crc & 1 else 0)
  return crc ^ 0xffffffff


def test_crc32c_known_answers():
  # RFC 3720 appendix B.4
  assert tb.crc32c(b"\x00" * 32) == 0x8a9136aa
  assert tb.crc32c(b"\xff" * 32) == 0x62a8ab43
  assert tb.crc32c(bytes(range(32))) == 0x46dd794e
  assert tb.crc32c(bytes(range(31, -1, -1))) == 0x113fdb5c
  assert tb.crc32c(b"123456789") == 0xe3069283
  assert tb.crc32c(b"") == 0


def test_crc32c_extend_alignment_and_arrays():
  rng = np.random.default_rng(0)
  data = rng.integers(0, 256, 4099, dtype=np.uint8).tobytes()
  want = _crc32c_bitwise(data)
  assert tb.crc32c(data) == want
  for cut in (0, 1, 7, 8, 9, 1000, 4098, 4099):
    assert tb.crc32c(data[cut:], tb.crc32c(data[:cut])) == want
  arr = np.frombuffer(data[3:4099], dtype=np.uint8)      # odd start address
  assert tb.crc32c(np.ascontiguousarray(arr)) == _crc32c_bitwise(data[3:])
  with pytest.raises(tb.BundleError):
    tb.crc32c(np.zeros((4, 4), np.float32)[:, ::2])


def test_crc_mask():
  # leveldb's documented property: masking is invertible and changes the value
  crc = tb.crc32c(b"foo")
  assert tb.mask_crc(crc) != crc
  assert tb.mask_crc(tb.mask_crc(crc)) != crc
  assert tb.unmask_crc(tb.mask_crc(crc)) == crc
  assert tb.unmask_crc(tb.unmask_crc(tb.mask_crc(tb.mask_crc(crc)))) == crc
  for value in (0, 1, 0xffffffff, 0x80000000, 0x12345678):
    assert tb.unmask_crc(tb.mask_crc(value)) == value
  assert tb.mask_crc(0) == 0xa282ead8


def test_table_layout_single_entry():
  table = tb.build_table([(b"key", b"value")])
  # one data block: entry (shared 0, unshared 3, value 5), restart [0], count 1
  block = b"\x00\x03\x05keyvalue" + struct.pack("<II", 0, 1)
  assert table[:len(block)] == block
  assert table[len(block)] == 0                                  # uncompressed
  stored = struct.unpack("<I", table[len(block) + 1:len(block) + 5])[0]
  assert tb.unmask_crc(stored) == _crc32c_bitwise(block + b"\x00")
  assert len(table) >= tb.FOOTER_BYTES
  assert table[-8:] == bytes.fromhex("57fb808b247547db")
  assert tb.read_table(table) == [(b"key", b"value")]


def test_table_many_blocks_and_prefix_compression():
  items = [(("layer_%03d/moe/wi/kernel" % i).encode(), os.urandom(i % 50))
           for i in range(500)]
  for block_bytes in (64, 1024, tb.BLOCK_BYTES):
    table = tb.build_table(items, block_bytes)
    assert tb.read_table(table) == items
  small = tb.build_table(items, 1 << 30)
  raw = sum(len(k) + len(v) for k, v in items)
  assert len(small) < raw                       # shared prefixes are elided
  assert tb.read_table(tb.build_table([])) == []
  with pytest.raises(tb.BundleError):
    tb.build_table([(b"b", b""), (b"a", b"")])


def test_table_corruption_is_detected():
  table = bytearray(tb.build_table([(b"a", b"1"), (b"b", b"2")]))
  bad = bytearray(table)
  bad[2] ^= 1
  with pytest.raises(tb.BundleError, match="checksum"):
    tb.read_table(bytes(bad))
  bad = bytearray(table)
  bad[-1] ^= 1
  with pytest.raises(tb.BundleError, match="magic"):
    tb.read_table(bytes(bad))
  with pytest.raises(tb.BundleError):
    tb.read_table(b"short")
  # a Snappy block is refused by name
  block = b"\x00\x01\x01a1" + struct.pack("<II", 0, 1)
  assert bytes(table[:len(block)]) != block    # (two entries in the real one)
  one = bytearray(tb.build_table([(b"a", b"1")]))
  assert bytes(one[:len(block)]) == block
  one[len(block)] = 1
  one[len(block) + 1:len(block) + 5] = struct.pack(
      "<I", tb.mask_crc(_crc32c_bitwise(block + b"\x01")))
  with pytest.raises(tb.BundleError, match="Snappy"):
    tb.read_table(bytes(one))


def test_entry_message_bytes():
  # dtype DT_FLOAT (1), shape [2, 3], offset 16, size 24, masked crc 0x01020304
  got = tb._serialize_entry(1, (2, 3), 0, 16, 24, 0x01020304)
  want = bytes([0x08, 0x01,                         # 1: varint 1
                0x12, 0x08,                         # 2: shape, 8 bytes
                0x12, 0x02, 0x08, 0x02,             #    dim {size: 2}
                0x12, 0x02, 0x08, 0x03,             #    dim {size: 3}
                0x20, 0x10,                         # 4: offset 16
                0x28, 0x18,                         # 5: size 24
                0x35, 0x04, 0x03, 0x02, 0x01])      # 6: fixed32
  assert got == want
  entry = tb._parse_entry(got)
  assert entry == tb.BundleEntry(1, (2, 3), 0, 16, 24, 0x01020304, False)
  # a slices field marks a partitioned variable
  assert tb._parse_entry(got + bytes([0x3a, 0x00])).sliced
  # header: num_shards 2, version {producer 1}
  assert tb._serialize_header(2) == bytes([0x08, 0x02, 0x1a, 0x02, 0x08, 0x01])
  assert tb._parse_header(bytes([0x08, 0x02, 0x10, 0x01])) == (2, 1)


@pytest.mark.parametrize("num_shards", [1, 3])
def test_bundle_round_trip(tmp_path, num_shards):
  rng = np.random.default_rng(1)
  tensors = {
      "encoder/block_000/layer_001/moe/wi/kernel":
          rng.standard_normal((4, 8, 16)).astype(np.float32),
      "encoder/block_000/layer_001/moe/wo/kernel":
          rng.standard_normal((4, 16, 8)).astype(np.float32),
      "encoder/block_000/layer_001/moe/top_2_gating/kernel":
          rng.standard_normal((8, 4)).astype(np.float32),
      "global_step": np.asarray(1234, np.int64),
      "f64": rng.standard_normal(5),
      "i32": rng.integers(-9, 9, (3, 2)).astype(np.int32),
      "u8": rng.integers(0, 255, 7).astype(np.uint8),
      "i8": rng.integers(-9, 9, 7).astype(np.int8),
      "i16": rng.integers(-9, 9, 7).astype(np.int16),
      "u16": rng.integers(0, 9, 7).astype(np.uint16),
      "u32": rng.integers(0, 9, 7).astype(np.uint32),
      "u64": rng.integers(0, 9, 7).astype(np.uint64),
      "f16": rng.standard_normal(6).astype(np.float16),
      "flag": np.asarray([True, False, True]),
      "empty": np.zeros((0, 4), np.float32),
      "big_endian": rng.standard_normal(4).astype(">f4"),
  }
  prefix = str(tmp_path / "sub" / "model.ckpt-1234")
  tb.write_bundle(prefix, tensors, num_shards=num_shards)
  assert os.path.exists(prefix + ".index")
  for s in range(num_shards):
    assert os.path.exists("%s.data-%05d-of-%05d" % (prefix, s, num_shards))
  reader = tb.BundleReader(prefix)
  assert reader.num_shards == num_shards
  assert reader.keys() == sorted(tensors)
  assert "global_step" in reader and "nope" not in reader
  for name, want in tensors.items():
    got = reader[name]
    assert got.shape == want.shape, name
    assert got.dtype == want.dtype.newbyteorder("="), name
    np.testing.assert_array_equal(got, want, err_msg=name)
    assert reader.shape(name) == want.shape
  assert reader.dtype_code("global_step") == 9
  assert reader.dtype_code("f16") == 19
  with pytest.raises(KeyError):
    reader["nope"]
  with pytest.raises(tb.BundleError):
    tb.write_bundle(prefix, {"s": np.asarray(["a"])})
  with pytest.raises(tb.BundleError):
    tb.write_bundle(prefix, {"": np.zeros(1)})


def test_bundle_data_corruption_and_unhandled_entries(tmp_path):
  prefix = str(tmp_path / "m")
  value = np.arange(12, dtype=np.float32).reshape(3, 4)
  tb.write_bundle(prefix, {"a": value, "b": value * 2})
  path = prefix + ".data-00000-of-00001"
  raw = bytearray(open(path, "rb").read())
  assert len(raw) == 2 * value.nbytes                 # no padding between them
  assert bytes(raw[:value.nbytes]) == value.tobytes()
  raw[5] ^= 0x40
  open(path, "wb").write(bytes(raw))
  with pytest.raises(tb.BundleError, match="checksum"):
    tb.BundleReader(prefix)["a"]
  np.testing.assert_array_equal(tb.BundleReader(prefix)["b"], value * 2)
  assert tb.BundleReader(prefix, verify_checksums=False)["a"].shape == (3, 4)
  open(path, "wb").write(bytes(raw[:-4]))
  with pytest.raises(tb.BundleError, match="truncated"):
    tb.BundleReader(prefix)["b"]
  # hand-made index: a bfloat16 tensor, a string tensor, a partitioned one
  bf = np.asarray([0x3f80, 0xc000, 0x0000, 0x7f80], np.uint16)   # 1, -2, 0, inf
  open(prefix + "2.data-00000-of-00001", "wb").write(bf.tobytes())
  items = [
      (b"", tb._serialize_header(1)),
      (b"bf", tb._serialize_entry(tb.DT_BFLOAT16, (2, 2), 0, 0, 8,
                                  tb.mask_crc(tb.crc32c(bf)))),
      (b"part", tb._serialize_entry(1, (2,), 0, 0, 8, 0) + bytes([0x3a, 0])),
      (b"str", tb._serialize_entry(7, (1,), 0, 0, 8, 0)),
      (b"wrong_size", tb._serialize_entry(1, (3,), 0, 0, 8, 0)),
  ]
  open(prefix + "2.index", "wb").write(tb.build_table(items))
  reader = tb.BundleReader(prefix + "2")
  got = reader["bf"]
  assert got.dtype == np.float32
  np.testing.assert_array_equal(got, [[1.0, -2.0], [0.0, np.inf]])
  for name, what in (("part", "partitioned"), ("str", "string"),
                     ("wrong_size", "bytes stored")):
    with pytest.raises(tb.BundleError, match=what):
      reader[name]
  open(prefix + "3.index", "wb").write(tb.build_table([(b"x", b"")]))
  with pytest.raises(tb.BundleError, match="header"):
    tb.BundleReader(prefix + "3")
  open(prefix + "4.index", "wb").write(tb.build_table(
      [(b"", bytes([0x08, 0x01, 0x10, 0x01]))]))
  with pytest.raises(tb.BundleError, match="big-endian"):
    tb.BundleReader(prefix + "4")


def test_latest_checkpoint(tmp_path):
  assert tb.latest_checkpoint(str(tmp_path)) is None
  prefix = str(tmp_path / "model.ckpt-7")
  tb.write_bundle(prefix, {"w": np.ones(3, np.float32)})
  tb.write_checkpoint_state(prefix)
  assert tb.latest_checkpoint(str(tmp_path)) == prefix
  text = open(str(tmp_path / "checkpoint")).read()
  assert text.splitlines()[0] == 'model_checkpoint_path: "model.ckpt-7"'
  (tmp_path / "checkpoint").write_text(
      'model_checkpoint_path: "/abs/model.ckpt-9"\n')
  assert tb.latest_checkpoint(str(tmp_path)) == "/abs/model.ckpt-9"


def test_hand_assembled_fixture(tmp_path):
  """tests/golden/hand_bundle.* were assembled byte by byte from the published
  format by tests/golden/make_bundle_fixture.py, which shares no code with the
  package: the reader must decode them, and the writer must reproduce them to
  the byte (a change that keeps reader and writer consistent with each other
  but moves either away from the format shows up here)."""
  golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
  prefix = os.path.join(golden, "hand_bundle")
  reader = tb.BundleReader(prefix)
  assert sorted(reader.keys()) == ["a/b", "a/c"]
  ab = reader.get_tensor("a/b")
  ac = reader.get_tensor("a/c")
  assert ab.dtype == np.float32 and ab.shape == (2, 3)
  np.testing.assert_array_equal(ab, np.arange(6, dtype=np.float32).reshape(2, 3))
  assert ac.dtype == np.int32 and ac.shape == (4,)
  np.testing.assert_array_equal(ac, np.array([7, -1, 0, 2 ** 31 - 1], np.int32))
  out = str(tmp_path / "rewritten")
  tb.write_bundle(out, {"a/c": ac, "a/b": ab})
  for suffix in (".index", ".data-00000-of-00001"):
    with open(prefix + suffix, "rb") as f, open(out + suffix, "rb") as g:
      assert f.read() == g.read(), suffix
