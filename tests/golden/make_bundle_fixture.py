"""Writes tests/golden/hand_bundle.index and hand_bundle.data-00000-of-00001:
a two-tensor TensorFlow tensor bundle assembled byte by byte from the
published format (tensorflow/core/lib/io/format.cc, block_builder.cc,
table_builder.cc; tensorflow/core/protobuf/tensor_bundle.proto;
tensorflow/core/lib/hash/crc32c.h), without the package's reader or writer.
The checksums come from the bitwise CRC-32C below (Castagnoli polynomial,
reflected: 0x82f63b78), not from the library.

  "a/b"  float32 [2, 3] = 0, 1, 2, 3, 4, 5        bytes  0 .. 23 of the data file
  "a/c"  int32   [4]    = 7, -1, 0, 2**31 - 1     bytes 24 .. 39

Run from the repository root: python tests/golden/make_bundle_fixture.py
"""

import os
import struct


def crc32c_bitwise(data):
  crc = 0xffffffff
  for byte in data:
    crc ^= byte
    for _ in range(8):
      crc = (crc >> 1) ^ (0x82f63b78 if crc & 1 else 0)
  return crc ^ 0xffffffff


def masked(data):
  """crc32c::Mask: rotate right by 15 bits, add 0xa282ead8."""
  crc = crc32c_bitwise(data)
  return (((crc >> 15) | (crc << 17)) + 0xa282ead8) & 0xffffffff


def with_trailer(block):
  """A table block as stored: the block, compression byte 0 (none), masked
  CRC-32C of both, little endian."""
  return block + b"\x00" + struct.pack("<I", masked(block + b"\x00"))


def main():
  here = os.path.dirname(os.path.abspath(__file__))
  ab = struct.pack("<6f", 0, 1, 2, 3, 4, 5)
  ac = struct.pack("<4i", 7, -1, 0, 2 ** 31 - 1)
  with open(os.path.join(here, "hand_bundle.data-00000-of-00001"), "wb") as f:
    f.write(ab + ac)

  # BundleHeaderProto {num_shards: 1, version {producer: 1}}; endianness
  # LITTLE = 0 is the default and not written
  header = bytes([0x08, 0x01,              # field 1 varint: num_shards = 1
                  0x1a, 0x02, 0x08, 0x01])  # field 3 message: version.producer = 1
  # BundleEntryProto of "a/b": dtype DT_FLOAT, shape [2, 3], shard 0 and
  # offset 0 (defaults, not written), size 24, crc32c
  entry_ab = bytes([0x08, 0x01,                            # dtype = 1
                    0x12, 0x08,                            # shape, 8 bytes:
                    0x12, 0x02, 0x08, 0x02,                #   dim {size: 2}
                    0x12, 0x02, 0x08, 0x03,                #   dim {size: 3}
                    0x28, 0x18,                            # size = 24
                    0x35]) + struct.pack("<I", masked(ab))  # crc32c (fixed32)
  # "a/c": dtype DT_INT32, shape [4], offset 24, size 16
  entry_ac = bytes([0x08, 0x03,                            # dtype = 3
                    0x12, 0x04, 0x12, 0x02, 0x08, 0x04,    # shape {dim {size: 4}}
                    0x20, 0x18,                            # offset = 24
                    0x28, 0x10,                            # size = 16
                    0x35]) + struct.pack("<I", masked(ac))
  # data block: entries (shared key bytes, unshared key bytes, value bytes,
  # key suffix, value), then the restart array [0] and its length 1
  data_block = (
      bytes([0x00, 0x00, len(header)]) + header +                  # key ""
      bytes([0x00, 0x03, len(entry_ab)]) + b"a/b" + entry_ab +     # key "a/b"
      bytes([0x02, 0x01, len(entry_ac)]) + b"c" + entry_ac +       # key "a/" + "c"
      struct.pack("<II", 0, 1))
  assert len(data_block) < 128          # its size is a one-byte varint below
  meta_block = struct.pack("<II", 0, 1)  # no entries
  stored_data = with_trailer(data_block)
  stored_meta = with_trailer(meta_block)
  # index block: the data block's last key -> its handle (offset 0, size)
  data_handle = bytes([0x00, len(data_block)])
  index_block = (bytes([0x00, 0x03, len(data_handle)]) + b"a/c" + data_handle +
                 struct.pack("<II", 0, 1))
  stored_index = with_trailer(index_block)
  meta_offset = len(stored_data)
  index_offset = meta_offset + len(stored_meta)
  assert index_offset < 128
  footer = bytes([meta_offset, len(meta_block), index_offset, len(index_block)])
  footer += b"\x00" * (40 - len(footer))
  footer += struct.pack("<Q", 0xdb4775248b80fb57)
  with open(os.path.join(here, "hand_bundle.index"), "wb") as f:
    f.write(stored_data + stored_meta + stored_index + footer)


if __name__ == "__main__":
  main()
