"""Reading and writing TensorFlow tensor-bundle ("V2") checkpoint files.

The reference restores and saves variables through TensorFlow
(tf.train.init_from_checkpoint at mesh_tensorflow/transformer/utils.py:947-972,
the saver hooks at mesh_tensorflow/ops.py:5740-5779); the files those calls
read and write are TensorFlow's tensor bundles.  TensorFlow is a dependency of
the reference that is not vendored in it and not installed here, so this module
restates the published file format (tensorflow/core/util/tensor_bundle and
tensorflow/core/lib/io/{format,block,table_builder}.cc, stable since 1.0):

  <prefix>.index                 a sorted string table (LevelDB table layout):
      data blocks of prefix-compressed (key, value) entries with restart
      points, one index block whose values are the data blocks' handles, an
      empty meta-index block, and a 48-byte footer ending in the magic number
      0xdb4775248b80fb57.  Every block is followed by one compression byte
      (0: none) and a masked CRC-32C of block + byte.  Key "" holds a
      BundleHeaderProto, every other key is a tensor name holding a
      BundleEntryProto (dtype, shape, shard, offset, size, masked CRC-32C).
  <prefix>.data-SSSSS-of-NNNNN   the tensors' bytes, little endian, row major.

PARITY UNPINNED: no file written by TensorFlow exists here to read back, and no
TensorFlow to read what this module writes.  What is checked: CRC-32C against
the known answers of RFC 3720, the checksum mask against its inverse, the
reader against the writer over every dtype, multi-block tables and multi-shard
bundles, and both against a two-tensor bundle assembled byte by byte from the
published format by a script that shares no code with this module
(tests/golden/make_bundle_fixture.py).

Not handled, each with its own error: Snappy-compressed table blocks
(TensorFlow's bundle writer writes none), partitioned variables (entries with
slices), string / variant / resource tensors, big-endian bundles.
"""

import collections
import os
import re
import struct

import numpy as np

from mesh_amd import moe_hip

TABLE_MAGIC = 0xdb4775248b80fb57
FOOTER_BYTES = 48
BLOCK_TRAILER_BYTES = 5
BLOCK_BYTES = 262144        # TensorFlow's table::Options::block_size
RESTART_INTERVAL = 16       # entries between restart points of a data block
_MASK_DELTA = 0xa282ead8

# tensorflow/core/framework/types.proto
_DTYPES = {
    1: np.dtype("<f4"), 2: np.dtype("<f8"), 3: np.dtype("<i4"),
    4: np.dtype("u1"), 5: np.dtype("<i2"), 6: np.dtype("i1"),
    9: np.dtype("<i8"), 10: np.dtype("?"), 17: np.dtype("<u2"),
    19: np.dtype("<f2"), 22: np.dtype("<u4"), 23: np.dtype("<u8"),
}
DT_BFLOAT16 = 14
_DTYPE_CODES = {v: k for k, v in _DTYPES.items()}
_UNREADABLE = {7: "string", 20: "resource", 21: "variant"}

BundleEntry = collections.namedtuple(
    "BundleEntry", ["dtype", "shape", "shard_id", "offset", "size", "crc32c",
                    "sliced"])


class BundleError(ValueError):
  """A tensor-bundle file is malformed or uses a feature not handled here."""


def crc32c(data, crc=0):
  """CRC-32C of a bytes-like object or a C-contiguous NumPy array, continued
  from `crc` (tensorflow/core/lib/hash/crc32c.h Extend).  Computed by the
  shared library; there is no Python fallback."""
  lib = moe_hip.load_library()
  if isinstance(data, np.ndarray):
    if not data.flags["C_CONTIGUOUS"]:
      raise BundleError("crc32c needs a C-contiguous array")
    return lib.mesh_moe_crc32c(crc, data.ctypes.data, data.nbytes)
  data = bytes(data)
  return lib.mesh_moe_crc32c(crc, data, len(data))


def mask_crc(crc):
  """The rotated and offset form checksums are stored in (crc32c.h Mask)."""
  return (((crc >> 15) | (crc << 17)) + _MASK_DELTA) & 0xffffffff


def unmask_crc(masked):
  rot = (masked - _MASK_DELTA) & 0xffffffff
  return ((rot >> 17) | (rot << 15)) & 0xffffffff


# --- varints and the three protocol-buffer messages of the format -----------

def _put_varint(value):
  if value < 0:
    value += 1 << 64
  out = bytearray()
  while value >= 0x80:
    out.append((value & 0x7f) | 0x80)
    value >>= 7
  out.append(value)
  return bytes(out)


def _get_varint(buf, pos):
  result = shift = 0
  while True:
    if pos >= len(buf) or shift > 63:
      raise BundleError("truncated or overlong varint")
    byte = buf[pos]
    pos += 1
    result |= (byte & 0x7f) << shift
    if byte < 0x80:
      return result, pos
    shift += 7


def _fields(buf):
  """Yields (field number, wire type, value) of a serialized message."""
  pos = 0
  while pos < len(buf):
    tag, pos = _get_varint(buf, pos)
    number, wire = tag >> 3, tag & 7
    if wire == 0:
      value, pos = _get_varint(buf, pos)
    elif wire == 1:
      value, pos = buf[pos:pos + 8], pos + 8
    elif wire == 2:
      size, pos = _get_varint(buf, pos)
      value, pos = buf[pos:pos + size], pos + size
    elif wire == 5:
      value, pos = buf[pos:pos + 4], pos + 4
    else:
      raise BundleError("unsupported wire type %d" % wire)
    if pos > len(buf):
      raise BundleError("truncated message")
    yield number, wire, value


def _signed(value):
  return value - (1 << 64) if value >= 1 << 63 else value


def _parse_shape(buf):
  dims = []
  for number, _, value in _fields(buf):
    if number == 2:                                   # repeated Dim dim
      size = 0
      for n2, _, v2 in _fields(value):
        if n2 == 1:
          size = _signed(v2)
      dims.append(size)
    elif number == 3 and value:
      raise BundleError("tensor of unknown rank")
  return tuple(dims)


def _parse_entry(buf):
  dtype = shard = offset = size = crc = 0
  shape, sliced = (), False
  for number, _, value in _fields(buf):
    if number == 1:
      dtype = value
    elif number == 2:
      shape = _parse_shape(value)
    elif number == 3:
      shard = value
    elif number == 4:
      offset = _signed(value)
    elif number == 5:
      size = _signed(value)
    elif number == 6:
      crc = struct.unpack("<I", value)[0]
    elif number == 7:
      sliced = True
  return BundleEntry(dtype, shape, shard, offset, size, crc, sliced)


def _parse_header(buf):
  num_shards, endianness = 0, 0
  for number, _, value in _fields(buf):
    if number == 1:
      num_shards = value
    elif number == 2:
      endianness = value
  return num_shards, endianness


def _message(number, payload):
  return _put_varint((number << 3) | 2) + _put_varint(len(payload)) + payload


def _serialize_entry(dtype_code, shape, shard_id, offset, size, masked_crc):
  out = _put_varint(1 << 3) + _put_varint(dtype_code)
  dims = b"".join(
      _message(2, (_put_varint(1 << 3) + _put_varint(d)) if d else b"")
      for d in shape)
  out += _message(2, dims)
  if shard_id:
    out += _put_varint(3 << 3) + _put_varint(shard_id)
  if offset:
    out += _put_varint(4 << 3) + _put_varint(offset)
  if size:
    out += _put_varint(5 << 3) + _put_varint(size)
  if masked_crc:
    out += _put_varint((6 << 3) | 5) + struct.pack("<I", masked_crc)
  return out


def _serialize_header(num_shards):
  # endianness LITTLE (0) is the default and omitted; version {producer: 1}
  version = _put_varint(1 << 3) + _put_varint(1)
  return _put_varint(1 << 3) + _put_varint(num_shards) + _message(3, version)


# --- the string table --------------------------------------------------------

def _read_block(buf, offset, size, verify):
  end = offset + size
  if offset < 0 or end + BLOCK_TRAILER_BYTES > len(buf):
    raise BundleError("block handle (%d, %d) outside the file" % (offset, size))
  kind = buf[end]
  if verify:
    stored = struct.unpack("<I", buf[end + 1:end + 5])[0]
    if unmask_crc(stored) != crc32c(buf[offset:end + 1]):
      raise BundleError("block checksum mismatch at offset %d" % offset)
  if kind == 1:
    raise BundleError("Snappy-compressed table block (not handled)")
  if kind != 0:
    raise BundleError("unknown block compression %d" % kind)
  return buf[offset:end]


def _block_entries(block):
  if len(block) < 4:
    raise BundleError("block too short")
  restarts = struct.unpack("<I", block[-4:])[0]
  limit = len(block) - 4 * (restarts + 1)
  if limit < 0:
    raise BundleError("bad restart count")
  pos, key = 0, b""
  while pos < limit:
    shared, pos = _get_varint(block, pos)
    unshared, pos = _get_varint(block, pos)
    vlen, pos = _get_varint(block, pos)
    if shared > len(key) or pos + unshared + vlen > limit:
      raise BundleError("corrupt block entry")
    key = key[:shared] + block[pos:pos + unshared]
    pos += unshared
    yield key, block[pos:pos + vlen]
    pos += vlen


def read_table(buf, verify=True):
  """[(key, value)] of a serialized string table, in key order."""
  buf = bytes(buf)
  if len(buf) < FOOTER_BYTES:
    raise BundleError("file too short for a table footer")
  footer = buf[-FOOTER_BYTES:]
  if struct.unpack("<Q", footer[-8:])[0] != TABLE_MAGIC:
    raise BundleError("bad table magic number")
  pos = 0
  _, pos = _get_varint(footer, pos)           # meta-index handle (unused)
  _, pos = _get_varint(footer, pos)
  index_offset, pos = _get_varint(footer, pos)
  index_size, pos = _get_varint(footer, pos)
  out = []
  for _, handle in _block_entries(
      _read_block(buf, index_offset, index_size, verify)):
    offset, p2 = _get_varint(handle, 0)
    size, _ = _get_varint(handle, p2)
    out.extend(_block_entries(_read_block(buf, offset, size, verify)))
  return out


class _BlockBuilder(object):

  def __init__(self, restart_interval):
    self._interval = restart_interval
    self.reset()

  def reset(self):
    self._buf = bytearray()
    self._restarts = [0]
    self._since_restart = 0
    self.last_key = b""
    self.empty = True

  def add(self, key, value):
    shared = 0
    if self._since_restart < self._interval:
      limit = min(len(key), len(self.last_key))
      while shared < limit and key[shared] == self.last_key[shared]:
        shared += 1
    else:
      self._restarts.append(len(self._buf))
      self._since_restart = 0
    self._buf += (_put_varint(shared) + _put_varint(len(key) - shared) +
                  _put_varint(len(value)) + key[shared:] + value)
    self._since_restart += 1
    self.last_key = key
    self.empty = False

  def size(self):
    return len(self._buf) + 4 * (len(self._restarts) + 1)

  def finish(self):
    return bytes(self._buf) + struct.pack(
        "<%dI" % (len(self._restarts) + 1),
        *(self._restarts + [len(self._restarts)]))


def build_table(items, block_bytes=BLOCK_BYTES):
  """Serializes [(key, value)] (bytes, sorted by key, keys distinct)."""
  out = bytearray()

  def emit(block):
    handle = _put_varint(len(out)) + _put_varint(len(block))
    trailer = b"\x00"
    out.extend(block + trailer +
               struct.pack("<I", mask_crc(crc32c(block + trailer))))
    return handle

  data = _BlockBuilder(RESTART_INTERVAL)
  index = _BlockBuilder(1)
  previous = None
  for key, value in items:
    if previous is not None and key <= previous:
      raise BundleError("table keys must be distinct and ascending")
    previous = key
    data.add(key, value)
    if data.size() >= block_bytes:
      # the block's own last key separates it from the next block
      index.add(data.last_key, emit(data.finish()))
      data.reset()
  if not data.empty:
    index.add(data.last_key, emit(data.finish()))
  meta_handle = emit(_BlockBuilder(1).finish())
  index_handle = emit(index.finish())
  footer = meta_handle + index_handle
  footer += b"\x00" * (FOOTER_BYTES - 8 - len(footer))
  out.extend(footer + struct.pack("<Q", TABLE_MAGIC))
  return bytes(out)


# --- bundles -------------------------------------------------------------------

def _data_path(prefix, shard, num_shards):
  return "%s.data-%05d-of-%05d" % (prefix, shard, num_shards)


def latest_checkpoint(directory):
  """The prefix named by model_checkpoint_path in `directory`/checkpoint (the
  text file tf.train.latest_checkpoint reads), or None."""
  state = os.path.join(directory, "checkpoint")
  if not os.path.exists(state):
    return None
  with open(state) as f:
    match = re.search(r'^model_checkpoint_path:\s*"(.*)"\s*$', f.read(), re.M)
  if not match:
    return None
  path = match.group(1)
  return path if os.path.isabs(path) else os.path.join(directory, path)


class BundleReader(object):
  """Read access to one bundle, with the interface of a name -> array mapping
  (`keys`, `in`, `[]`) plus `dtype_code(name)` and `shape(name)`.

  bfloat16 tensors come back as float32 (NumPy has no bfloat16); every other
  dtype as itself.  With verify_checksums every tensor read is checked against
  its stored CRC-32C, as TensorFlow's reader does.
  """

  def __init__(self, prefix, verify_checksums=True):
    self.prefix = prefix
    self._verify = verify_checksums
    with open(prefix + ".index", "rb") as f:
      items = read_table(f.read(), verify=True)
    if not items or items[0][0] != b"":
      raise BundleError("bundle header entry is missing")
    self.num_shards, endianness = _parse_header(items[0][1])
    if endianness != 0:
      raise BundleError("big-endian bundle (not handled)")
    self._entries = collections.OrderedDict(
        (key.decode("utf-8"), _parse_entry(value)) for key, value in items[1:])

  def keys(self):
    return list(self._entries)

  def __contains__(self, name):
    return name in self._entries

  def __iter__(self):
    return iter(self._entries)

  def __len__(self):
    return len(self._entries)

  def entry(self, name):
    return self._entries[name]

  def dtype_code(self, name):
    return self._entries[name].dtype

  def shape(self, name):
    return self._entries[name].shape

  def __getitem__(self, name):
    entry = self._entries[name]
    if entry.sliced:
      raise BundleError("%s is a partitioned variable (not handled)" % name)
    if entry.dtype in _UNREADABLE:
      raise BundleError("%s is a %s tensor (not handled)"
                        % (name, _UNREADABLE[entry.dtype]))
    if entry.dtype == DT_BFLOAT16:
      dtype = np.dtype("<u2")
    elif entry.dtype in _DTYPES:
      dtype = _DTYPES[entry.dtype]
    else:
      raise BundleError("%s has unknown dtype %d" % (name, entry.dtype))
    count = int(np.prod(entry.shape, dtype=np.int64)) if entry.shape else 1
    if count * dtype.itemsize != entry.size:
      raise BundleError("%s: %d bytes stored, shape %s needs %d"
                        % (name, entry.size, entry.shape,
                           count * dtype.itemsize))
    path = _data_path(self.prefix, entry.shard_id, self.num_shards)
    with open(path, "rb") as f:
      f.seek(entry.offset)
      value = np.fromfile(f, dtype=dtype, count=count)
    if value.size != count:
      raise BundleError("%s: data file %s is truncated" % (name, path))
    if self._verify and unmask_crc(entry.crc32c) != crc32c(value):
      raise BundleError("%s: tensor checksum mismatch" % name)
    if entry.dtype == DT_BFLOAT16:
      value = (value.astype(np.uint32) << 16).view(np.float32)
    return value.reshape(entry.shape)

  get_tensor = __getitem__


def write_bundle(prefix, tensors, num_shards=1, block_bytes=BLOCK_BYTES):
  """Writes {name: array} as <prefix>.index and <prefix>.data-*.  Tensors go
  to the shards round-robin in name order (one shard is what a TensorFlow 1
  saver on one host writes)."""
  if num_shards < 1:
    raise BundleError("num_shards must be positive")
  names = sorted(tensors, key=lambda n: n.encode("utf-8"))
  if "" in tensors:
    raise BundleError("the empty tensor name is reserved for the header")
  directory = os.path.dirname(prefix)
  if directory:
    os.makedirs(directory, exist_ok=True)
  files = [open(_data_path(prefix, s, num_shards), "wb")
           for s in range(num_shards)]
  offsets = [0] * num_shards
  items = [(b"", _serialize_header(num_shards))]
  try:
    for i, name in enumerate(names):
      value = np.asarray(tensors[name])
      dtype = value.dtype.newbyteorder("<") if value.dtype.byteorder == ">" \
          else value.dtype
      if np.dtype(dtype) not in _DTYPE_CODES:
        raise BundleError("%s: dtype %s cannot be stored" % (name, value.dtype))
      value = np.asarray(value, dtype=dtype, order="C")   # keeps rank 0
      shard = i % num_shards
      files[shard].write(value.reshape(-1).view(np.uint8))
      items.append((name.encode("utf-8"), _serialize_entry(
          _DTYPE_CODES[np.dtype(dtype)], value.shape, shard, offsets[shard],
          value.nbytes, mask_crc(crc32c(value)))))
      offsets[shard] += value.nbytes
  finally:
    for f in files:
      f.close()
  with open(prefix + ".index", "wb") as f:
    f.write(build_table(items, block_bytes))


def write_checkpoint_state(prefix):
  """Points `checkpoint` in the prefix's directory at it, as a saver does."""
  directory = os.path.dirname(prefix) or "."
  base = os.path.basename(prefix)
  with open(os.path.join(directory, "checkpoint"), "w") as f:
    f.write('model_checkpoint_path: "%s"\n' % base)
    f.write('all_model_checkpoint_paths: "%s"\n' % base)
