"""hnswlib index file format (cpp/src/cuhnsw_base.cu:159-365 of the reference):
closed-form byte layout of a hand-built 3-node index, written by the oracle and by
the product library's host-side reader/writer (which needs no GPU)."""
import os
import struct

import numpy as np
import pytest

from cuhnsw_amd import capi


def three_node_index(oracle):
  # D = 2, max_m = 2, max_m0 = 3; node 1 has one upper level
  vec = np.array([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], np.float32)
  levels = np.array([0, 1, 0], np.int32)
  links0 = np.array([[2, 1, 2, 0], [2, 0, 2, 0], [1, 1, 0, 0]], np.uint32)
  up = np.array([0, 0, 0], np.uint32)  # node 1, level 1: no links
  ix = oracle.OracleIndex("l2").from_arrays(vec, levels, links0, up, max_m=2, max_m0=3, maxlevel=1,
                                            enterpoint=1, labels=np.array([10, 11, 12], np.uint64),
                                            mult=0.5, efc=77)
  return ix, vec


def expected_bytes():
  size_links0 = 3 * 4 + 4
  size_data = size_links0 + 2 * 4 + 8
  header = struct.pack("<QQQQQQiIQQQdQ", 0, 3, 3, size_data, size_links0 + 8, size_links0, 1, 1, 2, 3, 2, 0.5, 77)
  assert len(header) == 96
  body = b""
  rows = [((2, 1, 2, 0), (1.0, 2.0), 10), ((2, 0, 2, 0), (3.0, 4.0), 11), ((1, 1, 0, 0), (5.0, 6.0), 12)]
  for links, v, label in rows:
    body += struct.pack("<4I2fQ", *links, *v, label)
  upper = struct.pack("<I", 0) + struct.pack("<I", 12) + struct.pack("<3I", 0, 0, 0) + struct.pack("<I", 0)
  return header + body + upper


def test_oracle_writer_bytes(oracle, tmp_path):
  ix, _ = three_node_index(oracle)
  p = str(tmp_path / "a.idx")
  ix.save(p)
  assert open(p, "rb").read() == expected_bytes()


def test_oracle_reader_roundtrip(oracle, tmp_path):
  p = str(tmp_path / "a.idx")
  open(p, "wb").write(expected_bytes())
  ix = oracle.OracleIndex("l2").load(p)
  assert (ix.num_data, ix.num_dims, ix.maxlevel, ix.enterpoint, ix.max_m, ix.max_m0) == (3, 2, 1, 1, 2, 3)
  assert list(ix.levels()) == [0, 1, 0]
  assert list(ix.labels()) == [10, 11, 12]
  assert list(ix.links(0, 0)) == [1, 2] and list(ix.links(2, 0)) == [1] and list(ix.links(1, 1)) == []
  q = str(tmp_path / "b.idx")
  ix.save(q)
  assert open(q, "rb").read() == expected_bytes()


def test_library_reader_writer_bytes(tmp_path):
  """The product's own host-side file code: load -> save is byte-identical."""
  p, q = str(tmp_path / "a.idx"), str(tmp_path / "b.idx")
  open(p, "wb").write(expected_bytes())
  e = capi.Engine()
  e.load_index(p)
  assert (e.num_data, e.num_dims, e.max_level, e.enter_point) == (3, 2, 1, 1)
  e.save_index(q)
  assert open(q, "rb").read() == expected_bytes()


def test_library_reads_hnswlib_count_word_flags(tmp_path):
  """hnswlib keeps the link count in the low 16 bits of the count word; the bits above are flags.
  Unknown flag bits are masked off.  Bit 0 of the third byte is hnswlib's delete mark: it is kept (the
  search walks through such an element and never returns it) and written back by save_index."""
  raw = bytearray(expected_bytes())
  struct.pack_into("<I", raw, 96, 2 | (1 << 17) | (1 << 31))
  p, q = str(tmp_path / "a.idx"), str(tmp_path / "b.idx")
  open(p, "wb").write(bytes(raw))
  e = capi.Engine()
  e.load_index(p)
  e.save_index(q)
  assert open(q, "rb").read() == expected_bytes()
  size_data = 3 * 4 + 4 + 2 * 4 + 8
  struct.pack_into("<I", raw, 96 + size_data, 2 | (1 << 16))     # node 1 marked deleted
  open(p, "wb").write(bytes(raw))
  assert e.num_deleted == 0
  e.load_index(p)
  assert e.num_data == 3 and e.num_deleted == 1
  e.save_index(q)
  marked = bytearray(expected_bytes())
  struct.pack_into("<I", marked, 96 + size_data, 2 | (1 << 16))
  assert open(q, "rb").read() == bytes(marked)                    # the mark is back, the unknown flags are not
  open(p, "wb").write(expected_bytes())
  e.load_index(p)
  assert e.num_deleted == 0                                       # the marks belong to the file they came from


def spare_capacity_bytes(spare=2):
  """The 3-node index as hnswlib writes it from an index created with max_elements = 3 + spare:
  the level-0 block has max_elements records (the unused ones are whatever the allocation held,
  here a pattern), the upper block one entry per existing element."""
  good = expected_bytes()
  size_data = 3 * 4 + 4 + 2 * 4 + 8
  header = bytearray(good[:96])
  struct.pack_into("<Q", header, 8, 3 + spare)                    # max_elements; cur_element_count stays 3
  body = good[96:96 + 3 * size_data]
  junk = bytes((0xA5 + i) & 0xFF for i in range(spare * size_data))
  return bytes(header) + body + junk + good[96 + 3 * size_data:]


def test_library_reads_files_with_spare_capacity(oracle, tmp_path):
  """max_elements > cur_element_count (an hnswlib index that was not filled up): the unused records
  are skipped, and saving writes the compact form."""
  p, q = str(tmp_path / "spare.idx"), str(tmp_path / "compact.idx")
  for spare in (1, 2, 1000):
    open(p, "wb").write(spare_capacity_bytes(spare))
    e = capi.Engine()
    e.load_index(p)
    assert (e.num_data, e.num_dims, e.max_level, e.enter_point) == (3, 2, 1, 1)
    e.save_index(q)
    assert open(q, "rb").read() == expected_bytes()
    ix = oracle.OracleIndex("l2").load(p)                         # the checker reads it the same way
    assert ix.num_data == 3 and list(ix.links(0, 0)) == [1, 2] and list(ix.labels()) == [10, 11, 12]
  raw = spare_capacity_bytes(2)
  open(p, "wb").write(raw[:len(raw) - 30])                        # spare records present, upper block cut short
  with pytest.raises(RuntimeError, match="truncated"):
    capi.Engine().load_index(p)
  header = bytearray(raw)
  struct.pack_into("<Q", header, 8, 2)                            # max_elements below cur_element_count
  open(p, "wb").write(bytes(header))
  with pytest.raises(RuntimeError, match="inconsistent header"):
    capi.Engine().load_index(p)


def test_library_rejects_bad_files(tmp_path):
  e = capi.Engine()
  with pytest.raises(RuntimeError, match="cannot open"):
    e.load_index(str(tmp_path / "missing.idx"))
  good = expected_bytes()
  for cut in (10, 95, 100, len(good) - 1):
    p = str(tmp_path / ("cut%d.idx" % cut))
    open(p, "wb").write(good[:cut])
    with pytest.raises(RuntimeError, match="truncated"):
      e.load_index(p)
  raw = bytearray(good)
  struct.pack_into("<I", raw, 96, 9)  # link count above max_m0
  p = str(tmp_path / "deg.idx")
  open(p, "wb").write(bytes(raw))
  with pytest.raises(RuntimeError, match="link count"):
    e.load_index(p)
  raw = bytearray(good)
  struct.pack_into("<I", raw, 100, 7)  # link id out of range
  p = str(tmp_path / "id.idx")
  open(p, "wb").write(bytes(raw))
  with pytest.raises(RuntimeError, match="out of range"):
    e.load_index(p)
  with pytest.raises(RuntimeError, match="no index"):
    capi.Engine().save_index(str(tmp_path / "x.idx"))


def test_bigger_roundtrip_oracle_to_library(oracle, tmp_path):
  from helpers import gauss_mixture
  x = gauss_mixture(500, 10, seed=3)
  rng = np.random.default_rng(0)
  levels = (-np.log(rng.uniform(size=500)) * 0.5).astype(np.int32)
  ix = oracle.OracleIndex("dot").build(x, levels, 4, 8, 20, 0.5, threads=1)
  p, q = str(tmp_path / "o.idx"), str(tmp_path / "l.idx")
  ix.save(p)
  e = capi.Engine()
  e.load_index(p)
  e.save_index(q)
  assert open(p, "rb").read() == open(q, "rb").read()
  assert os.path.getsize(p) == 96 + 500 * (8 * 4 + 4 + 10 * 4 + 8) + 500 * 4 + int(levels.sum()) * (4 * 4 + 4)
