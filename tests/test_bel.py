"""Graph file pair (.col / .dst): layout as the reference's reader expects it (benchmarks/bfs/main.cu:1238-1284)."""
import errno
import json
import os
import struct

import numpy as np
import pytest

from bam_amd import bel

G = os.path.join(os.path.dirname(__file__), "golden")


def test_layout_on_disk_and_round_trip(tmp_path):
    with open(os.path.join(G, "sample_graph.json")) as f:
        g = json.load(f)
    off = np.array(g["offsets"], dtype=np.uint64)
    nb = np.array(g["edges"], dtype=np.uint64)
    prefix = str(tmp_path / "sample.bel")
    bel.write(prefix, off, nb)
    # header: count, one ignored word, then the payload, all little-endian u64
    col = open(prefix + ".col", "rb").read()
    dst = open(prefix + ".dst", "rb").read()
    assert len(col) == 16 + 8 * len(off) and len(dst) == 16 + 8 * len(nb)
    assert struct.unpack("<Q", col[:8])[0] == len(off) and struct.unpack("<Q", dst[:8])[0] == len(nb)
    assert col[16:] == off.astype("<u8").tobytes() and dst[16:] == nb.astype("<u8").tobytes()
    assert bel.info(prefix) == (len(off), len(nb))
    assert np.array_equal(bel.read_offsets(prefix), off)
    assert np.array_equal(bel.read_edges(prefix), nb)
    assert np.array_equal(bel.read_edges(prefix, 5, 7), nb[5:12])
    assert len(bel.read_edges(prefix, len(nb), 0)) == 0


def test_a_file_written_by_hand_is_read(tmp_path):
    """the reader takes what any writer of the format produces; the second header word is ignored"""
    prefix = str(tmp_path / "hand")
    off = [0, 2, 2, 3]
    nb = [1, 2, 0]
    with open(prefix + ".col", "wb") as f:
        f.write(struct.pack("<QQ", len(off), 0xdeadbeef) + struct.pack("<%dQ" % len(off), *off))
    with open(prefix + ".dst", "wb") as f:
        f.write(struct.pack("<QQ", len(nb), 12345) + struct.pack("<%dQ" % len(nb), *nb))
    assert bel.info(prefix) == (4, 3)
    assert bel.read_offsets(prefix).tolist() == off and bel.read_edges(prefix).tolist() == nb


def test_bad_input_is_refused(tmp_path):
    prefix = str(tmp_path / "bad")
    with pytest.raises(OSError) as e:
        bel.info(prefix)
    assert e.value.errno == errno.ENOENT
    with pytest.raises(OSError):
        bel.write(prefix, [1, 2], [0, 0])                     # offsets must start at 0 and end at E
    # offsets that go down, or do not end at E
    for off in ([0, 3, 2, 3], [0, 1, 2, 2]):
        with open(prefix + ".col", "wb") as f:
            f.write(struct.pack("<QQ", 4, 0) + struct.pack("<4Q", *off))
        with open(prefix + ".dst", "wb") as f:
            f.write(struct.pack("<QQ", 3, 0) + struct.pack("<3Q", 1, 2, 0))
        with pytest.raises(OSError) as e:
            bel.read_offsets(prefix)
        assert e.value.errno == errno.EILSEQ
    with pytest.raises(OSError) as e:
        bel.read_edges(prefix, 2, 5)
    assert e.value.errno == errno.ERANGE
    # truncated payload
    with open(prefix + ".dst", "wb") as f:
        f.write(struct.pack("<QQ", 3, 0) + struct.pack("<2Q", 1, 2))
    with pytest.raises(OSError) as e:
        bel.read_edges(prefix)
    assert e.value.errno == errno.EIO


def test_empty_graph(tmp_path):
    prefix = str(tmp_path / "empty")
    bel.write(prefix, [0, 0, 0], [])
    assert bel.info(prefix) == (3, 0)
    assert bel.read_offsets(prefix).tolist() == [0, 0, 0] and len(bel.read_edges(prefix)) == 0
