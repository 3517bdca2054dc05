"""File formats of the search path: byte-level known answers built from the
layouts in the reference (src/disk.cpp:22-37, 155-179, 336-426; src/graph.cpp:316-351;
include/efanna2e/util.h:81-218; src/graph.cu:709-735), round trips, and the error
paths a loader must take on damaged input.  Runs without a GPU."""
import ctypes
import os
import struct

import numpy as np
import pytest

from coral_amd import capi, formats as F


def test_fbin_layout_and_padding(tmp_path):
    x = np.arange(15, dtype=np.float32).reshape(3, 5)
    p = tmp_path / "a.fbin"
    F.fbin_write(p, x)
    raw = p.read_bytes()
    assert raw[:8] == struct.pack("<II", 3, 5) and raw[8:] == x.tobytes()
    assert F.fbin_meta(p) == (3, 5)
    y = F.fbin_read(p)  # padded to a multiple of 4 like load_data (util.h:194-208)
    assert y.shape == (3, 8) and np.array_equal(y[:, :5], x) and not y[:, 5:].any()


def test_fbin_errors(tmp_path):
    with pytest.raises(capi.CoralError) as e:
        F.fbin_meta(tmp_path / "missing.fbin")
    assert e.value.code == capi.ERR_IO
    p = tmp_path / "short.fbin"
    p.write_bytes(struct.pack("<II", 10, 4) + b"\0" * 16 * 9)  # one row short
    with pytest.raises(capi.CoralError, match="Data file size wrong"):
        F.fbin_meta(p)
    p.write_bytes(b"\1\0\0")
    with pytest.raises(capi.CoralError):
        F.fbin_meta(p)


def test_gt_layout_and_trailing_distances_ignored(tmp_path):
    ids = np.array([[5, 2, 9], [1, 0, 3]], np.int32)
    p = tmp_path / "gt.bin"
    F.gt_write(p, ids)
    assert p.read_bytes() == struct.pack("<II", 2, 3) + ids.tobytes()
    with open(p, "ab") as f:
        f.write(np.ones(6, np.float32).tobytes())  # comp_gt appends distances
    assert np.array_equal(F.gt_read(p), ids)
    p.write_bytes(struct.pack("<II", 2, 3) + ids.tobytes()[:-4])
    with pytest.raises(capi.CoralError):
        F.gt_read(p)


# ------------------------------------------------------------------ LZ4

def test_lz4_known_answer_blocks():
    # literals only: token 0x50, five literals
    assert F.lz4_decompress(b"\x50hello", 5) == b"hello"
    # one match: "abcd" then copy 8 bytes from offset 4 (overlapping), then 5 literals
    blk = b"\x44abcd\x04\x00" + b"\x50vwxyz"
    assert F.lz4_decompress(blk, 17) == b"abcd" + b"abcdabcd" + b"vwxyz"
    # long literal run (15 + 255 + 10 = 280) and long match (4 + 15 + 255 + 3 = 277) length bytes
    lit = bytes(range(256)) + bytes(24)
    blk = b"\xff" + b"\xff\x0a" + lit + b"\x01\x00" + b"\xff\x03" + b"\x50tail!"
    out = F.lz4_decompress(blk, 280 + 277 + 5)
    assert out == lit + bytes([lit[-1]]) * 277 + b"tail!"


@pytest.mark.parametrize("blk,size", [
    (b"", 4),                      # empty input
    (b"\x50hell", 5),              # literals run past the input
    (b"\x40abcd\x00\x00\x00", 16),  # offset 0
    (b"\x40abcd\x09\x00\x00", 16),  # offset before the start of output
    (b"\x4fabcd\x04\x00", 64),     # match length bytes missing
    (b"\x50hello", 3),             # output too small
])
def test_lz4_rejects_malformed(blk, size):
    with pytest.raises(ValueError):
        F.lz4_decompress(blk, size)


def _payloads():
    rng = np.random.RandomState(0)
    yield b""
    yield b"a"
    yield b"abcdefghijkl"  # 12 bytes: below the match limit
    yield b"a" * 13
    yield b"ab" * 300
    for n in (5, 64, 132, 260, 1000, 70000):
        yield rng.bytes(n)
        yield bytes(rng.randint(0, 3, n).astype(np.uint8))
    # a serialised graph row: deg, 32 ids, 32 distances
    yield struct.pack("<i32i32f", 32, *range(1000, 1032), *[0.5] * 32)


@pytest.mark.parametrize("raw", list(_payloads()), ids=lambda b: "len%d" % len(b))
def test_lz4_round_trip(raw):
    c = F.lz4_compress(raw)
    assert len(c) <= F._L().coral_lz4_compress_bound(len(raw))
    assert F.lz4_decompress(c, len(raw)) == raw


def _system_lz4():
    try:
        z = ctypes.CDLL("liblz4.so.1")
    except OSError:
        return None
    z.LZ4_compress_default.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
    z.LZ4_decompress_safe.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
    return z


@pytest.mark.parametrize("raw", [p for p in _payloads() if p], ids=lambda b: "len%d" % len(b))
def test_lz4_interoperates_with_system_liblz4(raw):
    """The reference writes blocks with LZ4_compress_default and reads them with
    LZ4_decompress_safe (src/disk.cpp:370,400): both directions must interoperate."""
    z = _system_lz4()
    if z is None:
        pytest.skip("liblz4.so.1 not present")
    out = ctypes.create_string_buffer(len(raw))
    ours = F.lz4_compress(raw)
    assert z.LZ4_decompress_safe(ours, out, len(ours), len(raw)) == len(raw) and out.raw == raw
    buf = ctypes.create_string_buffer(len(raw) + len(raw) // 255 + 32)
    n = z.LZ4_compress_default(raw, buf, len(raw), len(buf))
    assert F.lz4_decompress(buf.raw[:n], len(raw)) == raw


# ------------------------------------------------------------- index directory

def _graph(n, R, seed):
    rng = np.random.RandomState(seed)
    g = rng.randint(0, n, (n, R)).astype(np.int32)
    d = rng.rand(n, R).astype(np.float32)
    deg = rng.randint(0, R + 1, n)
    deg[0], deg[1] = 0, R
    for i in range(n):
        g[i, deg[i]:] = -1
        d[i, deg[i]:] = 0
    return g, d, deg


def test_index_directory_bytes(tmp_path):
    g, d, deg = _graph(50, 8, 1)
    F.graph_dir_write(tmp_path / "idx", g, d)
    names = sorted(os.listdir(tmp_path / "idx"))
    assert names == ["graph.batch_id", "graph.part0.append", "graph.part0.data", "graph.part0.idx"]
    idx = (tmp_path / "idx" / "graph.part0.idx").read_bytes()
    data = (tmp_path / "idx" / "graph.part0.data").read_bytes()
    assert len(idx) == 50 * 16  # {uint64 offset; uint32 size; int32 pos}
    for i in range(50):
        off, size, pos = struct.unpack_from("<QIi", idx, 16 * i)
        if deg[i] == 0:
            assert size == 0
            continue
        assert pos == 0
        node_id, raw_size = struct.unpack_from("<iI", data, off)
        assert node_id == i and raw_size == 4 + 8 * deg[i]
        raw = F.lz4_decompress(data[off + 8:off + size], raw_size)
        assert struct.unpack_from("<i", raw)[0] == deg[i]
        assert raw[4:4 + 4 * deg[i]] == g[i, :deg[i]].tobytes()
        assert raw[4 + 4 * deg[i]:] == d[i, :deg[i]].tobytes()
    g2, d2 = F.graph_dir_read(tmp_path / "idx", 50, 8, want_dists=True)
    assert np.array_equal(g, g2) and np.array_equal(d, d2)


def test_index_directory_reads_append_file_and_foreign_blocks(tmp_path):
    """A block written the way DiskPartition::write_node_append does (pos = APPEND,
    compressed by the system liblz4 when present) must load."""
    g, d, deg = _graph(20, 8, 2)
    F.graph_dir_write(tmp_path / "idx", g, d)
    z = _system_lz4()
    new_row = np.array([7, 3, 11], np.int32)
    new_d = np.array([0.25, 0.5, 0.75], np.float32)
    raw = struct.pack("<i", 3) + new_row.tobytes() + new_d.tobytes()
    if z is not None:
        buf = ctypes.create_string_buffer(len(raw) + 32)
        n = z.LZ4_compress_default(raw, buf, len(raw), len(buf))
        comp = buf.raw[:n]
    else:
        comp = F.lz4_compress(raw)
    block = struct.pack("<iI", 5, len(raw)) + comp
    (tmp_path / "idx" / "graph.part0.append").write_bytes(b"\xee" * 10 + block)
    ip = tmp_path / "idx" / "graph.part0.idx"
    table = bytearray(ip.read_bytes())
    struct.pack_into("<QIi", table, 16 * 5, 10, len(block), 1)
    ip.write_bytes(bytes(table))
    g2, d2 = F.graph_dir_read(tmp_path / "idx", 20, 8, want_dists=True)
    want = g.copy()
    want[5] = -1
    want[5, :3] = new_row
    assert np.array_equal(g2, want) and np.array_equal(d2[5, :3], new_d)


def test_index_directory_errors(tmp_path):
    g, d, _ = _graph(30, 8, 3)
    F.graph_dir_write(tmp_path / "idx", g, d)
    with pytest.raises(capi.CoralError, match="cannot open"):
        F.graph_dir_read(tmp_path / "nowhere", 30, 8)
    with pytest.raises(capi.CoralError, match="entries"):
        F.graph_dir_read(tmp_path / "idx", 31, 8)  # truncated .idx for this n
    with pytest.raises(capi.CoralError, match="degree exceeds"):
        F.graph_dir_read(tmp_path / "idx", 30, 4)
    dp = tmp_path / "idx" / "graph.part0.data"
    blob = bytearray(dp.read_bytes())
    off, size, _ = struct.unpack_from("<QIi", (tmp_path / "idx" / "graph.part0.idx").read_bytes(), 16)
    blob[off + 8] ^= 0xF0  # damage node 1's first token
    dp.write_bytes(bytes(blob))
    with pytest.raises(capi.CoralError, match="node 1"):
        F.graph_dir_read(tmp_path / "idx", 30, 8)
    dp.write_bytes(bytes(blob[:off + 4]))  # file ends inside node 1's block
    with pytest.raises(capi.CoralError, match="outside its file"):
        F.graph_dir_read(tmp_path / "idx", 30, 8)


def test_start_ids_text(tmp_path):
    os.makedirs(tmp_path / "idx")
    F.start_ids_write(tmp_path / "idx", [12, 7, 99])
    assert (tmp_path / "idx" / "graph.search_start_ids").read_text() == "3 12 7 99 "
    assert F.start_ids_read(tmp_path / "idx").tolist() == [12, 7, 99]
    # missing file and short list both leave no start ids (src/graph.cpp:329-351)
    assert F.start_ids_read(tmp_path / "elsewhere").size == 0
    (tmp_path / "idx" / "graph.search_start_ids").write_text("4 1 2")
    assert F.start_ids_read(tmp_path / "idx").size == 0


def test_hits_file(tmp_path):
    """hits.bin = int64 n + uint32[n] (include/ivf.cuh:639-656); a file of more counts serves a smaller index"""
    os.makedirs(tmp_path / "idx")
    hits = np.array([3, 0, 7, 4000000000, 1], np.uint32)
    F.hits_write(tmp_path / "idx", hits)
    raw = (tmp_path / "idx" / "hits.bin").read_bytes()
    assert raw == struct.pack("<q", 5) + hits.tobytes()
    assert F.hits_read(tmp_path / "idx", 5).tolist() == hits.tolist()
    assert F.hits_read(tmp_path / "idx", 3).tolist() == hits[:3].tolist()
    with pytest.raises(Exception) as e:
        F.hits_read(tmp_path / "idx", 6)
    assert "holds 5 counts" in str(e.value)
    (tmp_path / "idx" / "hits.bin").write_bytes(raw[:-2])
    with pytest.raises(Exception) as e:
        F.hits_read(tmp_path / "idx", 5)
    assert "truncated" in str(e.value)
    with pytest.raises(Exception) as e:
        F.hits_read(tmp_path / "elsewhere", 5)
    assert "elsewhere" in str(e.value)


def test_roargraph_file(tmp_path):
    g, _, deg = _graph(12, 6, 4)
    p = tmp_path / "roar.index"
    F.roargraph_write(p, g, 9)
    raw = p.read_bytes()
    assert struct.unpack_from("<II", raw) == (9, 12)
    g2, ep = F.roargraph_read(p, 12, 6)
    assert ep == 9 and np.array_equal(g2, g)
    g3, _ = F.roargraph_read(p, 12, 4)  # degrees above R are truncated (src/graph.cu:724-728)
    assert np.array_equal(g3, g[:, :4])
    p.write_bytes(raw[:-3])
    with pytest.raises(capi.CoralError, match="truncated"):
        F.roargraph_read(p, 12, 6)


def test_normalize_and_recall_match_oracle(orc):
    x = np.random.RandomState(1).randn(40, 12).astype(np.float32)
    x[3] = 0
    y = x.copy()
    orc.lib().oracle_normalize_l2(y.ctypes.data, 40, 12)
    assert np.array_equal(F.normalize_l2(x), y)
    rng = np.random.RandomState(2)
    res = rng.randint(0, 30, (20, 5)).astype(np.int32)
    gt = rng.randint(0, 30, (20, 9)).astype(np.int32)
    want = sum(len(set(gt[i, :5].tolist()) & set(res[i].tolist())) for i in range(20))
    # rows with repeated gt ids count each occurrence, as the reference's loop does
    assert F.recall_hits(res, gt, 5) == orc.recall_hits(res, gt, 5)
    uniq = np.array([rng.permutation(30)[:9] for _ in range(20)], np.int32)
    ures = np.array([rng.permutation(30)[:5] for _ in range(20)], np.int32)
    want = sum(len(set(uniq[i, :5].tolist()) & set(ures[i].tolist())) for i in range(20))
    assert F.recall_hits(ures, uniq, 5) == want == orc.recall_hits(ures, uniq, 5)
