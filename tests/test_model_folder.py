"""The model-folder reader (csrc/model_folder.c) against: a folder written by the reference's own writer (committed under
tests/golden/model_folder, made by tests/golden/make_folder_golden.py), the reference's reader live where the compiled
reference is present, the cases of the reference's tests/test_model_st.c (rejections, affine groups, crafted headers) and
tests/test_moe.c:116-152 (.blk / .blk4 bank streams).  No GPU needed: nothing is launched."""
import ctypes as C
import json
import os
import shutil
import struct

import numpy as np
import pytest

from nanoseedlm_amd import folder

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden", "model_folder")
MANIFEST = json.load(open(os.path.join(HERE, "golden", "model_folder.json")))
SPECS = [tuple(s) for s in MANIFEST["specs"]]


def pattern(t, s, n):
    i = np.arange(n, dtype=np.uint64)
    return ((i * 131 + (i >> 8) * 29 + t * 17 + s * 5) & 255).astype(np.uint8)


def write_safetensors(path, entries, pad_to=0):
    """entries: [(name, dtype, shape, bytes)] -> one safetensors file (8-byte header length, JSON header, data)."""
    head, off = {}, 0
    for name, dtype, shape, data in entries:
        head[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + len(data)]}
        off += len(data)
    h = json.dumps(head).encode()
    if pad_to:
        h += b" " * ((-(8 + len(h))) % pad_to)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"".join(bytes(d) for _, _, _, d in entries))


def check_folder(path):
    m = folder.ModelFolder(path)
    assert m.shards > 1 and len(m) == len(SPECS)
    names = [m.at(i).name.decode() for i in range(len(m))]
    assert names == sorted(names)
    for ti, (name, enc, S, R, Cc) in enumerate(SPECS):
        t = m.find(name)
        assert t is not None, name
        assert (t.enc, t.slices, t.rows, t.cols) == (enc, S, R, Cc), name
        assert t.group == (64 if enc in (folder.Q8, folder.Q4) else 0)
        for s in range(4):
            n = folder.stream_len(enc, S, R, Cc, s)
            assert t.s[s].len == n, (name, s)
            assert np.array_equal(t.stream(s), pattern(ti, s, n)), (name, s)
            if n and n % folder.PAGE == 0:
                assert m.mappable(t.s[s]), (name, s)            # the writer puts page-multiple streams on page boundaries
    assert m.find("nope.weight") is None
    m.close()


def test_golden_folder_written_by_the_reference_writer():
    check_folder(GOLD)


def test_stream_lengths():
    # nslm/model_st.h:5-17: bytes of each stream
    assert [folder.stream_len(folder.SEED4P4, 4, 64, 256, s) for s in range(4)] == [16384, 16384, 16, 4096]
    assert [folder.stream_len(folder.SEED4, 4, 64, 128, s) for s in range(4)] == [8192, 8192, 16, 0]
    assert [folder.stream_len(folder.SEED6P8, 1, 64, 256, s) for s in range(4)] == [4096, 8192, 4, 1024]
    assert [folder.stream_len(folder.Q4, 3, 64, 128, s) for s in range(4)] == [12288, 768, 768, 0]
    assert [folder.stream_len(folder.Q8, 1, 96, 128, s) for s in range(4)] == [12288, 384, 384, 0]
    assert [folder.stream_len(folder.BF16, 2, 32, 64, s) for s in range(4)] == [8192, 0, 0, 0]


def test_reader_matches_the_reference_reader_live(oracle, tmp_path):
    """Where the compiled reference is present: a fresh folder from its writer, read by both readers."""
    ref = oracle.ref()
    if ref is None or not hasattr(ref, "ns_open"):
        pytest.skip("compiled reference not present")

    class NsModel(C.Structure):
        _fields_ = [("sh", C.c_void_p), ("nsh", C.c_int), ("t", C.POINTER(folder.Tensor)), ("n", C.c_int)]
    rm, err = NsModel(), C.create_string_buffer(512)
    ref.ns_open.argtypes = [C.POINTER(NsModel), C.c_char_p, C.c_char_p, C.c_int]
    assert ref.ns_open(C.byref(rm), GOLD.encode(), err, 512) == 0, err.value
    m = folder.ModelFolder(GOLD)
    assert rm.n == len(m) and rm.nsh == m.shards
    for i in range(rm.n):
        a, b = rm.t[i], m.at(i)
        assert (a.name, a.enc, a.slices, a.rows, a.cols, a.group) == (b.name, b.enc, b.slices, b.rows, b.cols, b.group)
        for s in range(4):
            assert (a.s[s].len, a.s[s].off, a.s[s].shard) == (b.s[s].len, b.s[s].off, b.s[s].shard)
            assert np.array_equal(a.stream(s), b.stream(s))
    m.close()
    ref.ns_close.argtypes = [C.POINTER(NsModel)]
    ref.ns_close(C.byref(rm))


def _copy(tmp_path, name):
    dst = tmp_path / name
    shutil.copytree(GOLD, dst)
    return dst


def test_rejects_a_truncated_shard_and_a_wrong_dtype(tmp_path):
    # tests/test_model_st.c:147-156
    d = _copy(tmp_path, "trunc")
    p = d / "model-00001-of-00003.safetensors"
    data = p.read_bytes()
    p.write_bytes(data[:-100])
    with pytest.raises(ValueError, match="out of bounds"):
        folder.ModelFolder(d)
    d = _copy(tmp_path, "dtype")
    p = d / "model-00001-of-00003.safetensors"
    data = bytearray(p.read_bytes())
    hn = struct.unpack("<Q", data[:8])[0]
    head = bytes(data[8:8 + hn])
    assert b'"U32"' in head
    data[8:8 + hn] = head.replace(b'"U32"', b'"I32"')
    p.write_bytes(bytes(data))
    with pytest.raises(ValueError, match="missing, or not U32"):
        folder.ModelFolder(d)


def test_missing_folder_and_empty_folder(tmp_path):
    with pytest.raises(ValueError):
        folder.ModelFolder(tmp_path / "absent")
    (tmp_path / "empty").mkdir()
    with pytest.raises(ValueError, match="no safetensors"):
        folder.ModelFolder(tmp_path / "empty")


def test_affine_groups_and_the_config_override(tmp_path):
    """MLX affine groups (tests/test_model_st.c:186-223): Q4 group 32, Q8 group 64, Q4 group 64 from the shapes; a
    config.json entry turns the ambiguous shape into Q8 group 32; a config the shapes contradict is refused."""
    d = tmp_path / "groups"
    d.mkdir()
    z = lambda n: pattern(1, 0, n).tobytes()
    ents = [("a.weight", "U32", (2, 8, 16), z(2 * 8 * 16 * 4)), ("a.scales", "BF16", (2, 8, 4), z(2 * 8 * 4 * 2)), ("a.biases", "BF16", (2, 8, 4), z(128)),
            ("b.weight", "U32", (4, 32), z(4 * 32 * 4)), ("b.scales", "BF16", (4, 2), z(16)), ("b.biases", "BF16", (4, 2), z(16)),
            ("c.weight", "U32", (4, 16), z(4 * 16 * 4)), ("c.scales", "BF16", (4, 2), z(16)), ("c.biases", "BF16", (4, 2), z(16))]
    write_safetensors(d / "model.safetensors", ents)
    m = folder.ModelFolder(d)
    a, b, c = m.find("a.weight"), m.find("b.weight"), m.find("c.weight")
    assert (a.enc, a.group, a.slices, a.rows, a.cols) == (folder.Q4, 32, 2, 8, 128)
    assert (b.enc, b.group, b.rows, b.cols) == (folder.Q8, 64, 4, 128)
    assert (c.enc, c.group, c.rows, c.cols) == (folder.Q4, 64, 4, 128)
    assert a.s[1].len == 128 and a.stream(1)[3] == pattern(1, 0, 4)[3]
    assert len(m) == 3                                          # scales and biases are streams, not tensors
    m.close()
    (d / "config.json").write_text('{"quantization": {"group_size": 64, "bits": 4, "c": {"group_size": 32, "bits": 8}}}')
    m = folder.ModelFolder(d)
    c = m.find("c.weight")
    assert (c.enc, c.group, c.rows, c.cols) == (folder.Q8, 32, 4, 64)
    m.close()
    (d / "config.json").write_text('{"text_config": {"quantization": {"c": {"group_size": 32, "bits": 8}}}}')
    m = folder.ModelFolder(d)
    assert m.find("c.weight").enc == folder.Q8
    m.close()
    (d / "config.json").write_text('{"quantization": {"c": {"group_size": 64, "bits": 8}}}')
    with pytest.raises(ValueError, match="c:"):
        folder.ModelFolder(d)


CRAFTED = [
    ("shorter than the length", b"", -1),
    ("a header longer than the file", b"{}", 1 << 20),
    ("a header without its end", b'{"a":{"dtype":"BF16","shape":[2,2],"data_offsets":[0,8', 0),
    ("a negative shape", b'{"a":{"dtype":"BF16","shape":[-2,2],"data_offsets":[0,8]}}', 0),
    ("an offset past the file", b'{"a":{"dtype":"BF16","shape":[2,2],"data_offsets":[0,800]}}', 0),
    ("an end near 2^64", b'{"a":{"dtype":"BF16","shape":[2,2],"data_offsets":[1,18446744073709551615]}}', 0),
    ("a shape past 2^40 values", b'{"a":{"dtype":"BF16","shape":[1048577,1048577],"data_offsets":[0,8]}}', 0),
    ("a truncated literal in the metadata", b'{"__metadata__":{"a":tru', 0),
    ("trailing bytes after the header object", b'{"a":{"dtype":"BF16","shape":[2,2],"data_offsets":[0,8]}} x', 0),
]


@pytest.mark.parametrize("name,head,hn", CRAFTED, ids=[c[0] for c in CRAFTED])
def test_crafted_files_are_refused(tmp_path, name, head, hn):
    # tests/test_model_st.c:224-249: each is refused with a message, and none reads past the file
    d = tmp_path / "crafted"
    d.mkdir()
    if hn < 0:
        (d / "model.safetensors").write_bytes(b"\x00" * 4)
    else:
        (d / "model.safetensors").write_bytes(struct.pack("<Q", hn if hn > 0 else len(head)) + head + (b"" if hn else b"\x00" * 8))
    with pytest.raises(ValueError) as e:
        folder.ModelFolder(d)
    assert str(e.value)


@pytest.mark.parametrize("text", ['[1,t', '{"weight_map":{"a":fals', '{"weight_map":[nul', 'tru', '{"weight_map":{"a":"model.safetensors"'])
def test_truncated_index_is_refused(tmp_path, text):
    # tests/test_model_st.c:252-264: truncated JSON literals
    d = tmp_path / "idx"
    d.mkdir()
    write_safetensors(d / "model.safetensors", [("x", "BF16", (2, 2), b"\0" * 8)])
    (d / "model.safetensors.index.json").write_text(text)
    with pytest.raises(ValueError):
        folder.ModelFolder(d)


def test_seed_encodings_by_their_entries(tmp_path):
    """No .codes: P = 3; .coefs as U32: P = 8; else P = 4 (nslm/lib_model_st.c:228-236); 1-D BF16 is [1][1][n]; scalars and
    4-D tensors are skipped; a name twice (two shards) is refused."""
    d = tmp_path / "enc"
    d.mkdir()
    nb = 2 * 8 * 4                                               # [2 slices][8 rows][32 cols / 8]
    ents = [("p3.seeds", "U16", (2, 8, 4), b"\1" * (2 * nb)), ("p3.nibbles", "U16", (2, 8, 4), b"\2" * (2 * nb)), ("p3.exp_bias", "I32", (2,), b"\3" * 8),
            ("p4.seeds", "U16", (2, 8, 4), b"\1" * (2 * nb)), ("p4.coefs", "U16", (2, 8, 4), b"\2" * (2 * nb)), ("p4.exp_bias", "I32", (2,), b"\3" * 8),
            ("p4.codes", "U8", (2, 8, 2), b"\4" * (nb // 2)),
            ("p8.seeds", "U16", (2, 8, 4), b"\1" * (2 * nb)), ("p8.coefs", "U32", (2, 8, 4), b"\2" * (4 * nb)), ("p8.exp_bias", "I32", (2,), b"\3" * 8),
            ("p8.codes", "U8", (2, 8, 2), b"\4" * (nb // 2)),
            ("v.weight", "BF16", (6,), b"\5" * 12), ("scalar", "BF16", (), b"\6" * 2), ("conv", "BF16", (1, 2, 1, 2), b"\7" * 8), ("f", "F32", (2,), b"\0" * 8)]
    write_safetensors(d / "model.safetensors", ents)
    m = folder.ModelFolder(d)
    assert [m.at(i).name.decode() for i in range(len(m))] == ["p3.weight", "p4.weight", "p8.weight", "v.weight"]
    assert [m.at(i).enc for i in range(4)] == [folder.SEED4, folder.SEED4P4, folder.SEED6P8, folder.BF16]
    p4 = m.find("p4.weight")
    assert (p4.slices, p4.rows, p4.cols) == (2, 8, 32) and p4.stream(3)[0] == 4 and p4.stream(2).view(np.int32)[1] == 0x03030303
    v = m.find("v.weight")
    assert (v.slices, v.rows, v.cols) == (1, 1, 6)
    m.close()
    write_safetensors(d / "model-2.safetensors", [("p4.seeds", "U16", (2, 8, 4), b"\1" * (2 * nb))])
    with pytest.raises(ValueError, match="appears twice"):
        folder.ModelFolder(d)


def bank_image(p, E, R, Cc):
    nb = R * Cc // 8
    img = np.zeros(56 + 12 * E + (5 if p == 4 else 4) * nb * E, dtype=np.uint8)
    img[:8] = np.frombuffer(b"NSLMBLK4" if p == 4 else b"NSLMBLKM", dtype=np.uint8)
    img[8:20] = np.array([R, Cc, E], dtype=np.uint32).view(np.uint8)
    return img, nb


def test_blk4_and_blk_bank_streams(oracle):
    # the vectors of tests/test_moe.c:116-152
    E, R, Cc = 2, 2, 16
    img, nb = bank_image(4, E, R, Cc)
    b = 56
    img[b:b + 8] = np.array([-20, -19], dtype=np.int32).view(np.uint8)
    k = np.arange(nb * E)
    img[b + 12 * E:b + 12 * E + 2 * nb * E] = (100 + k).astype(np.uint16).view(np.uint8)
    img[b + 12 * E + 2 * nb * E:b + 12 * E + 4 * nb * E] = (0x1000 + k).astype(np.uint16).view(np.uint8)
    img[b + 12 * E + 4 * nb * E:] = k.astype(np.uint8)
    s0 = folder.blk_stream(img, 4, E, R, Cc, 0, 2 * nb * E).view(np.uint16)
    s1 = folder.blk_stream(img, 4, E, R, Cc, 1, 2 * nb * E).view(np.uint16)
    s2 = folder.blk_stream(img, 4, E, R, Cc, 2, 4 * E).view(np.int32)
    s3 = folder.blk_stream(img, 4, E, R, Cc, 3, nb * E // 2)
    assert s0[5] == 105 and s1[7] == 0x1007 and s2[1] == -19 and s3[0] == 0x10 and s3[3] == 0x76
    assert folder.blk_stream(img, 4, E, R, 2 * Cc, 0, 4 * nb * E) is None         # a bank of another shape
    assert folder.blk_stream(img[:-1], 4, E, R, Cc, 0, 2 * nb * E) is None        # a short file
    ref = oracle.ref()
    if ref is not None and hasattr(ref, "nslm_blk_stream"):                       # the reference's function on the same image
        for s, n in ((0, 2 * nb * E), (1, 2 * nb * E), (2, 4 * E), (3, nb * E // 2)):
            dst = np.zeros(n, dtype=np.uint8)
            assert ref.nslm_blk_stream(img.ctypes.data_as(C.c_void_p), C.c_size_t(img.size), 4, E, R, Cc, s, dst.ctypes.data_as(C.c_void_p)) == 0
            assert np.array_equal(dst, folder.blk_stream(img, 4, E, R, Cc, s, n))
    img3, nb = bank_image(3, E, R, Cc)
    img3[b + 12 * E:b + 12 * E + 2 * nb * E] = (7 + k).astype(np.uint16).view(np.uint8)
    img3[b + 12 * E + 2 * nb * E:] = (0x2000 + k).astype(np.uint16).view(np.uint8)
    assert folder.blk_stream(img3, 3, E, R, Cc, 0, 2 * nb * E).view(np.uint16)[3] == 10
    assert folder.blk_stream(img3, 3, E, R, Cc, 1, 2 * nb * E).view(np.uint16)[6] == 0x2006
    assert folder.blk_stream(img3, 4, E, R, Cc, 0, 2 * nb * E) is None            # a .blk read as .blk4
    assert folder.blk_stream(img3, 3, E, R, Cc, 3, nb * E) is None                # P = 3 has no code stream
