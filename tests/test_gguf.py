"""The GGUF weight source (include/infr_gguf.h) on files written by tests/gguf_writer.py.  The
cases follow the reference loader's own tests (crates/infr-gguf/src/lib.rs:1040-2040): round trip of
metadata and tensors, every malformed-file refusal, and gguf-split shard sets.  CPU only."""
import os
import re
import struct

import numpy as np
import pytest

import moe4all_amd as M
from moe4all_amd import gguf as G

import gguf_writer as W
import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _meta(extra=()):
    return [("general.architecture", W.STR, "qwen3moe"), ("general.alignment", W.U32, 32)] + list(extra)


def test_header_symbols_are_exported_and_bound():
    src = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "infr_gguf.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(infr_gguf_[a-z0-9_]+)\s*\(", src)))
    lib = M.load_library()
    for s in declared:
        assert hasattr(lib, s), f"{s} declared in include/infr_gguf.h but not exported"
    assert sorted(G._SIGS) == declared


def test_round_trip_of_metadata_and_tensors(tmp_path):
    rng = np.random.default_rng(0)
    f32 = rng.standard_normal(24).astype(np.float32)
    q8 = H.synth_weight(H.Q8_0, 64, 1)
    q4k = H.synth_weight(H.Q4K, 512, 2)
    i32 = np.arange(6, dtype=np.int32)
    meta = _meta([("a.u8", W.U8, 7), ("a.i8", W.I8, -3), ("a.u16", W.U16, 65535), ("a.i16", W.I16, -2), ("a.i32", W.I32, -70000),
                  ("a.f32", W.F32, 0.5), ("a.bool", W.BOOL, 1), ("a.u64", W.U64, 2 ** 40), ("a.i64", W.I64, -2 ** 40),
                  ("a.f64", W.F64, 1e-300), ("a.arr", W.ARR, (W.U32, [1, 2, 3])), ("a.strs", W.ARR, (W.STR, ["x", "yz", ""])),
                  ("a.nested", W.ARR, (W.ARR, [(W.I8, [1, 2]), (W.I8, [])])), ("a.empty", W.STR, "")])
    tensors = [("t.f32", (6, 4), W.GGML["F32"], f32.tobytes()), ("t.q8", (32, 2), W.GGML["Q8_0"], q8.tobytes()),
               ("t.q4k", (256, 2, 1), W.GGML["Q4K"], q4k.tobytes()), ("t.i32", (6,), W.GGML["I32"], i32.tobytes())]
    p = tmp_path / "m.gguf"
    W.write(p, meta, tensors)
    with G.Gguf(p) as g:
        assert g.n_shards == 1
        assert g.meta_str("general.architecture") == "qwen3moe" and g.meta_str("a.empty") == ""
        assert g.meta_u64("a.u8") == 7 and g.meta_i64("a.i8") == -3 and g.meta_u64("a.u16") == 65535
        assert g.meta_i64("a.i16") == -2 and g.meta_i64("a.i32") == -70000 and g.meta_f64("a.f32") == 0.5
        assert g.meta_bool("a.bool") is True and g.meta_u64("a.u64") == 2 ** 40 and g.meta_i64("a.i64") == -2 ** 40
        assert g.meta_f64("a.f64") == 1e-300
        assert g.meta_array_len("a.arr") == 3 and g.meta_array_len("a.strs") == 3 and g.meta_array_len("a.nested") == 2
        # a negative integer is not an unsigned value; an absent key and a kind mismatch read as None
        assert g.meta_u64("a.i8") is None and g.meta_u64("nope") is None and g.meta_str("a.u8") is None
        infos = g.tensors()
        assert [t.name for t in infos] == ["t.f32", "t.q8", "t.q4k", "t.i32"]
        assert [t.dtype for t in infos] == [int(M.DType.F32), int(M.DType.Q8_0), int(M.DType.Q4K), int(M.DType.I32)]
        assert infos[0].shape == (6, 4) and infos[2].shape == (256, 2, 1) and infos[2].numel == 512
        assert [t.nbytes for t in infos] == [96, 68, 288, 24]
        assert all(t.offset % 32 == 0 for t in infos) and infos[0].offset < infos[1].offset
        assert np.array_equal(g.tensor_bytes("t.f32").view(np.float32), f32)
        assert np.array_equal(g.tensor_bytes("t.q8"), q8.view(np.uint8))
        assert np.array_equal(g.tensor_bytes("t.q4k"), q4k.view(np.uint8))
        assert np.array_equal(g.tensor_bytes("t.i32").view(np.int32), i32)
        assert g.find("t.q8") == infos[1] and g.has("t.q8") and not g.has("t.q9")
        with pytest.raises(G.LoaderError, match="tensor not found"):
            g.find("t.q9")
        # what the file says lies at the offset is what the mapping hands out
        raw = open(p, "rb").read()
        assert raw[infos[2].offset:infos[2].offset + 288] == q4k.tobytes()


def test_version_2_and_default_alignment(tmp_path):
    p = tmp_path / "v2.gguf"
    W.write(p, [("general.architecture", W.STR, "x")], [("t", (4,), 0, np.arange(4, dtype=np.float32).tobytes())], version=2)
    with G.Gguf(p) as g:
        assert g.find("t").offset % 32 == 0
        assert np.array_equal(g.tensor_bytes("t").view(np.float32), np.arange(4, dtype=np.float32))


def test_block_layouts_match_the_ggml_formulas():
    # decode_spec.rs:455-504: bytes of a block from its fields
    want = {M.DType.Q4_0: (32, 2 + 16), M.DType.Q4_1: (32, 4 + 16), M.DType.Q5_0: (32, 2 + 4 + 16), M.DType.Q5_1: (32, 4 + 4 + 16),
            M.DType.Q8_0: (32, 2 + 32), M.DType.Q2K: (256, 16 + 64 + 4), M.DType.Q3K: (256, 32 + 64 + 12 + 2),
            M.DType.Q4K: (256, 4 + 12 + 128), M.DType.Q5K: (256, 4 + 12 + 32 + 128), M.DType.Q6K: (256, 128 + 64 + 16 + 2),
            M.DType.F32: (1, 4), M.DType.F16: (1, 2), M.DType.Bf16: (1, 2), M.DType.I32: (1, 4)}
    for dt, layout in want.items():
        assert G.block_layout(dt) == layout
    assert G.block_layout(28) == (32, 17) and G.block_layout(29) == (64, 36)   # Mxfp4, Nvfp4
    with pytest.raises(M.Unsupported):
        G.block_layout(26)   # I2S has no block layout


@pytest.mark.parametrize("kw,msg", [
    (dict(magic=0x46554746), "not a GGUF file"),
    (dict(version=1), "unsupported GGUF version 1"),
    (dict(version=4), "unsupported GGUF version 4"),
    (dict(dims_override=5), "declares 5 dimensions"),
    (dict(declared_tensors=3), "unexpected end of file"),
])
def test_malformed_headers_are_refused(tmp_path, kw, msg):
    p = tmp_path / "bad.gguf"
    W.write(p, _meta(), [("t", (4,), 0, b"\0" * 16)], **kw)
    with pytest.raises(G.LoaderError, match=msg):
        G.Gguf(p)


@pytest.mark.parametrize("align,msg", [(0, "positive power of two"), (24, "positive power of two"), (1 << 40, "cap")])
def test_alignment_rules(tmp_path, align, msg):
    p = tmp_path / "bad.gguf"
    W.write(p, [("general.alignment", W.U64, align)], [("t", (4,), 0, b"\0" * 16)], alignment=32)
    with pytest.raises(G.LoaderError, match=msg):
        G.Gguf(p)


def test_other_refusals(tmp_path):
    p = tmp_path / "bad.gguf"
    # a quantised tensor must be a whole number of blocks (lib.rs:855-872)
    W.write(p, _meta(), [("t", (100,), W.GGML["Q4K"], b"\0" * 144)])
    with pytest.raises(G.LoaderError, match="whole number of blocks"):
        G.Gguf(p)
    W.write(p, _meta(), [("t", (6,), W.GGML["I2S"], b"\0" * 8)])
    with pytest.raises(G.LoaderError, match="multiple of 4"):
        G.Gguf(p)
    W.write(p, _meta(), [("t", (4,), 0, b"\0" * 16), ("t", (4,), 0, b"\0" * 16)])
    with pytest.raises(G.LoaderError, match="duplicate tensor name 't'"):
        G.Gguf(p)
    W.write(p, _meta(), [("t", (4,), 99, b"\0" * 16)])
    with pytest.raises(G.LoaderError, match="unsupported ggml type 99"):
        G.Gguf(p)
    W.write(p, _meta(), [("t", (2 ** 40, 2 ** 40), 0, b"")])
    with pytest.raises(G.LoaderError, match="overflows"):
        G.Gguf(p)
    raw = bytearray(W.build(_meta([("k", W.U8, 1)]), []))
    raw[raw.index(b"k") + 1:raw.index(b"k") + 5] = struct.pack("<I", 13)   # an unknown value type
    p.write_bytes(raw)
    with pytest.raises(G.LoaderError, match="unknown metadata value type 13"):
        G.Gguf(p)
    with pytest.raises(G.LoaderError):
        G.Gguf(tmp_path / "missing.gguf")
    (tmp_path / "empty.gguf").write_bytes(b"")
    with pytest.raises(G.LoaderError, match="not a GGUF file"):
        G.Gguf(tmp_path / "empty.gguf")
    # a directory entry may point past the end of the file: the open succeeds, the read is refused (lib.rs:960-975)
    W.write(p, _meta(), [("t", (64,), 0, b"\0" * 16)])
    with G.Gguf(p) as g:
        with pytest.raises(G.LoaderError, match="exceeds"):
            g.tensor_bytes("t")


def test_array_nesting_depth_is_bounded(tmp_path):
    def nest(depth):
        v = (W.U8, [1])
        for _ in range(depth - 1):
            v = (W.ARR, [v])
        return v
    p = tmp_path / "n.gguf"
    W.write(p, _meta([("deep", W.ARR, nest(64))]), [])
    with G.Gguf(p) as g:
        assert g.meta_array_len("deep") == 1
    W.write(p, _meta([("deep", W.ARR, nest(65))]), [])
    with pytest.raises(G.LoaderError, match="nest deeper"):
        G.Gguf(p)
    # 85,000 levels in about a megabyte: refused by the bound, no stack to overflow
    raw = W.build(_meta([("bomb", W.U8, 1)]), [])
    cut = raw.index(b"bomb") + 4
    p.write_bytes(raw[:cut] + struct.pack("<I", W.ARR) + struct.pack("<IQ", W.ARR, 1) * 85000)
    with pytest.raises(G.LoaderError, match="nest deeper"):
        G.Gguf(p)


def test_every_truncation_is_an_error_not_a_crash(tmp_path):
    raw = W.build(_meta([("a.strs", W.ARR, (W.STR, ["x", "yz"])), ("a.f", W.F64, 2.0)]),
                  [("t.a", (32, 2), W.GGML["Q8_0"], b"\1" * 68), ("t.b", (4,), 0, b"\2" * 16)])
    directory_end = raw.index(b"t.b") + 3 + 4 + 8 + 4 + 8
    p = tmp_path / "cut.gguf"
    for cut in range(0, directory_end):
        p.write_bytes(raw[:cut])
        with pytest.raises(G.LoaderError):
            G.Gguf(p)
    # cut inside the data region: the directory parses, the tensor whose bytes are gone is refused
    p.write_bytes(raw[:len(raw) - 8])
    with G.Gguf(p) as g:
        assert g.tensor_bytes("t.a").tobytes() == b"\1" * 68
        with pytest.raises(G.LoaderError, match="exceeds"):
            g.tensor_bytes("t.b")
    # a length prefix near 2^64 must be an error, not an overflow
    bad = bytearray(raw)
    k = raw.index(b"general.architecture") - 8
    struct.pack_into("<Q", bad, k, 2 ** 64 - 3)
    p.write_bytes(bad)
    with pytest.raises(G.LoaderError):
        G.Gguf(p)


# ------------------------------------------------------------------------------------ shard sets
def _shards(tmp_path, n=2, base="model", width=5, no=None, count=None, tensors_count=None, names=None, name_total=None):
    """n shards, one f32 tensor each; only the first carries the model's own metadata (gguf-split)."""
    paths = []
    for i in range(n):
        meta = [("split.no", W.U16, i if no is None else no[i]), ("split.count", W.U16, n if count is None else count[i])]
        if tensors_count is not False:
            meta.append(("split.tensors.count", W.I32, n if tensors_count is None else tensors_count))
        if i == 0:
            meta = [("general.architecture", W.STR, "qwen3moe")] + meta
        tname = names[i] if names else f"t{i}"
        data = np.full(8 + i, float(i + 1), np.float32)
        fname = f"{base}-{i + 1:0{width}d}-of-{(name_total or n):0{width}d}.gguf"
        p = tmp_path / fname
        W.write(p, meta, [(tname, (8 + i,), 0, data.tobytes())])
        paths.append(p)
    return paths


def test_a_shard_set_reads_each_tensor_from_its_own_file(tmp_path):
    paths = _shards(tmp_path, 3)
    for opened in paths:   # any shard opens the whole model, re-rooted at shard 1 (lib.rs:495-503)
        with G.Gguf(opened) as g:
            assert g.n_shards == 3 and [t.name for t in g.tensors()] == ["t0", "t1", "t2"]
            assert g.meta_str("general.architecture") == "qwen3moe"
            sizes = [os.path.getsize(p) for p in paths]
            for i, t in enumerate(g.tensors()):
                assert np.array_equal(g.tensor_bytes(t.name).view(np.float32), np.full(8 + i, float(i + 1), np.float32))
                # offsets live in the set's concatenated address space (lib.rs:923-936)
                assert sum(sizes[:i]) <= t.offset < sum(sizes[:i + 1])


def test_shard_set_refusals(tmp_path):
    paths = _shards(tmp_path, 2)
    os.remove(paths[1])
    with pytest.raises(G.LoaderError, match="shard 2 of 2"):
        G.Gguf(paths[0])
    for kw, msg in [(dict(no=[0, 0]), "declares split.no = 0"), (dict(count=[2, 3]), "rest of the set declares 2"),
                    (dict(name_total=3, count=[2, 2]), "one of 3 shards but declares split.count = 2"),
                    (dict(tensors_count=5), "split.tensors.count = 5"), (dict(tensors_count=False), "no split.tensors.count"),
                    (dict(names=["same", "same"]), "duplicate tensor name 'same'")]:
        d = tmp_path / re.sub(r"\W", "", msg)[:24]
        d.mkdir()
        paths = _shards(d, 2, **kw)
        with pytest.raises(G.LoaderError, match=msg):
            G.Gguf(paths[0])
    # split metadata in a file whose name cannot name the other shards
    d = tmp_path / "plainname"
    d.mkdir()
    paths = _shards(d, 2)
    os.rename(paths[0], d / "model.gguf")
    with pytest.raises(G.LoaderError, match="shard name"):
        G.Gguf(d / "model.gguf")
    # a shard index outside its own set
    d = tmp_path / "outside"
    d.mkdir()
    paths = _shards(d, 2)
    os.rename(paths[1], d / "model-00003-of-00002.gguf")
    with pytest.raises(G.LoaderError, match="numbered 3 of 2"):
        G.Gguf(d / "model-00003-of-00002.gguf")


def test_a_shard_shaped_name_without_split_metadata_is_one_file(tmp_path):
    p = tmp_path / "model-00001-of-00002.gguf"
    W.write(p, _meta(), [("t", (4,), 0, b"\0" * 16)])
    with G.Gguf(p) as g:
        assert g.n_shards == 1 and len(g.tensors()) == 1
