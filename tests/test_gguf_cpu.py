"""GGUF reader: header rules of the reference's inspector (icn-models/src/gguf.rs:76-238 - magic,
versions 2/3, metadata value types, bounds, general.alignment) plus payload location."""
import struct

import numpy as np
import pytest

from magnitude_amd import gguf


def blocks(rng, gtype, shape):
    return rng.integers(0, 256, gguf.tensor_storage_bytes(gtype, shape), dtype=np.uint8)


@pytest.mark.parametrize("version,alignment", [(3, 32), (2, 32), (3, 64), (3, 4096)])
def test_round_trip_locates_every_payload(tmp_path, version, alignment):
    rng = np.random.default_rng(version * 100 + alignment)
    spec = [("blk.0.attn_q.weight", (512, 64), 12), ("blk.0.ffn_down.weight", (256, 48), 14),
            ("output.weight", (96, 10), 8), ("blk.0.ffn_gate_exps.weight", (256, 24, 4), 12),
            ("blk.0.attn_norm.weight", (512,), 0)]
    data = {n: blocks(rng, t, s) for n, s, t in spec}
    meta = {"general.architecture": "llama", "general.name": "synthetic", "llama.context_length": 4096,
            "general.file_type": 15, "tokenizer.ggml.tokens": ["<s>", "</s>", "a"], "x.floats": [0.5, 1.5],
            "x.big": 2 ** 40, "x.neg": -7, "x.flag": True, "x.pi": 3.25}
    p = tmp_path / "m.gguf"
    gguf.write(str(p), [(n, s, t, data[n]) for n, s, t in spec], meta, version=version, alignment=alignment)
    with gguf.GgufFile(str(p)) as g:
        assert g.version == version and g.alignment == alignment and g.data_offset % alignment == 0
        assert g.metadata["general.architecture"] == "llama" and g.metadata["x.big"] == 2 ** 40
        assert g.metadata["tokenizer.ggml.tokens"] == ["<s>", "</s>", "a"] and g.metadata["x.neg"] == -7
        assert g.metadata["x.flag"] is True and g.metadata["x.pi"] == 3.25
        for n, s, t in spec:
            info = g.tensors[n]
            assert info.shape == s and info.ggml_type == t and info.offset % alignment == 0
            assert np.array_equal(g.tensor_bytes(n), data[n])
        assert [t.name for t in g.projection_tensors()] == [n for n, s, t in spec if t in (8, 12, 14)]


def test_storage_bytes_formula():
    assert gguf.tensor_storage_bytes(12, (4096, 14336)) == 33_030_144      # gate/up of the 8B layer
    assert gguf.tensor_storage_bytes(14, (14336, 4096)) == 48_168_960      # down
    assert gguf.tensor_storage_bytes(8, (4096, 4096)) == 17_825_792
    with pytest.raises(gguf.GgufError):
        gguf.tensor_storage_bytes(12, (100, 4))        # not whole blocks
    with pytest.raises(gguf.GgufError):
        gguf.tensor_storage_bytes(99, (256, 4))


def test_rejects_what_the_inspector_rejects(tmp_path):
    def put(name, b):
        p = tmp_path / name
        p.write_bytes(b)
        return str(p)
    head = lambda ver, nt, nm: b"GGUF" + struct.pack("<IQQ", ver, nt, nm)
    with pytest.raises(gguf.GgufError, match="magic"):
        gguf.GgufFile(put("a", b"GGML" + b"\0" * 40))
    with pytest.raises(gguf.GgufError, match="version"):
        gguf.GgufFile(put("b", head(1, 0, 0) + b"\0" * 40))
    with pytest.raises(gguf.GgufError, match="tensor count"):
        gguf.GgufFile(put("c", head(3, 10_000_001, 0) + b"\0" * 40))
    with pytest.raises(gguf.GgufError, match="metadata count"):
        gguf.GgufFile(put("d", head(3, 0, 1_000_001) + b"\0" * 40))
    with pytest.raises(gguf.GgufError, match="beyond end"):
        gguf.GgufFile(put("e", head(3, 0, 1) + struct.pack("<Q", 100) + b"ab"))          # truncated key
    bad_type = head(3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13) + b"\0" * 32
    with pytest.raises(gguf.GgufError, match="value type"):
        gguf.GgufFile(put("f", bad_type))
    zero_dims = head(3, 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<I", 0) + b"\0" * 64
    with pytest.raises(gguf.GgufError, match="dimension"):
        gguf.GgufFile(put("g", zero_dims))
    bad_align = head(3, 0, 1) + struct.pack("<Q", 17) + b"general.alignment" + struct.pack("<II", 4, 24) + b"\0" * 64
    with pytest.raises(gguf.GgufError, match="alignment"):
        gguf.GgufFile(put("h", bad_align))
    # a tensor whose payload would lie past the end of the file
    t = head(3, 1, 0) + struct.pack("<Q", 1) + b"w" + struct.pack("<IQQIQ", 2, 256, 4, 12, 0)
    with pytest.raises(gguf.GgufError, match="outside the file"):
        gguf.GgufFile(put("i", t + b"\0" * 64))
