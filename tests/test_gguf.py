"""GGUF container reader: hand-assembled files (bytes laid out in the test itself, following the
public specification, independently of the writer), writer -> reader round trips, and malformed
files.  CPU only.  The reference holds no GGUF file or loader (its loader is in go-huggingface),
so there is no reference vector for this format."""
import struct

import numpy as np
import pytest

from gomlx_amd import ggml, gguf, synth


def s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def hand_made(alignment=64, version=3):
    """Two tensors and five key/value pairs, every field written out by hand."""
    q8 = synth.weights(ggml.Q8_0, 1, 3, 64)                      # [3, 68] bytes: ne = [64, 3]
    f32 = np.array([1.5, -2.0, 0.25, 8.0], "<f4")
    head = b"GGUF" + struct.pack("<IQQ", version, 2, 5)
    head += s("general.architecture") + struct.pack("<I", 8) + s("llama")
    head += s("general.alignment") + struct.pack("<II", 4, alignment)
    head += s("llama.rope.freq_base") + struct.pack("<If", 6, 10000.0)
    head += s("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, 3) + s("<s>") + s("a") + s("bc")
    head += s("tokenizer.ggml.scores") + struct.pack("<IIQ", 9, 6, 3) + struct.pack("<3f", 0.0, -1.0, -2.5)
    head += s("blk.0.attn_q.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 64, 3) + struct.pack("<IQ", 8, 0)
    second = (q8.size + alignment - 1) // alignment * alignment
    head += s("blk.0.attn_norm.weight") + struct.pack("<I", 1) + struct.pack("<Q", 4) + struct.pack("<IQ", 0, second)
    pad = -len(head) % alignment
    data = q8.tobytes() + b"\0" * (second - q8.size) + f32.tobytes()
    return head + b"\0" * pad + data, q8, f32


def test_hand_made_file(tmp_path):
    blob, q8, f32 = hand_made()
    p = tmp_path / "hand.gguf"
    p.write_bytes(blob)
    with gguf.GGUFFile(str(p)) as g:
        assert g.version == 3 and g.alignment == 64
        assert g.metadata["general.architecture"] == "llama"
        assert g.metadata["llama.rope.freq_base"] == 10000.0
        assert g.metadata["tokenizer.ggml.tokens"] == ["<s>", "a", "bc"]
        assert np.array_equal(g.metadata["tokenizer.ggml.scores"], np.array([0.0, -1.0, -2.5], np.float32))
        assert list(g.tensors) == ["blk.0.attn_q.weight", "blk.0.attn_norm.weight"]
        ti = g.tensors["blk.0.attn_q.weight"]
        assert ti.ne == (64, 3) and ti.shape == (3, 64) and ti.type_name == "Q8_0" and ti.nbytes == 3 * 68
        assert g.data_start % 64 == 0
        rows = g.rows("blk.0.attn_q.weight")
        assert rows.shape == (3, ggml.row_bytes(ggml.Q8_0, 64)) and np.array_equal(rows, q8)
        assert np.array_equal(g.array("blk.0.attn_norm.weight"), f32)
        with pytest.raises(gguf.GGUFError):
            g.array("blk.0.attn_q.weight")


def test_version_2_and_default_alignment(tmp_path):
    q = synth.weights(ggml.Q4_0, 2, 5, 96)
    head = b"GGUF" + struct.pack("<IQQ", 2, 1, 0) + s("w") + struct.pack("<I", 2) + struct.pack("<QQ", 96, 5) + struct.pack("<IQ", 2, 0)
    p = tmp_path / "v2.gguf"
    p.write_bytes(head + b"\0" * (-len(head) % 32) + q.tobytes())
    with gguf.GGUFFile(str(p)) as g:
        assert g.version == 2 and g.alignment == 32 and g.data_start == len(head) + (-len(head) % 32)
        assert np.array_equal(g.rows("w"), q)


def test_round_trip_all_formats(tmp_path):
    K, N = 512, 7
    tensors, want = [], {}
    for t in (ggml.Q4_0, ggml.Q8_0, ggml.Q4_K, ggml.Q6_K, ggml.IQ4_NL):
        W = synth.weights(t, 10 + t, N, K)
        name = f"blk.0.{ggml.name(t)}.weight"
        tensors.append((name, t, (K, N), W))
        want[name] = W
    gain = synth.normal(3, 0, K).astype(np.float32)
    tensors.append(("blk.0.ffn_norm.weight", 0, (K,), gain))
    half = np.arange(12, dtype="<f2").reshape(3, 4)
    tensors.append(("half", 1, (4, 3), half))
    stacked = synth.weights(ggml.Q8_0, 4, 6, 64)                 # ne = [64, 3, 2]: two experts of three rows
    tensors.append(("experts", ggml.Q8_0, (64, 3, 2), stacked))
    meta = {"general.name": "synthetic", "llama.block_count": np.uint32(1), "llama.attention.layer_norm_rms_epsilon": 1e-5,
            "flag": True, "big": 1 << 63, "neg": -5, "ids": np.arange(4, dtype=np.int32), "names": ["x", "yz"]}
    for alignment in (32, 256):
        p = tmp_path / f"rt{alignment}.gguf"
        gguf.write_gguf(str(p), meta, tensors, alignment=alignment)
        with gguf.GGUFFile(str(p)) as g:
            assert g.alignment == alignment
            for name, W in want.items():
                assert np.array_equal(g.rows(name), W)
                assert (g.data_start + g.tensors[name].offset) % alignment == 0
            assert np.array_equal(g.array("blk.0.ffn_norm.weight"), gain)
            assert np.array_equal(g.array("half"), half)
            assert g.tensors["experts"].shape == (2, 3, 64) and np.array_equal(g.rows("experts"), stacked)
            m = g.metadata
            assert m["general.name"] == "synthetic" and m["llama.block_count"] == 1 and m["flag"] is True
            assert m["big"] == 1 << 63 and m["neg"] == -5 and m["names"] == ["x", "yz"]
            assert abs(m["llama.attention.layer_norm_rms_epsilon"] - 1e-5) < 1e-12
            assert np.array_equal(m["ids"], np.arange(4))


def test_block_geometry_table_matches_the_library():
    for t in (ggml.Q4_0, ggml.Q8_0, ggml.Q4_K, ggml.Q6_K, ggml.IQ4_NL):
        name, vpb, bpb = gguf.GGML_TYPES[t]
        assert name == ggml.name(t) and vpb == ggml.values_per_block(t) and bpb == ggml.bytes_per_block(t)
        assert gguf.tensor_nbytes(t, (1024, 3)) == 3 * ggml.row_bytes(t, 1024)


def test_malformed_files(tmp_path):
    blob, _, _ = hand_made()

    def load(b):
        p = tmp_path / "bad.gguf"
        p.write_bytes(b)
        with gguf.GGUFFile(str(p)):
            pass

    load(blob)
    for bad in (b"GGUX" + blob[4:],                       # magic
                blob[:4] + struct.pack("<I", 1) + blob[8:],  # version 1
                blob[:4] + struct.pack(">I", 3) + blob[8:],  # big-endian file
                blob[:40],                                 # ends inside the header
                blob[:-8],                                 # last tensor runs past the end
                b"GGUF"):
        with pytest.raises(gguf.GGUFError):
            load(bad)
    # an offset that is not a multiple of the alignment
    i = blob.index(b"blk.0.attn_norm.weight") + len(b"blk.0.attn_norm.weight") + 4 + 8 + 4
    off = struct.unpack_from("<Q", blob, i)[0]
    with pytest.raises(gguf.GGUFError):
        load(blob[:i] + struct.pack("<Q", off + 4) + blob[i + 8:])
    # K that is not a whole number of blocks
    head = b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + s("w") + struct.pack("<I", 2) + struct.pack("<QQ", 48, 5) + struct.pack("<IQ", 2, 0)
    with pytest.raises(gguf.GGUFError):
        load(head + b"\0" * 4096)
    with pytest.raises(gguf.GGUFError):
        gguf.write_gguf(str(tmp_path / "w.gguf"), {}, [("w", ggml.Q8_0, (64, 3), np.zeros(10, np.uint8))])


def test_round_trip_property(tmp_path):
    """Random files: any mix of tensor types, ranks and alignments written by write_gguf reads back byte for byte."""
    from hypothesis import given, settings, strategies as st, HealthCheck

    types = [ggml.Q4_0, ggml.Q8_0, ggml.Q4_K, ggml.Q6_K, ggml.IQ4_NL, 0, 1, 24, 26, 30]
    tensor = st.tuples(st.sampled_from(types), st.integers(1, 3), st.lists(st.integers(1, 5), min_size=0, max_size=2), st.integers(0, 2 ** 31))
    counter = [0]

    @settings(max_examples=40, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
    @given(st.lists(tensor, min_size=0, max_size=6), st.sampled_from([32, 64, 4096]),
           st.dictionaries(st.text(min_size=1, max_size=12), st.one_of(st.integers(-2 ** 62, 2 ** 62), st.text(max_size=20), st.booleans()), max_size=5))
    def run(tensors, alignment, meta):
        meta = {k: v for k, v in meta.items() if k != "general.alignment"}
        specs, want = [], {}
        for i, (t, blocks, outer, seed) in enumerate(tensors):
            _, vpb, bpb = gguf.GGML_TYPES[t]
            ne = (blocks * vpb, *outer)
            n = gguf.tensor_nbytes(t, ne)
            data = np.random.default_rng(seed).integers(0, 256, size=n, dtype=np.uint8)
            specs.append((f"t{i}", t, ne, data))
            want[f"t{i}"] = (ne, data)
        counter[0] += 1
        path = str(tmp_path / f"p{counter[0]}.gguf")
        gguf.write_gguf(path, meta, specs, alignment=alignment)
        with gguf.GGUFFile(path) as g:
            assert g.alignment == alignment and list(g.tensors) == list(want)
            for name, (ne, data) in want.items():
                assert g.tensors[name].ne == tuple(ne)
                assert np.array_equal(g.raw(name), data)
                assert (g.data_start + g.tensors[name].offset) % alignment == 0
            for k, v in meta.items():
                assert g.metadata[k] == v

    run()
