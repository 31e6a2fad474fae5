"""GGUF reader / writer (host logic, no GPU): the file format of the reference's StreamingGGUFReader -- header, metadata
value types, tensor infos with aligned relative offsets, block geometry -- checked by round trips through the writer,
by hand-built byte strings, and by the reader's error behaviour on damaged files."""
import os
import struct

import numpy as np
import pytest

from skainet_amd import gguf, kernels


def small_file(tmp_path, alignment=32):
    rng = np.random.default_rng(0)
    w = gguf.GGUFWriter(alignment=alignment)
    w.add_string("general.architecture", "llama")
    w.add_u32("llama.block_count", 2)
    w.add_f32("llama.rope.freq_base", 500000.0)
    w.add_array_i32("tokenizer.ggml.token_type", [1, 2, 3, -4])
    w.add_array_string("tokenizer.ggml.tokens", ["<s>", "héllo", ""])
    dense = rng.standard_normal((3, 64)).astype(np.float32)
    q4 = kernels.quantize("Q4_K", rng.standard_normal((5, 512)).astype(np.float32))
    q6 = kernels.quantize("Q6_K", rng.standard_normal((2, 256)).astype(np.float32))
    q8 = kernels.quantize("Q8_0", rng.standard_normal((7, 96)).astype(np.float32))
    half = rng.standard_normal((4, 8)).astype(np.float16)
    w.add_tensor("dense.weight", "F32", (3, 64), dense)
    w.add_tensor("a.q4", "Q4_K", (5, 512), q4)
    w.add_tensor("b.q6", "Q6_K", (2, 256), q6)
    w.add_tensor("c.q8", "Q8_0", (7, 96), q8)
    w.add_tensor("d.f16", "F16", (4, 8), half)
    path = str(tmp_path / "small.gguf")
    w.write(path)
    return path, dict(dense=dense, q4=q4, q6=q6, q8=q8, half=half)


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_round_trip(tmp_path, alignment):
    path, src = small_file(tmp_path, alignment)
    with gguf.GGUFReader(path) as r:
        assert r.version == 3 and r.alignment == alignment
        assert r.fields["general.architecture"] == "llama"
        assert r.fields["llama.block_count"] == 2
        assert r.fields["llama.rope.freq_base"] == pytest.approx(500000.0)
        assert r.fields["tokenizer.ggml.token_type"].tolist() == [1, 2, 3, -4]
        assert r.fields["tokenizer.ggml.tokens"] == ["<s>", "héllo", ""]
        assert r.names() == ["dense.weight", "a.q4", "b.q6", "c.q8", "d.f16"]
        for t in r.tensors:
            assert t.offset % alignment == 0 and t.offset >= r.data_offset
        t = r.info("a.q4")
        assert (t.type_name, t.shape, t.rows, t.cols, t.n_bytes) == ("Q4_K", (512, 5), 5, 512, 5 * 2 * 144)
        assert r.info("b.q6").n_bytes == 2 * 210 and r.info("c.q8").n_bytes == 7 * 3 * 34
        assert np.array_equal(r.tensor_bytes("a.q4"), src["q4"])
        assert np.array_equal(r.tensor_bytes("b.q6"), src["q6"])
        assert np.array_equal(r.tensor_bytes("c.q8"), src["q8"])
        assert np.array_equal(r.tensor_f32("dense.weight"), src["dense"])
        assert np.array_equal(r.tensor_f32("d.f16"), src["half"].astype(np.float32))
        assert not r.tensor_bytes("a.q4").flags.writeable          # a view of the mapping, not a copy
        with pytest.raises(KeyError):
            r.info("missing")
        with pytest.raises(gguf.GGUFError):
            r.tensor_f32("a.q4")


def test_header_layout_is_the_published_one(tmp_path):
    """A file assembled by hand (not by the writer): magic, version, counts, one u32 key, one F32 tensor."""
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b
    head = struct.pack("<IIQQ", 0x46554747, 2, 1, 1) + s("k") + struct.pack("<II", 4, 7)
    head += s("t") + struct.pack("<I", 2) + struct.pack("<QQ", 4, 3) + struct.pack("<IQ", 0, 0)
    data = np.arange(12, dtype="<f4")
    raw = head + b"\0" * (-len(head) % 32) + data.tobytes()
    path = tmp_path / "hand.gguf"
    path.write_bytes(raw)
    with gguf.GGUFReader(str(path)) as r:
        assert r.version == 2 and r.fields == {"k": 7}
        assert r.info("t").shape == (4, 3) and r.info("t").rows == 3 and r.info("t").cols == 4
        assert np.array_equal(r.tensor_f32("t"), data.reshape(3, 4))


def test_bf16_and_unknown_types(tmp_path):
    w = gguf.GGUFWriter()
    vals = np.array([1.0, -2.5, 3.140625, 0.0], np.float32)
    w.add_tensor("b", "BF16", (4,), (vals.view(np.uint32) >> 16).astype("<u2"))
    w.add_tensor("q", "Q3_K", (1, 256), np.zeros(110, np.uint8))
    path = str(tmp_path / "t.gguf")
    w.write(path)
    with gguf.GGUFReader(path) as r:
        assert np.array_equal(r.tensor_f32("b"), vals)
        assert r.info("q").type_name == "Q3_K" and r.info("q").n_bytes == 110
        with pytest.raises(gguf.GGUFError):
            r.upload("q")                                            # not an encoding the device kernels take


def test_damaged_files_are_rejected(tmp_path):
    path, _ = small_file(tmp_path)
    raw = open(path, "rb").read()

    def reject(b, name):
        p = tmp_path / name
        p.write_bytes(b)
        with pytest.raises(gguf.GGUFError):
            gguf.GGUFReader(str(p))

    reject(b"GGUX" + raw[4:], "magic.gguf")
    reject(raw[:4] + struct.pack("<I", 1) + raw[8:], "version.gguf")
    reject(raw[:40], "short_header.gguf")
    reject(raw[:-64], "short_data.gguf")
    reject(b"", "empty.gguf")
    w = gguf.GGUFWriter()
    with pytest.raises(gguf.GGUFError):
        w.add_tensor("bad", "Q4_K", (2, 256), np.zeros(100, np.uint8))   # byte count does not match the shape


FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "test_experiment.gguf")


def test_reference_fixture_parses_as_the_reference_reader_asserts():
    """The 512-byte file the reference's own reader tests run on
    (/root/reference/skainet-io/skainet-io-gguf/src/jvmTest/resources/test_experiment.gguf, kept here as a data fixture),
    with the assertions of StreamingGGUFReaderTest.kt:39-185: version, tensor count, names, shapes, types, offsets at or
    behind the data section, positive sizes, every tensor loadable at its full size, two loads of a tensor identical,
    a load into a larger buffer at an offset leaves the prefix alone."""
    assert os.path.getsize(FIXTURE) == 512
    with gguf.GGUFReader(FIXTURE) as r:
        assert r.version == 3 and r.version > 0
        assert len(r.tensors) == 3 == len(r.names())
        assert sorted(r.names()) == ["result", "x", "y"]
        assert r.fields["general.architecture"] == "llama"
        assert r.fields["general.name"] == "addition_op" and r.fields["general.description"] == "Simple addition"
        assert r.data_offset > 0 and r.data_offset % r.alignment == 0
        expected_offsets = {"x": 320, "y": 384, "result": 448}
        for t in r.tensors:
            assert t.shape == (3, 3) and t.type_name == "F32" and t.type_id == 0
            assert t.offset >= r.data_offset and t.offset == expected_offsets[t.name]
            assert t.n_bytes == 36 > 0 and t.n_elements == 9
            data = np.array(r.tensor_bytes(t.name))
            assert data.size == t.n_bytes
            assert np.array_equal(data, np.array(r.tensor_bytes(t.name)))          # loading twice gives the same bytes
            buf = np.zeros(t.n_bytes + 100, np.uint8)
            buf[10:10 + t.n_bytes] = r.tensor_bytes(t.name)
            assert not buf[:10].any() and np.array_equal(buf[10:10 + t.n_bytes], data) and not buf[10 + t.n_bytes:].any()
        # the file is a recorded addition: result = x + y, which pins the element order and the float decoding
        x, y, res = r.tensor_f32("x"), r.tensor_f32("y"), r.tensor_f32("result")
        assert x.shape == (3, 3) and np.isfinite(res).all()
        assert np.allclose(x + y, res, rtol=0, atol=1e-6)
        with pytest.raises(gguf.GGUFError):
            r.upload("x")                                                          # dense F32 is not a packed matmul weight
