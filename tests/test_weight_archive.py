"""`weights.llmopt` reader/writer (llmopt_amd/weight_archive.py) against the index of an archive the
reference's own tests hold, and against the reference reader's rejection rules
(lib/weight_archive.ml:165-296)."""
import json
import os
import struct

import numpy as np
import pytest

from llmopt_amd import weight_archive as wa

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def golden():
    meta = json.load(open(os.path.join(GOLDEN, "weight_archive_index_mul1_3bit.json")))
    data = open(os.path.join(GOLDEN, "weight_archive_index_mul1_3bit.bin"), "rb").read()
    return meta, data


def test_reads_the_index_of_a_reference_written_archive():
    """test/fixtures/exl3/mul1-3bit.llmopt, written by the reference's Python exporter: the entry list
    below was read off that file's bytes (names, dtype tags 1/0/7, shapes, 256-aligned offsets)."""
    meta, data = golden()
    assert len(data) == meta["index_bytes"] == 512
    entries = wa.parse_index(data, meta["file_size"])
    assert [e.name for e in entries] == ["codebook", "decoded", "expected", "input", "weight.exl3", "weight.suh",
                                         "weight.svh", "weight.trellis"]
    assert entries[0] == wa.TensorEntry("codebook", "float16", (65536,), 512, 131072)
    assert entries[2] == wa.TensorEntry("expected", "float32", (9, 128), 164352, 4608)
    assert entries[7] == wa.TensorEntry("weight.trellis", "uint8", (8, 8, 96), 172032, 6144)
    assert entries[7].offset + entries[7].byte_length == meta["file_size"] == 178176
    for entry, want in zip(entries, meta["entries"]):
        assert (entry.name, entry.dtype, list(entry.shape), entry.offset, entry.byte_length) == (
            want["name"], want["dtype"], want["shape"], want["offset"], want["byte_length"])


def test_writer_output_is_what_the_reader_accepts_and_layout_is_the_documented_one(tmp_path):
    rng = np.random.default_rng(0)
    tensors = {"model.layers.0.q.weight": rng.integers(0, 256, size=(64, 32), dtype=np.uint8),
               "model.layers.0.q.scale": rng.uniform(0.005, 0.02, size=(64, 1)).astype(np.float16),
               "model.norm.weight": rng.standard_normal(64).astype(np.float16),
               "positions": np.arange(5, dtype=np.int64)}
    path = str(tmp_path / "weights.llmopt")
    written = wa.write_archive(path, tensors)
    entries = wa.read_index(path)
    assert entries == written
    raw = open(path, "rb").read()
    assert raw[:8] == b"LLMOPTWT" and struct.unpack_from("<HHIQ", raw, 8) == (1, 0, 4, 256)
    assert [e.name for e in entries] == sorted(tensors)  # ASCII names: byte order = str order
    for entry in entries:
        assert entry.offset % 256 == 0
        assert raw[entry.offset:entry.offset + entry.byte_length] == tensors[entry.name].tobytes()
    assert len(raw) == entries[-1].offset + entries[-1].byte_length  # nothing after the last payload


def corrupt(data: bytes, offset: int, replacement: bytes) -> bytes:
    return data[:offset] + replacement + data[offset + len(replacement):]


@pytest.mark.parametrize("mutate,message", [
    (lambda d: corrupt(d, 0, b"LLMOPTWX"), "invalid weight-archive magic"),
    (lambda d: corrupt(d, 8, struct.pack("<H", 2)), "unsupported weight-archive version: 2"),
    (lambda d: corrupt(d, 10, struct.pack("<H", 1)), "unsupported weight-archive flags: 1"),
    (lambda d: corrupt(d, 12, struct.pack("<I", 0)), "weight archive contains no tensors"),
    (lambda d: corrupt(d, 24 + 6, struct.pack("<H", 7)), "weight archive tensor reserved field is non-zero"),
    (lambda d: corrupt(d, 24 + 4, bytes([200])), "unknown weight-archive dtype tag: 200"),
    (lambda d: corrupt(d, 24 + 8, b"zodebook"), "weight archive tensor names are not strictly sorted"),
    (lambda d: corrupt(d, 24 + 8 + 8 + 8, struct.pack("<Q", 513)), "weight archive tensor codebook offset is not aligned"),
    (lambda d: corrupt(d, 24 + 8 + 8 + 8, struct.pack("<Q", 768)),
     "weight archive tensor codebook has an unexpected payload offset"),
    (lambda d: corrupt(d, 24 + 8 + 8 + 16, struct.pack("<Q", 131070)),
     "weight archive tensor codebook byte length disagrees with its dtype and shape"),
    (lambda d: corrupt(d, 511, b"\x01"), "weight archive index padding contains non-zero bytes"),
])
def test_rejections_carry_the_reference_messages(mutate, message):
    meta, data = golden()
    with pytest.raises(wa.ArchiveError) as caught:
        wa.parse_index(mutate(data), meta["file_size"])
    assert str(caught.value) == message


def test_file_size_rules():
    meta, data = golden()
    with pytest.raises(wa.ArchiveError, match="trailing or missing payload bytes"):
        wa.parse_index(data, meta["file_size"] + 1)
    with pytest.raises(wa.ArchiveError, match="weight.trellis exceeds the file"):
        wa.parse_index(data, meta["file_size"] - 1)
    with pytest.raises(wa.ArchiveError, match="index extends beyond the file"):
        wa.parse_index(data, 100)
    with pytest.raises(wa.ArchiveError, match="file is too short"):
        wa.parse_index(data[:10], 10)


@pytest.mark.gpu
def test_mapped_archive_feeds_the_w4a16_kernel(tmp_path):
    """Views of one mapped file as weight / scale / activation buffers of llmopt_w4a16_linear_f16_g64."""
    import oracle
    from llmopt_amd.native import Runtime
    from tests.gpu_util import assert_close_to_oracle, linear_grid, u32s, w4_case
    rng = np.random.default_rng(4)
    x, packed, scale, _ = w4_case(rng, 1, 192, 576)
    path = str(tmp_path / "weights.llmopt")
    wa.write_archive(path, {"proj.weight": packed, "proj.scale": scale, "x": x})
    runtime = Runtime()
    try:
        archive = wa.WeightArchive(runtime, path)
        assert archive.entry("proj.weight").shape == (192, 288)
        np.testing.assert_array_equal(archive.numpy("proj.scale"), scale)
        weight, scales = archive.w4a16_pair("proj.weight", "proj.scale")
        out = runtime.create_buffer(192 * 2)
        runtime.dispatch("llmopt_w4a16_linear_f16_g64", [archive.buffer("x"), weight, scales, scales, out],
                         u32s(1, 192, 576, 0, 0), grid=(linear_grid(192), 1, 1), group=(256, 1, 1))
        assert_close_to_oracle(out.numpy(np.float16, (1, 192)), oracle.w4a16_linear(x, packed, scale, None),
                               "GEMV on mapped archive views")
        with pytest.raises(wa.ArchiveError):
            archive.w4a16_pair("proj.scale", "proj.weight")
    finally:
        runtime.close()
