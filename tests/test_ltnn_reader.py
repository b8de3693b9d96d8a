"""The reader of a LiteNN model archive's variable table (host code in the library, no GPU): files
written by the independent writer in tests/ltnn_writer.py are parsed back through the same handle
and accessors as a GGUF file.  Layout: src/LiteNN/Serialization/ModelIO.h:1291-1341 (header, names,
metadata, variables), :592-612 (tensor), :281-338 (quantisation record), :27-39,447-505 (metadata
values); the 18-byte Q4_0 payload with expressed shape [32] is the case the reference round-trips
in tests/QuantizationTest.cpp:233-275.  The reference holds no .ltnn file, so the byte layout is
pinned by these sources only."""
import struct

import numpy as np
import pytest

import ltnn_writer as lw
from litenn_amd import synth
from litenn_amd._lib import LiteNNHipError
from litenn_amd.formats import Q4_0, Q4_K
from litenn_amd.gguf import GGUFFile

RAW_18 = np.arange(1, 19, dtype=np.uint8)  # the payload of QuantizationTest.cpp:235-236


def test_block_payload_and_record_survive(tmp_path):
    path = lw.write_ltnn(tmp_path / "one.ltnn", [("general.architecture", lw.K_STRING, "llama")],
                         [("w", RAW_18, (Q4_0, (32,))),
                          ("norm", np.linspace(0.5, 1.5, 7, dtype=np.float32), None),
                          ("half", np.arange(6, dtype=np.float16).reshape(2, 3), None),
                          ("mask", np.array([True, False, True]), None)])
    with GGUFFile(path) as f:
        assert f.version == 18 and f.tensor_count == 4 and f.metadata_count == 1
        t = f.tensor("w")
        assert t.shape == (32,) and t.quantized and t.fmt == Q4_0 and t.dtype == -1 and t.bytes == 18
        assert f.payload(0).tobytes() == RAW_18.tobytes()
        n = f.tensor("norm")
        assert n.shape == (7,) and not n.quantized and n.fmt == -1 and n.dtype == lw.F32 and n.bytes == 28
        assert np.array_equal(f.payload(1).view(np.float32), np.linspace(0.5, 1.5, 7, dtype=np.float32))
        h = f.tensor("half")
        assert h.shape == (2, 3) and h.dtype == lw.F16
        assert np.array_equal(f.payload(2).view(np.float16), np.arange(6, dtype=np.float16))
        m = f.tensor("mask")
        assert m.shape == (3,) and m.dtype == lw.BOOL and m.bytes == 3


def test_metadata_kinds(tmp_path):
    md = [("a.i", lw.K_I64, -5), ("a.u", lw.K_U64, 2 ** 40), ("a.f", lw.K_F64, 0.125), ("a.b", lw.K_BOOL, True),
          ("a.s", lw.K_STRING, "text"), ("a.il", lw.K_I64_LIST, [1, -2, 3]), ("a.ul", lw.K_U64_LIST, [4, 5]),
          ("a.fl", lw.K_F64_LIST, [0.5]), ("a.bl", lw.K_BOOL_LIST, [True, False]),
          ("a.sl", lw.K_STRING_LIST, ["x", "yy", "zzz"])]
    path = lw.write_ltnn(tmp_path / "md.ltnn", md, [("w", RAW_18, (Q4_0, (32,)))])
    with GGUFFile(path) as f:
        assert f.keys() == [k for k, _, _ in md]
        assert f.get_double("a.i") == -5.0 and f.get_size("a.u") == 2 ** 40 and f.get_double("a.f") == 0.125
        assert f.get_bool("a.b") is True and f.get_string("a.s") == "text"
        with pytest.raises(LiteNNHipError, match="must be non-negative"):
            f.get_size("a.i")
        assert f.get_array_info("a.il")[1] == 3 and f.get_array_info("a.ul")[1] == 2 and f.get_array_info("a.fl")[1] == 1
        assert f.get_array_info("a.bl")[1] == 2 and f.get_array_info("a.sl")[1] == 3
        assert f.tensor("w").bytes == 18  # the variables after the metadata are still found


def test_llama_archive_gives_the_hyperparameters(tmp_path):
    cfg = synth.tiny_llama(Q4_K)
    path = lw.llama_ltnn(tmp_path / "m.ltnn", cfg, 3)
    with GGUFFile(path) as f:
        p = f.llama_params()
        assert (p.block_count, p.embedding_length, p.head_count, p.head_count_kv) == (
            cfg.block_count, cfg.embedding_length, cfg.head_count, cfg.head_count_kv)
        assert p.feed_forward_length == cfg.feed_forward_length and p.vocab_size == cfg.vocab
        assert p.context_length == cfg.context_length
        t = f.tensor("blk.0.attn_q.weight")
        assert t.quantized and t.fmt == cfg.fmt("attn_q") and t.shape == cfg.tensor_shapes()["attn_q"]


def test_broken_archives_are_refused(tmp_path):
    good = lw.write_ltnn(tmp_path / "good.ltnn", [], [("w", RAW_18, (Q4_0, (32,)))])
    raw = open(good, "rb").read()
    cases = {
        "version0": raw[:8] + struct.pack("<I", 0) + raw[12:],
        "version19": raw[:8] + struct.pack("<I", 19) + raw[12:],
        "version5": raw[:8] + struct.pack("<I", 5) + raw[12:],
        "truncated": raw[:len(raw) // 2],
    }
    expect = {"version0": "Unsupported LiteNN model version", "version19": "Unsupported LiteNN model version",
              "version5": "version 6 or later", "truncated": "truncated or unreadable"}
    for name, data in cases.items():
        p = tmp_path / f"{name}.ltnn"
        p.write_bytes(data)
        with pytest.raises(LiteNNHipError, match=expect[name]):
            GGUFFile(p)
    # payload size that does not match the block format and expressed shape
    bad = lw.write_ltnn(tmp_path / "size.ltnn", [], [("w", RAW_18, (Q4_0, (64,)))])
    with pytest.raises(LiteNNHipError, match="invalid serialized byte size"):
        GGUFFile(bad)
    # a block format this reader has no layout for (an IQ format id)
    iq = lw.write_ltnn(tmp_path / "iq.ltnn", [], [("w", RAW_18, (13, (32,)))])
    with pytest.raises(LiteNNHipError, match="no layout"):
        GGUFFile(iq)
    # names and variables disagree
    head = raw.index(struct.pack("<Q", 1) + struct.pack("<Q", 1))
    names_bad = raw[:head + 8] + struct.pack("<Q", 0) + raw[head + 16 + 8 + 1:]
    p = tmp_path / "names.ltnn"
    p.write_bytes(names_bad)
    with pytest.raises(LiteNNHipError):
        GGUFFile(p)
