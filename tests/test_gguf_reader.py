"""The GGUF container reader (host code in the library, no GPU): files written by the
independent writer in tests/gguf_writer.py are parsed back; behaviour follows the reference's
importer (tools/gguf/GGUFImporter.cpp) -- shape reversal (:206-221, pinned by
tests/GGUFImporterTest.cpp:513-519), raw payload import (:457-502, the 18-byte Q4_0 fixture of
tests/GGUFImporterTest.cpp:173-178,521-534), metadata widening (:339-437), hyper-parameter defaults,
checks and messages (:505-642)."""
import numpy as np
import pytest

import gguf_writer as gw
from litenn_amd import synth
from litenn_amd import _lib
from litenn_amd._lib import LiteNNHipError
from litenn_amd.formats import Q4_0, Q4_K, Q6_K, Q8_0
from litenn_amd.gguf import GGUFFile

Q4_0_FIXTURE = bytes([0x10, 0x00, 0x22, 0x44, 0x66, 0x88, 0xaa, 0xcc, 0xee, 0x11, 0x33, 0x55, 0x77, 0x99, 0xbb, 0xdd,
                      0xff, 0x7f])


def test_q4_0_payload_fixture_round_trips(tmp_path):
    """The reference's raw-import fixture: one Q4_0 block, shape [32], bytes kept verbatim."""
    path = gw.write_gguf(tmp_path / "one.gguf", [("general.architecture", gw.STRING, "llama")],
                         [("blk.0.attn_q.weight", "q4_0", (32,), np.frombuffer(Q4_0_FIXTURE, np.uint8))])
    with GGUFFile(path) as f:
        assert f.version == 3 and f.tensor_count == 1 and f.metadata_count == 1
        t = f.tensor("blk.0.attn_q.weight")
        assert t.shape == (32,) and t.quantized and t.fmt == Q4_0 and t.dtype == -1 and t.bytes == 18
        raw = f.payload(0)
        assert raw[0] == 0x10 and raw[17] == 0x7f  # what the reference's test asserts
        assert raw.tobytes() == Q4_0_FIXTURE
        assert t.file_offset % 32 == 0


def test_shapes_are_reversed_and_payloads_aligned(tmp_path):
    rng = np.random.default_rng(0)
    a = rng.standard_normal((3, 5)).astype(np.float32)           # stored as ne = [5, 3]
    q = synth.quant_weights(Q6_K, 7, 512, 1)
    path = gw.write_gguf(tmp_path / "s.gguf", [], [("a", "f32", (3, 5), a), ("q", "q6_k", (7, 512), q),
                                                    ("v", "f32", (4,), np.arange(4, dtype=np.float32))], alignment=64,
                         declare_alignment=True)
    with GGUFFile(path) as f:
        ta, tq, tv = f.tensor("a"), f.tensor("q"), f.tensor(2)
        assert ta.shape == (3, 5) and ta.dtype == 0 and not ta.quantized and ta.fmt == -1
        assert np.array_equal(f.payload("a").view(np.float32).reshape(3, 5), a)
        assert tq.shape == (7, 512) and tq.fmt == Q6_K and tq.bytes == 7 * 2 * 210
        assert np.array_equal(f.payload("q"), q.reshape(-1))
        assert tv.name == "v" and tv.shape == (4,)
        assert all(t.file_offset % 64 == 0 for t in f.tensors())
        assert f.get_size("general.alignment") == 64


def test_metadata_is_widened_like_the_reference(tmp_path):
    md = [("u8", gw.U8, 200), ("i8", gw.I8, -5), ("u16", gw.U16, 60000), ("i16", gw.I16, -300), ("u32", gw.U32, 7),
          ("i32", gw.I32, 12), ("f32", gw.F32, 0.5), ("b", gw.BOOL, 1), ("s", gw.STRING, "hello"),
          ("u64", gw.U64, 2 ** 40), ("i64", gw.I64, -2 ** 40), ("f64", gw.F64, 1e-300),
          ("arr", gw.ARRAY, (gw.I32, [1, 2, 3])), ("names", gw.ARRAY, (gw.STRING, ["a", "bc"]))]
    path = gw.write_gguf(tmp_path / "m.gguf", md, [])
    with GGUFFile(path) as f:
        assert f.keys() == [k for k, _, _ in md]
        assert f.get_size("u8") == 200 and f.get_size("u16") == 60000 and f.get_size("i32") == 12
        assert f.get_size("u64") == 2 ** 40
        assert f.get_double("f32") == 0.5 and f.get_double("f64") == 1e-300 and f.get_double("i8") == -5.0
        assert f.get_string("s") == "hello" and f.get_bool("b") is True
        assert f.get_array_info("arr") == (gw.I32, 3) and f.get_array_info("names") == (gw.STRING, 2)
        for key, msg in [("i8", "must be non-negative"), ("f32", "must be an integer"), ("s", "must be an integer")]:
            with pytest.raises(LiteNNHipError, match=f"GGUF metadata key '{key}' {msg}"):
                f.get_size(key)
        with pytest.raises(LiteNNHipError, match="GGUF metadata key 's' must be numeric"):
            f.get_double("s")
        with pytest.raises(LiteNNHipError, match="GGUF metadata key 'u8' must be a string"):
            f.get_string("u8")
        with pytest.raises(LiteNNHipError, match="Missing GGUF metadata key 'nope'"):
            f.get_size("nope")
        with pytest.raises(LiteNNHipError, match="Missing GGUF tensor 'nope'"):
            f.tensor("nope")


def test_llama_hyperparameters_defaults_and_checks(tmp_path):
    cfg = synth.tiny_llama(Q4_K, block_count=1, d_model=256, heads=4, kv_heads=2, ff=512, vocab=300, context_length=77)
    with GGUFFile(gw.llama_gguf(tmp_path / "t.gguf", cfg, 1)) as f:
        p = f.llama_params()
        assert (p.block_count, p.embedding_length, p.head_count, p.head_count_kv, p.feed_forward_length) == \
               (1, 256, 4, 2, 512)
        assert p.vocab_size == 300 and p.context_length == 77
        assert p.rope_dimension_count == 64  # defaults to the head dimension
        assert p.rms_norm_epsilon == float(np.float32(cfg.rms_eps))  # f32 key widened to double
        assert p.rope_freq_base == cfg.rope_freq_base and p.rope_freq_scale == 1.0
        assert f.get_string("general.architecture") == "llama"

    # linear rope scaling: freq_scale = 1 / factor; another architecture prefix works the same way
    extra = [("qwen2.rope.scaling.type", gw.STRING, "LINEAR"), ("qwen2.rope.scaling.factor", gw.F32, 4.0)]
    with GGUFFile(gw.llama_gguf(tmp_path / "l.gguf", cfg, 1, extra_metadata=extra, arch="qwen2")) as f:
        assert f.llama_params().rope_freq_scale == 0.25

    bad = [
        ([("llama.rope.scaling.type", gw.STRING, "yarn")], "only executes none/linear scaling, got 'yarn'"),
        ([("llama.rope.scaling.type", gw.STRING, "weird")], "Unsupported LLaMA rope.scaling.type 'weird'"),
        ([("llama.rope.dimension_count", gw.U32, 63)], "rope.dimension_count must be an even value"),
        ([("llama.rope.scaling.factor", gw.F32, -1.0)], "rope.scaling.factor must be non-negative"),
    ]
    for i, (extra, msg) in enumerate(bad):
        with GGUFFile(gw.llama_gguf(tmp_path / f"bad{i}.gguf", cfg, 1, extra_metadata=extra)) as f:
            with pytest.raises(LiteNNHipError, match=msg):
                f.llama_params()
    cfg_bad = synth.tiny_llama(Q4_0, block_count=1, d_model=256, heads=4, kv_heads=3, ff=512, vocab=300)
    with GGUFFile(gw.llama_gguf(tmp_path / "kv.gguf", cfg_bad, 1, skip=("attn_k", "attn_v"))) as f:
        with pytest.raises(LiteNNHipError, match="attention.head_count 4 must be divisible by attention.head_count_kv 3"):
            f.llama_params()


def test_broken_files_are_refused(tmp_path):
    with pytest.raises(LiteNNHipError, match="Failed to open GGUF file"):
        GGUFFile(tmp_path / "missing.gguf")
    p = tmp_path / "junk.gguf"
    p.write_bytes(b"GGUX" + b"\0" * 64)
    with pytest.raises(LiteNNHipError, match="Failed to open GGUF file"):
        GGUFFile(p)
    good = gw.write_gguf(tmp_path / "g.gguf", [], [("a", "f32", (64,), np.zeros(64, np.float32))])
    raw = open(good, "rb").read()
    cut = tmp_path / "cut.gguf"
    cut.write_bytes(raw[:-100])  # payload truncated
    with pytest.raises(LiteNNHipError, match="Failed to read 256 bytes for GGUF tensor 'a'"):
        GGUFFile(cut)
    odd = gw.write_gguf(tmp_path / "odd.gguf", [], [("q", "q4_k", (2, 256), np.zeros(288, np.uint8))])
    with GGUFFile(odd) as f:
        assert f.tensor("q").bytes == 288
    # an unknown ggml type id
    patched = bytearray(open(odd, "rb").read())
    idx = patched.find(b"q" + (2).to_bytes(4, "little"))  # name 'q' followed by rank 2
    type_pos = idx + 1 + 4 + 16
    patched[type_pos:type_pos + 4] = (99).to_bytes(4, "little")
    bad = tmp_path / "type.gguf"
    bad.write_bytes(bytes(patched))
    with pytest.raises(LiteNNHipError, match="Unsupported ggml tensor type '99' for tensor 'q'"):
        GGUFFile(bad)


@pytest.mark.parametrize("kind", ["gguf", "ltnn"])
def test_mutated_images_are_refused_or_read_never_crash(tmp_path, kind):
    """Both container readers parse files from outside: truncations anywhere, random bytes and huge
    counts in the header region, single bit flips.  Every mutant either opens (and every accessor
    then works on it) or is refused with an error; a fault in the reader would take the test
    process down.  (The same mutations, tens of thousands per format, were also run once against
    a host-sanitizer build of the reader.)"""
    import ltnn_writer as lw
    cfg = synth.tiny_llama(Q4_K, block_count=1, d_model=256, heads=2, kv_heads=1, ff=256, vocab=64,
                           formats={"default": Q4_K, "attn_v": Q6_K, "token_embd": Q8_0})
    base = tmp_path / ("base." + kind)
    (gw.llama_gguf if kind == "gguf" else lw.llama_ltnn)(base, cfg, 3)
    image = open(base, "rb").read()
    rng = np.random.default_rng(17)
    head = min(len(image), 8192)
    opened = 0
    for it in range(400):
        m = bytearray(image)
        how = it % 5
        if how == 0:
            m = m[:int(rng.integers(0, len(m) + 1))]
        elif how == 1:
            m = m[:int(rng.integers(0, head + 1))]
        elif how == 2:
            for _ in range(int(rng.integers(1, 9))):
                m[int(rng.integers(0, head))] = int(rng.integers(0, 256))
        elif how == 3:
            at = int(rng.integers(0, head - 8))
            value = (1 << 64) - 1 if it % 4 == 0 else int(rng.integers(0, 1 << 62)) >> int(rng.integers(0, 62))
            m[at:at + 8] = value.to_bytes(8, "little")
        else:
            for _ in range(int(rng.integers(1, 5))):
                m[int(rng.integers(0, len(m)))] ^= 1 << int(rng.integers(0, 8))
        p = tmp_path / "mutant.bin"
        p.write_bytes(bytes(m))
        try:
            with GGUFFile(p) as f:
                opened += 1
                for i in range(f.tensor_count):
                    try:
                        t = f.tensor(i)
                        assert len(f.payload(i)) == t.bytes
                    except (LiteNNHipError, UnicodeDecodeError):
                        pass
                for i in range(f.metadata_count):
                    raw_key = _lib.load().litenn_gguf_metadata_key(f._h, i)
                    try:
                        key = raw_key.decode()
                    except UnicodeDecodeError:
                        continue
                    for get in (f.get_size, f.get_double, f.get_string, f.get_bool, f.get_array_info):
                        try:
                            get(key)
                        except (LiteNNHipError, UnicodeDecodeError):
                            pass
                try:
                    f.llama_params()
                except LiteNNHipError:
                    pass
        except LiteNNHipError:
            pass
    assert 0 < opened < 400


def _raw_gguf(path, tensors, pad_to=0, tail=b""):
    """A version-3 image with a hand-made tensor directory: tensors = (name, ne fastest first, ggml type id, offset)."""
    import struct
    head = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), 0)
    for name, ne, type_id, offset in tensors:
        head += struct.pack("<Q", len(name)) + name.encode() + struct.pack("<I", len(ne))
        for n in ne:
            head += struct.pack("<Q", n)
        head += struct.pack("<IQ", type_id, offset)
    start = (len(head) + 31) // 32 * 32
    with open(path, "wb") as f:
        f.write(head + b"\0" * (start - len(head)) + tail + b"\0" * pad_to)
    return path, start


def test_offsets_and_shapes_that_wrap_64_bits_are_refused(tmp_path):
    """Directory entries whose offset + size, or whose element count, does not fit 64 bits must not
    pass a bound check through wrap-around (the reference reads through ggml's checked reader)."""
    data = np.arange(16, dtype=np.float32).tobytes()
    # one f32[4] tensor at an offset just below 2^64: data_offset + offset + 16 wraps to a small number
    for offset in (2 ** 64 - 72, 2 ** 64 - 64, 2 ** 64 - 32, 2 ** 63):
        path, start = _raw_gguf(tmp_path / "wrap.gguf", [("t", (4,), 0, offset)], tail=data)
        with pytest.raises(LiteNNHipError) as e:
            GGUFFile(path)
        assert "Failed to read" in str(e.value), str(e.value)
    # a 2^32 x 2^32 f32 tensor: the element count wraps to 0
    path, _ = _raw_gguf(tmp_path / "big.gguf", [("t", (2 ** 32, 2 ** 32), 0, 0)], tail=data)
    with pytest.raises(LiteNNHipError) as e:
        GGUFFile(path)
    assert "more elements than the file has room for" in str(e.value)
    # four dimensions of 2^40: far past any wrap
    path, _ = _raw_gguf(tmp_path / "big4.gguf", [("t", (2 ** 40,) * 4, 0, 0)], tail=data)
    with pytest.raises(LiteNNHipError):
        GGUFFile(path)
    # a quantised shape whose element count wraps to a whole number of blocks
    path, _ = _raw_gguf(tmp_path / "bigq.gguf", [("t", (2 ** 40, 2 ** 24), 12, 0)], tail=data)
    with pytest.raises(LiteNNHipError):
        GGUFFile(path)
    # the honest neighbour still opens: same tensor at offset 32
    path, start = _raw_gguf(tmp_path / "ok.gguf", [("t", (4,), 0, 32)], tail=b"\0" * 32 + data[:16])
    with GGUFFile(path) as f:
        t = f.tensor("t")
        assert t.file_offset == start + 32 and t.bytes == 16
        assert np.array_equal(f.payload("t").view(np.float32), np.arange(4, dtype=np.float32))


def test_unaligned_tensor_offsets_are_refused(tmp_path):
    """ggml refuses a file whose tensor data does not start on a multiple of general.alignment."""
    data = np.arange(16, dtype=np.float32).tobytes()
    path, _ = _raw_gguf(tmp_path / "unaligned.gguf", [("t", (4,), 0, 8)], tail=data)
    with pytest.raises(LiteNNHipError) as e:
        GGUFFile(path)
    assert "not a multiple of the alignment" in str(e.value)
