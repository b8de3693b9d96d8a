"""A minimal GGUF (version 3) writer for tests, written from the published container layout and
independent of the library's reader: header, key/value table, tensor directory, payloads aligned to
general.alignment.  Tensor shapes are given slowest dimension first ([N, K]); the file stores them
fastest first, as ggml does."""
from __future__ import annotations

import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
GGML_TYPE = {"f32": 0, "f16": 1, "q4_0": 2, "q4_1": 3, "q5_0": 6, "q5_1": 7, "q8_0": 8, "q2_k": 10, "q3_k": 11,
             "q4_k": 12, "q5_k": 13, "q6_k": 14, "i32": 26}
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
           I64: "<q", F64: "<d"}


def _string(s: str) -> bytes:
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype: int, value) -> bytes:
    if vtype == STRING:
        return _string(value)
    if vtype == ARRAY:
        etype, items = value
        out = struct.pack("<IQ", etype, len(items))
        for it in items:
            out += _value(etype, it)
        return out
    return struct.pack(_SCALAR[vtype], value)


def write_gguf(path, metadata, tensors, alignment: int = 32, version: int = 3, declare_alignment: bool = False):
    """metadata: list of (key, type id, value); tensors: list of (name, ggml type name, shape slowest
    first, payload bytes/ndarray)."""
    if declare_alignment:
        metadata = list(metadata) + [("general.alignment", U32, alignment)]
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata))
    for key, vtype, value in metadata:
        head += _string(key) + struct.pack("<I", vtype) + _value(vtype, value)
    payloads, offset, infos = [], 0, b""
    for name, tname, shape, payload in tensors:
        raw = np.ascontiguousarray(payload).view(np.uint8).reshape(-1).tobytes()
        offset = (offset + alignment - 1) // alignment * alignment
        infos += _string(name) + struct.pack("<I", len(shape))
        for n in reversed(shape):
            infos += struct.pack("<Q", n)
        infos += struct.pack("<IQ", GGML_TYPE[tname], offset)
        payloads.append((offset, raw))
        offset += len(raw)
    head += infos
    data_start = (len(head) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (data_start - len(head)))
        pos = 0
        for off, raw in payloads:
            f.write(b"\0" * (off - pos))
            f.write(raw)
            pos = off + len(raw)
    return path


FORMAT_NAMES = {1: "q4_0", 2: "q4_1", 3: "q5_0", 4: "q5_1", 5: "q8_0", 7: "q2_k", 8: "q3_k", 9: "q4_k", 10: "q5_k",
                11: "q6_k", 27: "f32", 25: "f16"}


def llama_gguf(path, cfg, seed, extra_metadata=(), skip=(), arch="llama", alignment=32):
    """A GGUF file of the synthetic decoder `cfg` (litenn_amd.synth): metadata keys of
    ParseLLaMAHyperparameters and tensor names of the reference's builder."""
    from litenn_amd import synth
    md = [
        ("general.architecture", STRING, arch),
        (f"{arch}.context_length", U32, cfg.context_length),
        (f"{arch}.embedding_length", U32, cfg.embedding_length),
        (f"{arch}.block_count", U32, cfg.block_count),
        (f"{arch}.feed_forward_length", U32, cfg.feed_forward_length),
        (f"{arch}.attention.head_count", U32, cfg.head_count),
        (f"{arch}.attention.head_count_kv", U32, cfg.head_count_kv),
        (f"{arch}.attention.layer_norm_rms_epsilon", F32, cfg.rms_eps),
        (f"{arch}.rope.freq_base", F32, cfg.rope_freq_base),
        ("tokenizer.ggml.tokens", ARRAY, (STRING, ["<s>", "</s>", "a"])),
        ("general.file_type", U32, 2),
    ] + list(extra_metadata)
    if getattr(cfg, "rope_freq_scale", 1.0) != 1.0:
        md += [(f"{arch}.rope.scaling.type", STRING, "linear"),
               (f"{arch}.rope.scaling.factor", F32, 1.0 / cfg.rope_freq_scale)]
    if getattr(cfg, "rope_dimension_count", 0):
        md.append((f"{arch}.rope.dimension_count", U32, cfg.rope_dimension_count))
    tensors = []
    for kind, layer, fmt, payload, n, k in synth.llama_tensors(cfg, seed):
        if kind in skip:
            continue
        name = f"{kind}.weight" if layer < 0 else f"blk.{layer}.{kind}.weight"
        shape = (k,) if kind.endswith("norm") else (n, k)
        tensors.append((name, FORMAT_NAMES[fmt], shape, payload))
    return write_gguf(path, md, tensors, alignment=alignment, declare_alignment=alignment != 32)
