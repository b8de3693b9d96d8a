"""A minimal writer of the variable table of a LiteNN model archive (.ltnn, version 18) for tests,
written from the serializer's layout (src/LiteNN/Serialization/ModelIO.h:1291-1341: header, names,
metadata entries, per variable a tensor and an optional quantisation record, then slots and
subgraphs) and independent of the library's reader.  The graph part is one empty subgraph-less
tail: readers of the variable table stop before it."""
from __future__ import annotations

import struct

import numpy as np

# DataType (src/LiteNN/DType.h:17-30)
F32, F64, I32, I64, BOOL, F16, BF16, F8E4M3, F8E5M2, I8, U8 = range(11)
_NP_DTYPE = {np.dtype(np.float32): F32, np.dtype(np.float64): F64, np.dtype(np.int32): I32, np.dtype(np.int64): I64,
             np.dtype(np.float16): F16, np.dtype(np.int8): I8, np.dtype(np.uint8): U8, np.dtype(np.bool_): BOOL}
# MetadataValueKind (ModelIO.h:27-39)
K_I64, K_U64, K_F64, K_BOOL, K_STRING, K_I64_LIST, K_U64_LIST, K_F64_LIST, K_BOOL_LIST, K_STRING_LIST = range(10)
SCHEME_BLOCK, GRANULARITY_PER_TENSOR = 1, 0


def _size(n: int) -> bytes:
    return struct.pack("<Q", n)


def _string(s: str) -> bytes:
    b = s.encode()
    return _size(len(b)) + b


def _metadata_value(kind: int, value) -> bytes:
    out = struct.pack("<I", kind)
    if kind == K_I64:
        return out + struct.pack("<q", value)
    if kind == K_U64:
        return out + struct.pack("<Q", value)
    if kind == K_F64:
        return out + struct.pack("<d", value)
    if kind == K_BOOL:
        return out + struct.pack("<B", 1 if value else 0)
    if kind == K_STRING:
        return out + _string(value)
    out += _size(len(value))
    for v in value:
        out += {K_I64_LIST: lambda x: struct.pack("<q", x), K_U64_LIST: lambda x: struct.pack("<Q", x),
                K_F64_LIST: lambda x: struct.pack("<d", x), K_BOOL_LIST: lambda x: struct.pack("<B", 1 if x else 0),
                K_STRING_LIST: _string}[kind](v)
    return out


def _tensor(array: np.ndarray) -> bytes:
    a = np.ascontiguousarray(array)
    out = struct.pack("<I", _NP_DTYPE[a.dtype]) + _size(a.ndim)
    for d in a.shape:
        out += _size(d)
    return out + a.tobytes()


def _quantization(block_format: int, expressed_shape, expressed_type=F32) -> bytes:
    out = struct.pack("<IIIII", SCHEME_BLOCK, GRANULARITY_PER_TENSOR, block_format, U8, expressed_type)
    out += struct.pack("<q", -1) + _size(0)          # axis, group size
    out += _size(0) + _size(0)                       # scales, zero points
    out += _size(len(expressed_shape))
    for d in expressed_shape:
        out += _size(d)
    return out


def write_ltnn(path, metadata, variables, version: int = 18, input_names=("tokens",), output_names=("logits",),
               trailing: bytes | None = None):
    """metadata: list of (key, kind, value); variables: list of (name, ndarray, None) for plain tensors
    or (name, uint8 payload, (block format id, expressed shape)) for block-quantised ones."""
    out = b"LTNNMDL\0" + struct.pack("<I", version)
    out += _size(0) + struct.pack("<B", 0)           # forward subgraph 0, no backward
    for names in (input_names, output_names):
        out += _size(len(names))
        for n in names:
            out += _string(n)
    out += _size(len(variables))
    out += _size(len(variables))
    for name, _, _ in variables:
        out += _string(name)
    out += _size(len(metadata))
    for key, kind, value in metadata:
        out += _string(key) + _metadata_value(kind, value)
    for _, array, quant in variables:
        out += _tensor(np.asarray(array))
        if quant is None:
            out += struct.pack("<B", 0)
        else:
            out += struct.pack("<B", 1) + _quantization(*quant)
    # activation slots, tape slots, subgraphs: empty tables stand in for the graph
    out += (_size(0) + _size(0) + _size(0)) if trailing is None else trailing
    with open(path, "wb") as f:
        f.write(out)
    return path


def llama_ltnn(path, cfg, seed, skip=(), arch="llama"):
    """The archive ImportGGUFArchive + SaveModel would give for the synthetic decoder `cfg`: GGUF
    key/values widened to Int64 / UInt64 / Float64 / String entries (tools/gguf/GGUFImporter.cpp:339-437),
    tensors as variables under their GGUF names, block-quantised ones as raw UInt8 payloads with format
    and expressed shape (:478-491)."""
    from litenn_amd import synth
    md = [
        ("general.architecture", K_STRING, arch),
        (f"{arch}.context_length", K_U64, cfg.context_length),
        (f"{arch}.embedding_length", K_U64, cfg.embedding_length),
        (f"{arch}.block_count", K_U64, cfg.block_count),
        (f"{arch}.feed_forward_length", K_U64, cfg.feed_forward_length),
        (f"{arch}.attention.head_count", K_U64, cfg.head_count),
        (f"{arch}.attention.head_count_kv", K_U64, cfg.head_count_kv),
        (f"{arch}.attention.layer_norm_rms_epsilon", K_F64, float(np.float32(cfg.rms_eps))),
        (f"{arch}.rope.freq_base", K_F64, float(np.float32(cfg.rope_freq_base))),
        ("tokenizer.ggml.tokens", K_STRING_LIST, ["<s>", "</s>", "a"]),
        ("general.file_type", K_U64, 2),
    ]
    variables = []
    for kind, layer, fmt, payload, n, k in synth.llama_tensors(cfg, seed):
        if kind in skip:
            continue
        name = f"{kind}.weight" if layer < 0 else f"blk.{layer}.{kind}.weight"
        if kind.endswith("norm"):
            variables.append((name, np.asarray(payload, np.float32).reshape(k), None))
        elif fmt == 27:
            variables.append((name, np.asarray(payload).view(np.float32).reshape(n, k), None))
        elif fmt == 25:
            variables.append((name, np.asarray(payload).view(np.float16).reshape(n, k), None))
        else:
            variables.append((name, np.asarray(payload).view(np.uint8).reshape(-1), (fmt, (n, k))))
    return write_ltnn(path, md, variables)
