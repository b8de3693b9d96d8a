"""The ggml block formats that run through the per-element kernels (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K,
Q5_K; src/LiteNN/Quantization.h:31-62,186-217): dequantise, row gather, matmul for one row and for
several, and a decoder whose tensors use them, against the CPU checker through the C ABI.

Tolerances: dequantised values and gathered rows bit for bit (the decoders are written with the
same separately rounded steps); matmul rel-L2 <= 1e-3 (only the summation order differs, measured
~1e-6); greedy tokens exact."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q2_K, Q3_K, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, row_bytes
from llama_util import hip_model, oracle_model

pytestmark = pytest.mark.gpu
FORMATS = [Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K]


@pytest.mark.parametrize("fmt", FORMATS)
def test_dequantize_and_get_rows_bitwise(hip, oracle, fmt):
    rows, k = 37, 1024
    raw = synth.quant_weights(fmt, rows, k, 7, fmt)
    want = oracle.dequantize(fmt, raw, rows, k)
    got = hip.dequantize(fmt, hip.Tensor.from_numpy(raw), rows, k).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # every field uniformly random (NaN scale patterns included)
    rnd = np.random.default_rng(fmt).integers(0, 256, size=(rows, row_bytes(fmt, k)), dtype=np.uint8)
    want = oracle.dequantize(fmt, rnd, rows, k)
    got = hip.dequantize(fmt, hip.Tensor.from_numpy(rnd), rows, k).numpy()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    ids = np.array([36, 0, 5, 5, 17], np.int32)
    picked = hip.get_rows_q(fmt, hip.Tensor.from_numpy(raw), rows, k, hip.Tensor.from_numpy(ids)).numpy()
    assert np.array_equal(picked, oracle.dequantize(fmt, raw, rows, k)[ids])


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(1, 64, 256), (1, 100, 4096), (1, 4096, 4096), (3, 33, 11008), (20, 70, 512)])
def test_matmul_matches_checker(hip, oracle, fmt, m, n, k):
    wq = synth.quant_weights(fmt, n, k, n + k, 1)
    x = synth.activations(m, k, n + k, 2)
    res = synth.activations(m, n, n + k, 3)
    y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x),
                      residual=hip.Tensor.from_numpy(res)).numpy()
    assert rel_l2(y, res + oracle.mul_mat_q(fmt, wq, n, k, x)) <= 1e-3


def test_small_blocks_ragged_rows(hip, oracle):
    """32-element formats at widths that are not multiples of 256."""
    for fmt in (Q4_1, Q5_0, Q5_1):
        for n, k in ((1, 32), (3, 96), (7, 32 * 37)):
            wq = synth.quant_weights(fmt, n, k, k, 1)
            x = synth.activations(1, k, k, 2)
            y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x)).numpy()
            assert rel_l2(y, oracle.mul_mat_q(fmt, wq, n, k, x)) <= 1e-3


def test_q8_1_and_q8_k_are_refused(hip):
    """ggml has no dequantizer for them; the reference's lowering refuses such tensors
    (tools/gguf/LLaMABuilder.cpp:95-101)."""
    for fmt, nbytes, k in ((6, 40, 32), (12, 292, 256)):
        with pytest.raises(hip.LiteNNHipError, match="unsupported block format"):
            hip.dequantize(fmt, hip.Tensor.from_numpy(np.zeros(nbytes, np.uint8)), 1, k)


def test_decoder_with_mixed_formats(hip, oracle, tmp_path):
    """A Q5_K_M-like mix (Q5_K projections, Q6_K value / down projections, Q4_1 embedding, Q5_0
    head): logits against the CPU checker, greedy tokens exact with healthy margins, and the same
    model through a GGUF file."""
    import gguf_writer as gw
    cfg = synth.tiny_llama(Q5_K, block_count=2, d_model=512, heads=4, kv_heads=2, ff=768, vocab=288, context_length=48,
                           formats={"default": Q5_K, "attn_v": Q6_K, "ffn_down": Q6_K, "attn_k": Q3_K, "ffn_up": Q2_K,
                                    "attn_output": Q5_1, "token_embd": Q4_1, "output": Q5_0})
    toks = synth.prompt_tokens(cfg, 9, 4)
    dev, ref = hip_model(hip, cfg, 17), oracle_model(oracle, cfg, 17)
    assert rel_l2(dev.eval(toks), ref.eval(toks)) < 1e-4
    dev.reset()
    ref.reset()
    want, margins = ref.generate(toks, 8)
    got, _, _ = dev.generate(toks, 8)
    assert got.tolist() == want.tolist()
    loaded = hip.LLaMA.from_gguf(str(gw.llama_gguf(tmp_path / "mix.gguf", cfg, 17)))
    dev.reset()
    assert np.array_equal(loaded.eval(toks), dev.eval(toks))
    loaded.close()
    dev.close()
