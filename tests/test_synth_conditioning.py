"""Why the synthetic decoder models draw their scales the way litenn_amd.synth.model_weights does
(CPU only, numpy float64 through tests/np_llama.py).

With the law of the single-matrix benchmarks (positive scales |N(0,1)| * 0.02, uniform codes) a
decoder's attention scores reach the thousands and the softmax is a hard maximum.  The matrix-core
prompt path rounds q / sqrt(d) and the keys to Float16 (two roundings of relative 2^-11 / sqrt(3)
each, about 3e-4 of a score): where the two best keys of a row score within a few times that
distance of each other the mixture of values the row receives changes by a large factor, and
the row's logits differ by several per cent although nothing is wrong.  That is what a randomised
comparison once showed for one row of one model (768 wide, 8 query heads on one KV head of 96,
Q8_0, second of seven rows after the prompt): reproduced here from the shape.  With model_weights
the scores are of order one and the same rounding moves a softmax weight by a fraction of a per
cent, so the comparisons of the decoder tests can hold every row to one bar."""
import numpy as np

from litenn_amd import synth
from litenn_amd.formats import F32, Q8_0
from np_llama import NumpyLLaMA

HALF_OPERANDS = 3e-4  # relative perturbation of a score with Float16 q and k (two roundings of 2^-11 / sqrt(3))


def _old_law_tensors(cfg, seed):
    shapes = cfg.tensor_shapes()
    ones = np.ones(cfg.embedding_length, np.float32)
    for kind_id, kind in enumerate(("token_embd", "output")):
        n, k = shapes[kind]
        yield kind, -1, cfg.fmt(kind), synth.quant_weights(cfg.fmt(kind), n, k, seed, 1000 + kind_id), n, k
    yield "output_norm", -1, F32, ones, 1, cfg.embedding_length
    for layer in range(cfg.block_count):
        for kind_id, kind in enumerate(synth.TENSOR_KINDS):
            n, k = shapes[kind]
            yield kind, layer, cfg.fmt(kind), synth.quant_weights(cfg.fmt(kind), n, k, seed, layer, kind_id), n, k
        yield "attn_norm", layer, F32, ones, 1, cfg.embedding_length
        yield "ffn_norm", layer, F32, ones, 1, cfg.embedding_length


def _top2(model, tokens):
    """[(layer, head, row, best score, runner-up)] for every row that sees at least two keys."""
    model.trace = []
    model.eval(tokens)
    out = []
    for layer, head, scores in model.trace:
        for row in range(scores.shape[0]):
            s = np.sort(scores[row][np.isfinite(scores[row])])
            if s.size >= 2:
                out.append((layer, head, row, float(s[-1]), float(s[-2])))
    return out


def test_positive_scales_saturate_the_softmax_and_signed_normalised_scales_do_not():
    cfg = synth.tiny_llama(Q8_0, block_count=2, d_model=768, heads=8, kv_heads=1, ff=1280, vocab=663, context_length=96)
    cfg.rope_dimension_count = 16
    toks = synth.prompt_tokens(cfg, 10, 39)[:9]
    old = _top2(NumpyLLaMA(cfg, list(_old_law_tensors(cfg, 39))), toks)
    new = _top2(NumpyLLaMA(cfg, list(synth.llama_tensors(cfg, 39))), toks)
    # old law: scores in the thousands; some row has its two best keys closer than a few times what
    # Float16 operands move a score by, so its softmax weights move by a factor, not a fraction
    assert max(abs(b) for *_, b, _ in old) > 1000.0
    close = [(l, h, r, b, s) for l, h, r, b, s in old if b - s < 3.0 * HALF_OPERANDS * abs(b)]
    assert close, "expected a near-tie under the saturated law"
    assert any(r == 6 for _, _, r, _, _ in close)  # the row the randomised comparison singled out
    # new law: scores of order one, so the rounding moves an exponent by about 1e-3 at most
    assert max(abs(b) for *_, b, _ in new) < 20.0
    assert max(HALF_OPERANDS * abs(b) for *_, b, _ in new) < 1e-2


def test_model_weights_have_unit_gain_in_every_format():
    """A dequantised decoder matrix has entries of rms 1/sqrt(k) whatever its block format, and no
    common offset (the rank-one part that made greedy decoding repeat one token)."""
    import np_decoders
    from litenn_amd.formats import Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K
    for fmt in (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K):
        n, k = 192, 1024
        w = np_decoders.decode(fmt, synth.model_weights(fmt, n, k, 3, fmt), k).astype(np.float64)
        rms = float(np.sqrt(np.mean(w * w)))
        assert 0.85 / np.sqrt(k) < rms < 1.15 / np.sqrt(k), (fmt, rms * np.sqrt(k))
        assert abs(float(w.mean())) < 0.05 * rms, (fmt, w.mean() / rms)
