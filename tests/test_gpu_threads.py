"""Every export may be called from several host threads at once (the reference runs one
read-only graph from many threads with an interpreter each, tests/ThreadSafetyTest.cpp:49-103):
concurrent calls on shared read-only weights give, bit for bit, what the same calls give alone,
and two decoder instances can generate side by side."""
import threading

import numpy as np
import pytest

from litenn_amd import synth
from litenn_amd.formats import DT_F16, Q4_K, Q6_K, Q8_0
from llama_util import hip_model

pytestmark = pytest.mark.gpu
WORKERS = 4
ROUNDS = 12


def run_workers(fn):
    errors = []

    def body(i):
        try:
            fn(i)
        except Exception as e:  # reported in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=body, args=(i,)) for i in range(WORKERS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors


def test_concurrent_operator_calls_on_shared_weights(hip):
    rng = np.random.default_rng(21)
    n, k = 1024, 2048
    weights = {fmt: hip.Tensor.from_numpy(synth.quant_weights(fmt, n, k, fmt)) for fmt in (Q4_K, Q6_K, Q8_0)}
    norm_w = hip.Tensor.from_numpy(rng.standard_normal(k).astype(np.float32))
    inputs = [[rng.standard_normal((m, k)).astype(np.float32) for m in (1, 3, 32)] for _ in range(WORKERS)]

    def work(i):
        out = []
        for x in inputs[i]:
            tx = hip.Tensor.from_numpy(x)
            out.append(hip.rmsnorm(tx, norm_w, 1e-5).numpy())
            for fmt, w in weights.items():
                out.append(hip.mul_mat_q(fmt, w, n, k, tx).numpy())
        return out

    alone = [work(i) for i in range(WORKERS)]

    def worker(i):
        for r in range(ROUNDS):
            got = work(i)
            for j, (g, a) in enumerate(zip(got, alone[i])):
                assert np.array_equal(g, a), (i, r, j)

    run_workers(worker)


def test_errors_stay_with_the_thread_that_made_them(hip):
    from litenn_amd import LiteNNHipError
    x = hip.Tensor.from_numpy(np.zeros((1, 100), np.float32))
    w = hip.Tensor.from_numpy(np.zeros(4 * 144, np.uint8))
    good_x = hip.Tensor.from_numpy(np.ones((1, 256), np.float32))

    def worker(i):
        for _ in range(50):
            if i % 2:
                with pytest.raises(LiteNNHipError, match="block size"):
                    hip.mul_mat_q(Q4_K, w, 4, 100, x)
            else:
                assert hip.mul_mat_q(Q4_K, w, 4, 256, good_x).numpy().shape == (1, 4)

    run_workers(worker)


def test_two_decoders_generate_side_by_side(hip):
    cfg = synth.tiny_llama(Q4_K, block_count=2, d_model=512, heads=4, kv_heads=2, ff=1024, vocab=500)
    prompts = [synth.prompt_tokens(cfg, 12, seed) for seed in range(WORKERS)]
    alone = []
    for i in range(WORKERS):
        m = hip_model(hip, cfg, 30 + i % 2, kv_dtype=DT_F16)
        alone.append(m.generate(prompts[i], 24)[0])

    def worker(i):
        m = hip_model(hip, cfg, 30 + i % 2, kv_dtype=DT_F16)
        for r in range(3):
            m.reset()
            tokens = m.generate(prompts[i], 24)[0]
            assert np.array_equal(tokens, alone[i]), (i, r)

    run_workers(worker)
