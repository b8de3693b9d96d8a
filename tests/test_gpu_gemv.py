"""Parity of the quantised GEMV (through the C ABI) with the CPU checker.

Tolerance: relative L2 error <= 1e-3 on matmul outputs with f32 accumulation (the bar the
benchmark definition states); the measured error is ~1e-6 because only the summation order and
the factoring of per-block scales differ."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import F16, F32, Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, row_bytes

pytestmark = pytest.mark.gpu
TOL = 1e-3
FORMATS = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]


def run_case(hip, oracle, fmt, n, k, m=1, seed=0, residual=False, flags=0):
    wq = synth.quant_weights(fmt, n, k, seed, 1)
    x = synth.activations(m, k, seed, 2)
    res = synth.activations(m, n, seed, 3) if residual else None
    y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x),
                      residual=hip.Tensor.from_numpy(res) if residual else None, flags=flags).numpy()
    ref = oracle.mul_mat_q(fmt, wq, n, k, x)
    if residual:
        ref = res + ref
    assert y.shape == (m, n)
    return rel_l2(y, ref)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("n,k", [(64, 256), (100, 4096), (33, 11008), (17, 14336), (256, 8192), (5, 32768)])
def test_gemv_matches_checker(hip, oracle, fmt, n, k):
    assert run_case(hip, oracle, fmt, n, k, seed=n + k) <= TOL


def test_config1_q8_0_4096x4096(hip, oracle):
    """BASELINE config 1 at full size."""
    assert run_case(hip, oracle, Q8_0, 4096, 4096, seed=1) <= TOL


@pytest.mark.parametrize("fmt", [Q4_0, Q4_K])
@pytest.mark.parametrize("n,k", [(11008, 4096), (4096, 11008)])
def test_config2_ffn_shapes(hip, oracle, fmt, n, k):
    """BASELINE config 2 at full size."""
    assert run_case(hip, oracle, fmt, n, k, seed=2) <= TOL


def test_north_star_shape_q4_k_4096x14336(hip, oracle):
    assert run_case(hip, oracle, Q4_K, 14336, 4096, seed=3) <= TOL
    assert run_case(hip, oracle, Q6_K, 4096, 14336, seed=4) <= TOL


@pytest.mark.parametrize("fmt", FORMATS)
def test_ragged_shapes_take_the_generic_kernel(hip, oracle, fmt):
    """K not a multiple of 256 (single blocks, odd block counts) and tiny N."""
    for n, k in [(1, 32), (3, 96), (7, 32 * 37)] if fmt in (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0) else [(1, 256), (3, 768)]:
        assert run_case(hip, oracle, fmt, n, k, seed=k) <= TOL


@pytest.mark.parametrize("fmt", FORMATS)
def test_small_batches_and_residual(hip, oracle, fmt):
    assert run_case(hip, oracle, fmt, 96, 1024, m=5, seed=9) <= TOL
    assert run_case(hip, oracle, fmt, 96, 4096, m=2, seed=10, residual=True) <= TOL


def test_plain_float_weights(hip, oracle):
    rng = np.random.default_rng(0)
    w = rng.standard_normal((48, 300)).astype(np.float32)
    x = rng.standard_normal((2, 300)).astype(np.float32)
    for fmt, payload in ((F32, w), (F16, w.astype(np.float16))):
        y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(payload.view(np.uint8).reshape(-1)), 48, 300,
                          hip.Tensor.from_numpy(x)).numpy()
        assert rel_l2(y, oracle.mul_mat_q(fmt, payload, 48, 300, x)) <= 1e-5


def test_linearity_and_one_hot_at_full_size(hip):
    """Size-independent properties at the north-star shape: W.e_k reproduces column k of the
    dequantised weight, and W.(a x1 + b x2) = a W.x1 + b W.x2."""
    n, k = 14336, 4096
    wq = synth.quant_weights(Q4_K, n, k, 11)
    wt = hip.Tensor.from_numpy(wq)
    deq = hip.dequantize(Q4_K, wt, n, k).numpy()
    for col in (0, 77, 4095):
        e = np.zeros((1, k), np.float32)
        e[0, col] = 1.0
        y = hip.mul_mat_q(Q4_K, wt, n, k, hip.Tensor.from_numpy(e)).numpy()[0]
        assert np.allclose(y, deq[:, col], rtol=1e-6, atol=1e-6)
    x1, x2 = synth.activations(1, k, 12), synth.activations(1, k, 13)
    f = lambda v: hip.mul_mat_q(Q4_K, wt, n, k, hip.Tensor.from_numpy(v)).numpy().astype(np.float64)
    assert rel_l2(f(2.0 * x1 - 0.5 * x2), 2.0 * f(x1) - 0.5 * f(x2)) < 1e-5


@pytest.mark.parametrize("fmt", FORMATS)
def test_device_dequantize_is_bit_exact(hip, oracle, fmt):
    wq = synth.quant_weights(fmt, 9, 1024, 21)
    got = hip.dequantize(fmt, hip.Tensor.from_numpy(wq), 9, 1024).numpy()
    want = oracle.dequantize(fmt, wq, 9, 1024)
    if fmt in (Q4_0, Q8_0):
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    else:  # d*sc*q - dmin*m may contract into an fma on the device
        assert np.allclose(got, want, rtol=1e-6, atol=1e-7)


def test_get_rows_q_and_range_check(hip, oracle):
    wq = synth.quant_weights(Q4_0, 50, 256, 5)
    ids = np.array([49, 0, 7, 7], np.int32)
    got = hip.get_rows_q(Q4_0, hip.Tensor.from_numpy(wq), 50, 256, hip.Tensor.from_numpy(ids)).numpy()
    assert np.array_equal(got, oracle.dequantize(Q4_0, wq, 50, 256)[ids])
    with pytest.raises(hip.LiteNNHipError, match="GetRows index out of range"):
        hip.get_rows_q(Q4_0, hip.Tensor.from_numpy(wq), 50, 256, hip.Tensor.from_numpy(np.array([50], np.int32)))


def test_errors_and_empty_inputs(hip):
    wq = hip.Tensor.from_numpy(np.zeros(144, np.uint8))
    x = hip.Tensor.from_numpy(np.zeros((1, 256), np.float32))
    with pytest.raises(hip.LiteNNHipError, match="payload size"):
        hip.mul_mat_q(Q4_K, wq, 2, 256, x)
    with pytest.raises(hip.LiteNNHipError, match="unsupported block format"):
        hip.mul_mat_q(6, wq, 1, 256, x)  # Q8_1: no dequantizer
    with pytest.raises(hip.LiteNNHipError, match="block size"):
        hip.mul_mat_q(Q4_K, wq, 1, 128, x)
    empty = hip.mul_mat_q(Q4_K, hip.Tensor.from_numpy(np.zeros(0, np.uint8)), 0, 256, x)
    assert empty.shape == (1, 0)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("k,ns", [(4096, (4096, 1024, 1024)), (4096, (256, 256, 256)), (11008, (96,)), (512, (40, 24))])
def test_linear_group_norm_and_concat(hip, oracle, fmt, k, ns):
    """RMSNorm folded into up to three projections that share the input (the q/k/v group)."""
    ws = [synth.quant_weights(fmt, n, k, 31, i) for i, n in enumerate(ns)]
    x = synth.activations(1, k, 32) * 3.0
    nw = (1.0 + 0.1 * synth.activations(1, k, 33)).reshape(-1)
    eps = float(np.float32(1e-5))
    outs = hip.linear_group(fmt, [hip.Tensor.from_numpy(w) for w in ws], list(ns), k, hip.Tensor.from_numpy(x),
                            norm_w=hip.Tensor.from_numpy(nw), eps=eps)
    xn = oracle.rmsnorm(x, nw, eps)
    for w, n, out in zip(ws, ns, outs):
        assert rel_l2(out.numpy(), oracle.mul_mat_q(fmt, w, n, k, xn)) <= TOL
    # without the norm
    outs = hip.linear_group(fmt, [hip.Tensor.from_numpy(w) for w in ws], list(ns), k, hip.Tensor.from_numpy(x))
    for w, n, out in zip(ws, ns, outs):
        assert rel_l2(out.numpy(), oracle.mul_mat_q(fmt, w, n, k, x)) <= TOL


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("n,k", [(11008, 4096), (14336, 4096), (300, 8192), (50, 512)])
def test_linear_group_swiglu(hip, oracle, fmt, n, k):
    """RMSNorm -> gate/up -> silu(gate) * up in one launch (front half of the SwiGLU MLP)."""
    wg, wu = synth.quant_weights(fmt, n, k, 41, 0), synth.quant_weights(fmt, n, k, 41, 1)
    x = synth.activations(1, k, 42)
    nw = np.ones(k, np.float32)
    eps = float(np.float32(1e-5))
    out, = hip.linear_group(fmt, [hip.Tensor.from_numpy(wg), hip.Tensor.from_numpy(wu)], [n, n], k,
                            hip.Tensor.from_numpy(x), norm_w=hip.Tensor.from_numpy(nw), eps=eps, silu_mul=True)
    xn = oracle.rmsnorm(x, nw, eps)
    want = oracle.silu_mul(oracle.mul_mat_q(fmt, wg, n, k, xn), oracle.mul_mat_q(fmt, wu, n, k, xn))
    assert rel_l2(out.numpy(), want) <= TOL


def test_linear_group_residual_and_errors(hip, oracle):
    n, k = 4096, 11008
    w = synth.quant_weights(Q4_0, n, k, 51)
    x = synth.activations(1, k, 52)
    res = synth.activations(1, n, 53)
    out, = hip.linear_group(Q4_0, [hip.Tensor.from_numpy(w)], [n], k, hip.Tensor.from_numpy(x),
                            residual=hip.Tensor.from_numpy(res))
    assert rel_l2(out.numpy(), res + oracle.mul_mat_q(Q4_0, w, n, k, x)) <= TOL
    wt = hip.Tensor.from_numpy(w)
    with pytest.raises(hip.LiteNNHipError, match="equal height"):
        hip.linear_group(Q4_0, [wt, wt, wt], [n, n, n], k, hip.Tensor.from_numpy(x), silu_mul=True)
    with pytest.raises(hip.LiteNNHipError, match="single matrix"):
        hip.linear_group(Q4_0, [wt, wt], [n, n], k, hip.Tensor.from_numpy(x), residual=hip.Tensor.from_numpy(res))


@pytest.mark.parametrize("fmt,n", [(Q6_K, 128256), (Q4_0, 32000)])
def test_lm_head_shapes(hip, oracle, fmt, n):
    """The vocabulary projections of BASELINE configs 5 and 4 at full size (431 MB / 74 MB)."""
    assert run_case(hip, oracle, fmt, n, 4096, seed=n) <= TOL


def test_gemv_properties_at_full_size(hip):
    """Size-independent checks at the north-star shape: linearity in x, and y(e_k) = column k of the
    dequantised matrix (so y over all one-hot inputs of a block reproduces litenn_hip_dequantize)."""
    n, k = 14336, 4096
    wq = hip.Tensor.from_numpy(synth.quant_weights(Q4_K, n, k, 8, 1))
    y = lambda x: hip.mul_mat_q(Q4_K, wq, n, k, hip.Tensor.from_numpy(np.ascontiguousarray(x, np.float32))).numpy()
    x1, x2 = synth.activations(1, k, 8, 2), synth.activations(1, k, 8, 3)
    assert rel_l2(y(3.0 * x1 - x2), 3.0 * y(x1) - y(x2)) <= 1e-5
    deq = hip.dequantize(Q4_K, wq, n, k).numpy()
    for col in (0, 31, 32, 255, 256, 4095):
        e = np.zeros((1, k), np.float32)
        e[0, col] = 1.0
        assert np.array_equal(y(e)[0], deq[:, col]), col
    # all-ones input: row sums (f32 summation order differs: tolerance, not equality)
    assert rel_l2(y(np.ones((1, k), np.float32))[0], deq.astype(np.float64).sum(axis=1).astype(np.float32)) <= 1e-5


@pytest.mark.parametrize("fmt", [Q4_K, Q6_K, Q8_0])
@pytest.mark.parametrize("m", [1, 3, 32])
def test_sixteen_bit_activations_are_widened_exactly(hip, oracle, fmt, m):
    """Float16 / BFloat16 activations give what their exact Float32 values give."""
    from litenn_amd.formats import DT_BF16
    n, k = 96, 1024
    wq = synth.quant_weights(fmt, n, k, 5, 1)
    x = synth.activations(m, k, 5, 2)
    w = hip.Tensor.from_numpy(wq)
    half = x.astype(np.float16)
    want = hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(half.astype(np.float32))).numpy()
    got = hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(half)).numpy()
    assert np.array_equal(got, want)
    assert rel_l2(got, oracle.mul_mat_q(fmt, wq, n, k, half.astype(np.float32))) <= TOL
    bits = (x.view(np.uint32) >> 16).astype(np.uint16)  # BFloat16 by truncation: exactly representable
    bf = hip.Tensor((m, k), DT_BF16)
    hip.DeviceTraits.CopyFromCPU(bf.device, DT_BF16, bf.ptr, DT_BF16, bits, bits.size)
    wide = (bits.astype(np.uint32) << 16).view(np.float32)
    want = hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(wide)).numpy()
    assert np.array_equal(hip.mul_mat_q(fmt, w, n, k, bf).numpy(), want)
    with pytest.raises(hip.LiteNNHipError, match="Float32, Float16 or BFloat16"):
        hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(np.zeros((1, k), np.float64)))
