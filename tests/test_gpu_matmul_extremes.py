"""The quantised matmul on activations far from unit scale, through the C ABI, against the CPU
checker: rows of very large and very small magnitude, an outlier inside a row, rows of zeros, and
non-finite values.  The reference path is plain f32 arithmetic (src/LiteNN/Device.h:645-658), so a
row's scale must not matter beyond f32's own range; the matrix-core path rounds activations to
Float16 after scaling each row by a power of two, which these cases are aimed at."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q4_0, Q4_K, Q6_K, Q8_0

pytestmark = pytest.mark.gpu
FORMATS = [Q4_0, Q8_0, Q4_K, Q6_K]


def _rows_rel_l2(got, want):
    return np.array([rel_l2(got[i], want[i]) for i in range(got.shape[0])])


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [1, 16, 40])
def test_row_scale_does_not_matter(hip, oracle, fmt, m):
    """Each row carries its own magnitude, 1e-30 to 1e30: every row is held to the bar on its own
    (a whole-matrix norm would hide the small rows).  m = 1 takes the f32 GEMV, 16 the streaming
    matrix-core form, 40 the tiled one."""
    n, k = 192, 1024
    wq = synth.quant_weights(fmt, n, k, 3, 1)
    x = synth.activations(m, k, 4, 2)
    scales = np.array([1e-30, 1e-12, 1e-4, 1.0, 37.0, 1e6, 1e19, 1e30], np.float32)
    x *= scales[np.arange(m) % len(scales), None]
    got = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x)).numpy()
    want = oracle.mul_mat_q(fmt, wq, n, k, x)
    assert np.all(np.isfinite(got))
    err = _rows_rel_l2(got, want)
    assert err.max() <= (1e-5 if m == 1 else 1e-3), err


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [1, 16, 40])
def test_outlier_zero_rows_and_sign(hip, oracle, fmt, m):
    n, k = 160, 768
    wq = synth.quant_weights(fmt, n, k, 5, 1)
    x = synth.activations(m, k, 6, 2)
    x[0, 17] = 3.0e4        # one feature three thousand times the rest: small ones keep >= 10 bits below it
    if m > 1:
        x[1] = 0.0          # a row of zeros gives zeros
        x[2] = -x[3]        # negation commutes with the product (up to the matrix cores' own accumulation)
    got = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x)).numpy()
    want = oracle.mul_mat_q(fmt, wq, n, k, x)
    assert rel_l2(got[0], want[0]) <= (1e-5 if m == 1 else 1e-3)
    if m > 1:
        assert np.all(got[1] == 0.0)
        assert rel_l2(got[2], -got[3]) <= 1e-5
        assert _rows_rel_l2(got[2:], want[2:]).max() <= 1e-3


@pytest.mark.parametrize("fmt", [Q4_0, Q4_K])
@pytest.mark.parametrize("m", [1, 16, 40])
def test_non_finite_activations_stay_in_their_rows(hip, oracle, fmt, m):
    """An infinity or a NaN in one row makes that row's products non-finite, as in the reference's
    f32 loop, and leaves every other row as it was."""
    n, k = 128, 512
    wq = synth.quant_weights(fmt, n, k, 7, 1)
    x = synth.activations(m, k, 8, 2)
    clean = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x)).numpy()
    bad = x.copy()
    bad[0, 5] = np.inf
    if m > 1:
        bad[m - 1, 300] = np.nan
    got = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(bad)).numpy()
    want = oracle.mul_mat_q(fmt, wq, n, k, bad)
    # (a zero weight times infinity is NaN, any other weight gives an infinity: neither is finite)
    assert not np.any(np.isfinite(want[0]))
    assert np.array_equal(np.isfinite(got[0]), np.isfinite(want[0]))
    if m > 1:
        assert np.all(np.isnan(got[m - 1])) and np.all(np.isnan(want[m - 1]))
        assert np.array_equal(got[1:m - 1], clean[1:m - 1])


@pytest.mark.parametrize("fmt", FORMATS)
def test_decoder_group_on_scaled_activations(hip, oracle, fmt):
    """RMSNorm in front of the matrices takes the scale out again: the fused group launch on a row
    of magnitude 1e20 agrees with the checker's norm followed by its matmul."""
    n, k = 256, 1024
    wq = synth.quant_weights(fmt, n, k, 9, 1)
    x = synth.activations(1, k, 10, 2) * np.float32(1e20)
    w = synth.norm_weights(k, 11)
    eps = float(np.float32(1e-5))
    got = hip.linear_group(fmt, [hip.Tensor.from_numpy(wq)], [n], k, hip.Tensor.from_numpy(x),
                           norm_w=hip.Tensor.from_numpy(w), eps=eps)[0].numpy()
    want = oracle.mul_mat_q(fmt, wq, n, k, oracle.rmsnorm(x, w, eps))
    assert rel_l2(got, want) <= 1e-5
