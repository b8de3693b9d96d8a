"""Randomised differential test of litenn_hip_mul_mat_q against the CPU checker: formats, ragged row
counts, every number of activation rows around the thresholds between its kernels (single-row GEMV,
row-by-row GEMV below 4 rows, streaming and tiled matrix-core forms), K from one chunk to 8192,
residual on or off, 16-bit activations now and then.  Seeds are fixed, so a failure names its case;
the address arithmetic of every fetch pattern these shapes reach is walked on the host for whole
launches by tests/cpp/fetch_bounds_test.cpp, which is where an over-fetch would be found first."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, block_layout, row_bytes
from litenn_amd.llama import MATMUL_PRECISE

pytestmark = pytest.mark.gpu
FORMATS = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]


def draw_case(seed):
    rng = np.random.default_rng(1000 + seed)
    fmt = FORMATS[seed % len(FORMATS)]
    k = int(rng.choice([256, 512, 768, 1024, 2048, 2304, 4096, 6144, 8192]))
    m = int(rng.choice([1, 2, 3, 4, 5, 7, 15, 16, 17, 24, 31, 32, 33, 40, 64, 100]))
    n = int(rng.choice([1, 5, 16, 31, 100, 257, 1000, 2051, 4100]))
    if k >= 4096 and m >= 33:
        n = min(n, 1000)  # bounds the checker's time
    return fmt, m, n, k, bool(rng.integers(2)), bool(rng.integers(4) == 0), bool(rng.integers(5) == 0)


@pytest.mark.parametrize("seed", range(60))
def test_random_matmul_matches_checker(hip, oracle, seed):
    fmt, m, n, k, residual, half_x, precise = draw_case(seed)
    what = f"seed {seed}: format {fmt} m {m} n {n} k {k} residual {residual} half {half_x} precise {precise}"
    print(what, flush=True)
    assert k % block_layout(fmt)[0] == 0 and row_bytes(fmt, k) > 0
    wq = synth.quant_weights(fmt, n, k, seed, 1)
    x = synth.activations(m, k, seed, 2)
    if half_x:
        x = x.astype(np.float16).astype(np.float32)
    res = synth.activations(m, n, seed, 3) if residual else None
    xt = hip.Tensor.from_numpy(x.astype(np.float16) if half_x else x)
    y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, xt,
                      residual=hip.Tensor.from_numpy(res) if residual else None,
                      flags=MATMUL_PRECISE if precise else 0).numpy()
    want = oracle.mul_mat_q(fmt, wq, n, k, x)
    if residual:
        want = res + want
    err = rel_l2(y, want)
    print("  rel-L2 %.2e" % err, flush=True)
    # f32 operands (fewer than 4 rows, a K that is no whole number of 256-element chunks, or the flag):
    # summation order only; matrix cores: the stated bar for Float16 operands
    assert err <= (1e-5 if (m < 4 or precise) else 1e-3), what


def draw_tile_case(seed):
    """Shapes on both sides of the tile rules of the tiled matrix-core form: 64 and 128-row tiles, one or
    two weight groups, two groups of wavefronts per tile, K walked in one, two or four ranges."""
    rng = np.random.default_rng(5000 + seed)
    fmt = FORMATS[seed % len(FORMATS)]
    k = int(rng.choice([1024, 1536, 2048, 4096, 4352, 8192, 11008]))
    m = int(rng.choice([49, 64, 65, 96, 128, 130, 192, 256, 300, 512, 600]))
    n = int(rng.choice([1024, 2048, 4096, 5120, 8192, 12288, 14336, 22016, 4100, 13000]))
    if m * n * k > 512 * 14336 * 4096:
        n = 4096
    return fmt, m, n, k, bool(rng.integers(2))


@pytest.mark.parametrize("seed", range(40))
def test_random_tiles_match_the_float32_path(hip, seed):
    """The matrix-core product against the device's own Float32-operand path (held to the CPU checker by
    the tests above), so that large shapes stay cheap: within the Float16-operand bar overall and with no
    outlier element, with and without a residual."""
    fmt, m, n, k, residual = draw_tile_case(seed)
    what = f"seed {seed}: format {fmt} m {m} n {n} k {k} residual {residual}"
    print(what, flush=True)
    wq = hip.Tensor.from_numpy(synth.quant_weights(fmt, n, k, seed, 1))
    x = hip.Tensor.from_numpy(synth.activations(m, k, seed, 2))
    res = hip.Tensor.from_numpy(synth.activations(m, n, seed, 3)) if residual else None
    exact = hip.mul_mat_q(fmt, wq, n, k, x, residual=res, flags=MATMUL_PRECISE).numpy()
    got = hip.mul_mat_q(fmt, wq, n, k, x, residual=res).numpy()
    import ctypes as C
    from litenn_amd._lib import check, load
    buf = C.create_string_buffer(256)
    check(load().litenn_hip_gemm_last_launch(buf, len(buf)))
    print("  " + buf.value.decode(), flush=True)
    assert rel_l2(got, exact) <= 1e-3, what
    assert float(np.abs(got - exact).max()) < 0.02 * float(np.abs(exact).max()), what
