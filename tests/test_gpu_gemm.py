"""Parity of the batched quantised matmul (prefill, M >= 16, matrix cores) with the CPU checker,
through the C ABI.

Tolerance: relative L2 error <= 1e-3 on the output (the bar the benchmark definition states).
The kernel rounds every dequantised weight and every activation to fp16 once and accumulates in
f32, so the expected error is about 4e-4 (two independent roundings of relative RMS 2^-11/sqrt 3);
a wrong element order, scale or sign gives errors of order 1."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, row_bytes
from litenn_amd.llama import MATMUL_PRECISE
from llama_util import hip_model, oracle_model

pytestmark = pytest.mark.gpu
TOL = 1e-3
FORMATS = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]


def last_gemm_launch():
    """The instance and grid of the calling thread's last matrix-core launch, as the library reports it."""
    import ctypes as C
    from litenn_amd._lib import check, load
    buf = C.create_string_buffer(256)
    check(load().litenn_hip_gemm_last_launch(buf, len(buf)))
    return buf.value.decode()


def run_case(hip, oracle, fmt, m, n, k, seed=0, residual=False, rows=None, flags=0):
    """rows: compare only these weight rows (they are independent), to bound the checker's time."""
    wq = synth.quant_weights(fmt, n, k, seed, 1)
    x = synth.activations(m, k, seed, 2)
    res = synth.activations(m, n, seed, 3) if residual else None
    y = hip.mul_mat_q(fmt, hip.Tensor.from_numpy(wq), n, k, hip.Tensor.from_numpy(x),
                      residual=hip.Tensor.from_numpy(res) if residual else None, flags=flags).numpy()
    assert y.shape == (m, n)
    if rows is not None:
        rb = row_bytes(fmt, k)
        sub = np.ascontiguousarray(wq.reshape(n, rb)[rows]).reshape(-1)
        ref = oracle.mul_mat_q(fmt, sub, len(rows), k, x)
        y = y[:, rows]
        if residual:
            ref = res[:, rows] + ref
    else:
        ref = oracle.mul_mat_q(fmt, wq, n, k, x)
        if residual:
            ref = res + ref
    return rel_l2(y, ref)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(16, 64, 256), (16, 256, 512), (17, 100, 256), (33, 67, 768), (64, 512, 1024),
                                   (100, 300, 2048), (133, 260, 512), (256, 1024, 256), (300, 96, 4096)])
def test_gemm_matches_checker(hip, oracle, fmt, m, n, k):
    err = run_case(hip, oracle, fmt, m, n, k, seed=m + n + k)
    assert err <= TOL, err
    assert err > 1e-6  # the fp16 path ran, not the f32 GEMV


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(4, 100, 256), (5, 999, 2048), (11, 64, 768), (15, 300, 4096)])
def test_four_to_fifteen_rows_take_the_matrix_cores(hip, oracle, fmt, m, n, k):
    """From four rows on the call pads the rows to a 16-row tile (the padding rows are zeros and are
    never stored); two and three rows go row by row through the Float32 GEMV."""
    err = run_case(hip, oracle, fmt, m, n, k, seed=m + n + k)
    assert 1e-6 < err <= TOL, err
    assert run_case(hip, oracle, fmt, m, n, k, seed=m + n + k + 1, residual=True) <= TOL
    assert run_case(hip, oracle, fmt, m, n, k, seed=m + n + k, flags=MATMUL_PRECISE) <= 1e-5
    assert run_case(hip, oracle, fmt, 3, n, k, seed=n + k) <= 1e-5


@pytest.mark.parametrize("fmt", FORMATS)
def test_gemm_residual_and_precise_flag(hip, oracle, fmt):
    assert run_case(hip, oracle, fmt, 48, 200, 512, seed=9, residual=True) <= TOL
    # the flag keeps f32 activations (GEMV path): error drops to summation-order level
    assert run_case(hip, oracle, fmt, 48, 200, 512, seed=9, flags=MATMUL_PRECISE) <= 1e-5


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(16, 999, 2048),    # one chunk per wavefront, ragged rows
                                   (23, 4100, 4096),   # two activation tiles, two chunks per wavefront
                                   (32, 777, 2048),
                                   (16, 260, 8192),    # four chunks per wavefront (where the slots fit LDS)
                                   (17, 20000, 2048)])  # runs of 80 rows: the partial products meet in several rounds
def test_streaming_form_for_few_activation_rows(hip, oracle, fmt, m, n, k):
    """Up to 32 activation rows against a single matrix whose K is a multiple of 2048 take the streaming
    form (one workgroup per CU, K cut over its eight wavefronts, partial products added in LDS);
    where its slots do not fit LDS the tiled kernel takes the shape: same bar either way."""
    rows = None
    if n > 5000:
        rows = np.sort(np.random.default_rng(n).choice(n, 640, replace=False))
        rows[0], rows[-1] = 0, n - 1
    err = run_case(hip, oracle, fmt, m, n, k, seed=m + n + k, rows=rows)
    assert 1e-6 < err <= TOL, err
    assert run_case(hip, oracle, fmt, m, n, k, seed=m + n + k + 1, residual=True, rows=rows) <= TOL


@pytest.mark.parametrize("m", [16, 64, 512])
def test_config3_q4_k_14336x4096(hip, oracle, m):
    """BASELINE config 3: K=4096, N=14336 Q4_K at full size (a 768-row sample of N is checked)."""
    rows = np.sort(np.random.default_rng(m).choice(14336, 768, replace=False))
    rows[0], rows[-1] = 0, 14335
    assert run_case(hip, oracle, Q4_K, m, 14336, 4096, seed=30 + m, rows=rows) <= TOL


@pytest.mark.parametrize("m", [16, 64, 512])
def test_config3_q6_k_4096x4096(hip, oracle, m):
    """BASELINE config 3: K=4096, N=4096 Q6_K at full size (a 768-row sample of N is checked)."""
    rows = np.sort(np.random.default_rng(m).choice(4096, 768, replace=False))
    rows[0], rows[-1] = 0, 4095
    assert run_case(hip, oracle, Q6_K, m, 4096, 4096, seed=40 + m, rows=rows) <= TOL


@pytest.mark.parametrize("fmt,n", [(Q4_K, 14336), (Q6_K, 4096)])
def test_config3_bf16_activations_at_full_size(hip, oracle, fmt, n):
    """BASELINE config 3 names fp32 and bf16 activations: M = 64, K = 4096, both matrices at full size
    with BFloat16 activations (src/LiteNN/DType.h:17-30), bit-equal to the call on their exact
    Float32 values and within the bar of the CPU checker on a 768-row sample of N."""
    from litenn_amd.formats import DT_BF16
    m, k = 64, 4096
    wq = synth.quant_weights(fmt, n, k, 50 + n % 7, 1)
    x = synth.activations(m, k, 51, 2)
    bits = ((x.view(np.uint32) + 0x8000) >> 16).astype(np.uint16)  # the nearest BFloat16 (no ties to worry about)
    wide = (bits.astype(np.uint32) << 16).view(np.float32)
    assert 1e-3 < rel_l2(wide, x) < 4e-3  # really rounded to eight bits
    w = hip.Tensor.from_numpy(wq)
    bf = hip.Tensor((m, k), DT_BF16)
    hip.DeviceTraits.CopyFromCPU(bf.device, DT_BF16, bf.ptr, DT_BF16, bits, bits.size)
    got = hip.mul_mat_q(fmt, w, n, k, bf).numpy()
    want = hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(wide)).numpy()
    assert got.shape == (m, n) and np.array_equal(got, want)
    rows = np.sort(np.random.default_rng(n).choice(n, 768, replace=False))
    rows[0], rows[-1] = 0, n - 1
    sub = np.ascontiguousarray(wq.reshape(n, row_bytes(fmt, k))[rows]).reshape(-1)
    err = rel_l2(got[:, rows], oracle.mul_mat_q(fmt, sub, len(rows), k, wide))
    print("BFloat16 activations, M=64, %d x %d: %.2e" % (n, k, err), flush=True)
    assert 1e-6 < err <= TOL


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(144, 26400, 512),    # 128-row tiles, one row group per wavefront
                                   (130, 52500, 256),    # 128-row tiles, two row groups (nibble formats)
                                   (50, 13200, 768)])    # 64-row tiles
def test_gemm_every_tile_shape(hip, oracle, fmt, m, n, k):
    """Shapes chosen so that the launcher's tile choice reaches each of its variants for every
    format (ragged in M and N, odd chunk counts); a 512-row sample of N is checked."""
    rows = np.sort(np.random.default_rng(n).choice(n, 512, replace=False))
    rows[0], rows[-1] = 0, n - 1
    assert run_case(hip, oracle, fmt, m, n, k, seed=n % 97, rows=rows, residual=(k == 512)) <= TOL


def check_k_ranges(hip, oracle, fmt, m, n, k, products):
    """One product with a workspace that has no room for K ranges and one with room for `products`
    more products: the two must differ (another summation order: the ranges ran) by no more than
    f32 summation noise, the in-place form (residual aliases y, the way the decoder calls it) must
    equal the second bit for bit, and a sample of weight rows must match the CPU checker."""
    import ctypes as C
    from litenn_amd._lib import Exec, check, load
    wq = synth.quant_weights(fmt, n, k, k % 89, 1)
    x = synth.activations(m, k, 5, 2)
    res = synth.activations(m, n, 6, 3)
    lib = load()
    w_t, x_t, r_t = hip.Tensor.from_numpy(wq), hip.Tensor.from_numpy(x), hip.Tensor.from_numpy(res)
    base = lib.litenn_hip_mul_mat_q_workspace_bytes(m, k)
    roomy = (base + 15) // 16 * 16 + 4 * m * n * products
    ws = hip.Tensor(((roomy + 3) // 4,))
    opts = Exec(None, 1)
    outs = []
    for ws_bytes in (base, roomy):
        y = hip.Tensor((m, n))
        check(lib.litenn_hip_mul_mat_q_ws(0, fmt, w_t.ptr, n, k, x_t.ptr, 0, m, y.ptr, r_t.ptr, 0, ws.ptr, ws_bytes,
                                          C.byref(opts)))
        outs.append(y.numpy())
    plain, split = outs
    import re
    assert int(re.search(r"grid \d+ x \d+ x (\d+)", last_gemm_launch()).group(1)) > 1, last_gemm_launch()  # K in ranges
    assert rel_l2(split - res, plain - res) < 1e-5
    assert not np.array_equal(split, plain)  # the ranges ran
    y = hip.Tensor.from_numpy(res)
    check(lib.litenn_hip_mul_mat_q_ws(0, fmt, w_t.ptr, n, k, x_t.ptr, 0, m, y.ptr, y.ptr, 0, ws.ptr, roomy,
                                      C.byref(opts)))
    assert np.array_equal(y.numpy(), split)
    rows = np.sort(np.random.default_rng(k).choice(n, min(n, 256), replace=False))
    rows[0], rows[-1] = 0, n - 1
    sub = np.ascontiguousarray(wq.reshape(n, row_bytes(fmt, k))[rows]).reshape(-1)
    ref = oracle.mul_mat_q(fmt, sub, len(rows), k, x)
    assert rel_l2(split[:, rows] - res[:, rows], ref) <= TOL
    # without a workspace the call takes its own room and must give the same product
    y = hip.mul_mat_q(fmt, w_t, n, k, x_t, residual=r_t).numpy()
    assert rel_l2(y - res, plain - res) < 1e-5


@pytest.mark.parametrize("fmt,k", [(Q4_0, 11008), (Q6_K, 14336), (Q4_K, 8192)])
@pytest.mark.parametrize("m", [512, 400])
def test_long_k_is_walked_in_two_halves(hip, oracle, fmt, k, m):
    """The down projections of the benchmark shapes (N = 4096, K = 11008 / 14336) at prompt sizes:
    with room for a second product in the workspace two workgroups per tile share the K walk."""
    check_k_ranges(hip, oracle, fmt, m, 4096, k, 1)


@pytest.mark.parametrize("fmt,m,n,k", [
    (Q6_K, 64, 4096, 4096),     # 64-row tiles, four ranges of four chunks: one workgroup per CU
    (Q4_K, 64, 5120, 4096),     # two ranges
    (Q4_0, 128, 4096, 11008),   # four ranges of a long K, two workgroups per CU
    (Q6_K, 256, 1024, 4096),    # k / v of a grouped-head model
    (Q4_K, 512, 4096, 4096),    # 128-row tiles, two ranges of a short K
    (Q4_0, 256, 4096, 11008),   # 128-row tiles, four ranges
    (Q5_K, 70, 4000, 4352),     # ragged rows on both sides, 17 chunks
    (Q2_K, 64, 4096, 2048),     # ranges of four chunks with the 84-byte blocks
    (Q8_0, 100, 2048, 8192)])
def test_k_ranges_on_few_weight_rows(hip, oracle, fmt, m, n, k):
    """A matrix of few rows (N = 1024 ... 5120: output, down and grouped k / v projections) gives the
    tall tiles fewer workgroups than the card has CUs; with room for three more products K is walked
    in up to four ranges at once."""
    check_k_ranges(hip, oracle, fmt, m, n, k, 3)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m,n,k", [(64, 14336, 4096),    # the benchmark's 64-row case: 224 tiles, no ranges
                                   (100, 5000, 1536),    # ragged on both sides, six chunks (three per group)
                                   (64, 5120, 4096),     # with two K ranges on top: four chunks per group
                                   (256, 4096, 2048)])   # one tile per CU, four row blocks
def test_two_groups_of_wavefronts_share_a_tile(hip, oracle, fmt, m, n, k):
    """64 x 64 output tiles that give a CU at most one workgroup are worked by eight wavefronts in two
    groups, each on half of the tile's K range, the second group's accumulators handed to the first
    through LDS.  Against the checker on a sample of weight rows, with a residual, and against the
    Float32-operand path on everything."""
    rng = np.random.default_rng(n + k)
    rows = np.sort(rng.choice(n, 192, replace=False))
    rows[0], rows[-1] = 0, n - 1
    assert run_case(hip, oracle, fmt, m, n, k, seed=7, residual=True, rows=rows) <= TOL
    wq = hip.Tensor.from_numpy(synth.quant_weights(fmt, n, k, 7, 1))
    x = hip.Tensor.from_numpy(synth.activations(m, k, 7, 2))
    exact = hip.mul_mat_q(fmt, wq, n, k, x, flags=MATMUL_PRECISE).numpy()
    got = hip.mul_mat_q(fmt, wq, n, k, x).numpy()
    launch = last_gemm_launch()
    assert rel_l2(got, exact) <= TOL
    assert float(np.abs(got - exact).max()) < 0.02 * float(np.abs(exact).max())
    # the tile this test is about ran (on a card of 256 CUs; the rule counts tiles against CUs)
    if "256 CUs" in hip.DeviceTraits.Info(hip.HIP(0)):
        assert launch.startswith("gemm_q_kernel<4, 1, 8, 2>"), launch
        assert ("x 2," in launch) == ((m, n, k) == (64, 5120, 4096)), launch  # two K ranges for that case only


@pytest.mark.parametrize("fmt", FORMATS)
def test_many_small_workgroups_share_a_cu(hip, fmt):
    """Few activation rows against a wide matrix: small tiles, several workgroups resident on every
    CU (with room for more products the K walk is also split), so LDS traffic is at its densest.
    A wavefront's weight slot must not be refilled while reads of it are still queued: no output
    may be an outlier against the f32-operand path, launch after launch."""
    for m, n, k in [(64, 4096, 4096), (32, 8192, 2048), (64, 16384, 1024)]:
        wq = hip.Tensor.from_numpy(synth.quant_weights(fmt, n, k, 3, 1))
        x = hip.Tensor.from_numpy(synth.activations(m, k, 4, 2))
        exact = hip.mul_mat_q(fmt, wq, n, k, x, flags=MATMUL_PRECISE).numpy()
        bound = 0.02 * float(np.abs(exact).max())
        for _ in range(3):
            got = hip.mul_mat_q(fmt, wq, n, k, x).numpy()
            assert rel_l2(got, exact) <= TOL
            assert float(np.abs(got - exact).max()) < bound


def test_gemm_is_linear_in_x_at_full_size(hip):
    """Size-independent property at the full north-star shape: Y(a x1 + x2) = a Y(x1) + Y(x2) up to
    the fp16 rounding of the activations."""
    n, k, m = 14336, 4096, 64
    wq = hip.Tensor.from_numpy(synth.quant_weights(Q4_K, n, k, 5, 1))
    x1, x2 = synth.activations(m, k, 5, 2), synth.activations(m, k, 5, 3)
    y = lambda x: hip.mul_mat_q(Q4_K, wq, n, k, hip.Tensor.from_numpy(x)).numpy()
    assert rel_l2(y(2.0 * x1 + x2), 2.0 * y(x1) + y(x2)) <= TOL


@pytest.mark.parametrize("fmt", [Q4_0, Q4_K, Q5_K])
def test_prefill_through_the_matrix_cores(hip, oracle, fmt):
    """The runtime's multi-row pass with fp16 matmul operands: logits stay within the matmul bar
    of the checker's f32 pass per layer (looser after three blocks), the cache matches, and decoding
    continues from it."""
    cfg = synth.tiny_llama(fmt, block_count=3, d_model=512, heads=4, kv_heads=2, ff=1024, vocab=777)
    toks = synth.prompt_tokens(cfg, 49, 2)
    ref = oracle_model(oracle, cfg, 2, kv_f16=True)
    dev = hip_model(hip, cfg, 2)
    want = ref.eval(toks[:32])
    got = dev.eval(toks[:32], precise=False)
    assert rel_l2(got, want) < 5e-3
    kd, vd = dev.get_kv(2)
    kr, vr = ref.get_kv(2)
    assert rel_l2(kd, kr) < 5e-3 and rel_l2(vd, vr) < 5e-3
    for t in toks[32:36]:
        assert rel_l2(dev.eval([t])[0], ref.eval([t])[0]) < 5e-3
    # short multi-row passes: four rows and more take the matrix cores as well (padded tile), fewer
    # go row by row through the GEMV
    for lo, hi in ((36, 40), (40, 47), (47, 49)):
        assert rel_l2(dev.eval(toks[lo:hi], precise=False), ref.eval(toks[lo:hi])) < 5e-3


@pytest.mark.parametrize("fmt,n,k", [(Q2_K, 512, 512), (Q3_K, 1024, 512), (Q6_K, 1024, 512), (Q2_K, 1024, 256),
                                     (Q2_K, 128, 2048), (Q3_K, 256, 2048), (Q6_K, 256, 4096)])  # the streaming form's
def test_weights_that_end_on_a_page_boundary(hip, oracle, fmt, n, k):
    """Blocks of 84, 110 and 210 bytes are fetched as 16-byte pieces from the boundary below them;
    no piece may lie wholly behind the tensor, where the next page need not be mapped (these
    tensors are a whole number of 4 KB pages)."""
    from litenn_amd.formats import row_bytes
    assert (n * row_bytes(fmt, k)) % 4096 == 0
    wq = synth.quant_weights(fmt, n, k, 9, 1)
    w = hip.Tensor.from_numpy(wq)
    for m in (16, 40):
        x = synth.activations(m, k, 9, m)
        y = hip.mul_mat_q(fmt, w, n, k, hip.Tensor.from_numpy(x)).numpy()
        assert rel_l2(y, oracle.mul_mat_q(fmt, wq, n, k, x)) <= 1e-3


def test_calls_without_a_workspace_queue_on_their_stream(hip, oracle):
    """Without a caller's workspace the matrix-core path takes its scratch from the device's memory
    pool in stream order: a run of calls with synchronize = 0 on one stream (different shapes, 16-bit
    activations among them, so that scratch of several sizes is taken and returned while earlier
    work is still queued) gives the same results as blocking calls."""
    from litenn_amd import hiprt
    from litenn_amd.formats import DT_F16
    stream = hiprt.Stream()
    cases = []
    for i, (fmt, m, n, k) in enumerate([(Q4_K, 16, 520, 2048), (Q6_K, 64, 300, 512), (Q4_0, 40, 1000, 1024),
                                        (Q8_0, 16, 64, 4096), (Q4_K, 130, 700, 256)] * 3):
        wq = synth.quant_weights(fmt, n, k, 70 + i, 1)
        x = synth.activations(m, k, 70 + i, 2)
        half = i % 4 == 1
        xt = hip.Tensor.from_numpy(x.astype(np.float16) if half else x)
        assert not half or xt.dtype == DT_F16
        w = hip.Tensor.from_numpy(wq)
        y = hip.mul_mat_q(fmt, w, n, k, xt, stream=stream.handle, synchronize=False)
        cases.append((fmt, wq, n, k, x.astype(np.float16).astype(np.float32) if half else x, y, w, xt))
    stream.synchronize()
    for fmt, wq, n, k, x, y, _, _ in cases:
        assert rel_l2(y.numpy(), oracle.mul_mat_q(fmt, wq, n, k, x)) <= TOL
    stream.destroy()
