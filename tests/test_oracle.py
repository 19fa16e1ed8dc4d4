"""Pins the CPU oracle (oracle/host_matmul.c) without retyping its formula in C: closed forms,
brute force in pure Python with explicit fp32 rounding, an independent library (numpy float64), and
invariants chosen so that a dropped term, a transposed operand or a wrong stride fails one of them.
The reference ships no golden vectors for this path (it has no test-suite at all)."""
import numpy as np
import pytest

from codegendemo_amd.kcg import SeededInputs as SI


def brute_force_f32(a_mk, b_kn):
    """Matmul.cc:41-65 spelled out: acc = 0; ascending k: acc = fl32(acc + fl32(a*b))."""
    M, K = a_mk.shape
    _, N = b_kn.shape
    c = np.zeros((M, N), np.float32)
    for i in range(M):
        for j in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + np.float32(a_mk[i, k] * b_kn[k, j]))
            c[i, j] = acc
    return c


SHAPES = [(1, 1, 1), (8, 8, 8), (13, 7, 5), (5, 9, 16), (16, 3, 33)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("a_trans", [0, 1])
def test_brute_force_tiny(oracle, M, N, K, a_trans):
    a = SI.uniform((M, K), 11)
    b = SI.uniform((K, N), 12)
    want = brute_force_f32(a, b)
    a_buf = SI.a_operand(a, a_trans)
    assert np.array_equal(oracle.ijk(a_buf, b, a_trans), want)
    assert np.array_equal(oracle.matmul(a_buf, b, a_trans), want)
    assert np.array_equal(oracle.matmul(a_buf, b, a_trans, nthreads=1), want)


@pytest.mark.parametrize("a_trans", [0, 1])
def test_reference_loop_equals_threaded_loop_bitwise(oracle, a_trans):
    """i-j-k (hostMatmul's order) and the threaded i-k-j loop add the same products in the same
    order per element.  Shape = the reference's own single-config test tile (test.py:32-57)."""
    M, N, K = 64, 48, 32
    a = SI.normal((M, K), 21)
    b = SI.normal((K, N), 22)
    a_buf = SI.a_operand(a, a_trans)
    assert np.array_equal(oracle.ijk(a_buf, b, a_trans), oracle.matmul(a_buf, b, a_trans))
    M, N, K = 96, 200, 257
    a = SI.normal((M, K), 23)
    b = SI.normal((K, N), 24)
    a_buf = SI.a_operand(a, a_trans)
    assert np.array_equal(oracle.ijk(a_buf, b, a_trans), oracle.matmul(a_buf, b, a_trans))


def test_identity_and_ones(oracle):
    n = 37
    b = SI.uniform((n, 53), 31)
    eye = np.eye(n, dtype=np.float32)
    for at in (0, 1):
        assert np.array_equal(oracle.matmul(eye, b, at), b)
    a = SI.uniform((29, n), 32)
    for at in (0, 1):
        assert np.array_equal(oracle.matmul(SI.a_operand(a, at), eye, at), a)
    K = 300
    ones_a, ones_b = np.ones((17, K), np.float32), np.ones((K, 19), np.float32)
    for at in (0, 1):
        assert np.array_equal(oracle.matmul(SI.a_operand(ones_a, at), ones_b, at), np.full((17, 19), K, np.float32))


def test_one_hot_probes_locate_indices(oracle):
    """A = e_i e_k^T picks row k of B into row i of C; catches swapped/transposed indices and
    wrong leading dimensions on non-square shapes."""
    M, N, K = 7, 11, 5
    b = np.arange(K * N, dtype=np.float32).reshape(K, N) + 1
    for (i, k) in [(0, 0), (6, 4), (3, 1), (2, 4)]:
        a = np.zeros((M, K), np.float32)
        a[i, k] = 2.0
        want = np.zeros((M, N), np.float32)
        want[i] = 2.0 * b[k]
        for at in (0, 1):
            assert np.array_equal(oracle.matmul(SI.a_operand(a, at), b, at), want)
            assert np.array_equal(oracle.ijk(SI.a_operand(a, at), b, at), want)


@pytest.mark.parametrize("M,N,K", [(64, 48, 32), (128, 128, 64), (33, 65, 1000)])
def test_small_integers_exact_against_int64(oracle, M, N, K):
    a = SI.small_ints((M, K), 41, lim=8)
    b = SI.small_ints((K, N), 42, lim=8)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for at in (0, 1):
        assert np.array_equal(oracle.matmul(SI.a_operand(a, at), b, at), want)
    assert np.array_equal(oracle.matmul_f64acc(a, b, 0), want.astype(np.float64))


def test_against_numpy_float64(oracle):
    M, N, K = 96, 80, 512
    a = SI.uniform((M, K), 51)
    b = SI.uniform((K, N), 52)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    got64 = oracle.matmul_f64acc(a, b, 0)
    assert np.abs(got64 - exact).max() <= 1e-12 * K
    got32 = oracle.matmul(a, b, 0)
    # sequential fp32 summation: |err| <= K * eps32 * sum|a||b| (first-order bound)
    bound = K * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
    assert (np.abs(got32 - exact) <= bound + 1e-30).all()
    # and it really is fp32 arithmetic, not a float64 sum rounded once
    assert np.abs(got32 - exact.astype(np.float32)).max() > 0


def test_row_panel_is_a_slice_of_the_full_product(oracle):
    M, N, K = 70, 40, 64
    a = SI.normal((M, K), 61)
    b = SI.normal((K, N), 62)
    full = oracle.matmul(a, b, 0)
    assert np.array_equal(oracle.matmul(a, b, 0, rows=(13, 29)), full[13:29])
    assert np.array_equal(oracle.ijk(a, b, 0, rows=(13, 29)), full[13:29])
    at = SI.a_operand(a, 1)
    assert np.array_equal(oracle.matmul(at, b, 1, rows=(64, 70)), full[64:70])


def test_linearity_and_f64_gemm(oracle):
    M, N, K = 24, 36, 48
    a1 = SI.small_ints((M, K), 71)
    a2 = SI.small_ints((M, K), 72)
    b = SI.small_ints((K, N), 73)
    assert np.array_equal(oracle.matmul(a1 + a2, b, 0), oracle.matmul(a1, b, 0) + oracle.matmul(a2, b, 0))
    ad = SI.uniform((M, K), 74).astype(np.float64)
    bd = SI.uniform((K, N), 75).astype(np.float64)
    assert np.allclose(oracle.matmul_f64(ad, bd, 0), ad @ bd, rtol=0, atol=1e-13 * K)
    assert np.array_equal(oracle.matmul_f64(np.ascontiguousarray(ad.T), bd, 1), oracle.matmul_f64(ad, bd, 0))


def test_reference_build_of_hostMatmul_is_bit_equal():
    """oracle/_ref: the reference's own hostMatmul, compiled from matmul.cpp:2349-2360 where it lies, against the
    restatement: the reference's single-config test tile (test.py:32-57) and two seeded shapes."""
    from tests import oracle_binding
    ref = oracle_binding.load_reference_build()
    if ref is None:
        pytest.skip("oracle/_ref was not built (no reference tree on this machine)")
    orc = oracle_binding.load()
    for (M, N, K), seeds in (((64, 48, 32), (81, 82)), ((96, 200, 257), (83, 84)), ((33, 17, 1000), (85, 86))):
        a = SI.normal((M, K), seeds[0])
        b = SI.normal((K, N), seeds[1])
        a_km = SI.a_operand(a, 1)
        want = ref(a_km, b)
        assert np.array_equal(orc.ijk(a_km, b, 1), want)
        assert np.array_equal(orc.matmul(a_km, b, 1), want)
        assert np.array_equal(orc.matmul(a, b, 0), want)          # the row-major layout of the same product


# ---- batched / strided GEMM with the alpha-beta epilogue: pinned by what the mathematics fixes -----------
def _batched_inputs(M, N, K, batch, ints=True):
    gen = (lambda shp, st: SI.small_ints(shp, st)) if ints else (lambda shp, st: SI.normal(shp, st))
    a = np.stack([gen((M, K), 100 + z) for z in range(batch)])
    b = np.stack([gen((K, N), 200 + z) for z in range(batch)])
    c0 = np.stack([gen((M, N), 300 + z) for z in range(batch)])
    return a, b, c0


@pytest.mark.parametrize("a_trans", [0, 1])
def test_batched_ab_alpha1_beta0_is_the_plain_product_per_slice(oracle, a_trans):
    M, N, K, batch = 24, 40, 56, 3
    a, b, c0 = _batched_inputs(M, N, K, batch, ints=False)
    a_buf = np.stack([SI.a_operand(a[z], a_trans) for z in range(batch)])
    c0[:] = np.nan                                   # beta == 0: C must not be read
    got = oracle.batched_ab(a_buf, b, c0, M, N, K, a_trans, batch, (M * K, K * N, M * N), 1.0, 0.0).reshape(batch, M, N)
    for z in range(batch):
        assert np.array_equal(got[z], oracle.matmul(a_buf[z], b[z], a_trans))


def test_batched_ab_strides(oracle):
    """Padding between the problems of a batch and a B shared by the whole batch (stride 0)."""
    M, N, K, batch = 8, 16, 24, 4
    a, b, c0 = _batched_inputs(M, N, K, batch)
    sa, sc = M * K + 5, M * N + 3
    a_flat = np.full(batch * sa, np.nan, np.float32)
    c_flat = np.full(batch * sc, -7.0, np.float32)
    for z in range(batch):
        a_flat[z * sa:z * sa + M * K] = a[z].ravel()
    got = oracle.batched_ab(a_flat, b[0], c_flat, M, N, K, 0, batch, (sa, 0, sc), 1.0, 0.0)
    for z in range(batch):
        assert np.array_equal(got[z * sc:z * sc + M * N].reshape(M, N), oracle.matmul(a[z], b[0], 0))
        assert (got[z * sc + M * N:(z + 1) * sc] == -7.0).all()          # the padding is not touched


def test_batched_ab_beta_and_alpha_exact_on_integers(oracle):
    M, N, K, batch = 16, 24, 32, 2
    a, b, c0 = _batched_inputs(M, N, K, batch)
    strides = (M * K, K * N, M * N)
    prod = np.stack([(a[z].astype(np.int64) @ b[z].astype(np.int64)) for z in range(batch)])
    for alpha, beta in ((1.0, 1.0), (2.0, -3.0), (-0.5, 0.25), (0.0, 1.0), (3.0, 0.0)):
        got = oracle.batched_ab(a, b, c0, M, N, K, 0, batch, strides, alpha, beta).reshape(batch, M, N)
        want = alpha * prod.astype(np.float64) + beta * c0.astype(np.float64)        # exact in fp64 and in fp32
        assert np.array_equal(got.astype(np.float64), want), (alpha, beta)


def test_batched_ab_linearity_in_alpha_on_powers_of_two(oracle):
    """Scaling by a power of two commutes with fp32 rounding: result(alpha = 2^p) = 2^p * result(alpha = 1)."""
    M, N, K = 12, 20, 300
    a, b, c0 = _batched_inputs(M, N, K, 1, ints=False)
    strides = (M * K, K * N, M * N)
    base = oracle.batched_ab(a, b, c0, M, N, K, 0, 1, strides, 1.0, 0.0)
    for p in (-3, 1, 5):
        assert np.array_equal(oracle.batched_ab(a, b, c0, M, N, K, 0, 1, strides, 2.0 ** p, 0.0), base * np.float32(2.0 ** p))
    # and beta = 1 adds C0 once, rounded once
    got = oracle.batched_ab(a, b, c0, M, N, K, 0, 1, strides, 1.0, 1.0)
    assert np.array_equal(got, (base + c0.ravel()).astype(np.float32))
