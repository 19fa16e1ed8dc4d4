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
