"""Pins the oracle's distance routines: fp64 closed form, special cases that a
dropped term / wrong index / wrong sign would break, agreement of the scalar and
SIMD forms, and bit equality with the reference's own DistanceL2 where built."""
import numpy as np
import pytest

DIMS = [4, 8, 12, 16, 20, 36, 64, 100, 128, 200, 256, 512, 1000]
ORDERS = [0, 1, 2, 3]  # GPU_SEQ, GPU_WARP32, CPU_AVX512, WAVE64


def _vec(seed, d):
    return np.random.RandomState(seed).randn(d).astype(np.float32)


@pytest.mark.parametrize("dim", DIMS)
@pytest.mark.parametrize("order", ORDERS)
def test_l2_matches_fp64(orc, dim, order):
    q, b = _vec(dim, dim), _vec(dim + 1, dim)
    want = float(((q.astype(np.float64) - b.astype(np.float64)) ** 2).sum())
    got = orc.dist(q, b, orc.L2, order)
    assert abs(got - want) <= 1e-5 * want


@pytest.mark.parametrize("dim", DIMS)
@pytest.mark.parametrize("order", [0, 1, 3])
def test_ip_matches_fp64(orc, dim, order):
    q, b = _vec(3 * dim, dim), _vec(3 * dim + 1, dim)
    want = float((q.astype(np.float64) * b.astype(np.float64)).sum())
    got = orc.dist(q, b, orc.IP, order)
    scale = float((np.abs(q.astype(np.float64) * b.astype(np.float64))).sum())
    assert abs(got - want) <= 1e-5 * scale


@pytest.mark.parametrize("order", ORDERS)
def test_identical_vectors_are_at_zero(orc, order):
    q = _vec(5, 200)
    assert orc.dist(q, q, orc.L2, order) == 0.0


@pytest.mark.parametrize("order", ORDERS)
@pytest.mark.parametrize("dim", [4, 36, 200])
def test_one_hot_exposes_every_coordinate(orc, order, dim):
    # e_i against 0 is exactly 1 for L2, and <2 e_i, 3 e_j> is 6 [i == j]: a skipped or
    # double-counted coordinate, or a transposed operand pair, changes an exact value
    zero = np.zeros(dim, np.float32)
    for i in range(dim):
        e = zero.copy()
        e[i] = 1.0
        assert orc.dist(e, zero, orc.L2, order) == 1.0
        assert orc.dist(zero, e, orc.L2, order) == 1.0
        if order != 2:
            f = zero.copy()
            f[(i + 1) % dim] = 3.0
            assert orc.dist(2 * e, 3 * e, orc.IP, order) == 6.0
            assert orc.dist(2 * e, f, orc.IP, order) == 0.0


@pytest.mark.parametrize("order", [0, 1, 3])
def test_unit_vectors_l2_is_2_minus_2ip(orc, order):
    q, b = _vec(11, 128), _vec(12, 128)
    q /= np.linalg.norm(q)
    b /= np.linalg.norm(b)
    l2 = orc.dist(q, b, orc.L2, order)
    ip = orc.dist(q, b, orc.IP, order)
    assert abs(l2 - (2.0 - 2.0 * ip)) < 1e-5


def test_cpu_order_ignores_metric(orc):
    # src/search_in_cpu.cpp:52 constructs DistanceL2 whatever the metric is
    q, b = _vec(1, 200), _vec(2, 200)
    assert orc.dist(q, b, orc.IP, 2) == orc.dist(q, b, orc.L2, 2)


@pytest.mark.parametrize("dim", list(range(1, 40)) + [100, 128, 200, 203, 512])
def test_avx512_forms_agree_bitwise(orc, dim):
    q, b = _vec(dim, dim), _vec(dim + 100, dim)
    simd = orc.dist(q, b, orc.L2, 2)
    scalar = float(orc.lib().oracle_dist_avx512_scalar(b.ctypes.data, q.ctypes.data, dim))
    assert np.float32(simd).tobytes() == np.float32(scalar).tobytes()


@pytest.mark.parametrize("dim", list(range(1, 40)) + [100, 128, 200, 203, 512])
def test_avx512_order_equals_reference_header(orc, ref, dim):
    q, b = _vec(dim, dim), _vec(dim + 100, dim)
    want = float(ref.ref_distance_l2(b.ctypes.data, q.ctypes.data, dim))
    got = orc.dist(q, b, orc.L2, 2)
    assert np.float32(got).tobytes() == np.float32(want).tobytes()


def test_wave64_group_sizes(orc):
    # chunks <= 16 -> 16 lanes, <= 32 -> 32 lanes, else 64: with a vector of ones the
    # result is exactly dim for every group size and tail shape
    for dim in (4, 60, 64, 68, 128, 132, 200, 256, 260, 512, 1024, 2048):
        one = np.ones(dim, np.float32)
        assert orc.dist(one, np.zeros(dim, np.float32), orc.L2, 3) == float(dim)
        assert orc.dist(one, one, orc.IP, 3) == float(dim)


def test_normalize_matches_numpy_restatement(orc):
    from coral_amd import synth
    x = np.random.RandomState(3).randn(50, 24).astype(np.float32)
    x[7] = 0.0
    y = x.copy()
    orc.lib().oracle_normalize_l2(y.ctypes.data, y.shape[0], y.shape[1])
    assert np.array_equal(y, synth.normalize_rows(x))
    assert not y[7].any()
    n = np.linalg.norm(y.astype(np.float64), axis=1)
    assert np.allclose(np.delete(n, 7), 1.0, atol=1e-6)


def test_cuda_summation_orders_known_answers(orc):
    """Inputs on which fp32 absorbs an addend (2^24 + 1 rounds back to 2^24), so that the ORDER of the additions
    decides the result and each result can be worked out by hand: the one-thread chain of include/utils.cuh:254-275
    and :307-323 (order 0) against the lane-strided partial sums and the shuffle-down tree, offsets 16 to 1, of
    src/search_gpu.cu:14-23 (order 1).  A chain summed as a tree, a lane stride other than 32 or a tree walked from
    offset 1 upwards gives the other value."""
    big = float(2 ** 24)
    ones = np.ones(64, np.float32)

    def vec(**at):
        b = np.zeros(64, np.float32)
        for i, x in at.items():
            b[int(i[1:])] = x
        return b

    # inner product with a vector of ones = the plain sum of b
    # chain: (2^24 + 1) - 2^24 = 0;  lanes 0, 1, 2 -> tree: (2^24 - 2^24) + 1 = 1
    b = vec(i0=big, i1=1.0, i2=-big)
    assert orc.dist(ones, b, orc.IP, 0) == 0.0 and orc.dist(ones, b, orc.IP, 1) == 1.0
    # chain: (2^24 - 2^24) + 1 = 1;  lane 0 holds coordinates 0 and 32: (2^24 + 1) - 2^24 = 0
    b = vec(i0=big, i1=-big, i32=1.0)
    assert orc.dist(ones, b, orc.IP, 0) == 1.0 and orc.dist(ones, b, orc.IP, 1) == 0.0
    # the tree adds lane 16 to lane 0 before lane 1: (2^24 - 2^24) + 1 = 1; from offset 1 upwards it would be 0.
    # chain: (2^24 + 1) - 2^24 = 0
    b = vec(i0=big, i1=1.0, i16=-big)
    assert orc.dist(ones, b, orc.IP, 1) == 1.0 and orc.dist(ones, b, orc.IP, 0) == 0.0
    # squared L2 from the origin: 4096^2 + 1 + 1.  chain: both ones absorbed; tree: lanes 1 and 3 meet first (2),
    # then 2^24 + 2 is exact.  The CPU routine (include/efanna2e/distance.h:39-89) ends in
    # (m0 + m1) + (m2 + m3) = (2^24 + 1) + (0 + 1): both absorbed
    zero = np.zeros(64, np.float32)
    b = vec(i0=4096.0, i1=1.0, i3=1.0)
    assert orc.dist(zero, b, orc.L2, 0) == big and orc.dist(zero, b, orc.L2, 1) == big + 2.0
    assert orc.dist(zero, b, orc.L2, 2) == big
    # ones in lanes 4 and 5 never meet each other in the shuffle-down tree: offset 4 brings lane 4 to lane 0
    # (absorbed) and lane 5 to lane 1, offset 1 adds lane 1 (absorbed).  A tree that pairs neighbours first
    # would give 2^24 + 2.  CPU: m2 = [2^24 + 1 -> 2^24, 1, 0, 0] -> 2^24 + 1 -> 2^24
    b = vec(i0=4096.0, i4=1.0, i5=1.0)
    assert orc.dist(zero, b, orc.L2, 1) == big and orc.dist(zero, b, orc.L2, 2) == big
