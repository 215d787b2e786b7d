"""gather / index_select / scatter on the GPU: bit-exact against the oracle and the reference's
goldens (zyx/tests/08_indexing.rs:181-300 gather, :303-435 scatter, :437-480 larger cases,
:597-627 index_select; zyx/tests/05_misc.rs:778-798)."""
import numpy as np
import pytest

from zyx_amd import BackendError, ErrorStatus
from zyx_amd.kernels import gather, index_select, scatter

pytestmark = pytest.mark.gpu


def test_gather_reference_goldens(hip):
    dev, pool = hip
    g = lambda x, ax, i: gather(dev, pool, x, ax, i).tolist()
    x = np.array([[10, 20, 30, 40, 50], [11, 21, 31, 41, 51], [12, 22, 32, 42, 52]], np.uint16)
    assert g(x, 1, np.array([[0, 2, 4], [1, 3, 0], [4, 1, 2]], np.uint16)) == [[10, 30, 50], [21, 41, 11], [52, 22, 32]]
    x = np.array([[1, 2, 3], [4, 5, 6], [7, 8, 9]], np.int32)
    assert g(x, 0, np.array([[0, 1], [1, 2], [0, 2]])) == [[1, 5], [4, 8], [1, 8]]
    assert g(np.array([10, 20, 30, 40, 50], np.int32), 0, np.array([0, 2, 4, 1], np.uint16)) == [10, 30, 50, 20]
    assert g(np.array([[1, 2, 3], [4, 5, 6]], np.int32), 1, np.array([[-1, 0], [1, -2]], np.int32)) == [[3, 1], [5, 5]]
    assert g(np.array([10, 20, 30], np.int32), 0, np.array([0, 0, 1, 1, 2, 0], np.uint16)) == [10, 10, 20, 20, 30, 10]
    x3 = np.array([[[1, 2], [3, 4]], [[5, 6], [7, 8]]], np.int32)
    assert g(x3, 2, np.array([[[0], [1]], [[1], [0]]])) == [[[1], [4]], [[6], [7]]]
    assert g(np.array([[1, 2, 3], [4, 5, 6]], np.int32), -1, np.array([[0, 2], [1, 0]])) == [[1, 3], [5, 4]]
    assert g(np.array([[1, 2], [3, 4], [5, 6]], np.int32), -2, np.array([[0], [0], [2]])) == [[1], [1], [5]]
    assert g(np.array([1.0, 2.0, 3.0, 4.0], np.float32), 0, np.array([0, 2, 3, 1], np.uint16)) == [1.0, 3.0, 4.0, 2.0]
    assert g(np.array([[1, 2], [3, 4]], np.int32), 1, np.array([[0, 0, 1], [1, 1, 0]])) == [[1, 1, 2], [4, 4, 3]]
    x4 = np.array([[[[1, 2], [3, 4]], [[5, 6], [7, 8]]]], np.int32)
    assert g(x4, 3, np.array([[[[0], [1]]]])) == [[[[1], [4]]]]
    assert g(np.array([1, 2, 3], np.int32), 0, np.array([0, 3, -4, 2])) == [1, 0, 0, 3]  # out of range reads 0


def test_scatter_reference_goldens(hip):
    dev, pool = hip
    s = lambda x, ax, i, v: scatter(dev, pool, x, ax, i, v).tolist()
    z = lambda *sh: np.zeros(sh, np.int32)
    assert s(z(3, 3), 0, np.array([[0, 1, 2], [0, 1, 2]], np.uint8), [[1, 2, 3], [4, 5, 6]]) == [[5, 0, 0], [0, 7, 0], [0, 0, 9]]
    assert s(z(3, 4), 1, np.array([[0, 3], [1, 2], [2, 1]], np.uint8), [[1, 2], [3, 4], [5, 6]]) == \
        [[1, 0, 0, 2], [0, 3, 4, 0], [0, 6, 5, 0]]
    assert s(z(5), 0, np.array([0, 0, 1, 1, 2, 4], np.uint8), [1, 2, 3, 4, 5, 6]) == [3, 7, 5, 0, 6]
    assert s(z(10), 0, np.array([0, 5, 9], np.uint8), [100, 200, 300]) == [100, 0, 0, 0, 0, 200, 0, 0, 0, 300]
    assert s(np.full((2, 3), 10, np.int32), 1, np.array([[0, 1, 2]], np.uint16), [[1, 2, 3]]) == [[11, 12, 13], [10, 10, 10]]
    assert s(z(3, 3), 1, np.array([[-1, -2], [0, 1]]), [[1, 2], [3, 4]]) == [[0, 2, 1], [3, 4, 0], [0, 0, 0]]
    assert s(z(2, 3, 4), 2, np.array([[[0, 3]], [[1, 2]]], np.int64), [[[1, 2]], [[3, 4]]]) == \
        [[[1, 0, 0, 2], [0, 0, 0, 0], [0, 0, 0, 0]], [[0, 3, 4, 0], [0, 0, 0, 0], [0, 0, 0, 0]]]
    r = scatter(dev, pool, z(10000), 0, np.array([0, 1, 5000, 9999, 0, 9999], np.uint16), [10, 20, 30, 40, 100, 200])
    assert (r[0], r[1], r[5000], r[9999]) == (110, 20, 30, 240) and r.sum() == 400
    assert s(z(3, 3), 0, np.array([[0, 1, 2]], np.uint8), [[1, 2, 3]]) == [[1, 0, 0], [0, 2, 0], [0, 0, 3]]
    assert s(np.zeros(3, np.float32), 0, np.array([0, 2], np.uint8), np.array([1.5, 2.5], np.float32)) == [1.5, 0.0, 2.5]
    with pytest.raises(ValueError):  # rank mismatch (scatter_error_rank_mismatch)
        scatter(dev, pool, z(3, 3), 0, np.array([0, 1]), np.array([1, 2]))
    with pytest.raises(ValueError):  # shape mismatch (scatter_error_shape_mismatch)
        scatter(dev, pool, z(3, 3), 0, np.array([[0, 1], [2, 0]]), np.array([[1, 2, 3]]))


def test_index_select_reference_goldens(hip):
    dev, pool = hip
    x = np.array([[1, 2, 3], [4, 5, 6], [7, 8, 9]], np.int32)
    sel = lambda ax, i: index_select(dev, pool, x, ax, np.array(i)).tolist()
    assert sel(0, [2, 0]) == [[7, 8, 9], [1, 2, 3]]
    assert sel(1, [2, 0]) == [[3, 1], [6, 4], [9, 7]]
    assert sel(0, [-1, -3]) == [[7, 8, 9], [1, 2, 3]]
    assert sel(1, [-2, -1]) == [[2, 3], [5, 6], [8, 9]]
    y = index_select(dev, pool, index_select(dev, pool, x, 0, np.array([1])), 1, np.array([2]))
    assert y.tolist() == [[6]]


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.int64, np.uint8, np.uint16, np.float64])
def test_random_against_oracle(hip, oracle, dtype):
    dev, pool = hip
    rng = np.random.default_rng(5)
    x = rng.integers(0, 200, size=(6, 37, 5, 19)).astype(dtype)
    for axis in range(4):
        ishape = [rng.integers(1, s + 1) for s in x.shape]
        ishape[axis] = int(rng.integers(1, 2 * x.shape[axis]))
        idx = rng.integers(-x.shape[axis] - 2, x.shape[axis] + 2, size=ishape)
        assert np.array_equal(gather(dev, pool, x, axis, idx), oracle.gather(x, axis, idx))
        sel = rng.integers(-x.shape[axis], x.shape[axis], size=11)
        assert np.array_equal(index_select(dev, pool, x, axis, sel), oracle.index_select(x, axis, sel))
        if dtype not in (np.uint8, np.uint16):
            src = rng.integers(-50, 50, size=ishape).astype(dtype)
            assert np.array_equal(scatter(dev, pool, x, axis, idx, src), oracle.scatter(x, axis, idx, src))


def test_mnist_like_batch_sampling(hip, oracle):
    """index_select of 64 random rows out of a [10000, 784] matrix: how the reference's example draws
    batches (zyx-examples/examples/mnist.rs:62-64)."""
    dev, pool = hip
    data = oracle.Rng(1).randn((10000, 784))
    idx = oracle.Rng(2).randint(64, 0, 10000)
    assert np.array_equal(index_select(dev, pool, data, 0, idx), data[idx])


def test_oversized_index_is_refused(hip):
    dev, pool = hip
    with pytest.raises(BackendError) as ei:  # index extent exceeds x outside the axis
        gather(dev, pool, np.zeros((2, 2), np.int32), 1, np.zeros((3, 2), np.int32))
    assert ei.value.status == ErrorStatus.KernelCompilation and "Shape mismatch" in ei.value.context
