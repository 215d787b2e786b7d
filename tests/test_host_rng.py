"""The backend library's host RNG (zyx/src/rng.rs restated in zyx_amd/csrc/host_rng.cpp) against the reference's
known answer and against the oracle's independent restatement, draw for draw. Runs without a GPU."""
import numpy as np

from zyx_amd import DType
from zyx_amd.rng import Rng


def test_reference_known_answer():
    # zyx/tests/05_misc.rs:768-774: manual_seed(69420); rand([3, 12], U8).slice((.., 8..=-2))
    x = Rng(69420).rand((3, 12), DType.U8)
    assert x[:, 8:11].tolist() == [[41, 171, 236], [212, 222, 77], [16, 125, 60]]


def test_splitmix_seeding_textbook_value():
    # splitmix64 from state 0: first output 0xe220a8397b1dcdaf (Vigna's reference implementation); xoshiro256++'s
    # first output from s = [a, b, c, d] is rotl(a + d, 23) + a
    r = Rng(0)
    s = list(r._s)
    assert s[0] == 0xE220A8397B1DCDAF and s[1] == 0x6E789E6AA1B965F4
    want = (((s[0] + s[3]) & (2**64 - 1)) << 23 | ((s[0] + s[3]) & (2**64 - 1)) >> 41) & (2**64 - 1)
    assert r.next_u64() == (want + s[0]) & (2**64 - 1)


def test_every_draw_equals_the_oracle(oracle):
    a, b = Rng(1234), oracle.Rng(1234)
    assert [a.next_u64() for _ in range(5)] == [b.next_u64() for _ in range(5)]
    assert np.array_equal(a.rand(1000), b.rand(1000))
    assert np.array_equal(a.uniform((7, 9), -1.0, 1.0), b.uniform((7, 9), -1.0, 1.0))
    assert np.array_equal(a.randint(500, 0, 10), b.randint(500, 0, 10))
    assert np.array_equal(a.rand(64, DType.U8), b.rand_u8(64))
    # randn goes through the host libm on both sides, built with different flags: a few ulp, and the same stream after
    x, y = a.randn((3, 1000), 3.0), b.randn((3, 1000), 3.0)
    assert np.allclose(x, y, rtol=1e-5, atol=1e-6)
    assert a.next_u64() == b.next_u64()


def test_ranges_and_moments():
    r = Rng()
    u = r.rand(200000)
    assert u.min() >= 0.0 and u.max() <= 1.0 and abs(u.mean() - 0.5) < 5e-3
    g = r.randn(200000)
    assert abs(g.mean()) < 1e-2 and abs(g.std() - 1.0) < 1e-2 and np.all(np.isfinite(g))
    k = r.randint(10000, -3, 4)
    assert k.min() == -3 and k.max() == 3
    assert r.randint(4, 5, 5).tolist() == [5] * 4
