"""safetensors reading / writing as zyx's Module::save and load_safetensors do it (zyx/src/module.rs:37-64,
436-530), against the data file the reference's own test holds (zyx/tests/05_misc.rs:639-661)."""
import json
import os
import struct

import numpy as np
import pytest

from zyx_amd import DType, safetensors_io

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_reads_the_reference_fixture(oracle):
    t = safetensors_io.load(os.path.join(GOLD, "xyz2.safetensors"))
    assert {k: (v[0], v[1].shape) for k, v in t.items()} == {"x": (DType.I64, (256, 512)), "y": (DType.I64, (512, 368)), "z": (DType.I64, (256, 368))}
    assert np.array_equal(t["x"][1] @ t["y"][1], t["z"][1])  # matmul_disk: z = x . y


def test_round_trip_and_layout(tmp_path):
    rng = np.random.default_rng(0)
    tensors = {"w": rng.standard_normal((3, 5)).astype(np.float32), "idx": np.arange(7, dtype=np.int64),
               "h": (DType.BF16, rng.integers(0, 65536, (2, 4)).astype(np.uint16)), "flag": np.array([True, False])}
    path = str(tmp_path / "m.safetensors")
    safetensors_io.save(path, tensors)
    raw = open(path, "rb").read()
    (n,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + n])
    assert list(header) == ["w", "idx", "h", "flag"] and header["h"] == {"dtype": "BF16", "shape": [2, 4], "data_offsets": [116, 132]}
    assert len(raw) == 8 + n + 60 + 56 + 16 + 2
    back = safetensors_io.load(path)
    assert back["h"][0] == DType.BF16 and np.array_equal(back["h"][1], tensors["h"][1])
    assert back["w"][0] == DType.F32 and np.array_equal(back["w"][1], tensors["w"])
    assert np.array_equal(back["idx"][1], tensors["idx"]) and np.array_equal(back["flag"][1], tensors["flag"])


def test_malformed_files_are_rejected(tmp_path):
    p = str(tmp_path / "bad.safetensors")
    open(p, "wb").write(b"\x01\x02")
    with pytest.raises(ValueError):
        safetensors_io.load(p)
    text = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(text)) + text + b"\0" * 8)
    with pytest.raises(ValueError):  # 4 x f32 needs 16 bytes
        safetensors_io.load(p)
    text = json.dumps({"a": {"dtype": "Q7", "shape": [1], "data_offsets": [0, 1]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(text)) + text + b"\0")
    with pytest.raises(ValueError):
        safetensors_io.load(p)


@pytest.mark.gpu
def test_load_to_pool_feeds_a_gemm(hip):
    """The fixture's x, y go from disk to HBM; their product on the device (i64 has no device GEMM here, so as f32
    on a slice whose values stay exact) matches z."""
    from zyx_amd.kernels import gemm
    dev, pool = hip
    bufs = safetensors_io.load_to_pool(os.path.join(GOLD, "xyz2.safetensors"), pool)
    assert bufs["x"][1:] == (DType.I64, (256, 512))
    x = np.empty((256, 512), np.int64)
    pool.pool_to_host(bufs["x"][0], x, [])
    t = safetensors_io.load(os.path.join(GOLD, "xyz2.safetensors"))
    assert np.array_equal(x, t["x"][1])
    got = gemm(dev, pool, t["x"][1].astype(np.float32), t["y"][1].astype(np.float32), dtype=DType.F32)
    assert np.allclose(got, t["z"][1].astype(np.float64), rtol=1e-5)
    for b, _, _ in bufs.values():
        pool.deallocate(b, [])
