"""The backend's host code (zyx_amd/csrc/*.cpp: event table, stream choice, block cache, plans, program scratch,
run-time compilation cache) built for the CPU against a host-only model of the HIP runtime (tests/fakehip/) and run
under AddressSanitizer + UBSan and under ThreadSanitizer. The model keeps a vector clock per stream and reports every
operation that touches a buffer without being ordered after the last conflicting access; the harness replays the
sequences zyx's runtime issues (zyx/src/graph/plan.rs:271-361, zyx/src/runtime.rs:2262-2300) under its event-map rule
(zyx/src/runtime.rs:1-16) plus random schedules, and must see none. Needs no GPU."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fakehip")


def _build(kind, out):
    r = subprocess.run(["make", "-C", HERE, kind, f"OUT={out}"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    return os.path.join(out, f"harness_{kind}")


def _run(exe, tmp, *args):
    env = dict(os.environ, ZYX_HIP_CACHE_DIR=os.path.join(tmp, "cache"), ASAN_OPTIONS="detect_leaks=1", LD_PRELOAD="")
    r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=600, env=env)
    assert r.returncode == 0 and "all scenarios passed" in r.stdout, r.stdout[-4000:] + r.stderr[-4000:]
    return r.stdout


@pytest.fixture(scope="module")
def out_dir(tmp_path_factory):
    return str(tmp_path_factory.mktemp("fakehip"))


def test_runtime_logic_under_address_and_ub_sanitizers(out_dir):
    exe = _build("asan", out_dir)
    out = _run(exe, out_dir)
    for scenario in ("execute_plan sequence", "consumed event still orders", "block cache", "random schedule, seed 12", "threads"):
        assert scenario in out
    # a second process finds the generated kernel's code object in the on-disk cache
    _run(exe, out_dir, "ir")
    assert any(f.endswith(".hsaco") for f in os.listdir(os.path.join(out_dir, "cache")))


def test_runtime_logic_under_thread_sanitizer(out_dir):
    exe = _build("tsan", out_dir)
    _run(exe, out_dir, "threads")
    _run(exe, out_dir, "random")
