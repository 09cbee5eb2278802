"""The `DELAY_CPU` backend (NumPy node by node, like the reference's cpu.py), which
is chosen at import time and therefore runs in a child process."""
import os
import subprocess
import sys
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCRIPT = textwrap.dedent("""
    import numpy as np
    import delayrepay as dnp
    from delayrepay import NPArray, array, full, ones, sum
    assert dnp.backend.__name__.endswith(".cpu")

    # reference tests/test.py:21-67 on the NumPy backend
    arr, np_arr = ones(64), np.ones(64)
    assert isinstance(arr + 1, dnp.DelayArray) and "array" not in (arr + 1).__dict__
    assert np.array_equal((arr + 1).get(), np_arr + 1)
    assert np.array_equal((8 * arr + 9).get(), 8 * np_arr + 9)
    assert np.array_equal((arr + arr * 3 + 9).get(), np_arr + np_arr * 3 + 9)
    assert np.array_equal(np.cos(arr).get(), np.cos(np_arr))
    a32 = arr.astype(np.float32)
    assert (a32 ** 2).get().dtype == np.float32
    x = np.random.RandomState(0).uniform(-3, 3, 1000).astype(np.float32)
    assert (array(x) ** 3).get().tobytes() == ((x * x) * x).tobytes()      # delayarray.py:316-324
    assert np.array_equal((np.sin(arr) ** 2 + np.cos(arr) ** 2).get(),
                          np.sin(np_arr) * np.sin(np_arr) + np.cos(np_arr) * np.cos(np_arr))
    # tests/test.py:70-111
    v, w = full((64,), 7).astype(np.float32), full((64,), 3).astype(np.float32)
    assert np.all((v + w).get() == 10) and np.all((v * w).get() == 21)
    assert sum(v) == 448 and float(v.dot(w)) == 7 * 3 * 64 and float(v @ w) == 1344
    m = full((64, 64), 7).astype(np.float32)
    assert np.array_equal((m @ v).get(), np.full((64, 64), 7, np.float32) @ np.full(64, 7, np.float32))
    # tests/test.py:143-162
    raw = np.array([1, 2, 3])
    assert NPArray(raw) is NPArray(raw)
    z = array([1, 2, 3])
    assert np.sin(z) is np.sin(z)

    # slices, fused assignment, reductions, several roots: same front end, NumPy underneath
    u0 = np.zeros((20, 30), np.float32)
    u0[1:-1, 1:-1] = np.random.RandomState(1).uniform(0, 1, (18, 28))
    u, ref = array(u0.copy()), u0.copy()
    for _ in range(3):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        ref[1:-1, 1:-1] = 0.25 * (ref[:-2, 1:-1] + ref[2:, 1:-1] + ref[1:-1, :-2] + ref[1:-1, 2:])
    assert u.get().tobytes() == ref.tobytes()
    a = array(np.arange(12.0).reshape(3, 4))
    assert np.array_equal(dnp.sum(a * 2, axis=0).get(), (np.arange(12.0).reshape(3, 4) * 2).sum(axis=0))
    assert float(dnp.mean(a)) == 5.5 and float(dnp.max(a)) == 11
    p, q = dnp.evaluate(a + 1, a * 2)
    assert np.array_equal(p.get(), np.arange(12.0).reshape(3, 4) + 1)
    assert np.array_equal(np.where(a > 5, a, 0.0).get(), np.where(np.arange(12.0).reshape(3, 4) > 5,
                                                                   np.arange(12.0).reshape(3, 4), 0.0))
    print("cpu-backend-ok")
""")


def test_delay_cpu_backend_runs_the_reference_suite():
    env = dict(os.environ, DELAY_CPU="1", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", SCRIPT], env=env, capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "cpu-backend-ok" in out.stdout


def test_hip_backend_is_the_default_and_fails_loudly_without_the_library(tmp_path):
    """No silent host fall-back: without libdrhip.so the default backend refuses to import."""
    pkg = tmp_path / "delayrepay_amd"
    pkg.mkdir()
    for name in os.listdir(os.path.join(ROOT, "delayrepay_amd")):
        if name.endswith(".py"):
            (pkg / name).write_text(open(os.path.join(ROOT, "delayrepay_amd", name)).read())
    env = {k: v for k, v in os.environ.items() if k != "DELAY_CPU"}
    env["PYTHONPATH"] = str(tmp_path)
    out = subprocess.run([sys.executable, "-c", "import delayrepay_amd"], env=env, cwd=str(tmp_path),
                         capture_output=True, text=True, timeout=300)
    assert out.returncode != 0
    assert "libdrhip.so is missing" in out.stderr and "no host fall-back" in out.stderr
