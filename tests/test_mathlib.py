"""Accuracy of the double-precision device math functions, on the CPU.

`mathlib.source(..., HOST_MACROS)` is the same text the kernels include, with the
reciprocal seed and the scalar-constant multiply-add spelled in plain C; it is built
here with g++ and compared with 40-digit values (mpmath) and with libm / SciPy.
The device build of the same text is checked against NumPy in the GPU tests."""
import ctypes
import subprocess

import mpmath as mp
import numpy as np
import pytest
import scipy.special

from delayrepay_amd import hip, mathlib


@pytest.fixture(scope="module")
def host(tmp_path_factory):
    """The device source built for the host with g++.  Arrays go through the 4-element
    pack (the form the kernels use) and the remainder through the 1-element form."""
    d = tmp_path_factory.mktemp("mathlib")
    src = "#include <math.h>\n" + mathlib.source(sorted(mathlib.FUNCTIONS), mathlib.HOST_MACROS, soft_div=True)
    src += ('extern "C" void v_div(const double* a, const double* b, double* y, long n)\n'
            "{ long i = 0;\n"
            "  for (; i + 4 <= n; i += 4) { const double p[4] = {a[i], a[i+1], a[i+2], a[i+3]}, "
            "q[4] = {b[i], b[i+1], b[i+2], b[i+3]}; double r[4]; dr_div_f8<4>(p, q, r); "
            "for (int e = 0; e < 4; e++) y[i+e] = r[e]; }\n"
            "  for (; i < n; i++) y[i] = dr_div_f8_1(a[i], b[i]); }\n")
    for name, (fn, _) in mathlib.FUNCTIONS.items():
        src += (f'extern "C" void v_{name}(const double* x, double* y, long n)\n'
                "{ long i = 0;\n"
                "  for (; i + 4 <= n; i += 4) { const double a[4] = {x[i], x[i+1], x[i+2], x[i+3]}; "
                f"double r[4]; {fn}<4>(a, r); for (int e = 0; e < 4; e++) y[i+e] = r[e]; }}\n"
                f"  for (; i < n; i++) y[i] = {fn}_1(x[i]); }}\n")
    src += ('extern "C" void v_sqrt_near(const double* x, double* y, long n)\n'
            "{ long i = 0;\n"
            "  for (; i + 4 <= n; i += 4) { const double a[4] = {x[i], x[i+1], x[i+2], x[i+3]}; "
            "double r[4]; dr_sqrt_near_f8<4>(a, r); for (int e = 0; e < 4; e++) y[i+e] = r[e]; }\n"
            "  for (; i < n; i++) y[i] = dr_sqrt_near_f8_1(x[i]); }\n")
    (d / "m.cpp").write_text(src)
    subprocess.run(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", str(d / "m.so"),
                    str(d / "m.cpp")], check=True)
    lib = ctypes.CDLL(str(d / "m.so"))

    def call(name, x, other=None):
        if name == "div":
            a = np.ascontiguousarray(x, dtype=np.float64)
            b = np.ascontiguousarray(other, dtype=np.float64)
            y = np.empty_like(a)
            lib.v_div(a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p),
                      y.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(a.size))
            return y
        x = np.ascontiguousarray(x, dtype=np.float64)
        y = np.empty_like(x)
        getattr(lib, "v_" + name)(x.ctypes.data_as(ctypes.c_void_p),
                                  y.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(x.size))
        return y
    return call


def mathlib_fit_ends(i):
    """The last double of interval i of the log table and the first of the next."""
    from delayrepay_amd.mathlib_fit import log_interval
    hi = log_interval(i)[1]
    return float(np.nextafter(hi, 0)), hi


def ulp_error(got, x, exact):
    """Largest |got - exact(x)| in units of the last place of the exact value."""
    mp.mp.dps = 40
    worst = 0.0
    for g, v in zip(got, x):
        e = exact(mp.mpf(float(v)))
        if e == 0:
            assert g == 0
            continue
        worst = max(worst, float(abs(mp.mpf(float(g)) - e) / mp.mpf(float(np.spacing(abs(float(e)))))))
    return worst


def test_log_accuracy_over_the_whole_range(host):
    rs = np.random.RandomState(3)
    x = np.concatenate([rs.uniform(1e-6, 1e6, 1 << 18), np.exp(rs.uniform(-744, 709, 1 << 18)),
                        rs.uniform(0.5, 2, 1 << 18), 1 + rs.uniform(-1e-6, 1e-6, 1 << 16),
                        [5e-324, 2.2250738585072014e-308, 1e-310, 1.0, np.nextafter(1, 2),
                         np.nextafter(1, 0), 1.7976931348623157e308, 0.7071067811865475,
                         0.7071067811865476, 1.4142135623730951]])
    got = host("log", x)
    ref = np.log(x)
    assert np.max(np.abs(got - ref) / np.spacing(np.abs(ref))) <= 1.0      # libm itself: < 1 ulp
    pick = np.r_[rs.choice(x.size - 10, 6000, replace=False), np.arange(x.size - 10, x.size)]
    assert ulp_error(got[pick], x[pick], mp.log) <= 1.0
    near = 1 + rs.uniform(-5e-3, 5e-3, 1 << 17)                 # the intervals around the centre one
    assert ulp_error(host("log", near)[:8000], near[:8000], mp.log) <= 0.8
    ends = np.array([v for i in range(0, 256, 5) for v in mathlib_fit_ends(i)])
    assert ulp_error(host("log", ends), ends, mp.log) <= 1.0


def test_log_special_values(host):
    got = host("log", [0.0, -0.0, -1.0, -np.inf, np.inf, np.nan, 1.0])
    assert got[0] == -np.inf and got[1] == -np.inf
    assert np.isnan(got[2]) and np.isnan(got[3]) and np.isnan(got[5])
    assert got[4] == np.inf and got[6] == 0.0 and not np.signbit(got[6])


def test_erf_accuracy(host):
    rs = np.random.RandomState(4)
    edges = np.arange(1, 97) / 16.0                               # where the table row changes
    x = np.concatenate([rs.uniform(-6.5, 6.5, 1 << 19), rs.uniform(-1, 1, 1 << 18),
                        rs.uniform(0, 1 / 16, 1 << 16), 10.0 ** rs.uniform(-300, 1, 1 << 16),
                        edges, np.nextafter(edges, 0), np.nextafter(edges, 10),
                        [5.9, 6.0, 6.1, 27.0, 1e300, 5e-324, 1e-310]])
    got = host("erf", x)
    ref = scipy.special.erf(x)
    assert np.max(np.abs(got - ref) / np.spacing(np.abs(ref))) <= 3.5      # SciPy's is off by up to 2.6
    assert np.all(np.abs(got) <= 1.0)
    pick = np.r_[rs.choice(x.size - 295, 12000, replace=False), np.arange(x.size - 295, x.size)]
    inner = np.abs(x[pick]) < 1 / 16       # the first row multiplies by 2/sqrt(pi): one more rounding
    assert ulp_error(got[pick][inner], x[pick][inner], mp.erf) <= 1.8
    assert ulp_error(got[pick][~inner], x[pick][~inner], mp.erf) <= 1.1
    # odd, and monotone from each row of the table to the next
    assert np.array_equal(host("erf", -x), -got)
    around = np.sort(np.concatenate([np.nextafter(edges, 0), edges, np.nextafter(edges, 10)]))
    assert np.all(np.diff(host("erf", around)) >= 0)
    # the pack and the one-element form are the same arithmetic
    assert np.array_equal(host("erf", x[:1001]), np.concatenate([host("erf", x[i:i + 1]) for i in range(1001)]))


def test_erf_special_values(host):
    got = host("erf", [0.0, -0.0, np.inf, -np.inf, np.nan, 40.0, -40.0])
    assert got[0] == 0 and not np.signbit(got[0]) and got[1] == 0 and np.signbit(got[1])
    assert got[2] == 1 and got[3] == -1 and np.isnan(got[4]) and got[5] == 1 and got[6] == -1


def test_exp_accuracy_and_limits(host):
    rs = np.random.RandomState(5)
    x = np.concatenate([rs.uniform(-20, 20, 1 << 18), rs.uniform(-745, 709.78, 1 << 18),
                        rs.uniform(-1e-3, 1e-3, 1 << 16),
                        [0.0, -0.0, 1.0, -1.0, 709.782712893384, 709.7827128933841, -708.3964185322641,
                         -745.1332191019411, -745.1332191019412, -744.0, 1e-320, 0.5 * np.log(2)]])
    got = host("exp", x)
    with np.errstate(over="ignore"):
        ref = np.exp(x)
    assert np.array_equal(np.isinf(got), np.isinf(ref))
    normal = (ref >= np.finfo(np.float64).tiny) & np.isfinite(ref)
    assert np.max(np.abs(got[normal] - ref[normal]) / np.spacing(ref[normal])) <= 1.0
    small = ref < np.finfo(np.float64).tiny
    assert np.max(np.abs(got[small] - ref[small]) / 5e-324) <= 1.0              # denormal results: one step
    pick = np.r_[rs.choice(x.size - 12, 6000, replace=False), np.arange(x.size - 12, x.size)]
    pick = pick[normal[pick]]
    assert ulp_error(got[pick], x[pick], mp.exp) <= 1.0
    got = host("exp", [np.inf, -np.inf, np.nan, 710.0, 1e300, -746.0, -1e300, 0.0])
    assert got[0] == np.inf and got[1] == 0 and np.isnan(got[2]) and got[3] == np.inf
    assert got[4] == np.inf and got[5] == 0 and got[6] == 0 and got[7] == 1.0


def test_sqrt_is_correctly_rounded(host):
    """The short square root against IEEE sqrt (NumPy's is the hardware instruction):
    equal bits on random arguments over the whole exponent range, on arguments next to
    perfect squares (where the rounding is decided by the last residual), and on the
    arguments that take the compiler's own path."""
    rs = np.random.RandomState(9)
    m = rs.uniform(1, 4, 1 << 20)
    exact = np.floor(rs.uniform(1, 2 ** 26, 1 << 16)) ** 2
    x = np.concatenate([m, np.ldexp(m, rs.randint(-766, 1020, m.size)), exact, np.nextafter(exact, 0),
                        np.nextafter(exact, np.inf), rs.uniform(0, 1e-300, 1 << 12),
                        [0.0, -0.0, np.inf, 4.0, 2.0, 1e-320, 5e-324, 2.0 ** -767, np.nextafter(2.0 ** -767, 0),
                         1.7976931348623157e308]])
    got = host("sqrt", x)
    assert got.tobytes() == np.sqrt(x).tobytes()
    bad = host("sqrt", [-1.0, -np.inf, np.nan])
    assert np.all(np.isnan(bad))


def test_device_source_compiles():
    for lds in (0, 256):
        src = mathlib.source(["log", "erf", "exp", "sqrt"], lds=lds)
        assert src.count("DR_STEP(") >= 13 and src.count("void dr_expm1_reduced(") == 1
        assert ("__shared__ DR_ALIGN16 double dr_erf_tab_lds[960]" in src) == bool(lds)
        stage = "DR_STAGE_TABLES(); " if lds else ""
        kernel = ('extern "C" __global__ void k(const double* a, double* o)\n'
                  "{ " + stage + "int i = threadIdx.x; const double x[2] = {a[2 * i], a[2 * i + 1]}; double p[2], q[2], r[2];\n"
                  "  dr_log_f8<2>(x, p); dr_erf_f8<2>(x, q); dr_exp_f8<2>(x, r); dr_sqrt_f8<2>(q, q);\n"
                  "  o[i] = p[0] + q[1] + r[0] + dr_log_f8_1(a[i]) + dr_erf_f8_1(a[i]) + dr_exp_f8_1(a[i]); }\n")
        assert len(hip.compile_source(src + kernel)) > 0


def test_packs_share_each_coefficient_between_their_elements():
    """The reason for packs: in the kernel's main loop a coefficient is moved into its
    scalar register pair once per pack.  Counted in the generated assembly: scalar moves
    per vector multiply-add must be well below the two that a lone element needs."""
    import re
    import shutil
    import tempfile
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = mathlib.source(["exp"]) + (
        'extern "C" __global__ void k(const double* a, double* o)\n'
        "{ const long i = 4L * (blockIdx.x * 256 + threadIdx.x);\n"
        "  const double x[4] = {a[i], a[i + 1], a[i + 2], a[i + 3]}; double r[4], k[4];\n"
        "  dr_expm1_reduced<4>(x, r, k); for (int e = 0; e < 4; e++) o[i + e] = r[e] + k[e]; }\n")
    with tempfile.TemporaryDirectory() as d:
        with open(f"{d}/k.hip", "w") as fh:
            fh.write(src)
        subprocess.run([hipcc, "-x", "hip", "-include", "hip/hip_runtime.h", "-O3", "-ffp-contract=off",
                        "--offload-arch=gfx950", "--cuda-device-only", "-S", "-o", f"{d}/k.s",
                        f"{d}/k.hip"], check=True, capture_output=True)
        asm = open(f"{d}/k.s").read()
    fma = len(re.findall(r"^\s+v_fma_f64", asm, re.M))
    smov = len(re.findall(r"^\s+s_mov_b32", asm, re.M))
    assert fma >= 4 * 9                       # the nine polynomial steps, per element
    assert smov < fma, (smov, fma)            # a lone element needs 2 moves per step


def test_erf_table_entries_are_what_they_claim():
    """Each row against 50-digit arithmetic: the point c lies inside its interval, the
    constant term is erf(c) rounded (within 0.25 ulp of it: the table adds little rounding of
    its own), the first row is centred on 0 with a zero constant term, and on a grid over
    the interval the row's polynomial is within 6e-17 of erf relative to erf.
    (`mathlib_fit.erf_table()` regenerates the table; it takes a few minutes.)"""
    import re
    nums = [float.fromhex(h) for h in re.findall(r"-?0x[01]\.[0-9a-f]+p[+-]\d+", mathlib.ERF_TABLE)]
    assert len(nums) == 960
    mp.mp.dps = 50
    assert nums[0] == 0.0 and nums[1] == 0.0
    for i in range(96):
        c, coef = nums[10 * i], nums[10 * i + 1:10 * i + 10]
        lo, hi = i / 16, (i + 1) / 16
        assert lo <= c < hi
        if i:
            exact = mp.erf(mp.mpf(c))
            assert float(exact) == coef[0]
            assert abs(exact - mp.mpf(coef[0])) <= mp.mpf("0.25") * mp.mpf(float(np.spacing(coef[0])))
        for k in range(0 if i else 1, 41):
            x = mp.mpf(lo) + (mp.mpf(hi) - mp.mpf(lo)) * k / 40
            t, p = x - mp.mpf(c), mp.mpf(0)
            for a in reversed(coef):
                p = p * t + mp.mpf(a)
            assert abs(p - mp.erf(x)) <= mp.mpf("6e-17") * mp.erf(x), (i, k)


def test_programs_name_the_functions_they_replace():
    from delayrepay_amd.codegen import Program
    ops = [("log", "f8", "f8", (("l", 0),)), ("erf", "f4", "f4", (("l", 1),))]
    prog = Program(["f8", "f4"], [], ops, [(("v", 0), "f8")])
    assert prog.own_math == ("log",)                 # float32 keeps the device library's erf
    plain = Program(["f8", "f4"], [], ops, [(("v", 0), "f8")], own_math=False)
    assert plain.own_math == () and plain.key() != prog.key()


def test_coefficients_are_the_ones_the_fit_script_prints(capsys):
    import re
    from delayrepay_amd import mathlib_fit
    mathlib_fit.main()
    printed = set(re.findall(r"-?0x1\.[0-9a-f]+p[+-]\d+", capsys.readouterr().out))
    used = set()
    for _, pieces in mathlib.FUNCTIONS.values():
        for piece in pieces:
            if piece not in (mathlib.LOG_TABLE, mathlib.ERF_TABLE):
                used |= set(re.findall(r"-?0x1\.[0-9a-f]+p[+-]\d+", piece))
    printed |= {"-" + h for h in printed}                       # -ln 2 (hi, lo)
    assert used - printed == {"0x1.7ffffffffffffp+2"}            # the last double below 6
    assert float.fromhex("0x1.7ffffffffffffp+2") == np.nextafter(6.0, 0)


def test_log_table_entries_are_what_they_claim():
    """Each entry against 60-digit arithmetic: log c is the double nearest to -log(1/c) and
    lies within 0.004 ulp of it; c sits within 2^-23 of its interval's centre; at the
    interval's ends |z/c - 1| stays at 2^-9; the interval around 1 has c = 1 exactly.
    (`mathlib_fit.log_table()` regenerates the table; it takes a minute.)"""
    import re
    from delayrepay_amd import mathlib_fit as mf
    nums = [float.fromhex(h) for h in re.findall(r"-?0x[01]\.[0-9a-f]+p[+-]\d+", mathlib.LOG_TABLE)]
    assert len(nums) == 2 * mf.LOG_INTERVALS
    mp.mp.dps = 60
    assert mf.log_interval(0)[0] == 0.7060546875 and mf.log_interval(255)[1] == 2 * 0.7060546875
    assert mf.log_interval(mf.LOG_CENTRE) == (1 - 2.0 ** -10, 1 + 2.0 ** -9)
    assert nums[2 * mf.LOG_CENTRE] == 1.0 and nums[2 * mf.LOG_CENTRE + 1] == 0.0
    for i in range(mf.LOG_INTERVALS):
        invc, logc = nums[2 * i], nums[2 * i + 1]
        lo, hi = mf.log_interval(i)
        assert abs(mp.mpf(invc) * (mp.mpf(lo) + mp.mpf(hi)) / 2 - 1) < mp.mpf(2) ** -23 or i == mf.LOG_CENTRE
        for z in (lo, hi):
            assert abs(mp.mpf(z) * mp.mpf(invc) - 1) <= mp.mpf(2) ** -9 * (1 + mp.mpf(2) ** -13)
        if i != mf.LOG_CENTRE:
            exact = -mp.log(mp.mpf(invc))
            assert float(exact) == logc
            assert abs(exact - mp.mpf(logc)) <= mp.mpf("0.0041") * mp.mpf(float(np.spacing(abs(logc))))
    assert "0x3fe69800u" in mathlib.LOG_CORE and mf.LOG_OFF >> 32 == 0x3fe69800 and mf.LOG_OFF & 0xffffffff == 0


# ---- float32 functions (mathlib32) ---------------------------------------------------------

@pytest.fixture(scope="module")
def host32(tmp_path_factory):
    """`mathlib32` built for the host: the two hardware functions (2^x, log2 x) are taken
    from libm here, so this checks the argument reductions, the polynomials and the
    special cases; the device's own 1-ulp versions are measured in the GPU tests."""
    from delayrepay_amd import mathlib32
    d = tmp_path_factory.mktemp("mathlib32")
    src = "#include <math.h>\n" + mathlib32.source(sorted(mathlib32.FUNCTIONS), mathlib32.HOST_MACROS,
                                                   soft_div=True)
    for name, (fn, _) in mathlib32.FUNCTIONS.items():
        src += (f'extern "C" void v_{name}(const float* x, float* y, long n)\n'
                f"{{ for (long i = 0; i < n; i++) y[i] = {fn}(x[i]); }}\n")
    # the short division: packs of four (the form the kernels use), then one at a time
    src += ('extern "C" void v_div(const float* a, const float* b, float* y, long n)\n'
            "{ long i = 0;\n"
            "  for (; i + 4 <= n; i += 4) { const float p[4] = {a[i], a[i+1], a[i+2], a[i+3]}, "
            "q[4] = {b[i], b[i+1], b[i+2], b[i+3]}; float r[4]; dr_div_f4_pack<4>(p, q, r); "
            "for (int e = 0; e < 4; e++) y[i+e] = r[e]; }\n"
            "  for (; i < n; i++) y[i] = dr_div_f4(a[i], b[i]); }\n")
    (d / "m.cpp").write_text(src)
    subprocess.run(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", str(d / "m.so"),
                    str(d / "m.cpp"), "-lm"], check=True)
    lib = ctypes.CDLL(str(d / "m.so"))

    def call(name, x, other=None):
        if name == "div":
            a, b = (np.ascontiguousarray(v, dtype=np.float32) for v in (x, other))
            y = np.empty_like(a)
            lib.v_div(a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p),
                      y.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(a.size))
            return y
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.empty_like(x)
        getattr(lib, "v_" + name)(x.ctypes.data_as(ctypes.c_void_p),
                                  y.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(x.size))
        return y
    return call


def ulp32(got, exact64):
    """Error of float32 results in float32 ulps of the exact value (given in float64)."""
    scale = np.spacing(np.abs(exact64).astype(np.float32)).astype(np.float64)
    return np.abs(got.astype(np.float64) - exact64) / scale


def test_float32_erf(host32):
    rs = np.random.RandomState(6)
    x = np.concatenate([rs.uniform(-4.5, 4.5, 1 << 20), rs.uniform(-1, 1, 1 << 19),
                        rs.uniform(0.87, 0.88, 1 << 16), 10.0 ** rs.uniform(-44, 0, 1 << 16),
                        [0.875, np.nextafter(np.float32(0.875), 0), 3.9, 4.0, 4.1, 1e-45, 1e30]]
                       ).astype(np.float32)
    got = host32("erf", x)
    exact = scipy.special.erf(x.astype(np.float64))
    assert ulp32(got, exact).max() <= 1.5
    assert np.all(np.abs(got) <= 1.0) and np.array_equal(host32("erf", -x), -got)
    near = np.sort(rs.uniform(0.8749, 0.8751, 4096).astype(np.float32))      # across the switch
    assert np.all(np.diff(host32("erf", near)) >= -np.spacing(np.float32(0.5)))
    sp = host32("erf", [0.0, -0.0, np.inf, -np.inf, np.nan, 40.0, -40.0])
    assert sp[0] == 0 and not np.signbit(sp[0]) and sp[1] == 0 and np.signbit(sp[1])
    assert sp[2] == 1 and sp[3] == -1 and np.isnan(sp[4]) and sp[5] == 1 and sp[6] == -1


def test_float32_exp(host32):
    rs = np.random.RandomState(7)
    x = np.concatenate([rs.uniform(-104, 89, 1 << 20), rs.uniform(-1, 1, 1 << 18),
                        [0.0, -0.0, 88.72283, 88.72284, -87.33654, -103.97, -104.1, 87.0, -87.0]]
                       ).astype(np.float32)
    got = host32("exp", x)
    with np.errstate(over="ignore", under="ignore"):
        exact = np.exp(x.astype(np.float64))
    normal = (exact >= np.finfo(np.float32).tiny) & (exact <= np.finfo(np.float32).max)
    assert ulp32(got[normal], exact[normal]).max() <= 1.0
    small = exact < np.finfo(np.float32).tiny
    assert np.max(np.abs(got[small].astype(np.float64) - exact[small]) / 1.401298464324817e-45) <= 1.0
    with np.errstate(over="ignore"):
        assert np.array_equal(np.isinf(got), np.isinf(np.exp(x)))
    sp = host32("exp", [np.inf, -np.inf, np.nan, 89.0, 1e30, -105.0, -1e30, 0.0])
    assert sp[0] == np.inf and sp[1] == 0 and np.isnan(sp[2]) and sp[3] == np.inf
    assert sp[4] == np.inf and sp[5] == 0 and sp[6] == 0 and sp[7] == 1.0


def test_float32_log(host32):
    rs = np.random.RandomState(8)
    x = np.concatenate([rs.uniform(1e-6, 1e6, 1 << 19), np.exp(rs.uniform(-103, 88, 1 << 19)),
                        rs.uniform(0.5, 2, 1 << 19), 1 + rs.uniform(-1e-3, 1e-3, 1 << 16),
                        [1e-45, 1.1754944e-38, 1e-40, 1.0, np.nextafter(np.float32(1), 2),
                         np.nextafter(np.float32(1), 0), 3.4028235e38]]).astype(np.float32)
    got = host32("log", x)
    exact = np.log(x.astype(np.float64))
    nz = exact != 0
    # the stand-in log2f is itself up to 0.8 ulp off, and that error passes straight through
    assert ulp32(got[nz], exact[nz]).max() <= 1.6 and np.all(got[~nz] == 0)
    sp = host32("log", [0.0, -0.0, -1.0, -np.inf, np.inf, np.nan, 1.0])
    assert sp[0] == -np.inf and sp[1] == -np.inf
    assert np.isnan(sp[2]) and np.isnan(sp[3]) and np.isnan(sp[5])
    assert sp[4] == np.inf and sp[6] == 0.0 and not np.signbit(sp[6])


def test_float32_device_source_compiles_to_the_hardware_functions():
    import re
    import shutil
    import tempfile
    from delayrepay_amd import mathlib32
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = mathlib32.source(["erf", "exp", "log"]) + (
        'extern "C" __global__ void k(const float* a, float* o)\n'
        "{ const int i = blockIdx.x * 256 + threadIdx.x;\n"
        "  o[i] = dr_erf_f4(a[i]) + dr_exp_f4(a[i]) * dr_log_f4(a[i]); }\n")
    assert len(hip.compile_source(src)) > 0
    with tempfile.TemporaryDirectory() as d:
        with open(f"{d}/k.hip", "w") as fh:
            fh.write(src)
        subprocess.run([hipcc, "-x", "hip", "-include", "hip/hip_runtime.h", "-O3", "-ffp-contract=off",
                        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                        "--offload-arch=gfx950", "--cuda-device-only", "-S", "-o", f"{d}/k.s",
                        f"{d}/k.hip"], check=True, capture_output=True)
        asm = open(f"{d}/k.s").read()
    assert len(re.findall(r"^\s+v_exp_f32", asm, re.M)) >= 2 and len(re.findall(r"^\s+v_log_f32", asm, re.M)) >= 1
    assert not re.findall(r"^\s+v_pk_\w+_f32", asm, re.M)


def test_quotients_that_only_inexact_functions_read(host):
    """`dr_div_f8` (eight operations instead of the correctly rounded division's thirteen):
    the correctly rounded quotient nearly always, never more than one ulp from it; zero,
    infinite, NaN, denormal and overflowing cases are NumPy's."""
    rs = np.random.RandomState(11)
    n = 1 << 20
    a = np.concatenate([rs.uniform(-100, 100, n), np.exp(rs.uniform(-300, 300, n)) * rs.choice([-1, 1], n)])
    b = np.concatenate([rs.uniform(0.1, 100, n) * rs.choice([-1, 1], n), np.exp(rs.uniform(-300, 300, n))])
    got, ref = host("div", a, b), a / b
    off = np.abs(got - ref) / np.spacing(np.abs(ref))
    assert off.max() <= 1.0
    assert np.count_nonzero(off) <= a.size // 50000         # measured: none in 2^21
    with np.errstate(all="ignore"):
        sa = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1.0, 0.0, np.inf, 1e308, 1e-308,
                       5e-324, 1.0, 1e-320, 3.0, 1e300, -1e-300, 2.0, 7.0, 1e-310, 5e-324, 3e-305])
        sb = np.array([1.0, 2.0, 0.0, -0.0, 2.0, -3.0, 1.0, np.nan, 0.0, np.inf, 1e-308, 1e308,
                       2.0, 5e-324, 1e-320, np.inf, 1e-300, 1e300, 1e-310, 1.7976931348623157e308,
                       1e-250, 1e-250, 7e-200])
        want = sa / sb
    res = host("div", sa, sb)
    assert np.array_equal(np.isnan(res), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(res[ok], want[ok]) and np.array_equal(np.signbit(res[ok]), np.signbit(want[ok]))
    # one at a time and in packs: the same arithmetic
    assert np.array_equal(host("div", a[:1001], b[:1001]),
                          np.concatenate([host("div", a[i:i + 1], b[i:i + 1]) for i in range(1001)]))


def test_square_roots_that_only_inexact_functions_read(host):
    """`dr_sqrt_near_f8` (seven operations instead of ten): the correctly rounded root nearly
    always, never more than one ulp from it; zero, negative, infinite, NaN and tiny
    arguments give what `sqrt` gives."""
    rs = np.random.RandomState(12)
    n = 1 << 20
    x = np.concatenate([rs.uniform(0, 100, n), np.exp(rs.uniform(-500, 700, n))])
    got, ref = host("sqrt_near", x), np.sqrt(x)
    off = np.abs(got - ref) / np.spacing(ref)
    assert off.max() <= 1.0
    assert np.count_nonzero(off) <= x.size // 50000
    with np.errstate(all="ignore"):
        sx = np.array([0.0, -0.0, -1.0, np.inf, -np.inf, np.nan, 5e-324, 1e-310, 2.2250738585072014e-308,
                       1e-250, 1.7976931348623157e308, 4.0, 2.0])
        want = np.sqrt(sx)
    res = host("sqrt_near", sx)
    assert np.array_equal(np.isnan(res), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(res[ok], want[ok]) and np.array_equal(np.signbit(res[ok]), np.signbit(want[ok]))


def test_only_quotients_that_no_root_can_see_are_computed_that_way():
    from delayrepay_amd import codegen as cg
    def soft(ops, roots):
        return cg.Program(["f8", "f8"], [], ops, roots).soft_div
    div = ("divide", "f8", "f8", (("l", 0), ("l", 1)))
    log = lambda j: ("log", "f8", "f8", (("v", j),))
    add = lambda i, j: ("add", "f8", "f8", (("v", i), ("v", j)))
    assert soft([div, log(0)], [(("v", 1), "f8")]) == (0,)                       # log(a / b)
    assert soft([div], [(("v", 0), "f8")]) == ()                                 # a / b itself
    assert soft([div, log(0), add(0, 1)], [(("v", 2), "f8")]) == ()              # a / b + log(a / b)
    assert soft([div, log(0)], [(("v", 1), "f8"), (("v", 0), "f8")]) == ()       # both are roots
    assert soft([div, ("sqrt", "f8", "f8", (("v", 0),))], [(("v", 1), "f8")]) == ()      # sqrt is exact
    root = ("sqrt", "f8", "f8", (("l", 0),))
    erf = lambda j: ("erf", "f8", "f8", (("v", j),))
    assert soft([root, erf(0)], [(("v", 1), "f8")]) == (0,)                      # erf(sqrt(a)): the root too
    assert soft([root, erf(0), add(0, 1)], [(("v", 2), "f8")]) == ()             # sqrt(a) + erf(sqrt(a))
    assert cg.Program(["f8", "f8"], [], [root, erf(0)], [(("v", 1), "f8")], own_math=False).soft_div == ()
    assert soft([div, ("multiply", "f8", "f8", (("v", 0), ("l", 0))), ("erf", "f8", "f8", (("v", 1),))],
                [(("v", 2), "f8")]) == (0,)                                      # erf(a / b * a)
    f4 = [("divide", "f4", "f4", (("l", 0), ("l", 1))), ("log", "f4", "f4", (("v", 0),))]
    assert soft(f4, [(("v", 1), "f4")]) == ()                                    # float32: only on request
    assert cg.Program(["f4", "f4"], [], f4, [(("v", 1), "f4")], soft_div=2).soft_div == (0,)
    assert cg.Program(["f8", "f8"], [], [div, log(0)], [(("v", 1), "f8")], soft_div=False).soft_div == ()


def test_float32_quotients_that_only_inexact_functions_read(host32):
    """`dr_div_f4`: within one ulp of the exact quotient (here with a correctly rounded
    reciprocal standing in for the hardware's, which is within one ulp: the device build is
    measured in the GPU tests), special cases as NumPy's."""
    rs = np.random.RandomState(12)
    n = 1 << 21
    a = np.concatenate([rs.uniform(-100, 100, n), np.exp(rs.uniform(-40, 40, n))]).astype(np.float32)
    b = np.concatenate([rs.uniform(0.1, 100, n) * rs.choice([-1, 1], n), np.exp(rs.uniform(-40, 40, n))]
                       ).astype(np.float32)
    got = host32("div", a, b)
    exact = a.astype(np.float64) / b.astype(np.float64)
    assert ulp32(got, exact).max() <= 1.0
    with np.errstate(all="ignore"):
        sa = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1.0, 0.0, np.inf, 1e38, 1e-38,
                       1e-45, 1.0, 1e-40, 3.0, 1e30, -1e-30, 2.0], dtype=np.float32)
        sb = np.array([1.0, 2.0, 0.0, -0.0, 2.0, -3.0, 1.0, np.nan, 0.0, np.inf, 1e-38, 1e38,
                       2.0, 1e-45, 1e-40, np.inf, 1e-30, 1e30, 1e-39], dtype=np.float32)
        want = sa / sb
    res = host32("div", sa, sb)
    assert np.array_equal(np.isnan(res), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(res[ok], want[ok]) and np.array_equal(np.signbit(res[ok]), np.signbit(want[ok]))
