"""GPU: brute force over the arithmetic shortcuts of the wave-scaling kernels.

The kernels divide integers through a float reciprocal, take a ceiling through
a float product, divide doubles by constants through a corrected multiplication
and raise 2 to a power through a polynomial.  Each shortcut's comment states
the domain it is exact (or accurate) on; tests/native/device_arith.hip compiles
the product's own device functions into checkers that walk that whole domain on
the GPU, or 2^30 operands where the domain is the doubles, against integer
division, IEEE division and the device library's exp2."""
import ctypes
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "_build",
                   "libdevice_arith.so")


@pytest.fixture(scope="module")
def arith():
    if not os.path.exists(LIB):
        pytest.fail("tests/native/_build/libdevice_arith.so is not built: run "
                    "`make -C tests/native` (or __graft_entry__.build()) first")
    lib = ctypes.CDLL(LIB)
    u64p = ctypes.POINTER(ctypes.c_uint64)
    lib.arith_fast_div.argtypes = [ctypes.c_int32, u64p]
    lib.arith_ceil_div.argtypes = [ctypes.c_int32, u64p]
    lib.arith_div_const.argtypes = [ctypes.c_int64, ctypes.c_uint64, ctypes.c_uint64, u64p]
    lib.arith_exp2.argtypes = [ctypes.c_double, ctypes.c_double, ctypes.c_uint64,
                               ctypes.POINTER(ctypes.c_double)]
    lib.arith_exp2_at.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p]
    lib.arith_occupancy_lattice.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint32), u64p]
    return lib


def test_reciprocal_division_is_exact_on_its_whole_domain(arith):
    """fast_div_r: every a >= 0, b > 0 with a + b <= 2^21, 2.2e12 pairs."""
    limit = 1 << 21
    out = (ctypes.c_uint64 * 4)()
    print("fast_div: all pairs with a + b <= 2^21 ...", flush=True)
    assert arith.arith_fast_div(limit, out) == 0
    checked, bad = out[0], out[1]
    print("fast_div: %d pairs, %d mismatches" % (checked, bad), flush=True)
    assert bad == 0, "a=%d b=%d" % (out[2], out[3])
    assert checked == limit * (limit + 1) // 2


def test_small_kernel_ceiling_is_exact_on_its_whole_domain(arith):
    """ceil_div_small: every multiprocessor count up to 2^14 and every block
    count below 64 waves' worth (the occupancy models give at most 40)."""
    sms_end = 1 << 14
    out = (ctypes.c_uint64 * 4)()
    assert arith.arith_ceil_div(sms_end, out) == 0
    checked, bad = out[0], out[1]
    print("ceil_div_small: %d pairs, %d mismatches" % (checked, bad), flush=True)
    assert bad == 0, "nb=%d sms=%d" % (out[2], out[3])
    assert checked == 64 * sms_end * (sms_end + 1) // 2


@pytest.mark.parametrize("constant", [100, 1_000_000_000])
def test_division_by_a_constant_is_the_ieee_quotient(arith, constant):
    """div_const: 2^30 operands as raw bit patterns (a quarter of them with
    short mantissas), bit for bit against the division it replaces, the
    sign of a zero aside."""
    out = (ctypes.c_uint64 * 4)()
    n = 1 << 30
    assert arith.arith_div_const(constant, n, 12345, out) == 0
    checked, bad = out[0], out[1]
    print("div_const<%d>: %d operands, %d mismatches, %d zeros of the other sign" %
          (constant, checked, bad, out[3]), flush=True)
    assert bad == 0, "x = %r" % np.array([out[2]], np.uint64).view(np.float64)[0]
    # x = -0.0 gives +0.0 where the division gives -0.0 (some 1 300 of the
    # operands are negative zeros); the kernels only compare the result with
    # 1e-9, which no zero passes
    assert out[3] < 3000
    # raw patterns: 1/2048 are inf/NaN, some 6 % lie below 2^-900
    assert 0.90 * n < checked < n


def test_power_of_two_polynomial(arith):
    """exp2_poly: relative error below 1e-13 (observed: printed) on 2^28 points
    over the normal range and on a fine grid around 0; exact at integers;
    finite arguments beyond the exponent range saturate, NaN stays NaN."""
    out = (ctypes.c_double * 2)()
    n = 1 << 28
    assert arith.arith_exp2(-1021.0, 2044.0 / n, n, out) == 0
    print("exp2_poly on [-1021, 1023): worst relative error %.3g over %d points" %
          (out[0], int(out[1])), flush=True)
    assert out[1] == n and out[0] < 1e-13
    assert arith.arith_exp2(-2.0, 4.0 / n, n, out) == 0
    print("exp2_poly on [-2, 2): worst relative error %.3g" % out[0], flush=True)
    assert out[1] == n and out[0] < 1e-13
    x = np.array([0.0, 1.0, -1.0, 10.0, 1023.0, -1022.0, 1024.0, 5000.0, 1e300,
                  -1100.0, -5000.0, -1e300, np.nan, 0.5, -0.5])
    y = np.empty_like(x)
    assert arith.arith_exp2_at(x.ctypes.data, len(x), y.ctypes.data) == 0
    assert list(y[:6]) == [1.0, 2.0, 0.5, 1024.0, 2.0 ** 1023, 2.0 ** -1022]
    assert np.all(np.isposinf(y[6:9]))
    assert np.all(y[9:12] == 0.0)
    assert np.isnan(y[12])
    assert abs(y[13] / 2 ** 0.5 - 1) < 1e-13 and abs(y[14] / 2 ** -0.5 - 1) < 1e-13


def test_32bit_occupancy_models_equal_the_64bit_ones_on_a_lattice(arith, occupancy_golden):
    """Every variant of the occupancy model the kernels can run for a device
    (32-bit arithmetic with reciprocal divisions, with and without the
    branches that are uniform over a launch) against the 64-bit model with
    plain divisions, which the CPU tests hold against the compiled reference:
    1102 block sizes x 302 register counts x 3098 shared-memory sizes per
    device, for the 15 device descriptions of the reference-built fixture and
    the compute-unit reading of the one that has one."""
    from habitat_amd import DeviceProperties
    from habitat_amd.analysis.wave_scaling.cdna import native_description
    _, described = occupancy_golden
    specs = []
    for name, kwargs in described.items():
        dev = DeviceProperties(name=name, **{k: v for k, v in kwargs.items() if k != "name"})
        specs.append((name, dev))
        native = native_description(dev)
        if native.compute_capability != dev.compute_capability:
            specs.append((name + " as compute units", native))
            odd = dict(native.as_dict(), warp_size=48)     # not a power of two: no lean form
            specs.append((name + " as compute units, 48 lanes",
                          DeviceProperties(name=name + "_48", **odd)))
    total, seen = 0, 0
    for name, dev in specs:
        out = (ctypes.c_uint64 * 4)()
        variants = ctypes.c_uint32(0)
        assert arith.arith_occupancy_lattice(ctypes.addressof(dev.spec), ctypes.byref(variants),
                                             out) == 0, name
        checked, bad = out[0], out[1]
        assert checked == 1102 * 302 * 3098
        assert bad == 0, "%s: block %d smem %d regs %d variants %#x" % (
            name, np.int32(out[2] >> 32), np.int32(out[2] & 0xffffffff), out[3] >> 32,
            out[3] & 0xff)
        total += checked * bin(variants.value).count("1")
        seen |= variants.value
    print("occupancy lattice: %d descriptions, %.3g (configuration, variant) pairs, variants %#x" %
          (len(specs), total, seen), flush=True)
    assert seen == 0x1f       # every variant ran for some device
