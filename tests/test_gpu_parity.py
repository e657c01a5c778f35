"""GPU parity: the HIP library, called through its C ABI, against the CPU
oracle on the same inputs.  Bit-exact for every integer result (sort, scan,
reduce, histogram) and for stable pair order; floating-point sums within the
tolerance written in each test."""
import sys

import numpy as np
import pytest

from ilgpu_amd import capi, datagen
from oracle import cpu_oracle as O
from tests.refcases import (ALL_KEY_DTYPES, ARRAY_SIZES, ATOMIC_NUMERIC_DTYPES,
                            compute_inverted_sequence, compute_sequence)

pytestmark = pytest.mark.gpu

D = capi.DeviceArray
INT_KEY_DTYPES = [d for d in ALL_KEY_DTYPES if np.dtype(d).kind in "iu"]
SCAN_DTYPES = ATOMIC_NUMERIC_DTYPES
OPS = [capi.OP_ADD, capi.OP_MAX, capi.OP_MIN]


def note(*args):
    print(*args, flush=True)
    sys.stdout.flush()


def sync():
    import torch
    torch.cuda.synchronize()


def random_ints(dtype, n, seed=0, lo=None, hi=None):
    info = np.iinfo(dtype)
    lo = info.min if lo is None else lo
    hi = info.max if hi is None else hi
    return np.random.default_rng(seed).integers(lo, hi, size=n, dtype=dtype,
                                                endpoint=True)


def random_float_bits(dtype, n, seed=0):
    """Arbitrary bit patterns (includes negatives, NaNs, infinities, -0)."""
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dtype).itemsize]
    return random_ints(u, n, seed).view(dtype)


# ------------------------------------------------------------------- reduce
def gpu_reduce(values, op):
    d_in = D.from_numpy(values)
    d_out = D.zeros(1, values.dtype)
    capi.reduce(d_in, d_out, op=op)
    sync()
    return d_out.numpy()[0]


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.uint32, np.uint64])
@pytest.mark.parametrize("op", OPS)
def test_reduce_integers_exact(dtype, op):
    for n in ARRAY_SIZES + [4096, 100003, (1 << 20) + 7]:
        note("reduce", np.dtype(dtype).name, op, n)
        v = random_ints(dtype, n, seed=n)
        assert gpu_reduce(v, op) == O.reduce(v, op=op), n


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", ARRAY_SIZES[:-1] + [1000])
def test_reduce_reference_float_sequences_exact(dtype, n):
    # ReductionExtensionTests.tt:41-106: small integers, every partial sum is
    # exactly representable, so the result must equal the left fold exactly.
    for start, step in [(0, 1), (1, 0)]:
        seq = compute_sequence(dtype, start, step, n)
        for op in OPS:
            assert gpu_reduce(seq, op) == O.reduce(seq, op=op)


@pytest.mark.parametrize("n", [1, 3, 1000, 65537, 1 << 22])
def test_reduce_float32_add_tolerance(n):
    # Contract: |gpu - float64 host sum| <= 1e-5 * |float64 host sum|.
    v = datagen.normal_f32(n, seed=n)
    exact = O.sum_f64(v)
    got = float(gpu_reduce(v, capi.OP_ADD))
    note("reduce f32 add", n, got, exact)
    # one float32 rounding of the exact sum is allowed on top
    assert abs(got - exact) <= 1e-5 * abs(exact) + abs(exact) * 2.0 ** -24


def test_reduce_float64_add_tolerance():
    v = np.random.default_rng(1).standard_normal(1 << 20)
    exact = O.sum_f64(v)
    assert abs(float(gpu_reduce(v, capi.OP_ADD)) - exact) <= 1e-10 * max(1.0, abs(exact))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reduce_float_max_min_semantics(dtype):
    v = np.random.default_rng(2).standard_normal(50000).astype(dtype)
    assert gpu_reduce(v, capi.OP_MAX) == v.max()
    assert gpu_reduce(v, capi.OP_MIN) == v.min()
    w = v.copy()
    w[12345] = np.nan  # Math.Max/Min propagate NaN
    assert np.isnan(gpu_reduce(w, capi.OP_MAX)) and np.isnan(gpu_reduce(w, capi.OP_MIN))
    z = np.array([0.0, -0.0, 0.0], dtype=dtype)
    assert np.signbit(gpu_reduce(z, capi.OP_MIN))
    assert not np.signbit(gpu_reduce(z, capi.OP_MAX))
    neg = np.full(100, -5.0, dtype=dtype)
    assert gpu_reduce(neg, capi.OP_MAX) == -5.0


def test_reduce_overwrites_output_and_accepts_unaligned_views():
    v = random_ints(np.int32, 10000, seed=3)
    d_all = D.from_numpy(v)
    for off, n in [(1, 9999), (3, 5), (2, 4097), (5, 1)]:
        d_out = D.from_numpy(np.array([12345, 777], dtype=np.int32))
        capi.reduce(d_all.subview(off, n), d_out)
        sync()
        out = d_out.numpy()
        with np.errstate(over="ignore"):
            assert out[0] == np.sum(v[off:off + n], dtype=np.int32)
        assert out[1] == 777  # only output[0] is written (ReductionExtensions.cs:156)


# --------------------------------------------------------------------- scan
def gpu_scan(values, op, inclusive, out_extra=0):
    d_in = D.from_numpy(values)
    d_out = D.from_numpy(np.full(values.size + out_extra, 77, dtype=values.dtype))
    capi.scan(d_in, d_out, op=op,
              kind=capi.SCAN_INCLUSIVE if inclusive else capi.SCAN_EXCLUSIVE)
    sync()
    return d_out.numpy()


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.uint32, np.uint64])
@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("inclusive", [True, False])
def test_scan_integers_exact(dtype, op, inclusive):
    for n in ARRAY_SIZES + [2048, 4095, 4096, 4097, 100003, (1 << 20) + 13]:
        note("scan", np.dtype(dtype).name, op, inclusive, n)
        v = random_ints(dtype, n, seed=n)
        got = gpu_scan(v, op, inclusive)
        assert np.array_equal(got, O.scan(v, op=op, inclusive=inclusive)), n


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("inclusive", [True, False])
def test_scan_reference_float_sequences_exact(dtype, inclusive):
    # ScanExtensionTests.tt:43-104 (floats up to 1000 elements): all partial
    # results are exactly representable, so equality is exact.
    for n in [1, 31, 33, 127, 1000]:
        for start, step in [(0, 1), (1, 0), (n, -1)]:
            seq = compute_sequence(dtype, start, step, n)
            for op in OPS:
                got = gpu_scan(seq, op, inclusive)
                assert np.array_equal(got, O.scan(seq, op=op, inclusive=inclusive))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_scan_float_add_tolerance(dtype):
    # The association order differs from the reference's 16-wide group scan;
    # tolerance: 1e-5 (f32) / 1e-12 (f64) of the running sum of |x|.
    n = 200003
    v = np.random.default_rng(5).standard_normal(n).astype(dtype)
    exact = np.cumsum(v.astype(np.float64))
    scale = np.cumsum(np.abs(v.astype(np.float64)))
    tol = 1e-5 if dtype == np.float32 else 1e-12
    got = gpu_scan(v, capi.OP_ADD, True).astype(np.float64)
    assert np.all(np.abs(got - exact) <= tol * scale + 1e-30)
    got = gpu_scan(v, capi.OP_ADD, False).astype(np.float64)
    assert got[0] == 0.0
    assert np.all(np.abs(got[1:] - exact[:-1]) <= tol * scale[:-1] + 1e-30)
    assert np.array_equal(gpu_scan(v, capi.OP_MAX, True), np.maximum.accumulate(v))
    assert np.array_equal(gpu_scan(v, capi.OP_MIN, True), np.minimum.accumulate(v))


def test_scan_longer_output_in_place_and_unaligned_views():
    v = random_ints(np.int32, 50000, seed=8)
    with np.errstate(over="ignore"):
        inc = np.cumsum(v, dtype=np.int32)
    # output longer than input: only the first n are written (ScanExtensions.cs:679)
    got = gpu_scan(v, capi.OP_ADD, True, out_extra=5)
    assert np.array_equal(got[:-5], inc) and np.all(got[-5:] == 77)
    # in place
    d = D.from_numpy(v)
    capi.scan(d, d)
    sync()
    assert np.array_equal(d.numpy(), inc)
    # element-aligned but not 16-byte aligned views
    d_in = D.from_numpy(v)
    d_out = D.zeros(v.size, np.int32)
    for off, n in [(1, 40001), (3, 4096), (2, 7)]:
        capi.scan(d_in.subview(off, n), d_out.subview(1, n), kind=capi.SCAN_EXCLUSIVE)
        sync()
        with np.errstate(over="ignore"):
            e = np.concatenate([[0], np.cumsum(v[off:off + n], dtype=np.int32)[:-1]])
        assert np.array_equal(d_out.numpy()[1:1 + n], e.astype(np.int32))


def test_scan_temp_buffer_can_be_reused_dirty():
    v = datagen.small_ints_i32(300000, seed=1)
    d_in, d_out = D.from_numpy(v), D.zeros(v.size, np.int32)
    temp = capi.temp_buffer(capi.scan_temp_bytes(v.size, np.int32))
    temp.bytes.fill_(0xFF)
    for _ in range(3):
        capi.scan(d_in, d_out, temp, kind=capi.SCAN_EXCLUSIVE)
        sync()
        assert np.array_equal(d_out.numpy(), O.scan(v, inclusive=False))


# ---------------------------------------------------------------- histogram
HIST_IN_DTYPES = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16,
                  np.uint32, np.uint64, np.float32, np.float64]
HIST_BIN_DTYPES = [np.int32, np.int64, np.uint32, np.uint64]


def gpu_histogram(values, bins, locator, overflow=0, checked=True):
    d_in, d_bins = D.from_numpy(values), D.from_numpy(bins)
    d_ov = D.from_numpy(np.array([overflow], dtype=np.int32))
    capi.histogram(d_in, d_bins, d_ov if checked else None, locator=locator)
    sync()
    return d_bins.numpy(), int(d_ov.numpy()[0])


@pytest.mark.parametrize("in_dtype", HIST_IN_DTYPES)
@pytest.mark.parametrize("bin_dtype", HIST_BIN_DTYPES)
def test_histogram_reference_cases(in_dtype, bin_dtype):
    # HistogramTests.tt:99-144 and :146-203.
    values = np.arange(1, 1025).astype(in_dtype)
    for num_bins in (64, 256):
        zero = np.zeros(num_bins, dtype=bin_dtype)
        assert_hist_equal(values, zero, capi.LOCATOR_MODULO)
    info = np.iinfo(bin_dtype)
    small = np.arange(1, 33).astype(in_dtype)
    start = np.array([info.max - 32 - 1], dtype=bin_dtype)
    bins1, ov1 = gpu_histogram(small, start, capi.LOCATOR_MODULO)
    e1, eo1 = O.histogram(small, start, locator=O.LOCATOR_MODULO)
    assert np.array_equal(bins1, e1) and ov1 == eo1 == 0
    bins2, ov2 = gpu_histogram(small, bins1, capi.LOCATOR_MODULO)
    e2, eo2 = O.histogram(small, e1, locator=O.LOCATOR_MODULO)
    assert np.array_equal(bins2, e2) and ov2 == eo2 == 1


def assert_hist_equal(values, bins, locator, overflow=0):
    got, ov = gpu_histogram(values, bins, locator, overflow)
    exp, eov = O.histogram(values, bins, locator=locator, overflow=overflow)
    assert np.array_equal(got, exp)
    assert ov == eov


@pytest.mark.parametrize("n", [1, 100, 4099, (1 << 20) + 3])
def test_histogram_bytes_256_bins(n):
    note("hist u8", n)
    v = datagen.bytes_u8(n, seed=n)
    pre = random_ints(np.int32, 256, seed=1, lo=0, hi=1000)
    assert_hist_equal(v, pre, capi.LOCATOR_IDENTITY)
    # skew: a constant input hits one bin
    assert_hist_equal(np.full(n, 200, dtype=np.uint8), pre, capi.LOCATOR_IDENTITY)


@pytest.mark.parametrize("n", [1000, (1 << 20) + 5])
def test_histogram_4096_bins_gaussian_mixture(n):
    v = datagen.gaussian_mixture_i32(n, seed=n)
    assert v.min() >= 0 and v.max() <= 4095
    assert_hist_equal(v, np.zeros(4096, dtype=np.int32), capi.LOCATOR_IDENTITY)
    assert_hist_equal(v, np.zeros(4096, dtype=np.uint64), capi.LOCATOR_IDENTITY)


def test_histogram_many_bins_uses_global_atomics():
    n, bins = 200000, 100000
    v = random_ints(np.int32, n, seed=4, lo=0, hi=bins - 1)
    assert_hist_equal(v, np.zeros(bins, dtype=np.int32), capi.LOCATOR_IDENTITY)
    w = random_ints(np.int64, n, seed=5)
    assert_hist_equal(w, np.zeros(bins, dtype=np.uint32), capi.LOCATOR_MODULO)


def test_histogram_modulo_negative_and_wide_inputs():
    for dtype in (np.int8, np.int32, np.int64, np.uint64):
        v = random_ints(dtype, 30000, seed=6)
        assert_hist_equal(v, np.zeros(100, dtype=np.int32), capi.LOCATOR_MODULO)
    f = (np.random.default_rng(7).standard_normal(30000) * 1000).astype(np.float32)
    assert_hist_equal(f, np.zeros(64, dtype=np.int32), capi.LOCATOR_MODULO)


def test_histogram_identity_ignores_out_of_range_and_unchecked_variant():
    v = np.array([-1, 0, 5, 256, 1000, 255, 255], dtype=np.int32)
    got, ov = gpu_histogram(v, np.zeros(256, dtype=np.int32), capi.LOCATOR_IDENTITY)
    exp = np.zeros(256, dtype=np.int32)
    exp[0], exp[5], exp[255] = 1, 1, 2
    assert np.array_equal(got, exp) and ov == 0
    # HistogramUnchecked: no overflow word at all
    start = np.array([np.iinfo(np.int32).max], dtype=np.int32)
    got, ov = gpu_histogram(np.zeros(4, dtype=np.int32), start,
                            capi.LOCATOR_IDENTITY, checked=False)
    assert got[0] == np.int32(np.iinfo(np.int32).min + 3) and ov == 0
    # the overflow word is OR-ed into
    _, ov = gpu_histogram(np.zeros(4, dtype=np.int32), np.zeros(1, dtype=np.int32),
                          capi.LOCATOR_IDENTITY, overflow=1)
    assert ov == 1


@pytest.mark.parametrize("bin_dtype", [np.float32, np.float64])
def test_histogram_floating_point_bins_take_their_ones_in_bin_precision(bin_dtype):
    # HistogramLaunchers.tt over AtomicNumericTypes: float and double bins get
    # 1.0 added per element, rounded in the bin's precision each time, so a
    # float bin stops at 2^24.  The oracle adds serially; the library computes
    # the same value without the serial additions.
    rng = np.random.default_rng(21)
    fmax = np.finfo(bin_dtype).max
    assorted = np.array([0.0, -0.0, 0.5, 0.1, -0.3, -2.5, 1.5, 3.999, 16777210.0, 16777215.0,
                         16777216.0, 16777218.0, -16777218.0, -16777220.0, -33554434.0,
                         8388607.5, -8388607.5, 1e-30, 1e10, -1e10, np.inf, -np.inf, fmax,
                         -40000.25, 2.0 ** 23 - 0.5, 65535.0], dtype=bin_dtype)
    # few bins (counters in LDS, one flush per block and bin)
    values = rng.integers(0, assorted.size, 300000).astype(np.int32)
    got, ov = gpu_histogram(values, assorted.copy(), capi.LOCATOR_IDENTITY)
    want, want_ov = O.histogram(values, assorted.copy())
    assert bits_equal(got, want)
    assert ov == want_ov == 1            # a bin held MaxValue
    # bins that saturate on the way: 2^24 is reached after 100000 of 250000 samples
    start = np.array([2.0 ** 24 - 100000, 5.0, -7.5, 2.0 ** 24 - 3], dtype=bin_dtype)
    values = (np.arange(1000000) % 4).astype(np.uint8)
    got, ov = gpu_histogram(values, start.copy(), capi.LOCATOR_IDENTITY)
    want, want_ov = O.histogram(values, start.copy())
    assert bits_equal(got, want) and ov == want_ov == 0
    if bin_dtype == np.float32:
        assert got[0] == 2.0 ** 24 and got[3] == 2.0 ** 24 and got[1] == 250005.0
    else:
        assert got[0] == 2.0 ** 24 + 150000 and got[1] == 250005.0
    # many bins (global atomics per element), NaN bins stay NaN, unchecked variant
    nbins = 20000
    before = (rng.integers(-50, 50, nbins) * 0.25).astype(bin_dtype)
    before[7] = np.nan
    values = rng.integers(0, nbins, 150000).astype(np.int32)
    got, _ = gpu_histogram(values, before.copy(), capi.LOCATOR_IDENTITY, checked=False)
    want, _ = O.histogram(values, before.copy())
    assert np.isnan(got[7]) and np.isnan(want[7])
    got[7] = want[7] = 0
    assert bits_equal(got, want)
    # every element for one of many bins: single increments go through the
    # hardware's floating-point add, which does not retry under contention
    values = np.full(2000000, 5, dtype=np.int32)
    got, ov = gpu_histogram(values, np.zeros(nbins, dtype=bin_dtype), capi.LOCATOR_IDENTITY)
    assert got[5] == 2000000.0 and got.sum() == 2000000.0 and ov == 0
    start = np.zeros(nbins, dtype=bin_dtype)
    start[5] = 2.0 ** 24 - 1000
    got, ov = gpu_histogram(values, start, capi.LOCATOR_IDENTITY)
    assert got[5] == (2.0 ** 24 if bin_dtype == np.float32 else 2.0 ** 24 + 1999000) and ov == 0
    # modulo locator and float input
    samples = rng.normal(0, 300, 50000).astype(np.float32)
    got, ov = gpu_histogram(samples, np.zeros(64, dtype=bin_dtype), capi.LOCATOR_MODULO)
    want, want_ov = O.histogram(samples, np.zeros(64, dtype=bin_dtype), O.LOCATOR_MODULO)
    assert bits_equal(got, want) and ov == want_ov == 0


# --------------------------------------------------------------- radix sort
def gpu_sort(keys, **kw):
    d = D.from_numpy(keys)
    capi.radix_sort_keys(d, **kw)
    sync()
    return d.numpy()


def gpu_sort_pairs(keys, values, **kw):
    dk, dv = D.from_numpy(keys), D.from_numpy(values)
    capi.radix_sort_pairs(dk, dv, **kw)
    sync()
    return dk.numpy(), dv.numpy()


def bits_equal(a, b):
    return np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
def test_sort_reference_cases(dtype):
    # RadixSortExtensionTests.tt:144-230, 370-432.
    for n in ARRAY_SIZES:
        note("sort ref", np.dtype(dtype).name, n)
        seq = compute_sequence(dtype, 0, 1, n)
        inv = compute_inverted_sequence(dtype, 0, 1, n)
        assert bits_equal(gpu_sort(inv), seq)
        assert bits_equal(gpu_sort(seq), seq)
        assert bits_equal(gpu_sort(seq, descending=True), inv)
        assert bits_equal(gpu_sort(inv, descending=True), inv)
        for start in (0, 1, -1):
            if np.dtype(dtype).kind == "u" and start < 0:
                continue
            const = compute_sequence(dtype, start, 0, n)
            assert bits_equal(gpu_sort(const), const)
        k, v = gpu_sort_pairs(inv, inv)  # :319-365, values == keys
        assert bits_equal(k, seq) and bits_equal(v, seq)


def test_sort_2pow20_uniform_u32_bit_exact():
    # Baseline config: 2^20 uniform uint32 keys, compared with the CPU path.
    keys = datagen.uniform_u32(1 << 20)
    assert np.array_equal(gpu_sort(keys), O.radix_sort(keys))


@pytest.mark.parametrize("dtype", INT_KEY_DTYPES)
@pytest.mark.parametrize("descending", [False, True])
def test_sort_integer_types_match_oracle(dtype, descending):
    for n in [1, 63, 64, 65, 4095, 4096, 4097, 8191, 8192, 8193, 50001]:
        note("sort", np.dtype(dtype).name, descending, n)
        keys = random_ints(dtype, n, seed=n)
        assert np.array_equal(gpu_sort(keys, descending=descending),
                              O.radix_sort(keys, descending=descending)), n


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
@pytest.mark.parametrize("descending", [False, True])
def test_sort_float_types_match_reference_order(dtype, descending):
    # Default float order = the reference's ExtractRadixBits as written (no
    # reference test has negative or Half keys; the oracle's transform is held
    # by the hand-evaluated golden vectors of tests/test_golden.py).
    keys = random_float_bits(dtype, 30011, seed=3)
    assert bits_equal(gpu_sort(keys, descending=descending),
                      O.radix_sort(keys, descending=descending))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
@pytest.mark.parametrize("descending", [False, True])
def test_sort_float_keys_when_passes_are_skipped(dtype, descending):
    # Float keys are converted to their ordered form by the first pass that runs
    # and back by the last one; passes whose digit is the same for every key do
    # not run at all.  Inputs that skip the top pass (one exponent), the bottom
    # passes (few mantissa bits), everything but one pass, and every pass.
    rng = np.random.default_rng(7)
    n = 70001
    one_exponent = (1.0 + rng.random(n)).astype(dtype)              # [1, 2): top digit constant
    coarse = (rng.integers(-8, 8, n) * 0.5).astype(dtype)           # low mantissa bytes all zero
    one_pass = np.where(rng.random(n) < 0.5, 1.0, 1.5).astype(dtype)
    constant = np.full(n, -2.5, dtype=dtype)
    for name, keys in [("one exponent", one_exponent), ("coarse", coarse),
                       ("two values", one_pass), ("constant", constant)]:
        note("float keys with skipped passes", np.dtype(dtype).name, descending, name)
        expect = O.radix_sort(keys, descending=descending)
        assert bits_equal(gpu_sort(keys, descending=descending), expect), name
        values = np.arange(n, dtype=np.uint32)
        ek, ev = O.radix_sort_pairs(keys, values, descending=descending)
        k, v = gpu_sort_pairs(keys, values, descending=descending)
        assert bits_equal(k, ek) and np.array_equal(v, ev), name
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dtype).itemsize]
    bits = coarse.view(u)
    sign = u(1) << u(np.dtype(dtype).itemsize * 8 - 1)
    ordered = np.where(bits & sign, ~bits, bits | sign)
    if descending:
        ordered = ~ordered
    expect = coarse[np.argsort(ordered, kind="stable")]
    assert bits_equal(gpu_sort(coarse, descending=descending, float_total_order=True), expect)


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
def test_sort_float_total_order_flag(dtype):
    # Extension without a reference counterpart: IEEE totalOrder.
    keys = random_float_bits(dtype, 20000, seed=4)
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dtype).itemsize]
    bits = keys.view(u)
    sign = u(1) << u(np.dtype(dtype).itemsize * 8 - 1)
    ordered = np.where(bits & sign, ~bits, bits | sign)
    expect = keys[np.argsort(ordered, kind="stable")]
    assert bits_equal(gpu_sort(keys, float_total_order=True), expect)
    assert bits_equal(gpu_sort(keys, float_total_order=True, descending=True),
                      keys[np.argsort(~ordered, kind="stable")])


@pytest.mark.parametrize("kind", ["zipf", "constant", "low16", "two_values"])
def test_sort_skewed_inputs(kind):
    n = (1 << 18) + 77
    if kind == "zipf":
        keys = datagen.zipf_u32(n)
    elif kind == "constant":
        keys = datagen.constant_u32(n)
    elif kind == "low16":
        keys = datagen.uniform_u32(n) & np.uint32(0xFFFF)
    else:
        keys = np.where(datagen.uniform_u32(n) & 1, np.uint32(0xFFFFFFFF), np.uint32(0))
    assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
    values = np.arange(n, dtype=np.uint32)
    k, v = gpu_sort_pairs(keys, values)
    perm = np.argsort(keys, kind="stable")
    assert np.array_equal(k, keys[perm]) and np.array_equal(v, values[perm])


@pytest.mark.parametrize("key_dtype,value_dtype", [
    (np.uint32, np.uint32), (np.uint64, np.uint32), (np.int32, np.float64),
    (np.uint8, np.uint16), (np.int16, np.uint8), (np.uint64, np.uint64),
    (np.float32, np.int32)])
@pytest.mark.parametrize("descending", [False, True])
def test_sort_pairs_stable_and_bit_exact(key_dtype, value_dtype, descending):
    for n in [1, 100, 8193, 70001]:
        note("pairs", np.dtype(key_dtype).name, np.dtype(value_dtype).name, n)
        if np.dtype(key_dtype).kind == "f":
            keys = np.abs(np.random.default_rng(n).integers(0, 50, n)).astype(key_dtype)
        else:
            keys = random_ints(key_dtype, n, seed=n, lo=0, hi=40)  # many ties
        values = np.arange(n).astype(value_dtype)
        k, v = gpu_sort_pairs(keys, values, descending=descending)
        ek, ev = O.radix_sort_pairs(keys, values, descending=descending)
        assert bits_equal(k, ek) and bits_equal(v, ev), n


def test_sort_pairs_16_byte_values():
    n = 20001
    keys = random_ints(np.uint32, n, seed=1, lo=0, hi=1000)
    values = np.zeros((n, 2), dtype=np.uint64)
    values[:, 0] = np.arange(n)
    values[:, 1] = ~np.arange(n, dtype=np.uint64)
    dk = D.from_numpy(keys)
    dv = D(n, np.dtype([("a", np.uint64), ("b", np.uint64)]),
           _bytes=D.from_numpy(values.reshape(-1)).bytes)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32, 16))
    capi.check(capi.lib().ilgpu_hip_radix_sort_pairs(
        None, dk.ptr, 1, dv.ptr, 1, n, capi.U32, 16, 0, capi.VALUES_FROM_VIEW,
        temp.ptr, temp.nbytes))
    sync()
    perm = np.argsort(keys, kind="stable")
    assert np.array_equal(dk.numpy(), keys[perm])
    got = dv.bytes.cpu().numpy().view(np.uint64).reshape(n, 2)
    assert np.array_equal(got, values[perm])


@pytest.mark.parametrize("value_dtype", [np.uint32, np.int64, np.int8, np.uint8, np.int16,
                                         np.uint16, np.float16, np.float32, np.float64])
def test_sort_pairs_values_from_index(value_dtype):
    # Sequencer form (RadixSortExtensions.cs:1017-1074): value[i] = (TValue)i,
    # whatever the values view held before.  Integer sequencers truncate the index
    # (Sequencers.tt:25-37); HalfSequencer, FloatSequencer and DoubleSequencer
    # convert it (Sequencer.cs:47-75: Half through float, so +inf from 65520 on).
    def sequencer(index):
        if np.dtype(value_dtype) == np.float16:
            return index.astype(np.float32).astype(np.float16)
        return index.astype(value_dtype)           # numpy truncates integers as C# does

    for keys in (datagen.uniform_u64(100003), datagen.constant_u32(5000),
                 datagen.uniform_u32(9000) & np.uint32(0xFF),
                 datagen.uniform_u32(18432 * 3 + 5)):          # several tiles: the passes
        n = keys.size
        dk = D.from_numpy(keys)
        dv = D.from_numpy(np.full(n, 99, dtype=value_dtype))
        with np.errstate(over="ignore"):
            expect = sequencer(np.argsort(keys, kind="stable"))
        capi.radix_sort_pairs(dk, dv, values_from_index=True)
        sync()
        assert np.array_equal(dk.numpy(), np.sort(keys, kind="stable"))
        assert bits_equal(dv.numpy(), expect), np.dtype(value_dtype).name
    # hand-evaluated: index 2049 is not a Half (rounds to even: 2048), 65519 rounds
    # to 65504, 65520 to infinity; 16777217 is not a float (rounds to 16777216)
    if np.dtype(value_dtype) == np.float16:
        n = 70000
        dk, dv = D.from_numpy(np.arange(n, dtype=np.uint32)), D.zeros(n, np.float16)
        capi.radix_sort_pairs(dk, dv, values_from_index=True)
        sync()
        got = dv.numpy().view(np.uint16)
        assert got[2049] == 0x6800 and got[2051] == 0x6802       # 2048, 2052
        assert got[65519] == 0x7BFF and got[65520] == 0x7C00     # 65504, +inf
    if np.dtype(value_dtype) == np.float32:
        n = (1 << 24) + 4
        dk, dv = D.from_numpy(np.arange(n, dtype=np.uint32)), D.zeros(n, np.float32)
        capi.radix_sort_pairs(dk, dv, values_from_index=True)
        sync()
        got = dv.numpy()
        assert got[16777217] == 16777216.0 and got[16777219] == 16777220.0


def test_sort_reuses_dirty_temp_and_unaligned_key_view():
    keys = datagen.uniform_u32(100001, seed=5)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(keys.size, np.uint32))
    temp.bytes.fill_(0xAB)
    for _ in range(2):
        d = D.from_numpy(keys)
        capi.radix_sort_keys(d, temp)
        sync()
        assert np.array_equal(d.numpy(), np.sort(keys))
    d = D.from_numpy(keys)
    view = d.subview(3, 50000)
    capi.radix_sort_keys(view)
    sync()
    out = d.numpy()
    assert np.array_equal(out[3:50003], np.sort(keys[3:50003]))
    assert np.array_equal(out[:3], keys[:3]) and np.array_equal(out[50003:], keys[50003:])


# ------------------------------------------------------ strided views (General)
# Stride1D.General with an element stride above one (ArrayViews.tt:114-119):
# element i of the view is base[i * stride].  The logical elements must match
# the oracle on the dense sequence, and the elements in between must be left
# exactly as they were.
SENTINEL = 0x5A


def strided_buffer(logical: np.ndarray, stride: int):
    """A physical buffer holding `logical` at multiples of `stride`, sentinel
    bytes elsewhere; returns (device array, strided view, host copy)."""
    phys = np.full(((logical.size - 1) * stride + 1) * logical.dtype.itemsize,
                   SENTINEL, dtype=np.uint8).view(logical.dtype).copy()
    phys[::stride] = logical
    dev = D.from_numpy(phys)
    return dev, dev.strided(stride), phys


def assert_gaps_untouched(after: np.ndarray, before: np.ndarray, stride: int):
    mask = np.ones(after.size, dtype=bool)
    mask[::stride] = False
    assert np.array_equal(after.view(np.uint8).reshape(after.size, -1)[mask],
                          before.view(np.uint8).reshape(before.size, -1)[mask])


@pytest.mark.parametrize("stride", [2, 3, 7])
@pytest.mark.parametrize("dtype", [np.uint32, np.int64, np.float32, np.uint8])
def test_sort_keys_strided(dtype, stride):
    for n in [1, 33, 1027, 50001]:
        note("sort strided", np.dtype(dtype).name, stride, n)
        keys = (random_float_bits(dtype, n, seed=n) if np.dtype(dtype).kind == "f"
                else random_ints(dtype, n, seed=n))
        dev, view, phys = strided_buffer(keys, stride)
        capi.radix_sort_keys(view)
        sync()
        out = dev.numpy()
        expect = O.radix_sort(keys)
        assert np.array_equal(np.ascontiguousarray(out[::stride]).view(np.uint8),
                              expect.view(np.uint8))
        assert_gaps_untouched(out, phys, stride)


@pytest.mark.parametrize("key_stride,value_stride", [(2, 1), (1, 3), (4, 5)])
def test_sort_pairs_strided(key_stride, value_stride):
    for n in [1, 127, 40000]:
        note("pairs strided", key_stride, value_stride, n)
        keys = random_ints(np.uint16, n, seed=n)        # many duplicates
        vals = np.arange(n, dtype=np.uint64) * 3 + 1
        kdev, kview, kphys = strided_buffer(keys, key_stride)
        vdev, vview, vphys = strided_buffer(vals, value_stride)
        capi.radix_sort_pairs(kview, vview)
        sync()
        ek, ev = O.radix_sort_pairs(keys, vals)
        kout, vout = kdev.numpy(), vdev.numpy()
        assert np.array_equal(kout[::key_stride], ek)
        assert np.array_equal(vout[::value_stride], ev)
        assert_gaps_untouched(kout, kphys, key_stride)
        assert_gaps_untouched(vout, vphys, value_stride)
        # sequencer form: values = stable permutation indices
        kdev, kview, _ = strided_buffer(keys, key_stride)
        idev, iview, iphys = strided_buffer(np.zeros(n, dtype=np.int32), value_stride)
        capi.radix_sort_pairs(kview, iview, values_from_index=True)
        sync()
        order = np.argsort(keys, kind="stable").astype(np.int32)
        iout = idev.numpy()
        assert np.array_equal(iout[::value_stride], order)
        assert_gaps_untouched(iout, iphys, value_stride)


@pytest.mark.parametrize("in_stride,out_stride", [(2, 1), (1, 2), (3, 5), (4, 4)])
@pytest.mark.parametrize("dtype", [np.int32, np.uint64, np.float64])
def test_scan_strided(dtype, in_stride, out_stride):
    for n in [1, 31, 1027, 70001]:
        for kind in (capi.SCAN_INCLUSIVE, capi.SCAN_EXCLUSIVE):
            for op in OPS:
                note("scan strided", np.dtype(dtype).name, in_stride, out_stride, n, kind, op)
                v = (random_ints(dtype, n, seed=n, lo=0, hi=1000)
                     if np.dtype(dtype).kind in "iu"
                     else np.random.default_rng(n).integers(-50, 50, n).astype(dtype))
                idev, iview, iphys = strided_buffer(v, in_stride)
                odev, oview, ophys = strided_buffer(np.zeros(n, dtype=dtype), out_stride)
                capi.scan(iview, oview, op=op, kind=kind)
                sync()
                expect = O.scan(v, op=op, inclusive=kind == capi.SCAN_INCLUSIVE)
                out = odev.numpy()
                assert np.array_equal(out[::out_stride], expect)
                assert_gaps_untouched(out, ophys, out_stride)
                assert np.array_equal(idev.numpy().view(np.uint8), iphys.view(np.uint8))


def test_scan_strided_in_place():
    v = random_ints(np.int32, 5000, seed=5, lo=-9, hi=9)
    dev, view, phys = strided_buffer(v, 3)
    capi.scan(view, view, kind=capi.SCAN_INCLUSIVE)
    sync()
    out = dev.numpy()
    assert np.array_equal(out[::3], O.scan(v, op=capi.OP_ADD, inclusive=True))
    assert_gaps_untouched(out, phys, 3)


@pytest.mark.parametrize("stride", [2, 5])
@pytest.mark.parametrize("dtype", [np.int32, np.uint64, np.float32])
def test_reduce_strided(dtype, stride):
    for n in [1, 63, 4097, 300001]:
        for op in OPS:
            note("reduce strided", np.dtype(dtype).name, stride, n, op)
            v = (random_ints(dtype, n, seed=n) if np.dtype(dtype).kind in "iu"
                 else np.random.default_rng(n).integers(-10, 10, n).astype(dtype))
            dev, view, _ = strided_buffer(v, stride)
            out = D.zeros(1, dtype)
            capi.reduce(view, out, op=op)
            sync()
            assert out.numpy()[0] == O.reduce(v, op=op)


@pytest.mark.parametrize("stride", [2, 9])
@pytest.mark.parametrize("num_bins", [64, 256, 20000])
def test_histogram_strided(num_bins, stride):
    for n in [1, 1024, 200003]:
        note("histogram strided", num_bins, stride, n)
        v = random_ints(np.int32, n, seed=n, lo=-5, hi=3 * num_bins)
        dev, view, _ = strided_buffer(v, stride)
        bins = D.zeros(num_bins, np.int32)
        ov = D.zeros(1, np.int32)
        capi.histogram(view, bins, ov, locator=capi.LOCATOR_MODULO)
        sync()
        eb, eo = O.histogram(v, np.zeros(num_bins, np.int32),
                             locator=O.LOCATOR_MODULO)
        assert np.array_equal(bins.numpy(), eb)
        assert ov.numpy()[0] == eo


# -------------------------------------- unique, initialize, sequence, reorder
def gpu_unique(values):
    d = D.from_numpy(values)
    out_len = D.zeros(1, np.int64)
    capi.unique(d, out_len)
    sync()
    kept = int(out_len.numpy()[0])
    return d.numpy()[:kept], d.numpy()[kept:], kept


def test_lds_atomics_serve_the_lanes_of_an_instruction_in_lane_order():
    # The hardware property the sort's ranking rests on (one returning LDS add per
    # key, equal digits must come back in lane order): checked on every compute
    # unit, under load, for six digit distributions.  Any lane served out of
    # order would make a pass unstable, which the pair-sort tests would show too.
    assert capi.selftest_lds_atomic_order(2048) == 0
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.selftest_lds_atomic_order(0)


def test_sorts_ask_the_device_once_and_refuse_one_that_fails():
    # The library runs the check of the LDS atomics itself before the first sort
    # on a device and keeps the answer.
    capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, -1)   # forget, ask again
    keys = random_ints(np.uint32, 50000, seed=1)
    assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))   # asks the device
    capi.sort_check_device()                                               # cached: passes
    capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, 0)    # stand-in for a device that fails
    try:
        with pytest.raises(capi.NotSupportedError):
            gpu_sort(keys)
        values = np.arange(keys.size, dtype=np.uint32)
        with pytest.raises(capi.NotSupportedError):
            gpu_sort_pairs(keys, values)
    finally:
        capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, -1)
    assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))


def test_sort_look_back_that_never_waits_counts_missing_tiles_itself():
    # A pass hands its tiles to eight fixed groups of blocks, so a tile's
    # look-back can meet a predecessor nobody has started; past a bound of polls
    # it counts that tile's digit itself from the source keys.  With the bound
    # at zero every empty status word takes that path; results must not change.
    capi.sort_set_parameter(capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, 0)
    try:
        for dtype, n in [(np.uint32, 18432 * 40 + 77), (np.uint8, 300000), (np.int16, 400001),
                         (np.uint64, 9216 * 33 + 5)]:
            note("sort with zero spin limit", np.dtype(dtype).name, n)
            keys = random_ints(dtype, n, seed=11)
            assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
        keys = random_float_bits(np.float32, 500000, seed=12)
        assert bits_equal(gpu_sort(keys, descending=True), O.radix_sort(keys, descending=True))
        # pairs: few distinct keys, so stability decides the value order
        keys = random_ints(np.uint32, 300000, seed=13, lo=0, hi=999)
        values = np.arange(keys.size, dtype=np.uint64)
        k, v = gpu_sort_pairs(keys, values)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(k, keys[order]) and np.array_equal(v, values[order])
        keys = random_ints(np.int64, 200000, seed=14)
        values = random_ints(np.uint8, keys.size, seed=15)
        k, v = gpu_sort_pairs(keys, values)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(k, keys[order]) and np.array_equal(v, values[order])
        # the same with full tiles where short ones are the default
        capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, 0)
        keys = random_ints(np.uint32, 18432 * 40 + 77, seed=19)
        assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
        capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, -1)
        # the same with 1024-thread blocks
        capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU, 0)
        keys = random_ints(np.uint32, 36864 * 20 + 77, seed=17)
        assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
        keys = random_ints(np.uint16, 300000, seed=18, lo=0, hi=99)
        values = np.arange(keys.size, dtype=np.uint32)
        k, v = gpu_sort_pairs(keys, values)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(k, keys[order]) and np.array_equal(v, values[order])
    finally:
        capi.sort_set_parameter(capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, -1)
        capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU, -1)
        capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, -1)
    # back on the defaults
    keys = random_ints(np.uint32, 18432 * 40 + 77, seed=16)
    assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.sort_set_parameter(7, 0)


@pytest.fixture
def no_one_tile_kernel():
    """Inputs of one tile go through histogram, plan and passes like longer ones
    (by default one block sorts them in one launch)."""
    capi.sort_set_parameter(capi.SORT_PARAM_ONE_TILE_KERNEL, 0)
    yield
    capi.sort_set_parameter(capi.SORT_PARAM_ONE_TILE_KERNEL, 1)


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
def test_sort_of_one_tile_through_the_passes_matches_oracle(no_one_tile_kernel, dtype):
    kinds = np.dtype(dtype).kind
    for n in [1, 2, 63, 64, 65, 1027, 4097, 9216, 18431, 18432]:
        note("one tile through the passes", np.dtype(dtype).name, n)
        keys = random_float_bits(dtype, n, seed=n) if kinds == "f" else random_ints(dtype, n, seed=n)
        for descending in (False, True):
            assert bits_equal(gpu_sort(keys, descending=descending),
                              O.radix_sort(keys, descending=descending)), (n, descending)
    keys = (random_ints(np.int32, 5000, seed=3, lo=-40, hi=40)).astype(dtype)
    values = np.arange(keys.size, dtype=np.uint32)
    k, v = gpu_sort_pairs(keys, values)
    ek, ev = O.radix_sort_pairs(keys, values)
    assert bits_equal(k, ek) and np.array_equal(v, ev)


@pytest.mark.parametrize("key_dtype,value_dtype", [
    (np.uint32, np.uint32), (np.uint64, np.uint32), (np.uint32, np.uint64), (np.int64, np.float64),
    (np.uint8, np.uint8), (np.int16, np.uint16), (np.float32, np.int32), (np.float16, np.uint64),
    (np.float64, np.uint8)])
def test_sort_pairs_of_one_tile_by_one_block(key_dtype, value_dtype):
    # sizes up to the tile of every pair type (4096 pairs with 16-byte values,
    # 5120 to 10240 otherwise) and just beyond, where the passes take over
    for n in [1, 2, 64, 65, 1000, 4095, 4096, 4097, 5120, 5121, 7168, 7169, 8192, 8193, 10240,
              10241]:
        note("one-tile pairs", np.dtype(key_dtype).name, np.dtype(value_dtype).name, n)
        keys = (random_ints(np.int32, n, seed=n, lo=-40, hi=40)).astype(key_dtype)
        values = np.arange(n).astype(value_dtype)
        for descending in (False, True):
            k, v = gpu_sort_pairs(keys, values, descending=descending)
            ek, ev = O.radix_sort_pairs(keys, values, descending=descending)
            assert bits_equal(k, ek) and bits_equal(v, ev), (n, descending)
    n = 4000
    keys = random_ints(np.uint32, n, seed=5, lo=0, hi=300)
    order = np.argsort(keys, kind="stable")
    values = np.zeros((n, 2), dtype=np.uint64)
    values[:, 0] = np.arange(n)
    values[:, 1] = ~np.arange(n, dtype=np.uint64)
    dk = D.from_numpy(keys)
    dv = D(n, np.dtype([("a", np.uint64), ("b", np.uint64)]),
           _bytes=D.from_numpy(values.reshape(-1)).bytes)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32, 16))
    capi.check(capi.lib().ilgpu_hip_radix_sort_pairs(
        None, dk.ptr, 1, dv.ptr, 1, n, capi.U32, 16, 0, capi.VALUES_FROM_VIEW,
        temp.ptr, temp.nbytes))
    sync()
    assert np.array_equal(dk.numpy(), keys[order])
    assert np.array_equal(dv.bytes.cpu().numpy().view(np.uint64).reshape(n, 2), values[order])
    dk2, dv2 = D.from_numpy(keys), D.zeros(n, np.uint64)
    capi.radix_sort_pairs(dk2, dv2, values_from_index=True, descending=True)
    sync()
    order_desc = np.argsort(~keys, kind="stable")
    assert np.array_equal(dk2.numpy(), keys[order_desc])
    assert np.array_equal(dv2.numpy(), order_desc.astype(np.uint64))


@pytest.fixture
def large_sort_blocks():
    """Sorts of any size take the 1024-thread kernels (by default only inputs of
    tens of millions of keys do)."""
    capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU, 0)
    yield
    capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU, -1)


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("descending", [False, True])
def test_sort_with_large_blocks_matches_oracle(large_sort_blocks, dtype, descending):
    kinds = np.dtype(dtype).kind
    for n in [1, 65, 36863, 36864, 36865, 100003]:
        note("large-block sort", np.dtype(dtype).name, descending, n)
        keys = random_float_bits(dtype, n, seed=n) if kinds == "f" else random_ints(dtype, n, seed=n)
        assert bits_equal(gpu_sort(keys, descending=descending),
                          O.radix_sort(keys, descending=descending)), n


# Keys without values that make at most 512 tiles (128 with 8-byte keys) of a
# shorter class (512 threads x 12, 18 or 24 keys of up to 4 bytes; 6, 8 or 12 of
# 8 bytes) take the shortest class that does, every block one tile without a
# ticket; longer inputs and pairs take full tiles.
@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("descending", [False, True])
def test_sort_with_short_tiles_matches_oracle(dtype, descending):
    kinds = np.dtype(dtype).kind
    for n in [18433, 30000, 6144 * 7 + 5, 3072 * 9 - 1, 100003, 400001]:
        note("short-tile sort", np.dtype(dtype).name, descending, n)
        keys = random_float_bits(dtype, n, seed=n) if kinds == "f" else random_ints(dtype, n, seed=n)
        assert bits_equal(gpu_sort(keys, descending=descending),
                          O.radix_sort(keys, descending=descending)), n


@pytest.mark.parametrize("dtype,sizes", [
    (np.uint32, [512 * 6144, 512 * 6144 + 1, 512 * 9216, 512 * 9216 + 1, 512 * 12288,
                 512 * 12288 + 1]),
    (np.int16, [512 * 6144 - 1, 512 * 9216 + 1, 512 * 12288 + 1]),
    (np.uint64, [128 * 3072, 128 * 3072 + 1, 128 * 4096, 128 * 4096 + 1, 128 * 6144,
                 128 * 6144 + 1])])
def test_sort_at_the_edges_of_the_short_tile_classes(dtype, sizes):
    # the longest input of every class and the shortest of the next one
    for n in sizes:
        note("short-tile class edge", np.dtype(dtype).name, n)
        keys = random_ints(dtype, n, seed=n & 0xFFFF)
        assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable")), n


@pytest.mark.parametrize("dtype", [np.uint16, np.uint32, np.int32, np.uint64, np.int64,
                                   np.float32, np.float64])
def test_sort_of_keys_that_agree_across_whole_waves(dtype):
    # The digit histogram counts vectors whose keys agree in every lane of a wave
    # (wholly, or in their upper half) as runs in registers; a wave looks for
    # them when its first vector is one.  Stretches of constant keys, of small
    # values and of varying keys, with odd lengths so that the stretches start
    # and end inside vectors and waves, in either order, and a view that starts
    # off a 16-byte boundary.
    dt = np.dtype(dtype)
    rng = np.random.default_rng(77)
    bits = dt.itemsize * 8
    udt = np.dtype(f"u{dt.itemsize}")

    def varying(m):
        return rng.integers(0, 1 << bits, size=m, dtype=np.uint64).astype(udt)

    def small(m):
        return rng.integers(0, 1 << (bits // 2), size=m, dtype=np.uint64).astype(udt)

    def constant(m, value):
        return np.full(m, value & ((1 << bits) - 1), dtype=udt)

    for order in (0, 1):
        parts = [constant(70001, 0xDEADBEEFCAFEF00D), constant(30011, 5), small(130003),
                 varying(90007), constant(50021, 0x8000000000000001), small(40009)]
        if order:
            parts = [varying(4099)] + parts[::-1]
        raw = np.concatenate(parts)
        if dt.kind == "f":   # no NaN payload games here: keep every exponent finite
            raw &= udt.type(~(1 << (bits - 2)) & ((1 << bits) - 1))
        keys = raw.view(dt)
        for off in (0, 1):
            k = keys[off:]
            note("keys that agree across waves", dt.name, order, off, k.size)
            big = D.from_numpy(keys)
            view = D(k.size, dt, _bytes=big.bytes[off * dt.itemsize:])
            capi.radix_sort_keys(view)
            sync()
            got = view.numpy()
            if dt.kind == "f":
                assert bits_equal(got, O.radix_sort(k)), (order, off)
            else:
                assert np.array_equal(got, np.sort(k, kind="stable")), (order, off)
    # long enough for the grid to have every block several rounds deep
    n = (1 << 23) + 12345
    keys = np.concatenate([constant(n // 2, 0x1234567812345678), small(n - n // 2)]).view(dt)
    if dt.kind != "f":
        assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))


def test_sorts_of_random_shapes_under_random_test_hooks_match_oracle():
    # 300 seeded cases: key type, length (one row to a few hundred tiles), key
    # distribution (full range, a handful of values, constant), direction, keys
    # or pairs, and every test hook that picks a code path (block size, one-tile
    # kernel, short-tile limit, look-back bound) drawn at random.
    rng = np.random.default_rng(20240607)
    value_types = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}
    for case in range(300):
        dtype = ALL_KEY_DTYPES[int(rng.integers(len(ALL_KEY_DTYPES)))]
        dt = np.dtype(dtype)
        n = int(rng.choice([rng.integers(1, 300), rng.integers(1, 40000),
                            rng.integers(1, 400000)]))
        spin = int(rng.choice([-1, -1, -1, 0])) if n <= 200000 else -1
        hooks = {capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU: int(rng.choice([-1, -1, 0, 2**31 - 1])),
                 capi.SORT_PARAM_ONE_TILE_KERNEL: int(rng.choice([1, 1, 0])),
                 capi.SORT_PARAM_SHORT_TILE_MAX_TILES: int(rng.choice([-1, -1, 0, 40, 300])),
                 capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT: spin}
        for parameter, value in hooks.items():
            capi.sort_set_parameter(parameter, value)
        mode = int(rng.integers(0, 3))
        if dt.kind == "f":
            keys = random_float_bits(dtype, n, seed=case) if mode == 0 else \
                rng.integers(-3, 4, n).astype(dtype)
        elif mode == 0:
            keys = random_ints(dtype, n, seed=case)
        elif mode == 1:
            keys = rng.integers(0, 6, n).astype(dtype)
        else:
            keys = np.full(n, rng.integers(0, 100), dtype=dtype)
        descending = bool(rng.integers(0, 2))
        pairs = bool(rng.integers(0, 2))
        note("random sort case", case, dt.name, n, mode, descending, pairs, sorted(hooks.items()))
        if pairs:
            values = np.arange(n).astype(value_types[int(rng.choice([1, 2, 4, 8]))])
            k, v = gpu_sort_pairs(keys, values, descending=descending)
            ek, ev = O.radix_sort_pairs(keys, values, descending=descending)
            assert bits_equal(k, ek) and np.array_equal(v, ev), case
        else:
            assert bits_equal(gpu_sort(keys, descending=descending),
                              O.radix_sort(keys, descending=descending)), case


@pytest.fixture
def no_short_tiles():
    """Short inputs of keys take full tiles like pairs and longer inputs do."""
    capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, 0)
    yield
    capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, -1)


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
def test_sort_of_short_inputs_with_full_tiles_matches_oracle(no_short_tiles, dtype):
    kinds = np.dtype(dtype).kind
    for n in [18433, 100003, 18432 * 12 + 77]:
        note("short input, full tiles", np.dtype(dtype).name, n)
        keys = random_float_bits(dtype, n, seed=n) if kinds == "f" else random_ints(dtype, n, seed=n)
        for descending in (False, True):
            assert bits_equal(gpu_sort(keys, descending=descending),
                              O.radix_sort(keys, descending=descending)), (n, descending)


def test_sort_with_more_tiles_than_blocks_draws_tickets():
    # 515 full tiles of keys and 600 of pairs on at most 512 resident blocks:
    # the blocks draw their tiles from the tickets, some of them two.
    n = 18432 * 515 + 3
    keys = random_ints(np.uint32, n, seed=21)
    assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable"))
    n = 8192 * 600 + 3
    keys = random_ints(np.uint32, n, seed=22, lo=0, hi=4999)
    values = np.arange(n, dtype=np.uint32)
    k, v = gpu_sort_pairs(keys, values)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k, keys[order]) and np.array_equal(v, values[order])


@pytest.mark.parametrize("dtype", [np.uint32, np.int64, np.float32, np.float16, np.uint8])
def test_one_tile_sort_at_the_edges_of_its_row_counts(dtype):
    # Inputs of one tile are sorted by one block whose threads hold 4, 12, 24 or
    # all of a tile's keys each, by the input's length: the lengths either side
    # of every switch (512 threads x 4, 12, 24 keys; pairs switch where their
    # shorter tiles allow).
    for n in [2047, 2048, 2049, 6144, 6145, 12288, 12289]:
        note("one-tile sort", np.dtype(dtype).name, n)
        keys = (random_float_bits(dtype, n, seed=n) if np.dtype(dtype).kind == "f"
                else random_ints(dtype, n, seed=n))
        assert bits_equal(gpu_sort(keys), O.radix_sort(keys)), n
        assert bits_equal(gpu_sort(keys, descending=True), O.radix_sort(keys, descending=True)), n
    for n in [2048, 2049, 4095, 6144, 6145]:
        # few distinct keys: stability decides the order of the values
        keys = random_ints(np.int32, n, seed=n, lo=-9, hi=9).astype(dtype)
        values = np.arange(n, dtype=np.uint32)
        ek, ev = O.radix_sort_pairs(keys, values)
        k, v = gpu_sort_pairs(keys, values)
        assert bits_equal(k, ek) and np.array_equal(v, ev), n


@pytest.mark.parametrize("dtype", [np.uint32, np.int32, np.uint64, np.int64, np.uint16, np.uint8])
def test_sort_with_scanning_blocks_matches_numpy(large_sort_blocks, dtype):
    # Keys without values in 1024-thread blocks take the pipelined form of the pass.
    # From 64 tiles on, four blocks of the grid scan the tiles' digit counts
    # instead of sorting; below that every block resolves its tiles itself.
    # Sizes: some 100 tiles and a ragged last one; keys uniform, few-valued
    # (dominant digits), in runs (whole rows of one digit) and constant.
    items = 18 if np.dtype(dtype).itemsize == 8 else 36
    tile = 15 * 64 * items
    for n in [63 * tile, 64 * tile + 1, 101 * tile + 12345]:
        note("pipelined sort", np.dtype(dtype).name, n)
        keys = random_ints(dtype, n, seed=n & 0xFFFF)
        assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable")), n
    n = 90 * tile + 777
    info = np.iinfo(dtype)
    few = random_ints(np.int64, n, seed=3, lo=0, hi=2).astype(dtype) * (info.max // 3)
    assert np.array_equal(gpu_sort(few, descending=True), np.sort(few, kind="stable")[::-1])
    runs = ((np.arange(n, dtype=np.uint64) // 1000) * 2654435761 % (int(info.max) // 2 + 1)).astype(dtype)
    assert np.array_equal(gpu_sort(runs), np.sort(runs, kind="stable"))
    const = np.full(n, info.max // 5, dtype=dtype)
    assert np.array_equal(gpu_sort(const), const)


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64])
@pytest.mark.parametrize("descending", [False, True])
def test_float_sort_with_scanning_blocks_matches_oracle(large_sort_blocks, dtype, descending):
    # Float keys take the pipelined form too: the first pass that runs converts
    # them to their ordered form as it ranks them, the last one converts them
    # back as it writes them.  Arbitrary bit patterns (NaNs, infinities, both
    # zeros), and inputs whose top or bottom passes are skipped, so that the
    # converting passes are not the first and the last of the key.
    items = 18 if np.dtype(dtype).itemsize == 8 else 36
    tile = 15 * 64 * items
    n = 66 * tile + 4321
    rng = np.random.default_rng(11)
    cases = [("bit patterns", random_float_bits(dtype, n, seed=5)),
             ("one exponent", (1.0 + rng.random(n)).astype(dtype)),
             ("coarse", (rng.integers(-8, 8, n) * 0.5).astype(dtype))]
    for name, keys in cases:
        note("pipelined float sort", np.dtype(dtype).name, descending, name, n)
        assert bits_equal(gpu_sort(keys, descending=descending),
                          O.radix_sort(keys, descending=descending)), name
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[np.dtype(dtype).itemsize]
    keys = cases[0][1]
    bits = keys.view(u)
    sign = u(1) << u(np.dtype(dtype).itemsize * 8 - 1)
    ordered = np.where(bits & sign, ~bits, bits | sign)
    if descending:
        ordered = ~ordered
    expect = keys[np.argsort(ordered, kind="stable")]
    assert bits_equal(gpu_sort(keys, descending=descending, float_total_order=True), expect)


def test_sort_with_scanning_blocks_never_waits_without_bound(large_sort_blocks):
    # With the bound on polls at zero the scanning blocks count every tile they
    # find unpublished themselves, and the sorting blocks stop waiting for them
    # at once and walk back themselves, counting in turn what they find missing.
    capi.sort_set_parameter(capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, 0)
    try:
        for dtype, tiles in [(np.uint32, 70), (np.uint64, 66), (np.uint8, 65)]:
            items = 18 if np.dtype(dtype).itemsize == 8 else 36
            n = tiles * 15 * 64 * items + 31
            note("pipelined sort, zero spin limit", np.dtype(dtype).name, n)
            keys = random_ints(dtype, n, seed=tiles)
            assert np.array_equal(gpu_sort(keys), np.sort(keys, kind="stable")), n
        # float keys: what a block counts itself comes from source keys that are
        # raw in the first pass and ordered afterwards
        n = 67 * 15 * 64 * 36 + 5
        keys = random_float_bits(np.float32, n, seed=9)
        note("pipelined float sort, zero spin limit", n)
        assert bits_equal(gpu_sort(keys), O.radix_sort(keys))
    finally:
        capi.sort_set_parameter(capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, -1)


@pytest.mark.parametrize("key_dtype,value_dtype", [
    (np.uint32, np.uint32), (np.uint64, np.uint32), (np.uint32, np.uint64), (np.int64, np.float64),
    (np.uint8, np.uint8), (np.int16, np.uint16), (np.float32, np.int32), (np.float16, np.uint64)])
def test_sort_pairs_with_large_blocks_are_stable(large_sort_blocks, key_dtype, value_dtype):
    for n in [1000, 8191 * 2 + 5, 120001]:
        note("large-block pairs", np.dtype(key_dtype).name, np.dtype(value_dtype).name, n)
        # few distinct keys: stability decides the value order
        keys = (random_ints(np.int32, n, seed=n, lo=-40, hi=40)).astype(key_dtype)
        values = np.arange(n).astype(value_dtype)
        k, v = gpu_sort_pairs(keys, values)
        ek, ev = O.radix_sort_pairs(keys, values)
        assert bits_equal(k, ek) and bits_equal(v, ev), n
    # 16-byte values and index-generated values
    n = 50000
    keys = random_ints(np.uint32, n, seed=5, lo=0, hi=300)
    order = np.argsort(keys, kind="stable")
    values = np.zeros((n, 2), dtype=np.uint64)
    values[:, 0] = np.arange(n)
    values[:, 1] = ~np.arange(n, dtype=np.uint64)
    dk = D.from_numpy(keys)
    dv = D(n, np.dtype([("a", np.uint64), ("b", np.uint64)]),
           _bytes=D.from_numpy(values.reshape(-1)).bytes)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32, 16))
    capi.check(capi.lib().ilgpu_hip_radix_sort_pairs(
        None, dk.ptr, 1, dv.ptr, 1, n, capi.U32, 16, 0, capi.VALUES_FROM_VIEW,
        temp.ptr, temp.nbytes))
    sync()
    assert np.array_equal(dk.numpy(), keys[order])
    assert np.array_equal(dv.bytes.cpu().numpy().view(np.uint64).reshape(n, 2), values[order])
    dk2, dv2 = D.from_numpy(keys), D.zeros(n, np.uint32)
    capi.radix_sort_pairs(dk2, dv2, values_from_index=True)
    sync()
    assert np.array_equal(dk2.numpy(), keys[order]) and np.array_equal(dv2.numpy(), order)


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("repeat", [1, 317, 1025])
def test_unique_reference_cases(dtype, repeat):
    # UniqueExtensionTests.tt:48-67 (1025 elements) and :69-90 (more elements
    # than one grid of groups covers; here: several tiles).
    for length in (1025, 300001):
        note("unique", np.dtype(dtype).name, repeat, length)
        vals = np.repeat(np.arange(1, length // repeat + 2), repeat)[:length]
        if np.dtype(dtype) == np.float16:
            vals = vals % 2000 + 1     # integers above 2048 are not exact in Half; runs still differ
        vals = (vals.astype(np.int64).astype(dtype) if np.dtype(dtype).kind in "iu"
                else vals.astype(dtype))
        kept, _, count = gpu_unique(vals)
        expect = O.unique(vals)
        assert count == expect.size
        assert np.array_equal(kept, expect)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.uint32, np.int64, np.float32, np.float64, np.float16])
def test_unique_random_runs(dtype):
    for n in [1, 2, 63, 64, 65, 8191, 8192, 8193, 1 << 20, (1 << 22) + 5]:
        note("unique runs", np.dtype(dtype).name, n)
        r = np.random.default_rng(n)
        runs = r.integers(1, 6, size=n)
        base = r.integers(0, 3, size=n)
        vals = np.repeat(base, runs)[:n].astype(dtype)
        if np.dtype(dtype).kind == "f" and n > 8:
            vals[3:6] = np.nan               # a run of NaNs is one value
            vals[6] = -0.0
            vals[7] = 0.0                    # equal to -0.0
        kept, _, count = gpu_unique(vals)
        expect = O.unique(vals)
        assert count == expect.size, n
        assert np.array_equal(kept.view(np.uint8), expect.view(np.uint8)), n


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.int32, np.int64, np.float64])
def test_unique_tile_edges(dtype):
    # a tile is 512 threads x 12 sixteen-byte vectors (4 for 1-byte elements, 8 for 2-byte ones)
    size = np.dtype(dtype).itemsize
    tile = 512 * {1: 4, 2: 8}.get(size, 12) * (16 // size)
    for n in sorted({tile * m + d for m in (1, 2) for d in (-1, 0, 1)}):
        note("unique tile edge", np.dtype(dtype).name, n)
        r = np.random.default_rng(n)
        vals = np.repeat(r.integers(0, 100, size=n), r.integers(1, 4, size=n))[:n].astype(dtype)
        kept, _, count = gpu_unique(vals)
        expect = O.unique(vals)
        assert count == expect.size, n
        assert np.array_equal(kept.view(np.uint8), expect.view(np.uint8)), n
    # a run that spans a whole tile and its two borders
    vals = np.concatenate([np.arange(tile - 2), np.full(tile + 5, 7), np.arange(9)]).astype(dtype)
    kept, _, count = gpu_unique(vals)
    expect = O.unique(vals)
    assert count == expect.size and np.array_equal(kept.view(np.uint8), expect.view(np.uint8))


def test_unique_all_equal_and_all_distinct_large():
    n = (1 << 24) + 3
    kept, _, count = gpu_unique(np.full(n, 7, dtype=np.int32))
    assert count == 1 and kept[0] == 7
    seq = np.arange(n, dtype=np.uint32)
    kept, _, count = gpu_unique(seq)
    assert count == n and np.array_equal(kept, seq)


def test_unique_unaligned_view():
    vals = np.repeat(np.arange(5000, dtype=np.int32), 3)
    base = D.from_numpy(np.concatenate([np.array([99], np.int32), vals]))
    view = base.subview(1, vals.size)
    out_len = D.zeros(1, np.int64)
    capi.unique(view, out_len)
    sync()
    got = base.numpy()
    assert got[0] == 99 and int(out_len.numpy()[0]) == 5000
    assert np.array_equal(got[1:5001], np.arange(5000, dtype=np.int32))


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES + [100003])
def test_sequence_reference_cases(dtype, n):
    # SequencerTests.tt:56-96 and the repeated/batched forms.
    d = D.zeros(n, dtype)
    capi.sequence(d)
    sync()
    assert np.array_equal(d.numpy().view(np.uint8), O.sequence(n, dtype).view(np.uint8))
    for seq_len, batch in [(5, 1), (n, 4), (7, 3)]:
        capi.sequence(d, sequence_length=seq_len, batch_length=batch)
        sync()
        assert np.array_equal(d.numpy().view(np.uint8),
                              O.sequence(n, dtype, seq_len, batch).view(np.uint8))


def test_sequence_strided_and_errors():
    phys = D.from_numpy(np.full(30, -1, dtype=np.int32))
    capi.sequence(phys.strided(3))
    sync()
    got = phys.numpy()
    assert np.array_equal(got[::3], np.arange(10, dtype=np.int32))
    assert np.all(np.delete(got, np.arange(0, 30, 3)) == -1)
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.sequence(phys, sequence_length=0)
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.sequence(phys, batch_length=0)
    with pytest.raises(capi.ArgumentNullError):
        capi.sequence(D(0, np.int32))


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("n", [1, 5, 127, 4099, 1 << 20])
def test_initialize(dtype, n):
    value = np.array([3], dtype=np.int64).astype(dtype)[0] if np.dtype(dtype).kind != "f" else np.dtype(dtype).type(-1.5)
    base = D.from_numpy(np.zeros(n + 2, dtype=dtype))
    capi.initialize(base.subview(1, n), value)        # unaligned start: head/tail paths
    sync()
    got = base.numpy()
    assert got[0] == 0 and got[-1] == 0
    assert np.array_equal(got[1:-1], O.initialize(n, value))


def test_initialize_strided_and_16_byte():
    phys = D.from_numpy(np.zeros(40, dtype=np.uint16))
    capi.initialize(phys.strided(4), 0xBEEF)
    sync()
    got = phys.numpy()
    assert np.all(got[::4] == 0xBEEF) and np.all(np.delete(got, np.arange(0, 40, 4)) == 0)
    pair = np.dtype([("a", np.uint64), ("b", np.uint64)])
    d = D(1000, pair)
    value = np.array([(1, 2)], dtype=pair)
    capi.lib().ilgpu_hip_initialize(None, d.ptr, 1000, 1, 16, value.ctypes.data)
    sync()
    assert np.all(d.numpy() == value[0])


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.int64])
def test_reorder(dtype):
    for n in [1, 33, 1027, 1 << 18]:
        src = np.random.default_rng(n).integers(0, 100, n).astype(dtype)
        order = np.random.default_rng(n + 1).permutation(n).astype(np.int32)
        tgt = D.zeros(n, dtype)
        capi.reorder(D.from_numpy(src), tgt, D.from_numpy(order))
        sync()
        assert np.array_equal(tgt.numpy(), O.reorder(src, order))
    # ReorderExtensions.cs:166-167: the order view must cover the source
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.reorder(D.zeros(10, dtype), D.zeros(10, dtype), D.zeros(5, np.int32))
    # TransformExtensions.cs:324-331: the target must hold one element per index
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.reorder(D.zeros(10, dtype), D.zeros(9, dtype), D.zeros(10, np.int32))


ALL_NUMERIC = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64,
               np.uint64, np.float16, np.float32, np.float64]


def _transform_input(dtype, n, seed):
    dt = np.dtype(dtype)
    if dt.kind == "f":
        # finite values of every magnitude the type holds, both signs, zeros, and
        # specials; doubles include values that fall between float16/float32 neighbours
        r = np.random.default_rng(seed)
        mag = np.exp(r.uniform(-40, 40, n)) if dt.itemsize > 2 else np.exp(r.uniform(-12, 11, n))
        v = (mag * r.choice([-1.0, 1.0], n)).astype(dt)
        v[:8] = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 65519.99], dtype=dt)[: min(8, n)]
        if dt.itemsize == 8 and n > 12:
            # just above the midpoint of two float16 neighbours: rounding to float32 first
            # would land on the midpoint and then round the wrong way
            v[8:12] = [1 + 2.0 ** -11 + 2.0 ** -40, -(1 + 2.0 ** -11 + 2.0 ** -40),
                       1 + 3 * 2.0 ** -11 - 2.0 ** -40, 2.0 ** -25 + 2.0 ** -60]
        return v
    v = random_ints(dtype, n, seed=seed)
    info = np.iinfo(dtype)
    edge = np.array([0, 1, info.max, info.min, info.max - 1], dtype=dtype)
    v[: min(5, n)] = edge[: min(5, n)]
    return v


def _same_bits(a, b):
    if a.dtype.kind == "f":   # NaN payloads are not pinned: compare NaN-ness, then the rest bitwise
        na, nb = np.isnan(a), np.isnan(b)
        return np.array_equal(na, nb) and np.array_equal(a[~na].view(np.uint8), b[~nb].view(np.uint8))
    return np.array_equal(a, b)


@pytest.mark.parametrize("sdt", ALL_NUMERIC)
def test_transform_every_type_pair_and_transformer(sdt):
    n = 5000
    src = _transform_input(sdt, n, seed=np.dtype(sdt).num)
    d_src = D.from_numpy(src)
    for tdt in ALL_NUMERIC:
        if np.dtype(sdt).kind == "f" and np.dtype(tdt).kind != "f":
            with pytest.raises(capi.NotSupportedError):
                capi.transform(d_src, D.zeros(n, tdt))
            continue
        for op, factor in ((capi.TRANSFORM_CONVERT, 0), (capi.TRANSFORM_NEGATE, 0),
                           (capi.TRANSFORM_BIT_COMPLEMENT, 0), (capi.TRANSFORM_MULTIPLY, 2),
                           (capi.TRANSFORM_MULTIPLY, -3)):
            if op == capi.TRANSFORM_BIT_COMPLEMENT and np.dtype(sdt).kind == "f":
                continue
            note("transform", np.dtype(sdt).name, np.dtype(tdt).name, op, factor)
            tgt = D.zeros(n, tdt)
            capi.transform(d_src, tgt, op, factor)
            sync()
            assert _same_bits(tgt.numpy(), O.transform(src, tdt, op, factor)), (sdt, tdt, op)


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.uint16, np.int16, np.uint32])
def test_transform_multiply_wraps_in_the_source_type(dtype):
    # Largest operands: 0xFFFF * 0xFFFF does not fit the int that 16-bit operands
    # are promoted to; the product must wrap in the source type all the same.
    # Expected values are worked out with Python integers.
    bits = np.dtype(dtype).itemsize * 8
    top = (1 << bits) - 1
    raw = [top, top - 1, 1 << (bits - 1), (1 << (bits - 1)) - 1, 3, 0]
    src = np.array(raw, dtype=np.dtype(f"uint{bits}")).view(dtype)
    for factor in (top, -1, (1 << (bits - 1)) + 1):
        signed = np.dtype(dtype).kind == "i"
        expect = []
        for r in raw:
            v = r - (1 << bits) if signed and r >> (bits - 1) else r
            expect.append((v * factor) % (1 << bits))
        tgt = D.zeros(len(raw), dtype)
        capi.transform(D.from_numpy(src), tgt, capi.TRANSFORM_MULTIPLY, factor)
        sync()
        got = tgt.numpy().view(np.dtype(f"uint{bits}")).tolist()
        assert got == expect, (dtype, factor)
        assert _same_bits(tgt.numpy(), O.transform(src, dtype, O.TRANSFORM_MULTIPLY, factor))


@pytest.mark.parametrize("n", ARRAY_SIZES + [1 << 20, (1 << 20) + 3])
def test_transform_reference_cases(n):
    # TransformerExtensionTests.tt:66-134
    seq = compute_sequence(np.int32, 42, 0, n)
    out = D.zeros(n, np.int32)
    capi.transform(D.from_numpy(seq), out, capi.TRANSFORM_NEGATE)
    out64 = D.zeros(n, np.int64)
    capi.transform(D.from_numpy(seq), out64)
    useq = compute_sequence(np.uint32, 0, 1, n)
    comp = D.zeros(n, np.int32)
    capi.transform(D.from_numpy(useq), comp, capi.TRANSFORM_BIT_COMPLEMENT)
    sync()
    assert np.array_equal(out.numpy(), np.full(n, -42, dtype=np.int32))
    assert np.array_equal(out64.numpy(), np.full(n, 42, dtype=np.int64))
    assert np.array_equal(comp.numpy(), (-1 - np.arange(n)).astype(np.int32))


def test_transform_in_place_strided_and_longer_target():
    n = 10007
    src = random_ints(np.int32, n, seed=9)
    d = D.from_numpy(src)
    capi.transform(d, d, capi.TRANSFORM_NEGATE)      # in place
    sync()
    assert np.array_equal(d.numpy(), O.transform(src, np.int32, O.TRANSFORM_NEGATE))
    # strided source and target views; elements between the strides stay untouched
    base = random_ints(np.int16, 3 * n, seed=10)
    out = np.full(2 * n + 5, 77, dtype=np.int64)
    d_base_in, d_base_out = D.from_numpy(base), D.from_numpy(out)
    d_in, d_out = d_base_in.strided(3), d_base_out.strided(2)
    assert d_in.length == n and d_out.length >= n
    capi.transform(d_in, d_out, capi.TRANSFORM_MULTIPLY, 2)
    sync()
    expect = out.copy()
    expect[0: 2 * n: 2] = O.transform(base[::3], np.int64, O.TRANSFORM_MULTIPLY, 2)
    assert np.array_equal(d_base_out.numpy(), expect)
    # TransformExtensions.cs:310-317: a short target is refused
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.transform(D.zeros(10, np.int32), D.zeros(9, np.int32))


@pytest.mark.parametrize("sdt,tdt", [(np.int32, np.int32), (np.uint8, np.uint8), (np.int32, np.int64),
                                     (np.uint8, np.uint64), (np.int64, np.int16), (np.float64, np.float16),
                                     (np.int16, np.float32)])
def test_transform_dense_vector_path_heads_and_tails(sdt, tdt):
    # the dense path moves 16-byte vectors: lengths around whole vectors, and views
    # that start off a vector boundary (which take the element-wise path)
    src = _transform_input(sdt, 70000, seed=31)
    d_src = D.from_numpy(src)
    for off_in, off_out, n in [(0, 0, 65536), (0, 0, 65537), (0, 0, 65551), (0, 0, 1), (0, 0, 15),
                               (1, 0, 40000), (0, 3, 40001), (5, 5, 4099), (16, 16, 8191)]:
        base = np.full(n + off_out + 4, 77, dtype=tdt)
        d_out = D.from_numpy(base)
        capi.transform(d_src.subview(off_in, n), d_out.subview(off_out, n), capi.TRANSFORM_MULTIPLY, 3)
        sync()
        expect = base.copy()
        expect[off_out:off_out + n] = O.transform(src[off_in:off_in + n], tdt, O.TRANSFORM_MULTIPLY, 3)
        assert _same_bits(d_out.numpy(), expect), (sdt, tdt, off_in, off_out, n)


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
def test_reorder_transform_reference_case_and_random_gather(dtype):
    # ReorderExtensionTests.tt:160-200: reversed order, value * 2
    for n in ARRAY_SIZES:
        for start, step in ((0, 0), (1, 0), (0, 1)):
            seq = compute_sequence(dtype, start, step, n)
            order = np.arange(n - 1, -1, -1, dtype=np.int32)
            tgt = D.zeros(n, dtype)
            capi.reorder_transform(D.from_numpy(seq), tgt, D.from_numpy(order),
                                   capi.TRANSFORM_MULTIPLY, 2)
            sync()
            with np.errstate(over="ignore"):
                expect = (seq + seq)[::-1]
            assert np.array_equal(tgt.numpy().view(np.uint8), np.ascontiguousarray(expect).view(np.uint8))
    # ReorderExtensionTests.tt:69-112: widening and bit-complement transformers, random order
    n = 1 << 18
    for sdt, tdt, op in ((np.int32, np.int64, capi.TRANSFORM_CONVERT),
                         (np.uint32, np.uint64, capi.TRANSFORM_CONVERT),
                         (np.uint32, np.int32, capi.TRANSFORM_BIT_COMPLEMENT),
                         (np.uint64, np.int64, capi.TRANSFORM_BIT_COMPLEMENT)):
        src = random_ints(sdt, n, seed=21)
        order = np.random.default_rng(22).permutation(n).astype(np.int32)
        tgt = D.zeros(n, tdt)
        capi.reorder_transform(D.from_numpy(src), tgt, D.from_numpy(order), op)
        sync()
        assert np.array_equal(tgt.numpy(), O.reorder_transform(src, order, tdt, op))


def test_sort_then_unique_pipeline():
    # the pipeline the two primitives are used for: distinct keys of a column
    keys = datagen.zipf_u32(1 << 22)
    d = D.from_numpy(keys)
    capi.radix_sort_keys(d)
    out_len = D.zeros(1, np.int64)
    capi.unique(d, out_len)
    sync()
    count = int(out_len.numpy()[0])
    assert np.array_equal(d.numpy()[:count], np.unique(keys))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("op", [capi.OP_MAX, capi.OP_MIN])
def test_scan_float_max_min_signed_zero_and_nan(dtype, op):
    # Math.Max/Math.Min (IntrinsicMath.cs:111-112, 207-208): -0.0 < +0.0, and
    # from the first NaN on every result is NaN.
    for n in [64, 5000, 300000]:
        r = np.random.default_rng(n)
        v = r.integers(-3, 3, n).astype(dtype)
        v[v == 0] = np.where(r.integers(0, 2, int((v == 0).sum())) == 0, 0.0, -0.0)
        d_in, d_out = D.from_numpy(v), D.zeros(n, dtype)
        capi.scan(d_in, d_out, op=op, kind=capi.SCAN_INCLUSIVE)
        sync()
        expect = O.scan(v, op=op, inclusive=True)
        assert np.array_equal(d_out.numpy().view(np.uint8), expect.view(np.uint8)), n
        w = v.copy()
        w[n // 2] = np.nan
        capi.scan(D.from_numpy(w), d_out, op=op, kind=capi.SCAN_INCLUSIVE)
        sync()
        got = d_out.numpy()
        assert np.array_equal(got[: n // 2].view(np.uint8), expect[: n // 2].view(np.uint8))
        assert np.isnan(got[n // 2:]).all()


# ------------------------------------------------------------- tile boundaries
# Lengths just below, at and just above one and two tiles of every tile shape
# the pass kernel uses (512 threads x 36, 20, 18, 16, 14 or 8 items).
TILE_EDGE_SIZES = sorted({t * m + d for t in (4096, 7168, 8192, 9216, 10240, 18432)
                          for m in (1, 2)
                          for d in (-1, 0, 1)})


@pytest.mark.parametrize("dtype", [np.uint8, np.uint32, np.uint64, np.float64])
def test_sort_keys_tile_edges(dtype):
    for n in TILE_EDGE_SIZES:
        note("sort edge", np.dtype(dtype).name, n)
        keys = (random_float_bits(dtype, n, seed=n) if np.dtype(dtype).kind == "f"
                else random_ints(dtype, n, seed=n))
        d = D.from_numpy(keys)
        capi.radix_sort_keys(d)
        sync()
        assert np.array_equal(d.numpy().view(np.uint8), O.radix_sort(keys).view(np.uint8)), n


@pytest.mark.parametrize("kdt,vdt", [(np.uint32, np.uint32), (np.uint64, np.uint32),
                                     (np.uint32, np.uint64), (np.uint16, np.uint8)])
def test_sort_pairs_tile_edges(kdt, vdt):
    for n in TILE_EDGE_SIZES:
        note("pairs edge", np.dtype(kdt).name, np.dtype(vdt).name, n)
        keys = random_ints(kdt, n, seed=n, lo=0, hi=500)        # duplicates: stability matters
        vals = (np.arange(n, dtype=np.uint64) * 7 + 3).astype(vdt)
        dk, dv = D.from_numpy(keys), D.from_numpy(vals)
        capi.radix_sort_pairs(dk, dv)
        sync()
        ek, ev = O.radix_sort_pairs(keys, vals)
        assert np.array_equal(dk.numpy(), ek) and np.array_equal(dv.numpy(), ev), n


def test_sort_pairs_16_byte_values_tile_edges():
    pair = np.dtype([("a", np.uint64), ("b", np.uint64)])
    for n in TILE_EDGE_SIZES:
        keys = random_ints(np.uint32, n, seed=n, lo=0, hi=300)
        vals = np.zeros(n, dtype=pair)
        vals["a"] = np.arange(n)
        vals["b"] = ~np.arange(n, dtype=np.uint64)
        dk, dv = D.from_numpy(keys), D.from_numpy(vals)
        capi.radix_sort_pairs(dk, dv)
        sync()
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(dk.numpy(), keys[order]), n
        assert np.array_equal(dv.numpy(), vals[order]), n


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.int64, np.uint64])
def test_scan_tile_edges(dtype):
    # a tile is 512 threads x 16 sixteen-byte vectors for 4-byte elements, x 10 for 8-byte ones
    tile = 512 * (16 * 4 if np.dtype(dtype).itemsize == 4 else 10 * 2)
    for n in sorted({tile * m + d for m in (1, 2, 3) for d in (-1, 0, 1)}):
        vals = random_ints(dtype, n, seed=n)
        for op in (capi.OP_ADD, capi.OP_MAX, capi.OP_MIN):
            for inclusive in (True, False):
                note("scan tile edge", np.dtype(dtype).name, n, op, inclusive)
                got = gpu_scan(vals, op, inclusive)
                assert np.array_equal(got[:n], O.scan(vals, op=op, inclusive=inclusive)), (n, op, inclusive)


# ------------------------------------------------------------- dominant digits
# A digit that holds an eighth of the keys or more is ranked by ballots instead
# of LDS slots (up to four such digits per pass).
@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.uint32, np.int64, np.float32])
@pytest.mark.parametrize("shares", [(1.0,), (0.6, 0.4), (0.5, 0.2, 0.2), (0.25, 0.25, 0.25, 0.25),
                                    (0.2, 0.2, 0.2, 0.2, 0.2), (0.13, 0.13)])
def test_sort_keys_with_dominant_digits(dtype, shares):
    r = np.random.default_rng(len(shares) * 131 + np.dtype(dtype).num)
    for n in (1, 777, 18431, 18432, 18433, 100003, (1 << 20) + 11):
        note("dominant digits", np.dtype(dtype).name, shares, n)
        # chosen values differ in every byte, 0xFF bytes included (the digit of the
        # padding keys in a partial tile); the rest of the keys are uniform
        pool = np.array([0xFFFFFFFFFFFFFFFF, 0x0101010101010101, 0x80FF80FF80FF80FF,
                         0x7F007F007F007F00, 0x55AA55AA55AA55AA], dtype=np.uint64)
        which = r.choice(len(shares) + 1, size=n, p=list(shares) + [max(0.0, 1.0 - sum(shares))])
        bits = np.where(which < len(shares), pool[np.minimum(which, len(pool) - 1)],
                        r.integers(0, 1 << 63, size=n, dtype=np.uint64))
        width = np.dtype(dtype).itemsize
        keys = (bits & np.uint64((1 << (8 * width)) - 1 if width < 8 else 0xFFFFFFFFFFFFFFFF)).astype(
            np.dtype("u%d" % width)).view(dtype)
        for desc in (False, True):
            d = D.from_numpy(keys)
            capi.radix_sort_keys(d, descending=desc)
            sync()
            assert np.array_equal(d.numpy().view(np.uint8),
                                  O.radix_sort(keys, descending=desc).view(np.uint8)), (n, desc)


@pytest.mark.parametrize("kdt,vdt", [(np.uint32, np.uint32), (np.uint64, np.uint32), (np.uint16, np.uint64)])
def test_sort_pairs_with_dominant_digits_is_stable(kdt, vdt):
    r = np.random.default_rng(77)
    for n in (5000, 100003, (1 << 20) + 5):
        keys = r.choice(np.array([0, 255, 256, 0xFFFF, 12345], dtype=np.uint64), size=n,
                        p=[0.5, 0.2, 0.15, 0.1, 0.05]).astype(kdt)
        dk, dv = D.from_numpy(keys), D.zeros(n, vdt)
        capi.radix_sort_pairs(dk, dv, values_from_index=True)
        sync()
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(dk.numpy(), keys[order])
        assert np.array_equal(dv.numpy(), order.astype(vdt))


@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.uint32, np.int64, np.float64])
@pytest.mark.parametrize("run", [2, 15, 16, 17, 64, 1000])
def test_sort_keys_in_runs_and_presorted(dtype, run):
    # Rows of sixteen neighbouring keys that share a digit take a shortcut in the
    # ranking: runs around the row length, runs that straddle rows, sorted and
    # reversed inputs.
    r = np.random.default_rng(run)
    for n in (run, 18432 + run // 2, 100003, (1 << 20) + 7):
        note("runs", np.dtype(dtype).name, run, n)
        starts = r.integers(0, 1 << 62, size=n // run + 2, dtype=np.uint64)
        bits = np.repeat(starts, run)[r.integers(0, run):][:n]
        width = np.dtype(dtype).itemsize
        keys = (bits >> np.uint64(64 - 8 * width)).astype(np.dtype("u%d" % width)).view(dtype)
        if np.dtype(dtype).kind == "f":
            keys = np.where(np.isnan(keys), np.dtype(dtype).type(1.5), keys)
        for variant in (keys, np.sort(keys), np.sort(keys)[::-1].copy()):
            d = D.from_numpy(variant)
            capi.radix_sort_keys(d)
            sync()
            assert np.array_equal(d.numpy().view(np.uint8), O.radix_sort(variant).view(np.uint8)), n


def test_sort_pairs_in_runs_is_stable():
    r = np.random.default_rng(5)
    for n in (40000, (1 << 20) + 3):
        keys = np.repeat(r.integers(0, 1 << 20, size=n // 50 + 1), 50)[:n].astype(np.uint32)
        dk, dv = D.from_numpy(keys), D.zeros(n, np.uint32)
        capi.radix_sort_pairs(dk, dv, values_from_index=True)
        sync()
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(dk.numpy(), keys[order])
        assert np.array_equal(dv.numpy(), order.astype(np.uint32))


# ------------------------------------------------------------- streams, graphs
def test_two_streams_run_independent_calls_concurrently():
    # Calls on different streams with different temps must not disturb each
    # other (the delegates are re-entrant across streams; only a temp buffer is
    # single-use at a time).
    import torch
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    n1, n2 = 3_000_017, 2_500_003
    keys = random_ints(np.uint32, n1, seed=41)
    vals = random_ints(np.int32, n2, seed=42, lo=-9, hi=9)
    samples = random_ints(np.uint8, n2, seed=43)
    d_keys = [D.from_numpy(keys) for _ in range(4)]
    d_vals = D.from_numpy(vals)
    d_scan = [D.zeros(n2, np.int32) for _ in range(4)]
    d_bins = [D.zeros(256, np.int32) for _ in range(4)]
    d_sum = [D.zeros(1, np.int32) for _ in range(4)]
    d_samples = D.from_numpy(samples)
    t_sort = capi.temp_buffer(capi.radix_sort_temp_bytes(n1, np.uint32))
    t_scan = capi.temp_buffer(capi.scan_temp_bytes(n2, np.int32))
    t_red = capi.temp_buffer(capi.reduce_temp_bytes(n2, np.int32))
    torch.cuda.synchronize()
    for i in range(4):
        with torch.cuda.stream(s1):
            capi.radix_sort_keys(d_keys[i], t_sort, descending=bool(i & 1))
        with torch.cuda.stream(s2):
            capi.scan(d_vals, d_scan[i], t_scan, kind=capi.SCAN_EXCLUSIVE)
            capi.histogram(d_samples, d_bins[i])
            capi.reduce(d_vals, d_sum[i], t_red)
    s1.synchronize()
    s2.synchronize()
    asc = O.radix_sort(keys)
    e_scan = O.scan(vals, inclusive=False)
    e_bins, _ = O.histogram(samples, np.zeros(256, dtype=np.int32))
    for i in range(4):
        assert np.array_equal(d_keys[i].numpy(), asc[::-1] if i & 1 else asc), i
        assert np.array_equal(d_scan[i].numpy(), e_scan), i
        assert np.array_equal(d_bins[i].numpy(), e_bins), i
        assert d_sum[i].numpy()[0] == O.reduce(vals), i


def test_two_sorts_on_two_streams_share_the_gpu():
    # Each sort's pass kernels are persistent and sized to fill the GPU, so two
    # of them on two streams can each hold only part of the compute units.  A
    # pass hands its tiles to fixed groups of blocks; no block may wait without
    # bound for a tile whose group is not resident (the look-back gives up on an
    # unpublished tile and counts it itself), so both sorts finish and are exact.
    import torch
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    n1, n2 = (1 << 24) + 11, (1 << 24) - 5
    a = datagen.uniform_u32(n1)
    b = datagen.uniform_u64(n2)
    d_a = [D.from_numpy(a) for _ in range(3)]
    d_b = [D.from_numpy(b) for _ in range(3)]
    d_v = [D.zeros(n2, np.uint32) for _ in range(3)]
    t_a = [capi.temp_buffer(capi.radix_sort_temp_bytes(n1, np.uint32)) for _ in range(3)]
    t_b = [capi.temp_buffer(capi.radix_sort_temp_bytes(n2, np.uint64, 4)) for _ in range(3)]
    torch.cuda.synchronize()
    note("two sorts on two streams", n1, n2)
    for i in range(3):
        with torch.cuda.stream(s1):
            capi.radix_sort_keys(d_a[i], t_a[i])
        with torch.cuda.stream(s2):
            capi.radix_sort_pairs(d_b[i], d_v[i], t_b[i], values_from_index=True)
    s1.synchronize()
    s2.synchronize()
    e_a = np.sort(a, kind="stable")
    order = np.argsort(b, kind="stable")
    for i in range(3):
        assert np.array_equal(d_a[i].numpy(), e_a), i
        assert np.array_equal(d_b[i].numpy(), b[order]), i
        assert np.array_equal(d_v[i].numpy(), order.astype(np.uint32)), i


def test_two_pipelined_sorts_on_two_streams_share_the_gpu():
    # Large keys-only sorts take the pipelined pass: one block per compute unit,
    # four of them scanning.  Two such sorts on two streams cannot both be
    # resident in full; a resolving wave polls its own row a bounded number of
    # times and then walks back itself, and a scanning block counts a tile that
    # nobody publishes, so both finish whatever the hardware interleaves.
    import torch
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    n1, n2 = (1 << 25) + 11, (1 << 24) + 12345
    a = datagen.uniform_u32(n1)
    b = datagen.uniform_u64(n2)
    d_a = [D.from_numpy(a) for _ in range(2)]
    d_b = [D.from_numpy(b) for _ in range(2)]
    t_a = [capi.temp_buffer(capi.radix_sort_temp_bytes(n1, np.uint32)) for _ in range(2)]
    t_b = [capi.temp_buffer(capi.radix_sort_temp_bytes(n2, np.uint64)) for _ in range(2)]
    torch.cuda.synchronize()
    note("two pipelined sorts on two streams", n1, n2)
    for i in range(2):
        with torch.cuda.stream(s1):
            capi.radix_sort_keys(d_a[i], t_a[i])
        with torch.cuda.stream(s2):
            capi.radix_sort_keys(d_b[i], t_b[i])
    s1.synchronize()
    s2.synchronize()
    e_a, e_b = np.sort(a, kind="stable"), np.sort(b, kind="stable")
    for i in range(2):
        assert np.array_equal(d_a[i].numpy(), e_a), i
        assert np.array_equal(d_b[i].numpy(), e_b), i


def test_calls_can_be_captured_into_a_graph_and_replayed():
    # Every call is stream-ordered kernels only (temp memory is cleared by a
    # fill kernel, nothing is allocated), so a sequence of calls can be
    # captured once and replayed.  Each replay runs on new input contents, with
    # eager work and synchronisations in between, and is checked on its own.
    import torch
    n = 1_200_007
    static_keys = torch.zeros(n, dtype=torch.int32, device="cuda:0")
    static_vals = torch.zeros(n, dtype=torch.int32, device="cuda:0")
    work = torch.zeros(n, dtype=torch.int32, device="cuda:0")
    uniq = torch.zeros(n, dtype=torch.int32, device="cuda:0")
    scanned = torch.zeros(n, dtype=torch.int32, device="cuda:0")
    bins = torch.zeros(4096, dtype=torch.int32, device="cuda:0")

    def wrap(t, dt):
        return D(t.numel(), dt, _bytes=t.view(torch.uint8))

    d_work, d_uniq = wrap(work, np.uint32), wrap(uniq, np.uint32)
    d_vals, d_scanned, d_bins = wrap(static_vals, np.int32), wrap(scanned, np.int32), wrap(bins, np.int32)
    d_total, d_count = D.zeros(1, np.int32), D.zeros(1, np.int64)
    t_sort = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32))
    t_scan = capi.temp_buffer(capi.scan_temp_bytes(n, np.int32))
    t_red = capi.temp_buffer(capi.reduce_temp_bytes(n, np.int32))
    t_uniq = capi.temp_buffer(capi.unique_temp_bytes(n, np.uint32))

    def sequence_of_calls():
        work.copy_(static_keys)
        capi.radix_sort_keys(d_work, t_sort)
        uniq.copy_(work)
        capi.unique(d_uniq, d_count, t_uniq)
        capi.scan(d_vals, d_scanned, t_scan, kind=capi.SCAN_INCLUSIVE)
        capi.reduce(d_vals, d_total, t_red)
        bins.zero_()
        capi.histogram(d_vals, d_bins)

    def fill(seed):
        k = random_ints(np.uint32, n, seed=seed, lo=0, hi=50_000)
        v = random_ints(np.int32, n, seed=seed + 1, lo=0, hi=4095)
        static_keys.copy_(torch.from_numpy(k.view(np.int32)))
        static_vals.copy_(torch.from_numpy(v))
        return k, v

    def check(k, v, tag):
        torch.cuda.synchronize()
        assert np.array_equal(d_work.numpy(), O.radix_sort(k)), tag
        e = O.unique(O.radix_sort(k))
        kept = int(d_count.numpy()[0])
        assert kept == e.size and np.array_equal(d_uniq.numpy()[:kept], e), tag
        assert np.array_equal(d_scanned.numpy(), O.scan(v)), tag
        assert d_total.numpy()[0] == O.reduce(v), tag
        eb, _ = O.histogram(v, np.zeros(4096, dtype=np.int32))
        assert np.array_equal(d_bins.numpy(), eb), tag

    k, v = fill(100)
    sequence_of_calls()                      # eager, also warms the one-time queries
    check(k, v, "eager")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            sequence_of_calls()
    torch.cuda.synchronize()
    for r in range(3):
        k, v = fill(200 + 10 * r)
        junk = torch.rand(1 << 20, device="cuda:0").sum().item()   # eager work between replays
        assert junk > 0
        graph.replay()
        check(k, v, ("replay", r))
