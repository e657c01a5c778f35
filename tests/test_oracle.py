"""Pins the CPU oracle against evidence that does not come from the oracle:
the reference's own test sequences and expectations, numpy's stable sort,
cumulative sums and bincount, and closed forms.  No GPU needed."""
import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.refcases import (ALL_KEY_DTYPES, ARRAY_SIZES, ATOMIC_NUMERIC_DTYPES,
                            compute_inverted_sequence, compute_sequence)

INT_KEY_DTYPES = [d for d in ALL_KEY_DTYPES if np.dtype(d).kind in "iu"]
SCAN_INT_DTYPES = [np.int32, np.int64, np.uint32, np.uint64]


def rng(seed=0):
    return np.random.default_rng(seed)


def random_ints(dtype, n, seed=0, lo=None, hi=None):
    info = np.iinfo(dtype)
    lo = info.min if lo is None else lo
    hi = info.max if hi is None else hi
    return rng(seed).integers(lo, hi, size=n, dtype=dtype, endpoint=True)


# ---------------------------------------------------------------- radix sort
@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
def test_sort_reference_worst_and_best_case(dtype, n):
    # RadixSortExtensionTests.tt:144-230: inverted sequence sorts to the
    # sequence; an already sorted sequence stays put.
    seq = compute_sequence(dtype, 0, 1, n)
    inv = compute_inverted_sequence(dtype, 0, 1, n)
    assert np.array_equal(O.radix_sort(inv), seq)
    assert np.array_equal(O.radix_sort(seq), seq)
    assert np.array_equal(O.radix_sort(seq, descending=True), inv)
    assert np.array_equal(O.radix_sort(inv, descending=True), inv)


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
@pytest.mark.parametrize("start", [0, 1, -1])
def test_sort_reference_constant_case(dtype, n, start):
    # RadixSortExtensionTests.tt:370-432 (start -1 only for signed/float types)
    if np.dtype(dtype).kind == "u" and start < 0:
        pytest.skip("unsigned types have no -1 case in the reference")
    seq = compute_sequence(dtype, start, 0, n)
    assert np.array_equal(O.radix_sort(seq), seq)


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
def test_sort_pairs_reference_case(dtype, n):
    # RadixSortExtensionTests.tt:319-365: values == keys, both end up sorted.
    seq = compute_sequence(dtype, 0, 1, n)
    inv = compute_inverted_sequence(dtype, 0, 1, n)
    k, v = O.radix_sort_pairs(inv, inv)
    assert np.array_equal(k, seq) and np.array_equal(v, seq)
    k, v = O.radix_sort_pairs(seq, seq, descending=True)
    assert np.array_equal(k, inv) and np.array_equal(v, inv)


def test_sort_sample_program():
    # Samples/AlgorithmsRadixSort/Program.cs:59-63: 32 reversed ints.
    data = np.arange(32, 0, -1, dtype=np.int32)
    assert np.array_equal(O.radix_sort(data), np.arange(1, 33, dtype=np.int32))


@pytest.mark.parametrize("dtype", INT_KEY_DTYPES)
@pytest.mark.parametrize("n", [1, 2, 17, 1000, 4099])
def test_sort_random_integers_match_numpy(dtype, n):
    keys = random_ints(dtype, n, seed=n)
    assert np.array_equal(O.radix_sort(keys), np.sort(keys, kind="stable"))
    assert np.array_equal(O.radix_sort(keys, descending=True),
                          np.sort(keys, kind="stable")[::-1])


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.uint32, np.int64])
@pytest.mark.parametrize("descending", [False, True])
def test_sort_pairs_is_the_stable_permutation(dtype, descending):
    # Few distinct keys, payload = original index: the value array must be the
    # unique stable permutation.  Descending order in the reference inverts the
    # digits (RadixSortOperations.tt:122-123), so equal keys still keep their
    # original order.
    n = 5000
    keys = random_ints(dtype, n, seed=7, lo=0, hi=9)
    values = np.arange(n, dtype=np.uint32)
    order_key = -keys.astype(np.int64) if descending else keys.astype(np.int64)
    perm = np.argsort(order_key, kind="stable")
    k, v = O.radix_sort_pairs(keys, values, descending=descending)
    assert np.array_equal(k, keys[perm])
    assert np.array_equal(v, values[perm])


@pytest.mark.parametrize("num_groups", [1, 3, 16, 64])
def test_sort_is_independent_of_the_virtual_group_count(num_groups):
    keys = random_ints(np.uint32, 3001, seed=3)
    assert np.array_equal(O.radix_sort(keys, num_groups=num_groups),
                          np.sort(keys, kind="stable"))


@pytest.mark.parametrize("dtype", INT_KEY_DTYPES)
def test_radix_bits_reassemble_to_numeric_order(dtype):
    # Concatenating the 2-bit digits, most significant first, must give a key
    # whose unsigned order is the numeric order of the values.
    vals = random_ints(dtype, 200, seed=11)
    bits = np.dtype(dtype).itemsize * 8
    keys = []
    for v in vals:
        k = 0
        for shift in range(bits - 2, -2, -2):
            k = (k << 2) | O.extract_radix_bits(np.array(v, dtype=dtype), False,
                                                shift, 3)
        keys.append(k)
    order = np.argsort(np.array(keys, dtype=object), kind="stable")
    assert np.array_equal(vals[order], np.sort(vals, kind="stable"))
    # descending digits are the complement
    d = O.extract_radix_bits(np.array(vals[0], dtype=dtype), False, 0, 3)
    assert O.extract_radix_bits(np.array(vals[0], dtype=dtype), True, 0, 3) == (~d & 3)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_float_sort_as_written_in_the_reference(dtype):
    # PARITY UNPINNED beyond non-negative integers and constant -1: no
    # reference test sorts negative or adjacent floats.  The expectation below
    # is a hand evaluation of RadixSortOperations.tt:81-89 (logical shift of
    # the unsigned bit pattern): negatives keep ascending MAGNITUDE order and
    # positives that differ only in the last mantissa bit swap.
    one_up = np.nextafter(dtype(1), dtype(2))
    data = np.array([-2, -1, -0.0, 0, 1, one_up, 2], dtype=dtype)
    expect = np.array([-0.0, -1, -2, 0, one_up, 1, 2], dtype=dtype)
    got = O.radix_sort(data)
    assert np.array_equal(got.view(np.uint8), expect.view(np.uint8))


# ---------------------------------------------------------------------- scan
def serial_fold(values, op, inclusive, identity):
    # CalcValues of ScanExtensionTests.tt:286-305.
    out = np.empty_like(values)
    acc = values.dtype.type(identity)
    with np.errstate(over="ignore"):
        for i, v in enumerate(values):
            if inclusive:
                acc = op(acc, v)
                out[i] = acc
            else:
                out[i] = acc
                acc = op(acc, v)
    return out


def identity_of(dtype, op):
    dtype = np.dtype(dtype)
    if op == O.OP_ADD:
        return 0
    if dtype.kind in "iu":
        info = np.iinfo(dtype)
        return info.min if op == O.OP_MAX else info.max
    info = np.finfo(dtype)
    return info.min if op == O.OP_MAX else info.max


NP_OPS = {O.OP_ADD: lambda a, b: a + b, O.OP_MAX: max, O.OP_MIN: min}


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
@pytest.mark.parametrize("op", [O.OP_ADD, O.OP_MAX, O.OP_MIN])
@pytest.mark.parametrize("inclusive", [True, False])
def test_scan_reference_sequences(dtype, n, op, inclusive):
    # ScanExtensionTests.tt:43-104: ascending, constant and descending
    # sequences; floats only up to 1000 elements (:52).
    if np.dtype(dtype).kind == "f" and n > 1000:
        pytest.skip("the reference caps float scans at 1000 elements")
    for start, step in [(0, 1), (1, 0), (n, -1)]:
        if np.dtype(dtype).kind == "u" and step < 0:
            seq = compute_sequence(dtype, n, 1, n)[::-1].copy()
        else:
            seq = compute_sequence(dtype, start, step, n)
        expect = serial_fold(seq, NP_OPS[op], inclusive, identity_of(dtype, op))
        got = O.scan(seq, op=op, inclusive=inclusive)
        assert np.array_equal(got, expect), (start, step)


def test_scan_sample_program():
    # Samples/AlgorithmsScan/Program.cs:32-33: scan of 32 twos.
    twos = np.full(32, 2, dtype=np.int32)
    assert np.array_equal(O.scan(twos, inclusive=True), 2 * np.arange(1, 33))
    assert np.array_equal(O.scan(twos, inclusive=False), 2 * np.arange(0, 32))


@pytest.mark.parametrize("dtype", SCAN_INT_DTYPES)
@pytest.mark.parametrize("n", [1, 15, 16, 17, 5000])
def test_scan_random_integers_wrap_like_numpy(dtype, n):
    v = random_ints(dtype, n, seed=n)  # full range: the sums wrap
    with np.errstate(over="ignore"):
        inc = np.cumsum(v, dtype=dtype)
    assert np.array_equal(O.scan(v, inclusive=True), inc)
    exc = np.concatenate([np.zeros(1, dtype=dtype), inc[:-1]])
    assert np.array_equal(O.scan(v, inclusive=False), exc)
    assert np.array_equal(O.scan(v, op=O.OP_MAX), np.maximum.accumulate(v))
    assert np.array_equal(O.scan(v, op=O.OP_MIN), np.minimum.accumulate(v))


@pytest.mark.parametrize("group_size", [2, 4, 16, 64])
def test_scan_is_independent_of_the_group_size_for_integers(group_size):
    v = random_ints(np.int32, 1000, seed=5)
    with np.errstate(over="ignore"):
        inc = np.cumsum(v, dtype=np.int32)
    assert np.array_equal(O.scan(v, group_size=group_size), inc)
    exc = np.concatenate([np.zeros(1, dtype=np.int32), inc[:-1]])
    assert np.array_equal(O.scan(v, inclusive=False, group_size=group_size), exc)


def test_float_max_min_follow_dotnet_math():
    # Math.Max / Math.Min: NaN wins, -0.0 < +0.0 (IntrinsicMath.cs:101-112,197-208).
    v = np.array([1.0, -0.0, 0.0, np.nan, 5.0], dtype=np.float32)
    got = O.scan(v, op=O.OP_MAX)
    assert got[0] == 1.0 and got[2] == 1.0 and np.isnan(got[3]) and np.isnan(got[4])
    z = np.array([0.0, -0.0], dtype=np.float64)
    assert np.signbit(O.scan(z, op=O.OP_MIN)[1])
    assert not np.signbit(O.scan(z[::-1].copy(), op=O.OP_MAX)[1])
    # identities are the finite extremes, not infinities
    assert O.scan(np.array([1.0], dtype=np.float32), op=O.OP_MAX,
                  inclusive=False)[0] == np.finfo(np.float32).min


# -------------------------------------------------------------------- reduce
@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
@pytest.mark.parametrize("op", [O.OP_ADD, O.OP_MAX, O.OP_MIN])
def test_reduce_reference_sequences(dtype, n, op):
    # ReductionExtensionTests.tt:41-106,205-212: left fold, exact equality.
    if np.dtype(dtype).kind == "f" and n > 1000:
        pytest.skip("the reference caps float reductions at 1000 elements")
    for start, step in [(0, 1), (1, 0)]:
        seq = compute_sequence(dtype, start, step, n)
        expect = serial_fold(seq, NP_OPS[op], True, identity_of(dtype, op))[-1]
        assert O.reduce(seq, op=op) == expect


def test_reduce_sample_program():
    # Samples/AlgorithmsReduce/Program.cs:29-31: sum of 0..63.
    assert O.reduce(np.arange(64, dtype=np.int32)) == 2016


@pytest.mark.parametrize("dtype", SCAN_INT_DTYPES)
def test_reduce_random_integers(dtype):
    v = random_ints(dtype, 10007, seed=2)
    with np.errstate(over="ignore"):
        assert O.reduce(v) == np.sum(v, dtype=dtype)
    assert O.reduce(v, op=O.OP_MAX) == v.max()
    assert O.reduce(v, op=O.OP_MIN) == v.min()


def test_reduce_float_add_within_tolerance_of_float64_sum():
    v = rng(4).standard_normal(100000).astype(np.float32)
    exact = O.sum_f64(v)
    assert exact == pytest.approx(float(np.sum(v.astype(np.float64))), rel=1e-12)
    assert abs(float(O.reduce(v)) - exact) <= 1e-3 * max(1.0, abs(exact))


# ----------------------------------------------------------------- histogram
HIST_IN_DTYPES = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16,
                  np.uint32, np.uint64, np.float32, np.float64]
HIST_BIN_DTYPES = [np.int32, np.int64, np.uint32, np.uint64]


@pytest.mark.parametrize("in_dtype", HIST_IN_DTYPES)
@pytest.mark.parametrize("bin_dtype", HIST_BIN_DTYPES)
@pytest.mark.parametrize("num_bins", [64, 256])
def test_histogram_reference_case(in_dtype, bin_dtype, num_bins):
    # HistogramTests.tt:42-47,83-144: inputs (T)1..(T)1024 (narrow types wrap
    # in the cast), modulo locator, bins start at zero.
    length = 1024
    values = np.arange(1, length + 1).astype(in_dtype)
    if np.dtype(in_dtype).kind == "f":
        located = np.abs(np.fmod(values, in_dtype(num_bins))).astype(np.int64)
    else:
        located = np.abs(values.astype(np.int64)) % num_bins
    expect = np.bincount(located, minlength=num_bins).astype(bin_dtype)
    bins, ov = O.histogram(values, np.zeros(num_bins, dtype=bin_dtype),
                           locator=O.LOCATOR_MODULO)
    assert np.array_equal(bins, expect) and ov == 0


@pytest.mark.parametrize("bin_dtype", HIST_BIN_DTYPES)
def test_histogram_reference_overflow_case(bin_dtype):
    # HistogramTests.tt:146-203: one bin preloaded with Max - 33, 32 samples:
    # no overflow the first time, overflow the second; the count wraps.
    info = np.iinfo(bin_dtype)
    values = np.arange(1, 33, dtype=np.int32)
    start = np.array([info.max - 32 - 1], dtype=bin_dtype)
    bins1, ov1 = O.histogram(values, start, locator=O.LOCATOR_MODULO)
    assert int(bins1[0]) == info.max - 1 and ov1 == 0
    bins2, ov2 = O.histogram(values, bins1, locator=O.LOCATOR_MODULO)
    wrapped = (info.max - 1 + 32) - (int(info.max) - int(info.min) + 1)
    assert int(bins2[0]) == wrapped and ov2 == 1


def test_histogram_accumulates_and_identity_locator():
    v = rng(9).integers(0, 4096, size=50000, dtype=np.int32)
    pre = rng(10).integers(0, 100, size=4096, dtype=np.int32)
    bins, ov = O.histogram(v, pre)
    assert np.array_equal(bins, pre + np.bincount(v, minlength=4096))
    assert ov == 0
    _, ov = O.histogram(v, pre, overflow=1)
    assert ov == 1  # the flag is OR-ed into, never cleared


# ----------------------------------------------------------------- temp sizes
def test_cpu_temp_size_formulas():
    # RadixSortExtensions.cs:419-447 with MaxNumThreads = 16, scan temp = 1.
    assert O.scan_temp_ints_cpu() == 1
    assert O.radix_sort_temp_ints_cpu(4, 1027) == 16 * 4 * 2 + 1027 + 1
    assert O.radix_sort_temp_ints_cpu(8, 33) == 128 + 66 + 1
    assert O.radix_sort_temp_ints_cpu(1, 5) == 128 + 2 + 1


@pytest.mark.parametrize("elem_bytes", [1, 2, 4, 8])
def test_temp_view_manager_alignment_rule(elem_bytes):
    # TempViewManagerTests.cs:51-84.
    rel = (elem_bytes + 3) // 4
    # AlignedAllocation: two allocations of T in a buffer of 2*rel ints succeed.
    n1 = O.temp_view_allocate(0, 2 * rel, elem_bytes, True, 1)
    assert n1 == rel
    assert O.temp_view_allocate(n1, 2 * rel, elem_bytes, True, 1) == 2 * rel
    # UnalignedAllocation: a byte first, then T: throws only for types wider
    # than an int.
    after_byte = O.temp_view_allocate(0, rel + 1, 1, True, 1)
    assert after_byte == 1
    got = O.temp_view_allocate(after_byte, rel + 1, elem_bytes, True, 1)
    assert got == (-2 if elem_bytes > 4 else 1 + rel)
    # Too small a temp view.
    assert O.temp_view_allocate(0, rel - 1 if rel > 1 else 0, elem_bytes, True, 1) == -1


# ------------------------------------------- unique, sequence, reorder (oracle)
def remove_consecutive_duplicates(a):
    # UniqueExtensionTests.tt:36-46, the reference test's own expectation.
    out = []
    for x in a.tolist():
        if not out or out[-1] != x:
            out.append(x)
    return np.array(out, dtype=a.dtype)


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("repeat", [1, 317, 1025])
def test_unique_reference_cases(dtype, repeat):
    # UniqueExtensionTests.tt:48-67: 1..length, each value repeated, cut at length.
    if np.dtype(dtype) == np.float16:
        pytest.skip("values above 2048 are not exact in Half")
    length = 1025
    vals = np.repeat(np.arange(1, length + 1), repeat)[:length]
    if np.dtype(dtype).kind in "iu":
        vals = vals.astype(np.int64).astype(dtype)     # wraps for 8-bit types, as (T)x
    else:
        vals = vals.astype(dtype)
    expect = remove_consecutive_duplicates(vals)
    for tile in (1, 16, 100, 4096):
        assert np.array_equal(O.unique(vals, tile=tile), expect)


@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.int32, np.uint64])
def test_unique_random_runs_any_tile(dtype):
    for seed in range(5):
        runs = rng(seed).integers(1, 9, size=300)
        vals = np.repeat(rng(seed + 1).integers(0, 4, size=300), runs).astype(dtype)
        keep = np.ones(vals.size, dtype=bool)
        keep[1:] = vals[1:] != vals[:-1]            # first element of every run
        for tile in (1, 7, 16, 1000):
            assert np.array_equal(O.unique(vals, tile=tile), vals[keep])


def test_unique_float_compare_to_semantics():
    # CompareTo: every NaN equals every NaN, -0.0 equals +0.0; the FIRST of a run stays.
    for dt in (np.float16, np.float32, np.float64):
        nan2 = np.array([np.nan], dtype=dt)
        nan2.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[nan2.itemsize])[0] |= 1
        v = np.concatenate([np.array([np.nan], dt), nan2, np.array([-0.0, 0.0, 1.0, 1.0, np.inf, -np.inf, -np.inf], dt)])
        out = O.unique(v, tile=3)
        assert out.size == 5
        assert np.isnan(out[0]) and np.signbit(out[1]) and out[1] == 0
        assert out[2] == 1 and out[3] == np.inf and out[4] == -np.inf


@pytest.mark.parametrize("dtype", ALL_KEY_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
def test_sequence_reference_cases(dtype, n):
    # SequencerTests.tt:56-96: expected[i] = (T)i.
    expect = np.arange(n, dtype=np.int64)
    expect = (expect.astype(np.uint64).astype(dtype) if np.dtype(dtype).kind == "u"
              else expect.astype(dtype))
    assert np.array_equal(O.sequence(n, dtype), expect)
    # Repeated / Batched (SequenceExtensions.cs:163-171): closed form
    got = O.sequence(n, dtype, sequence_length=5, batch_length=3)
    for i in (0, n // 2, n - 1):
        assert got[i] == np.dtype(dtype).type((i // 3) % 5)


def test_reorder_is_a_gather():
    src = rng(3).integers(0, 1000, 50).astype(np.int64)
    order = rng(4).permutation(50).astype(np.int32)
    out = O.reorder(src, order)
    for i in range(50):
        assert out[i] == src[order[i]]


# ------------------------------------------------------------------ transform
def _py_convert(values, sdt, tdt):
    """Integer conversion by Python big-int arithmetic: value mod 2^bits, read
    back in the target's signedness."""
    bits = np.dtype(tdt).itemsize * 8
    out = []
    for v in values:
        w = int(v) % (1 << bits)
        if np.dtype(tdt).kind == "i" and w >= 1 << (bits - 1):
            w -= 1 << bits
        out.append(w)
    return np.array(out, dtype=tdt)


@pytest.mark.parametrize("n", ARRAY_SIZES)
def test_transform_reference_cases(n):
    # TransformerExtensionTests.tt:66-86: 42, 42, ... -> -42.
    seq = compute_sequence(np.int32, 42, 0, n)
    assert np.array_equal(O.transform(seq, np.int32, O.TRANSFORM_NEGATE),
                          np.full(n, -42, dtype=np.int32))
    # :88-111: (long)x.
    got = O.transform(seq, np.int64)
    assert got.dtype == np.int64 and np.array_equal(got, np.full(n, 42, dtype=np.int64))
    # :113-134: (int)~x for x = 0, 1, 2, ... is -1 - x.
    useq = compute_sequence(np.uint32, 0, 1, n)
    assert np.array_equal(O.transform(useq, np.int32, O.TRANSFORM_BIT_COMPLEMENT),
                          (-1 - np.arange(n)).astype(np.int32))


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("n", ARRAY_SIZES)
def test_transform_cast_from_index_reference_case(dtype, n):
    # TransformerExtensionTests.tt:136-162 with Index1To<T>Transformer
    # (AlgorithmsTestData.tt:239-252): index i -> (T)i.
    idx = compute_sequence(np.int32, 0, 1, n)
    got = O.transform(idx, dtype)
    assert got.dtype == np.dtype(dtype)
    assert [float(x) for x in got] == [float(i) for i in range(n)]


@pytest.mark.parametrize("dtype", ATOMIC_NUMERIC_DTYPES)
@pytest.mark.parametrize("start,step", [(0, 0), (1, 0), (0, 1), (-1, 0), (0, -1)])
def test_reorder_transform_mul2_reverse_reference_case(dtype, start, step):
    # ReorderExtensionTests.tt:43-66, 160-200: reversed order, value * 2;
    # expectation built the reference's way, result[order[i]] = 2 * input[i].
    if np.dtype(dtype).kind == "u" and (start < 0 or step < 0):
        pytest.skip("the reference skips negative sequences for unsigned types")
    for n in ARRAY_SIZES:
        seq = compute_sequence(dtype, start, step, n)
        order = np.arange(n - 1, -1, -1, dtype=np.int32)
        expect = np.empty(n, dtype=dtype)
        with np.errstate(over="ignore"):
            for i in range(n):
                expect[order[i]] = seq[i] + seq[i]
        got = O.reorder_transform(seq, order, dtype, O.TRANSFORM_MULTIPLY, 2)
        assert np.array_equal(got.view(np.uint8), expect.view(np.uint8))


@pytest.mark.parametrize("sdt", INT_KEY_DTYPES)
@pytest.mark.parametrize("tdt", INT_KEY_DTYPES)
def test_transform_integer_semantics_by_big_int_arithmetic(sdt, tdt):
    info = np.iinfo(sdt)
    edge = np.array([0, 1, info.max, info.min, info.max - 1, info.min + 1 if info.min else 2],
                    dtype=sdt)
    vals = np.concatenate([edge, random_ints(sdt, 200, seed=5)])
    sbits = np.dtype(sdt).itemsize * 8

    def in_source(py_values):   # wrap to the source type first (op is closed in it)
        return _py_convert(py_values, sdt, sdt)

    assert np.array_equal(O.transform(vals, tdt), _py_convert(vals, sdt, tdt))
    neg = in_source([-int(v) for v in vals])
    assert np.array_equal(O.transform(vals, tdt, O.TRANSFORM_NEGATE), _py_convert(neg, sdt, tdt))
    comp = in_source([-1 - int(v) for v in vals])   # ~v = -1 - v
    assert np.array_equal(O.transform(vals, tdt, O.TRANSFORM_BIT_COMPLEMENT),
                          _py_convert(comp, sdt, tdt))
    for k in (2, -3, 1 << 40):
        mul = in_source([int(v) * k for v in vals])
        assert np.array_equal(O.transform(vals, tdt, O.TRANSFORM_MULTIPLY, k),
                              _py_convert(mul, sdt, tdt))
    assert sbits in (8, 16, 32, 64)


def test_transform_float_semantics():
    x = np.array([0.0, -0.0, 1.5, -2.25, 65519.0, 65520.0, 1e-8, np.inf, -np.inf, np.nan],
                 dtype=np.float64)
    h = O.transform(x, np.float16)
    assert h[4] == 65504 and h[5] == np.inf and h[6] == 0 and np.isnan(h[9])   # RNE, overflow, underflow
    assert np.signbit(O.transform(x, np.float32, O.TRANSFORM_NEGATE)[0])        # -(+0) = -0
    # one rounding, not two: just above a float16 midpoint goes up
    above = np.array([1 + 2.0 ** -11 + 2.0 ** -40], dtype=np.float64)
    assert float(O.transform(above, np.float16)[0]) == 1 + 2.0 ** -10
    assert np.array_equal(O.transform(x[2:4], np.float64, O.TRANSFORM_MULTIPLY, 2), [3.0, -4.5])
    # integer -> float rounds to nearest even: 2^24 + 1 -> 2^24, 2^24 + 3 -> 2^24 + 4
    i = np.array([(1 << 24) + 1, (1 << 24) + 3, -(1 << 24) - 1], dtype=np.int32)
    assert [float(v) for v in O.transform(i, np.float32)] == [16777216.0, 16777220.0, -16777216.0]
    u = np.array([(1 << 64) - 1, (1 << 53) + 1], dtype=np.uint64)
    assert [float(v) for v in O.transform(u, np.float64)] == [float(1 << 64), float(1 << 53)]
    with pytest.raises(ValueError):
        O.transform(x, np.int32)
    with pytest.raises(ValueError):
        O.transform(x, np.float64, O.TRANSFORM_BIT_COMPLEMENT)


def test_histogram_float_bins_add_one_per_element_and_saturate():
    # HistogramLaunchers.tt over AtomicNumericTypes (float, double): Atomic.Add(ref
    # bin, 1) per element in the bin's precision; worked by hand: 16777214 -> 15, 16
    # and then 16777216 + 1 rounds back to 16777216 (tie to the even mantissa).
    zeros = np.zeros(5, dtype=np.int32)
    b, ov = O.histogram(zeros, np.array([16777214.0, 0.5], dtype=np.float32))
    assert b.tolist() == [16777216.0, 0.5] and ov == 0
    b, ov = O.histogram(zeros, np.array([16777214.0, 0.5], dtype=np.float64))
    assert b.tolist() == [16777219.0, 0.5] and ov == 0
    b, ov = O.histogram(np.array([1, 1, 1, 0], dtype=np.uint8), np.array([-2.5, 0.5], dtype=np.float32))
    assert b.tolist() == [-1.5, 3.5] and ov == 0
    # -(2^24 + 2) has an odd mantissa: + 1 is a tie that rounds to -2^24, then steps are exact
    b, _ = O.histogram(np.zeros(3, dtype=np.int32), np.array([-16777218.0], dtype=np.float32))
    assert b.tolist() == [-16777214.0]
    # -(2^24 + 4) has an even one: stuck
    b, _ = O.histogram(np.zeros(3, dtype=np.int32), np.array([-16777220.0], dtype=np.float32))
    assert b.tolist() == [-16777220.0]
    fmax = np.finfo(np.float32).max
    b, ov = O.histogram(np.zeros(2, dtype=np.int32), np.array([fmax], dtype=np.float32))
    assert b[0] == fmax and ov == 1
    b, ov = O.histogram(np.zeros(2, dtype=np.int32), np.array([np.inf], dtype=np.float32))
    assert b[0] == np.inf and ov == 0
