"""Known-answer vectors (tests/golden/known_answers.json, written by
tests/golden/make_known_answers.py from the closed forms of the reference's own
tests and samples) against the CPU oracle (no GPU) and against the HIP library
through its C ABI (gpu)."""
import json
import os

import numpy as np
import pytest

from oracle import cpu_oracle as O

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")
with open(_PATH) as _f:
    CASES = json.load(_f)["cases"]
OPS = sorted({c["op"] for c in CASES})


def arr(values, dtype):
    return np.array(values, dtype=np.dtype(dtype))


def by_op(op):
    return [c for c in CASES if c["op"] == op]


def test_golden_file_covers_every_primitive():
    assert OPS == ["histogram", "reduce", "scan", "sort", "sort_float_bits", "sort_pairs",
                   "sort_pairs_float_bits", "transform"]
    assert len(CASES) > 300
    # Half, float and double keys, both orders, keys-only and pairs
    assert len(by_op("sort_float_bits")) == 6 and len(by_op("sort_pairs_float_bits")) == 6


_UINT_OF = {"float16": np.uint16, "float32": np.uint32, "float64": np.uint64}


def float_keys(bits, dtype):
    """Raw bit patterns of a golden case as an array of the float type."""
    return np.array(bits, dtype=_UINT_OF[dtype]).view(np.dtype(dtype))


def same_bits(got, bits, dtype):
    return np.array_equal(np.ascontiguousarray(got).view(_UINT_OF[dtype]),
                          np.array(bits, dtype=_UINT_OF[dtype]))


# ------------------------------------------------------------------ CPU oracle
def test_oracle_sort_against_golden():
    for c in by_op("sort"):
        got = O.radix_sort(arr(c["input"], c["dtype"]), descending=c["descending"])
        assert np.array_equal(got, arr(c["expected"], c["dtype"])), c["dtype"]
    for c in by_op("sort_pairs"):
        k, v = O.radix_sort_pairs(arr(c["input"], c["dtype"]), arr(c["values"], c["dtype"]))
        assert np.array_equal(k, arr(c["expected"], c["dtype"]))
        assert np.array_equal(v, arr(c["expected_values"], c["dtype"]))


def test_oracle_float_key_order_against_golden():
    # The Half, float and double branches of the oracle's ascending_bits
    # against the hand evaluation of RadixSortOperations.tt:81-89, 122-123
    # (tests/golden/make_known_answers.py: Python integers only).
    for c in by_op("sort_float_bits"):
        got = O.radix_sort(float_keys(c["input_bits"], c["dtype"]), descending=c["descending"])
        assert same_bits(got, c["expected_bits"], c["dtype"]), (c["dtype"], c["descending"])
    for c in by_op("sort_pairs_float_bits"):
        keys = float_keys(c["input_bits"], c["dtype"])
        k, v = O.radix_sort_pairs(keys, np.arange(keys.size, dtype=np.uint32),
                                  descending=c["descending"])
        assert same_bits(k, c["expected_bits"], c["dtype"]), (c["dtype"], c["descending"])
        assert v.tolist() == c["expected_index_values"], (c["dtype"], c["descending"])


def test_half_key_example_worked_by_hand():
    # Half keys: raw ^ (0xFFFE | !sign).  Positive values have every bit
    # flipped (they follow the negative ones, in DEscending order), negative
    # ones all but bit 0.
    case = [c for c in by_op("sort_float_bits")
            if c["dtype"] == "float16" and not c["descending"]][0]
    assert 0x3C00 ^ 0xFFFF == 0xC3FF and 0xBC00 ^ 0xFFFE == 0x43FE
    data = np.array([1, 2, -1, -2, .5, -.5], dtype=np.float16)
    got = O.radix_sort(data)
    assert got.tolist() == [-2, -1, -.5, 2, 1, .5]
    # the golden case holds the same six values in that relative order
    six = [b for b in case["expected_bits"] if b in (0x3C00, 0x4000, 0xBC00, 0xC000, 0x3800,
                                                       0xB800)]
    assert [x for i, x in enumerate(six) if x not in six[:i]] == [0xC000, 0xBC00, 0xB800,
                                                                    0x4000, 0x3C00, 0x3800]


_SCAN_OPS = {"add": O.OP_ADD, "max": O.OP_MAX, "min": O.OP_MIN}


def test_oracle_scan_and_reduce_against_golden():
    for c in by_op("scan"):
        got = O.scan(arr(c["input"], c["dtype"]), _SCAN_OPS[c["scan_op"]],
                     inclusive=c["kind"] == "inclusive")
        assert np.array_equal(got, arr(c["expected"], c["dtype"])), (c["dtype"], c["kind"])
    for c in by_op("reduce"):
        got = O.reduce(arr(c["input"], c["dtype"]), _SCAN_OPS[c["reduce_op"]])
        assert got == arr([c["expected"]], c["dtype"])[0], (c["dtype"], c["reduce_op"])


def test_oracle_histogram_and_transform_against_golden():
    for c in by_op("histogram"):
        bins, overflow = O.histogram(arr(c["input"], c["dtype"]),
                                     arr(c["bins_before"], c["bin_dtype"]), O.LOCATOR_MODULO)
        assert np.array_equal(bins, arr(c["expected"], c["bin_dtype"]))
        assert int(overflow != 0) == c["expected_overflow"]
    kinds = {"convert": O.TRANSFORM_CONVERT, "negate": O.TRANSFORM_NEGATE,
             "bit_complement": O.TRANSFORM_BIT_COMPLEMENT}
    for c in by_op("transform"):
        got = O.transform(arr(c["input"], c["dtype"]), c["target_dtype"], kinds[c["transformer"]])
        assert np.array_equal(got, arr(c["expected"], c["target_dtype"]))


# ------------------------------------------------------------------ HIP library
@pytest.mark.gpu
def test_library_against_golden():
    import torch
    from ilgpu_amd import capi
    D = capi.DeviceArray
    for c in by_op("sort"):
        d = D.from_numpy(arr(c["input"], c["dtype"]))
        capi.radix_sort_keys(d, descending=c["descending"])
        torch.cuda.synchronize()
        assert np.array_equal(d.numpy(), arr(c["expected"], c["dtype"])), ("sort", c["dtype"])
    for c in by_op("sort_pairs"):
        k, v = D.from_numpy(arr(c["input"], c["dtype"])), D.from_numpy(arr(c["values"], c["dtype"]))
        capi.radix_sort_pairs(k, v)
        torch.cuda.synchronize()
        assert np.array_equal(k.numpy(), arr(c["expected"], c["dtype"]))
        assert np.array_equal(v.numpy(), arr(c["expected_values"], c["dtype"]))
    for c in by_op("sort_float_bits"):
        d = D.from_numpy(float_keys(c["input_bits"], c["dtype"]))
        capi.radix_sort_keys(d, descending=c["descending"])
        torch.cuda.synchronize()
        assert same_bits(d.numpy(), c["expected_bits"], c["dtype"]), \
            ("sort", c["dtype"], c["descending"])
    for c in by_op("sort_pairs_float_bits"):
        keys = float_keys(c["input_bits"], c["dtype"])
        k = D.from_numpy(keys)
        v = D.zeros(keys.size, np.uint32)
        capi.radix_sort_pairs(k, v, descending=c["descending"], values_from_index=True)
        torch.cuda.synchronize()
        assert same_bits(k.numpy(), c["expected_bits"], c["dtype"]), ("pairs", c["dtype"])
        assert v.numpy().tolist() == c["expected_index_values"], ("pairs", c["dtype"])
        # the same values handed in as a view
        k = D.from_numpy(keys)
        v = D.from_numpy(np.arange(keys.size, dtype=np.uint64))
        capi.radix_sort_pairs(k, v, descending=c["descending"])
        torch.cuda.synchronize()
        assert same_bits(k.numpy(), c["expected_bits"], c["dtype"])
        assert v.numpy().tolist() == c["expected_index_values"]
    ops = {"add": capi.OP_ADD, "max": capi.OP_MAX, "min": capi.OP_MIN}
    for c in by_op("scan"):
        x = arr(c["input"], c["dtype"])
        out = D.zeros(x.size, c["dtype"])
        capi.scan(D.from_numpy(x), out, op=ops[c["scan_op"]],
                  kind=capi.SCAN_INCLUSIVE if c["kind"] == "inclusive" else capi.SCAN_EXCLUSIVE)
        torch.cuda.synchronize()
        assert np.array_equal(out.numpy(), arr(c["expected"], c["dtype"])), ("scan", c["dtype"])
    for c in by_op("reduce"):
        out = D.zeros(1, c["dtype"])
        capi.reduce(D.from_numpy(arr(c["input"], c["dtype"])), out, op=ops[c["reduce_op"]])
        torch.cuda.synchronize()
        assert out.numpy()[0] == arr([c["expected"]], c["dtype"])[0], ("reduce", c["dtype"])
    for c in by_op("histogram"):
        bins = D.from_numpy(arr(c["bins_before"], c["bin_dtype"]))
        overflow = D.zeros(1, np.int32)
        capi.histogram(D.from_numpy(arr(c["input"], c["dtype"])), bins, overflow,
                       locator=capi.LOCATOR_MODULO)
        torch.cuda.synchronize()
        assert np.array_equal(bins.numpy(), arr(c["expected"], c["bin_dtype"]))
        assert int(overflow.numpy()[0] != 0) == c["expected_overflow"]
    kinds = {"convert": capi.TRANSFORM_CONVERT, "negate": capi.TRANSFORM_NEGATE,
             "bit_complement": capi.TRANSFORM_BIT_COMPLEMENT}
    for c in by_op("transform"):
        x = arr(c["input"], c["dtype"])
        out = D.zeros(x.size, c["target_dtype"])
        capi.transform(D.from_numpy(x), out, kinds[c["transformer"]])
        torch.cuda.synchronize()
        assert np.array_equal(out.numpy(), arr(c["expected"], c["target_dtype"]))
