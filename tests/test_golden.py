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
    assert OPS == ["histogram", "reduce", "scan", "sort", "sort_pairs", "transform"]
    assert len(CASES) > 300


# ------------------------------------------------------------------ CPU oracle
def test_oracle_sort_against_golden():
    for c in by_op("sort"):
        got = O.radix_sort(arr(c["input"], c["dtype"]), descending=c["descending"])
        assert np.array_equal(got, arr(c["expected"], c["dtype"])), c["dtype"]
    for c in by_op("sort_pairs"):
        k, v = O.radix_sort_pairs(arr(c["input"], c["dtype"]), arr(c["values"], c["dtype"]))
        assert np.array_equal(k, arr(c["expected"], c["dtype"]))
        assert np.array_equal(v, arr(c["expected_values"], c["dtype"]))


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
