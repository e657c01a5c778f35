"""Writes tests/golden/known_answers.json: inputs and expected outputs of the
known-answer cases that the reference's own tests and sample programs define.

The reference (ILGPU.Algorithms) ships no golden files: every expectation is
computed inside its tests from a closed form.  This script restates those
closed forms with Python integers (no numpy arithmetic, no oracle, no HIP
library), so the vectors are independent of everything they are used to check:

  sort      RadixSortExtensionTests.tt:37-131: inverted sequence -> sequence;
            Samples/AlgorithmsRadixSort/Program.cs:59-63: 32 reversed ints
  pairs     RadixSortExtensionTests.tt:346-364: values == keys
  scan      ScanExtensionTests.tt:43-104, 286-305: x_i = start + i*step;
            Samples/AlgorithmsScan/Program.cs:32-33: 32 twos
  reduce    ReductionExtensionTests.tt:41-106; Samples/AlgorithmsReduce/Program.cs:29-31
  histogram HistogramTests.tt:42-103 (1..1024 into 64 / 256 bins by v % bins)
            and the overflow case :149-189
  transform TransformerExtensionTests.tt:66-134
  float key order  RadixSortOperations.tt:77-93, 122-123 evaluated literally,
            with C#'s integer promotions, on raw bit patterns of Half, float and
            double keys (signed zeros, subnormals, infinities, NaNs, neighbours
            in the last mantissa bit, negative values): no reference test sorts
            such keys, so the expectation is the formula itself worked out with
            Python integers, and a stable sort on the resulting key

Run from the repository root:  python tests/golden/make_known_answers.py
"""
import json
import os

SIZES = [1, 31, 33, 127, 1027]
INT_TYPES = {"int32": (32, True), "int64": (64, True), "uint32": (32, False), "uint64": (64, False)}


def wrap(v, bits, signed):
    v %= 1 << bits
    if signed and v >= 1 << (bits - 1):
        v -= 1 << bits
    return v


def sequence(start, step, n, bits, signed):
    return [wrap(start + i * step, bits, signed) for i in range(n)]


def csharp_float_sort_key(raw, bits):
    """ExtractRadixBits of Ascending{Half,Float,Double} over all NumBits,
    RadixSortOperations.tt:81-89, on the raw bit pattern `raw` of the key.

    Half: Interop.FloatAsInt(Half) is a ushort (Interop.cs:171); `~` promotes it
    to a 32-bit int, the (uint) cast binds before `>>`, so the shift is a
    logical one of 0xFFFFxxxx by 15: bits 1..16 of the mask are always set and
    bit 0 is the inverted sign.  float/double: `~` stays unsigned, the shift by
    NumBits-1 leaves only the inverted sign in bit 0.  The sort's passes read
    bits 0..NumBits-1 of `bits` two at a time (RadixSortExtensions.cs:1276-1334),
    so the key is `bits` modulo 2^NumBits.
    """
    if bits == 16:
        promoted = (-raw - 1) % (1 << 32)           # (uint)~(int)ushort
        ones = promoted >> 15
    else:
        ones = ((-raw - 1) % (1 << bits)) >> (bits - 1)
    sign_mask = 1 << (bits - 1)
    return (raw ^ (sign_mask | ones)) % (1 << bits)


def stable_order(keys):
    # insertion into buckets by key, ties in input order
    return [i for _, i in sorted((k, i) for i, k in enumerate(keys))]


FLOAT_PATTERNS = {
    # +0 -0 1 -1 2 -2 .5 -.5, smallest subnormals, infinities, NaNs (quiet,
    # negative quiet, signalling), largest finite values, neighbours of +-1 in
    # the last mantissa bit, and duplicates of 1, -1 and -0 (stability)
    "float16": (16, [0x3C00, 0x4000, 0xBC00, 0xC000, 0x3800, 0xB800, 0x0000, 0x8000, 0x0001,
                     0x8001, 0x7C00, 0xFC00, 0x7E00, 0xFE00, 0x7C01, 0x7BFF, 0xFBFF, 0x3C01,
                     0xBC01, 0x3C00, 0xBC00, 0x8000, 0x3BFF, 0xBBFF]),
    "float32": (32, [0x3F800000, 0x40000000, 0xBF800000, 0xC0000000, 0x3F000000, 0xBF000000,
                     0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x7F800000, 0xFF800000,
                     0x7FC00000, 0xFFC00000, 0x7F800001, 0x7F7FFFFF, 0xFF7FFFFF, 0x3F800001,
                     0xBF800001, 0x3F800000, 0xBF800000, 0x80000000, 0x3F7FFFFF, 0xBF7FFFFF,
                     0xC2F6E979, 0xC2F6E97A, 0xC47A0000, 0xC47A0000]),
    "float64": (64, [0x3FF0000000000000, 0x4000000000000000, 0xBFF0000000000000,
                     0xC000000000000000, 0x3FE0000000000000, 0xBFE0000000000000,
                     0x0000000000000000, 0x8000000000000000, 0x0000000000000001,
                     0x8000000000000001, 0x7FF0000000000000, 0xFFF0000000000000,
                     0x7FF8000000000000, 0xFFF8000000000000, 0x7FF0000000000001,
                     0x7FEFFFFFFFFFFFFF, 0xFFEFFFFFFFFFFFFF, 0x3FF0000000000001,
                     0xBFF0000000000001, 0x3FF0000000000000, 0xBFF0000000000000,
                     0x8000000000000000, 0x3FEFFFFFFFFFFFFF, 0xBFEFFFFFFFFFFFFF,
                     0xC05EDD2F1A9FBE77, 0xC05EDD2F1A9FBE76, 0xC08F400000000000,
                     0xC08F400000000000]),
}


def float_key_cases():
    cases = []
    for name, (bits, raw) in FLOAT_PATTERNS.items():
        mask = (1 << bits) - 1
        asc_keys = [csharp_float_sort_key(r, bits) for r in raw]
        for descending in (False, True):
            # Descending*: every extracted digit is complemented (:122-123),
            # i.e. the whole key is.
            keys = [(~k) & mask for k in asc_keys] if descending else asc_keys
            order = stable_order(keys)
            cases.append({"op": "sort_float_bits", "dtype": name, "descending": descending,
                          "input_bits": raw, "expected_bits": [raw[i] for i in order]})
            cases.append({"op": "sort_pairs_float_bits", "dtype": name,
                          "descending": descending, "input_bits": raw,
                          "expected_bits": [raw[i] for i in order],
                          "expected_index_values": order})
    return cases


def main():
    cases = float_key_cases()
    for name, (bits, signed) in INT_TYPES.items():
        for n in SIZES:
            asc = sequence(0, 1, n, bits, signed)
            cases.append({"op": "sort", "dtype": name, "descending": False,
                          "input": asc[::-1], "expected": asc})
            if n > 127:   # the long cases once per type; the file stays small
                x = sequence(0, 1, n, bits, signed)
                cases.append({"op": "scan", "dtype": name, "kind": "inclusive", "scan_op": "add",
                              "input": x,
                              "expected": [wrap((i + 1) * i // 2, bits, signed) for i in range(n)]})
                continue
            cases.append({"op": "sort", "dtype": name, "descending": True,
                          "input": asc, "expected": asc[::-1]})
            cases.append({"op": "sort_pairs", "dtype": name, "input": asc[::-1],
                          "values": asc[::-1], "expected": asc, "expected_values": asc})
            for start, step in ((0, 1), (1, 0)) + (((-1, 0), (0, -1)) if signed else ()):
                x = sequence(start, step, n, bits, signed)
                inc, acc = [], 0
                for v in x:
                    acc = wrap(acc + v, bits, signed)
                    inc.append(acc)
                cases.append({"op": "scan", "dtype": name, "kind": "inclusive", "scan_op": "add",
                              "input": x, "expected": inc})
                cases.append({"op": "scan", "dtype": name, "kind": "exclusive", "scan_op": "add",
                              "input": x, "expected": [0] + inc[:-1]})
                run_max = [max(x[: i + 1]) for i in range(n)]
                cases.append({"op": "scan", "dtype": name, "kind": "inclusive", "scan_op": "max",
                              "input": x, "expected": run_max})
                cases.append({"op": "reduce", "dtype": name, "reduce_op": "add", "input": x,
                              "expected": inc[-1]})
                cases.append({"op": "reduce", "dtype": name, "reduce_op": "max", "input": x,
                              "expected": max(x)})
                cases.append({"op": "reduce", "dtype": name, "reduce_op": "min", "input": x,
                              "expected": min(x)})
    # sample programs
    rev = list(range(31, -1, -1))
    cases.append({"op": "sort", "dtype": "int32", "descending": False, "input": rev,
                  "expected": sorted(rev)})
    cases.append({"op": "scan", "dtype": "int32", "kind": "inclusive", "scan_op": "add",
                  "input": [2] * 32, "expected": [2 * (i + 1) for i in range(32)]})
    cases.append({"op": "scan", "dtype": "int32", "kind": "exclusive", "scan_op": "add",
                  "input": [2] * 32, "expected": [2 * i for i in range(32)]})
    cases.append({"op": "reduce", "dtype": "int32", "reduce_op": "add", "input": list(range(64)),
                  "expected": 2016})
    # histogram: 1..1024 by v % bins; overflow: bins[0] = max - 33, then 32 samples twice
    for bins in (64, 256):
        cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "int32", "locator": "modulo",
                      "input": list(range(1, 1025)), "bins_before": [0] * bins,
                      "expected": [1024 // bins] * bins, "expected_overflow": 0})
    imax = (1 << 31) - 1
    cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "int32", "locator": "modulo",
                  "input": [0] * 32, "bins_before": [imax - 33, 0], "expected": [imax - 1, 0],
                  "expected_overflow": 0})
    cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "int32", "locator": "modulo",
                  "input": [0] * 32, "bins_before": [imax - 1, 0],
                  "expected": [wrap(imax - 1 + 32, 32, True), 0], "expected_overflow": 1})
    # Floating-point bins (HistogramLaunchers.tt over AtomicNumericTypes): 1.0 is added
    # per element in the bin's precision.  Worked by hand: integers below 2^24 (float) are
    # exact, so 1..1024 by v % 64 adds 16 to every bin whatever it held; 16777214 + 5
    # steps is 16777215, 16777216 and then 16777216 + 1 = 16777217, which lies halfway
    # between 16777216 and 16777218 and rounds to the even mantissa, 16777216: stuck;
    # -2.5 + 4 steps is 1.5; 0.5 + 3 steps is 3.5; a bin at float.MaxValue stays there and
    # reports overflow; double bins hold 2^24 + 5 exactly.
    for bin_dtype in ("float32", "float64"):
        cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": bin_dtype,
                      "locator": "modulo", "input": list(range(1, 1025)),
                      "bins_before": [float(i) / 2 for i in range(64)],
                      "expected": [float(i) / 2 + 16 for i in range(64)], "expected_overflow": 0})
    cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "float32", "locator": "modulo",
                  "input": [0] * 5 + [1] * 4 + [2] * 3, "bins_before": [16777214.0, -2.5, 0.5, 7.0],
                  "expected": [16777216.0, 1.5, 3.5, 7.0], "expected_overflow": 0})
    cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "float64", "locator": "modulo",
                  "input": [0] * 7, "bins_before": [16777214.0, 0.25],
                  "expected": [16777221.0, 0.25], "expected_overflow": 0})
    fmax = (2 - 2 ** -23) * 2.0 ** 127  # float.MaxValue, exact in a Python float
    cases.append({"op": "histogram", "dtype": "int32", "bin_dtype": "float32", "locator": "modulo",
                  "input": [0, 1], "bins_before": [fmax, 0.0], "expected": [fmax, 1.0],
                  "expected_overflow": 1})
    # transform
    for n in SIZES:
        cases.append({"op": "transform", "dtype": "int32", "target_dtype": "int32",
                      "transformer": "negate", "input": [42] * n, "expected": [-42] * n})
        cases.append({"op": "transform", "dtype": "int32", "target_dtype": "int64",
                      "transformer": "convert", "input": [42] * n, "expected": [42] * n})
        cases.append({"op": "transform", "dtype": "uint32", "target_dtype": "int32",
                      "transformer": "bit_complement", "input": list(range(n)),
                      "expected": [-1 - i for i in range(n)]})
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(out, "w") as f:
        json.dump({"cases": cases}, f, separators=(",", ":"))
    print(out, len(cases), "cases", os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
