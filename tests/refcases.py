"""The reference's own test data, restated as generators.

Sizes, sequences and expectations follow ILGPU.Algorithms.Tests:
  * ArraySizes = {1, 31, 33, 127, 1027}          (Generic/ConfigurationBase.tt:80)
  * ComputeSequence / ComputeInvertedSequence    (Generic/AlgorithmsTestData.tt:74-96)
  * element types int, long, uint, ulong, float, double
                                                 (TypeInformation.ttinclude:125-138)
"""
import numpy as np

ARRAY_SIZES = [1, 31, 33, 127, 1027]
ATOMIC_NUMERIC_DTYPES = [np.int32, np.int64, np.uint32, np.uint64,
                         np.float32, np.float64]
ALL_KEY_DTYPES = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16,
                  np.uint32, np.uint64, np.float16, np.float32, np.float64]


def compute_sequence(dtype, start, step, length):
    """sequence[0] = start; sequence[i] = sequence[i-1] + step (wrapping)."""
    dtype = np.dtype(dtype)
    with np.errstate(over="ignore"):
        i = np.arange(length)
        if dtype.kind in "iu":
            seq = (np.int64(start) + np.int64(step) * i.astype(np.int64))
            return seq.astype(dtype)
        return (dtype.type(start) + dtype.type(step) * i.astype(dtype)).astype(dtype)


def compute_inverted_sequence(dtype, start, step, length):
    """sequence[length-1] = start; sequence[i] = sequence[i+1] + step."""
    return compute_sequence(dtype, start, step, length)[::-1].copy()
