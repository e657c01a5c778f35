"""TEST INFRASTRUCTURE ONLY: numpy/ctypes front end of the C oracle.

Loads ``oracle/_build/libilgpu_cpu_oracle.so`` (built by ``oracle/Makefile``)
and exposes the CPU restatement of ILGPU's CPUAccelerator algorithms on numpy
arrays.  Only tests, the smoke check and the benchmark's CPU-baseline leg may
import this module; the HIP library never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libilgpu_cpu_oracle.so")

# Element type codes (TypeInformation.ttinclude:94-121 order used by the C side).
I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 = range(11)
OP_ADD, OP_MAX, OP_MIN = 0, 1, 2
LOCATOR_IDENTITY, LOCATOR_MODULO = 0, 1

CPU_WARP_SIZE = 4
CPU_GROUP_SIZE = 16
CPU_MAX_NUM_THREADS = 16

_NP_TO_TYPE = {
    np.dtype(np.int8): I8, np.dtype(np.int16): I16, np.dtype(np.int32): I32,
    np.dtype(np.int64): I64, np.dtype(np.uint8): U8, np.dtype(np.uint16): U16,
    np.dtype(np.uint32): U32, np.dtype(np.uint64): U64,
    np.dtype(np.float16): F16, np.dtype(np.float32): F32,
    np.dtype(np.float64): F64,
}


def type_code(dtype) -> int:
    return _NP_TO_TYPE[np.dtype(dtype)]


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (idempotent unless ``force``)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.oracle_elem_size.argtypes = [i32]
        L.oracle_extract_radix_bits.argtypes = [i32, i32, vp, i32, i32]
        L.oracle_radix_sort.argtypes = [i32, i32, vp, i64, i32]
        L.oracle_radix_sort_pairs.argtypes = [i32, i32, vp, vp, i32, i64, i32]
        L.oracle_scan.argtypes = [i32, i32, i32, vp, vp, i64, i32]
        L.oracle_reduce.argtypes = [i32, i32, vp, i64, vp, i32, i32]
        L.oracle_sum_f64.argtypes = [i32, vp, i64]
        L.oracle_sum_f64.restype = ctypes.c_double
        L.oracle_histogram.argtypes = [i32, i32, i32, vp, i64, vp, i64, vp]
        L.oracle_scan_temp_ints_cpu.restype = i64
        L.oracle_unique.argtypes = [i32, vp, i64, i64]
        L.oracle_unique.restype = i64
        L.oracle_radix_sort_temp_ints_cpu.argtypes = [i32, i64, i32]
        L.oracle_radix_sort_temp_ints_cpu.restype = i64
        L.oracle_temp_view_allocate.argtypes = [i64, i64, i32, i32, i64]
        L.oracle_temp_view_allocate.restype = i64
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def extract_radix_bits(value: np.ndarray, descending: bool, shift: int,
                       mask: int) -> int:
    """Digit of one element (``value`` is a 0-d or 1-element array)."""
    v = np.ascontiguousarray(value).reshape(-1)[:1].copy()
    return lib().oracle_extract_radix_bits(type_code(v.dtype), int(descending),
                                           _ptr(v), shift, mask)


def radix_sort(keys: np.ndarray, descending: bool = False,
               num_groups: int = CPU_MAX_NUM_THREADS) -> np.ndarray:
    out = np.ascontiguousarray(keys).copy()
    if out.size == 0:
        return out
    rc = lib().oracle_radix_sort(type_code(out.dtype), int(descending),
                                 _ptr(out), out.size, num_groups)
    if rc != 0:
        raise RuntimeError(f"oracle_radix_sort failed: {rc}")
    return out


def radix_sort_pairs(keys: np.ndarray, values: np.ndarray,
                     descending: bool = False,
                     num_groups: int = CPU_MAX_NUM_THREADS):
    k = np.ascontiguousarray(keys).copy()
    v = np.ascontiguousarray(values).copy()
    assert k.shape == v.shape and k.ndim == 1
    if k.size == 0:
        return k, v
    rc = lib().oracle_radix_sort_pairs(type_code(k.dtype), int(descending),
                                       _ptr(k), _ptr(v), v.dtype.itemsize,
                                       k.size, num_groups)
    if rc != 0:
        raise RuntimeError(f"oracle_radix_sort_pairs failed: {rc}")
    return k, v


def scan(values: np.ndarray, op: int = OP_ADD, inclusive: bool = True,
         group_size: int = CPU_GROUP_SIZE) -> np.ndarray:
    a = np.ascontiguousarray(values)
    out = np.empty_like(a)
    if a.size == 0:
        return out
    rc = lib().oracle_scan(type_code(a.dtype), op, int(inclusive), _ptr(a),
                           _ptr(out), a.size, group_size)
    if rc != 0:
        raise RuntimeError(f"oracle_scan failed: {rc}")
    return out


def reduce(values: np.ndarray, op: int = OP_ADD,
           group_size: int = CPU_GROUP_SIZE,
           warp_size: int = CPU_WARP_SIZE):
    a = np.ascontiguousarray(values)
    out = np.empty(1, dtype=a.dtype)
    rc = lib().oracle_reduce(type_code(a.dtype), op, _ptr(a), a.size,
                             _ptr(out), group_size, warp_size)
    if rc != 0:
        raise RuntimeError(f"oracle_reduce failed: {rc}")
    return out[0]


def sum_f64(values: np.ndarray) -> float:
    a = np.ascontiguousarray(values)
    return float(lib().oracle_sum_f64(type_code(a.dtype), _ptr(a), a.size))


def histogram(values: np.ndarray, bins: np.ndarray,
              locator: int = LOCATOR_IDENTITY, overflow: int = 0):
    """Returns (bins_after, overflow_after); ``bins`` is accumulated into a copy."""
    a = np.ascontiguousarray(values)
    b = np.ascontiguousarray(bins).copy()
    ov = np.array([overflow], dtype=np.int32)
    rc = lib().oracle_histogram(type_code(a.dtype), type_code(b.dtype),
                                locator, _ptr(a), a.size, _ptr(b), b.size,
                                _ptr(ov))
    if rc != 0:
        raise RuntimeError(f"oracle_histogram failed: {rc}")
    return b, int(ov[0])


def unique(values: np.ndarray, tile: int = CPU_GROUP_SIZE) -> np.ndarray:
    """UniqueExtensions.cs:59-118: the kept prefix after removing consecutive
    duplicates under Comparison<T> (CompareTo)."""
    a = np.ascontiguousarray(values).copy()
    if a.size == 0:
        return a
    kept = lib().oracle_unique(type_code(a.dtype), _ptr(a), a.size, tile)
    if kept < 0:
        raise RuntimeError("oracle_unique failed")
    return a[:kept]


def sequence(n: int, dtype, sequence_length=None, batch_length: int = 1) -> np.ndarray:
    """SequenceExtensions.cs:163-171 with the identity sequencers
    (Sequencers.tt:25-37): view[i] = (T)((i / batchLength) % sequenceLength);
    Sequence itself passes sequenceLength = view.Length, batchLength = 1
    (SequenceExtensions.cs:262-268).  The cast is C#'s unchecked conversion
    from long: wrap-around for integers, nearest value for floating point."""
    if sequence_length is None:
        sequence_length = n
    idx = (np.arange(n, dtype=np.int64) // batch_length) % sequence_length
    dt = np.dtype(dtype)
    if dt.kind in "iu":
        return idx.astype(np.uint64).astype(dt) if dt.kind == "u" else idx.astype(dt)
    with np.errstate(over="ignore"):   # Half: indices above 65504 become +inf
        return idx.astype(dt)


def initialize(n: int, value) -> np.ndarray:
    """InitializeExtensions.cs:63-69: view[i] = value."""
    v = np.asarray(value)
    return np.full(n, v, dtype=v.dtype)


def reorder(source: np.ndarray, order: np.ndarray) -> np.ndarray:
    """ReorderExtensions.cs:116-120 with IdentityTransformer:
    target[i] = source[reorderView[i]]."""
    return np.ascontiguousarray(source)[np.asarray(order, dtype=np.int64)]


TRANSFORM_CONVERT, TRANSFORM_NEGATE, TRANSFORM_BIT_COMPLEMENT, TRANSFORM_MULTIPLY = 0, 1, 2, 3


def transform(source: np.ndarray, target_dtype, transformer: int = TRANSFORM_CONVERT,
              factor: int = 0) -> np.ndarray:
    """TransformImplementation.Execute (TransformExtensions.cs:153-159) for the
    closed transformer set (TTarget)op((TSource)value): op in the source type
    (unchecked C#: integers wrap), then the explicit numeric conversion
    (integers truncate or extend by the source's sign; floating-point targets
    round to nearest even).  Covers IdentityTransformer (:42-55) and the test
    transformers of Generic/AlgorithmsTestData.tt:170-252."""
    src = np.ascontiguousarray(source)
    sdt, tdt = src.dtype, np.dtype(target_dtype)
    if sdt.kind == "f" and tdt.kind != "f":
        raise ValueError("floating point -> integer is unspecified in C#")
    with np.errstate(over="ignore"):
        if transformer == TRANSFORM_CONVERT:
            v = src
        elif transformer == TRANSFORM_NEGATE:
            v = -src if sdt.kind == "f" else (0 - src.astype(sdt)).astype(sdt)
        elif transformer == TRANSFORM_BIT_COMPLEMENT:
            if sdt.kind == "f":
                raise ValueError("~ of a floating-point value")
            v = ~src
        elif transformer == TRANSFORM_MULTIPLY:
            if sdt.kind == "f":
                v = src * sdt.type(factor)
            else:
                bits = sdt.itemsize * 8
                k = np.uint64(factor & ((1 << 64) - 1))
                wide = src.astype(np.int64).view(np.uint64) * k
                v = (wide & np.uint64((1 << bits) - 1)).astype(
                    np.dtype("u%d" % sdt.itemsize)).view(sdt)
        else:
            raise ValueError(transformer)
        v = np.asarray(v, dtype=sdt)
        if sdt.kind != "f" and tdt.kind != "f":
            wide = v.astype(np.int64 if sdt.kind == "i" else np.uint64).view(np.uint64)
            tbits = tdt.itemsize * 8
            mask = np.uint64((1 << tbits) - 1)
            return (wide & mask).astype(np.dtype("u%d" % tdt.itemsize)).view(tdt)
        return v.astype(tdt)


def reorder_transform(source: np.ndarray, order: np.ndarray, target_dtype,
                      transformer: int = TRANSFORM_CONVERT, factor: int = 0) -> np.ndarray:
    """ReorderTransformWrapper.Transform (ReorderExtensions.cs:91-95):
    target[i] = transformer(source[reorderView[i]])."""
    return transform(reorder(source, order), target_dtype, transformer, factor)


def scan_temp_ints_cpu() -> int:
    return int(lib().oracle_scan_temp_ints_cpu())


def radix_sort_temp_ints_cpu(elem_bytes: int, n: int,
                             max_num_threads: int = CPU_MAX_NUM_THREADS) -> int:
    return int(lib().oracle_radix_sort_temp_ints_cpu(elem_bytes, n,
                                                     max_num_threads))


def temp_view_allocate(num_ints: int, temp_len_ints: int, elem_bytes: int,
                       is_primitive: bool, length: int) -> int:
    return int(lib().oracle_temp_view_allocate(num_ints, temp_len_ints,
                                               elem_bytes, int(is_primitive),
                                               length))
