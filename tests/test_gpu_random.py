"""Seeded random cases through the C ABI against the CPU oracle (and numpy's
stable sort for the long ones): every key type, keys and pairs, both orders,
key distributions that exercise the dominant-digit, whole-row and skipped-pass
paths, with the sort's block size, its one-tile kernel and its look-back bound
switched at random (ilgpu_hip_sort_set_parameter)."""
import numpy as np
import pytest

from ilgpu_amd import capi
from oracle import cpu_oracle as O

pytestmark = pytest.mark.gpu
D = capi.DeviceArray
KEYS = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
        np.float16, np.float32, np.float64]


def _sync():
    import torch
    torch.cuda.synchronize()


def _keys(rng, dt, n):
    dt = np.dtype(dt)
    mode = int(rng.integers(0, 5))
    if dt.kind == "f":
        u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[dt.itemsize]
        if mode == 0:
            return rng.integers(0, np.iinfo(u).max, n, dtype=u, endpoint=True).view(dt)
        if mode == 1:
            return (rng.integers(-8, 8, n) * 0.5).astype(dt)
        if mode == 2:
            return (1.0 + rng.random(n)).astype(dt)
        return np.repeat((rng.integers(-300, 300, n // 500 + 1)).astype(dt), 500)[:n]
    info = np.iinfo(dt)
    if mode == 0:
        return rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
    if mode == 1:
        return rng.integers(0, min(info.max, 5), n).astype(dt)
    if mode == 2:
        return np.repeat(rng.integers(info.min, info.max, n // 700 + 1, dtype=dt, endpoint=True),
                         700)[:n]
    if mode == 3:
        return np.full(n, rng.integers(info.min, info.max, dtype=dt, endpoint=True), dtype=dt)
    a, b, c = (rng.integers(info.min, info.max, n, dtype=dt, endpoint=True) for _ in range(3))
    return a & b & c


@pytest.fixture
def sort_parameters():
    yield
    for p in (capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU):
        capi.sort_set_parameter(p, -1)
    capi.sort_set_parameter(capi.SORT_PARAM_ONE_TILE_KERNEL, 1)


def test_random_sorts_against_the_oracle(sort_parameters):
    rng = np.random.default_rng(20240607)
    for case in range(260):
        n = int(rng.choice([rng.integers(1, 300), rng.integers(1, 40000),
                            rng.integers(1, 250000)]))
        dt = KEYS[rng.integers(len(KEYS))]
        keys = _keys(rng, dt, n)
        large = int(rng.choice([-1, 0, 2 ** 31 - 1]))
        one_tile = int(rng.choice([1, 0]))
        spin = int(rng.choice([-1, -1, -1, 0]))
        capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU, large)
        capi.sort_set_parameter(capi.SORT_PARAM_ONE_TILE_KERNEL, one_tile)
        capi.sort_set_parameter(capi.SORT_PARAM_LOOKBACK_SPIN_LIMIT, spin)
        descending = bool(rng.integers(0, 2))
        tag = (case, np.dtype(dt).name, n, large, one_tile, spin, descending)
        print("random sort", *tag, flush=True)
        if rng.integers(0, 2):
            vb = int(rng.choice([1, 2, 4, 8]))
            vdt = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[vb]
            values = rng.integers(0, 255, n * vb, dtype=np.uint8).view(vdt)
            dk, dv = D.from_numpy(keys), D.from_numpy(values)
            capi.radix_sort_pairs(dk, dv, descending=descending)
            _sync()
            ek, ev = O.radix_sort_pairs(keys, values, descending=descending)
            assert np.array_equal(dk.numpy().view(np.uint8), ek.view(np.uint8)), tag
            assert np.array_equal(dv.numpy(), ev), tag
        else:
            d = D.from_numpy(keys)
            capi.radix_sort_keys(d, descending=descending)
            _sync()
            want = O.radix_sort(keys, descending=descending)
            assert np.array_equal(d.numpy().view(np.uint8), want.view(np.uint8)), tag


def test_random_long_sorts_against_numpy(sort_parameters):
    rng = np.random.default_rng(7)
    for case in range(24):
        n = int(rng.choice([rng.integers(1, 3000000), rng.integers(1, 30000000)]))
        dt = KEYS[rng.integers(8)]          # integer keys: numeric order
        keys = _keys(rng, dt, n)
        capi.sort_set_parameter(capi.SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU,
                                int(rng.choice([-1, 0, 2 ** 31 - 1])))
        descending = bool(rng.integers(0, 2))
        tag = (case, np.dtype(dt).name, n, descending)
        print("random long sort", *tag, flush=True)
        flipped = ~keys                      # reverses the order of signed and unsigned keys alike
        order = np.argsort(flipped if descending else keys, kind="stable")
        if rng.integers(0, 2):
            dk, dv = D.from_numpy(keys), D.zeros(n, np.uint32)
            capi.radix_sort_pairs(dk, dv, descending=descending, values_from_index=True)
            _sync()
            assert np.array_equal(dk.numpy(), keys[order]), tag
            assert np.array_equal(dv.numpy(), order.astype(np.uint32)), tag
        else:
            d = D.from_numpy(keys)
            capi.radix_sort_keys(d, descending=descending)
            _sync()
            assert np.array_equal(d.numpy(), keys[order]), tag
