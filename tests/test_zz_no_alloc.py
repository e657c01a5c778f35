"""ilgpu_hip_scan_static: the scan on the library's static scratch (no temp
view, no allocation) against ilgpu_hip_scan, bit for bit, through the C ABI.

Two calls in a row share the scratch array; the second one is smaller, so it
runs over status words the first one left behind.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(capi, torch, values, op, kind):
    D = capi.DeviceArray
    d_in = D.from_numpy(values)
    with_temp, static = D.zeros(values.size, values.dtype), D.zeros(values.size, values.dtype)
    capi.scan(d_in, with_temp, op=op, kind=kind)
    capi.scan_static(d_in, static, op=op, kind=kind)
    torch.cuda.synchronize()
    return with_temp.numpy(), static.numpy()


@pytest.mark.parametrize("dtype", [np.int32, np.uint64, np.float32])
def test_scan_static_matches_scan_on_two_calls_in_a_row(dtype):
    import torch
    from ilgpu_amd import capi
    from oracle import cpu_oracle as O
    rng = np.random.default_rng(7)
    # first call: many tiles (a tile is 128 KiB); second call: fewer tiles, ragged end
    sizes = [(1 << 22) + 12345, (1 << 17) + 77]
    for n in sizes:
        if np.dtype(dtype).kind == "f":
            values = rng.integers(-8, 9, size=n).astype(dtype)     # sums stay exact
        else:
            values = rng.integers(0, 16, size=n).astype(dtype)
        for op, kind in ((capi.OP_ADD, capi.SCAN_EXCLUSIVE), (capi.OP_MAX, capi.SCAN_INCLUSIVE)):
            a, b = _both(capi, torch, values, op, kind)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (dtype, n, op, kind)
        # and against the CPU oracle, on the smaller size
        if n < (1 << 20):
            _, b = _both(capi, torch, values, capi.OP_ADD, capi.SCAN_INCLUSIVE)
            assert np.array_equal(b, O.scan(values, O.OP_ADD, inclusive=True))


def test_scan_static_rejects_inputs_beyond_its_scratch():
    import torch
    from ilgpu_amd import capi
    n = capi.SCAN_STATIC_MAX_BYTES // 8 + 1          # one int64 too many
    big = torch.empty(n, dtype=torch.int64, device="cuda")
    view = capi.DeviceArray(n, np.int64, _bytes=big.view(torch.uint8))
    with pytest.raises(capi.NotSupportedError) as info:
        capi.scan_static(view, view)
    assert info.value.status == capi.ERROR_STATIC_LIMIT
    assert "static scratch" in str(info.value)
    # the largest input it takes: exactly the limit, in place
    n = capi.SCAN_STATIC_MAX_BYTES // 8
    big = torch.ones(n, dtype=torch.int64, device="cuda")
    view = capi.DeviceArray(n, np.int64, _bytes=big.view(torch.uint8))
    capi.scan_static(view, view, kind=capi.SCAN_INCLUSIVE)
    torch.cuda.synchronize()
    assert int(big[-1]) == n and int(big[0]) == 1 and int(big[n // 2]) == n // 2 + 1
    # the checks of ilgpu_hip_scan still come first
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.scan_static(capi.DeviceArray.zeros(8, np.int32), capi.DeviceArray.zeros(4, np.int32))
