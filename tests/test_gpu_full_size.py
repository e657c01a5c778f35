"""GPU checks at the full baseline sizes, through properties that do not need a
CPU pass over the data: sortedness plus a multiset checksum, encode-and-invert
round trips, totals, and linearity.  Inputs are generated on the GPU by the
seeded generators the benchmark uses."""
import sys

import numpy as np
import pytest

from ilgpu_amd import capi, datagen

pytestmark = pytest.mark.gpu
D = capi.DeviceArray


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def wrap(t, dtype):
    import torch
    return D(t.numel(), dtype, _bytes=t.view(torch.uint8))


def u32(t):
    import torch
    return t.to(torch.int64) & 0xFFFFFFFF


def test_sort_2p28_uniform_u32_sorted_and_same_multiset():
    import torch
    n = 1 << 28
    note("sort 2^28 uniform u32")
    src = datagen.uniform_u32_torch(n)
    work = src.clone()
    capi.radix_sort_keys(wrap(work, np.uint32))
    torch.cuda.synchronize()
    a, b = u32(work), u32(src)
    assert bool((a[1:] >= a[:-1]).all().item())
    # multiset equality through two independent checksums and the histogram of the top byte
    assert int(a.sum().item()) == int(b.sum().item())
    assert int((a * a % 1000003).sum().item()) == int((b * b % 1000003).sum().item())
    assert torch.equal(torch.bincount(a >> 24, minlength=256), torch.bincount(b >> 24, minlength=256))
    # idempotence: sorting the sorted array changes nothing
    again = work.clone()
    capi.radix_sort_keys(wrap(again, np.uint32))
    torch.cuda.synchronize()
    assert torch.equal(again, work)


def test_sort_2p28_zipf_against_its_value_counts_and_descending_is_the_reverse():
    import torch
    n = 1 << 28
    note("sort 2^28 zipf u32 ascending vs descending")
    src = datagen.zipf_u32_torch(n)
    asc, desc = src.clone(), src.clone()
    capi.radix_sort_keys(wrap(asc, np.uint32))
    capi.radix_sort_keys(wrap(desc, np.uint32), descending=True)
    torch.cuda.synchronize()
    assert torch.equal(torch.flip(desc, [0]), asc)
    # Against the source, independently of the library: the keys take 2^16
    # values, so the sorted array is fully determined by the value counts of
    # the input (torch.bincount): value v fills [start[v], start[v] + count[v]).
    a = u32(asc)
    counts = torch.bincount(u32(src), minlength=1 << 16)
    assert counts.numel() == 1 << 16
    assert bool((a[1:] >= a[:-1]).all().item())
    assert torch.equal(torch.bincount(a, minlength=1 << 16), counts)
    starts = torch.cumsum(counts, 0) - counts
    present = torch.nonzero(counts).flatten()
    assert torch.equal(a[starts[present]], present)                       # first key of every run
    assert torch.equal(a[starts[present] + counts[present] - 1], present)  # and its last


def test_sort_2p28_all_equal_keys_runs_no_pass_and_leaves_the_input():
    import torch
    n = 1 << 28
    note("sort 2^28 all-equal u32")
    src = torch.full((n,), -559038737, dtype=torch.int32, device="cuda:0")   # 0xDEADBEEF
    work = src.clone()
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32))
    capi.radix_sort_keys(wrap(work, np.uint32), temp)
    torch.cuda.synchronize()
    assert torch.equal(work, src)
    # every digit is the same for all keys: no pass runs
    assert capi.radix_sort_passes(temp, n, np.uint32) == (0, 4)
    # one key differs: its pass and only its pass runs, and the odd key moves to the front
    work[n // 3] = -559038737 - 1                                            # 0xDEADBEEE
    capi.radix_sort_keys(wrap(work, np.uint32), temp)
    torch.cuda.synchronize()
    assert capi.radix_sort_passes(temp, n, np.uint32) == (1, 3)
    assert int(work[0].item()) == -559038738 and bool((work[1:] == -559038737).all().item())


def test_histogram_2p28_i32_4096_bins_against_bincount():
    import torch
    n = 1 << 28
    note("histogram 2^28 i32 -> 4096 bins")
    g = datagen.gaussian_mixture_i32_torch(n)
    bins, ov = D.zeros(4096, np.int32), D.zeros(1, np.int32)
    capi.histogram(wrap(g, np.int32), bins, ov)
    torch.cuda.synchronize()
    expect = torch.zeros(4096, dtype=torch.int64, device="cuda:0")
    for lo in range(0, n, 1 << 26):                       # chunked: bincount widens to int64
        expect += torch.bincount(g[lo: lo + (1 << 26)].to(torch.int64), minlength=4096)
    assert np.array_equal(bins.numpy().astype(np.int64), expect.cpu().numpy())
    assert int(expect.sum().item()) == n and ov.numpy()[0] == 0
    # int64 bins and the modulo locator give the same counts (all keys are in [0, 4095])
    wide = D.zeros(4096, np.int64)
    capi.histogram(wrap(g, np.int32), wide, locator=capi.LOCATOR_MODULO)
    torch.cuda.synchronize()
    assert np.array_equal(wide.numpy(), expect.cpu().numpy())


def test_pairs_2p27_u64_index_values_invert_the_sort():
    import torch
    n = 1 << 27
    note("pairs 2^27 u64 + index")
    keys = datagen.splitmix64_torch(n)
    work = keys.clone()
    vals = torch.empty(n, dtype=torch.int32, device="cuda:0")
    capi.radix_sort_pairs(wrap(work, np.uint64), wrap(vals, np.uint32), values_from_index=True)
    torch.cuda.synchronize()
    # values are a permutation that reproduces the output from the input
    assert torch.equal(keys[vals.to(torch.int64)], work)
    flipped = work ^ (-(1 << 63))
    assert bool((flipped[1:] >= flipped[:-1]).all().item())
    ties = work[1:] == work[:-1]
    assert bool((vals[1:][ties] > vals[:-1][ties]).all().item())    # stable
    assert int(torch.bincount(vals.to(torch.int64) >> 20).max().item()) == 1 << 20  # a permutation


def test_scan_2p28_inclusive_exclusive_and_differences():
    import torch
    n = 1 << 28
    note("scan 2^28 i32")
    x = datagen.small_ints_i32_torch(n)
    inc, exc = torch.empty_like(x), torch.empty_like(x)
    capi.scan(wrap(x, np.int32), wrap(inc, np.int32), kind=capi.SCAN_INCLUSIVE)
    capi.scan(wrap(x, np.int32), wrap(exc, np.int32), kind=capi.SCAN_EXCLUSIVE)
    torch.cuda.synchronize()
    assert torch.equal(inc - exc, x)                       # inclusive = exclusive + input
    assert torch.equal(inc[1:] - inc[:-1], x[1:])          # differences give the input back
    assert int(exc[0].item()) == 0
    # values are 0..15, so the total stays below 2^31 and the int32 scan does not wrap
    assert int(inc[-1].item()) == int(x.sum(dtype=torch.int64).item())


def test_scan_2p28_max_is_monotone_and_bounded():
    import torch
    n = 1 << 28
    x = datagen.gaussian_mixture_i32_torch(n)
    out = torch.empty_like(x)
    capi.scan(wrap(x, np.int32), wrap(out, np.int32), op=capi.OP_MAX, kind=capi.SCAN_INCLUSIVE)
    torch.cuda.synchronize()
    assert bool((out[1:] >= out[:-1]).all().item())
    assert bool((out >= x).all().item())
    assert int(out[-1].item()) == int(x.max().item())


def test_reduce_2p28_f32_and_linearity():
    import torch
    n = 1 << 28
    note("reduce 2^28 f32")
    f = datagen.normal_f32_torch(n)
    out = D.zeros(1, np.float32)
    capi.reduce(wrap(f, np.float32), out)
    torch.cuda.synchronize()
    exact = float(f.sum(dtype=torch.float64).item())
    got = float(out.numpy()[0])
    # contract: within 1e-5 relative of the float64 sum (plus one float32 rounding)
    assert abs(got - exact) <= 1e-5 * abs(exact) + abs(exact) * 2.0 ** -24
    # the halves add up to the whole, in integers exactly
    x = datagen.small_ints_i32_torch(n)
    tot, lo, hi = D.zeros(1, np.int32), D.zeros(1, np.int32), D.zeros(1, np.int32)
    d = wrap(x, np.int32)
    capi.reduce(d, tot)
    capi.reduce(d.subview(0, n // 2), lo)
    capi.reduce(d.subview(n // 2, n // 2), hi)
    torch.cuda.synchronize()
    assert int(tot.numpy()[0]) == int(lo.numpy()[0]) + int(hi.numpy()[0])
    assert int(tot.numpy()[0]) == int(x.sum(dtype=torch.int64).item())


def test_histogram_2p30_u8_totals_and_accumulation():
    import torch
    n = 1 << 30
    note("histogram 2^30 u8")
    b = datagen.bytes_u8_torch(n)
    bins, ov = D.zeros(256, np.int32), D.zeros(1, np.int32)
    d = wrap(b, np.uint8)
    capi.histogram(d, bins, ov)
    torch.cuda.synchronize()
    h1 = bins.numpy().astype(np.int64)
    assert h1.sum() == n and ov.numpy()[0] == 0
    expect = torch.zeros(256, dtype=torch.int64, device="cuda:0")
    for c in range(4):
        expect += torch.bincount(b[c << 28:(c + 1) << 28].to(torch.int64), minlength=256)
    assert np.array_equal(h1, expect.cpu().numpy())
    # a second call accumulates: twice the counts, and 2^31 total overflows no int32 bin
    capi.histogram(d, bins, ov)
    torch.cuda.synchronize()
    assert np.array_equal(bins.numpy().astype(np.int64), 2 * h1) and ov.numpy()[0] == 0


def test_unique_after_sort_2p28_counts_distinct_keys():
    import torch
    n = 1 << 28
    note("sort + unique 2^28 zipf")
    keys = datagen.zipf_u32_torch(n)
    work = keys.clone()
    d = wrap(work, np.uint32)
    capi.radix_sort_keys(d)
    count = D.zeros(1, np.int64)
    capi.unique(d, count)
    torch.cuda.synchronize()
    kept = int(count.numpy()[0])
    present = torch.bincount(u32(keys), minlength=1 << 16) > 0
    assert kept == int(present.sum().item())
    assert torch.equal(u32(work[:kept]), torch.nonzero(present).flatten())


def test_sort_beyond_2p30_keys():
    # Per-digit inclusive counts pass 2^30 here (two key values only), which the
    # look-back status words must carry; sortedness and the value counts pin
    # the result.
    import torch
    n = (1 << 30) + 12345
    note("sort 2^30 + 12345 u32, two distinct values")
    idx = torch.arange(n, device="cuda:0", dtype=torch.int64)
    src = torch.where(idx % (1 << 20) == 5,
                      torch.tensor(7, device="cuda:0"), torch.tensor(0x01000003, device="cuda:0")).to(torch.int32)
    del idx
    sevens = int((src == 7).sum().item())
    assert n - sevens > 1 << 30            # one digit's count passes 2^30
    work = src.clone()
    del src
    capi.radix_sort_keys(wrap(work, np.uint32))
    torch.cuda.synchronize()
    assert bool((work[:sevens] == 7).all().item())
    assert bool((work[sevens:] == 0x01000003).all().item())


def test_maximum_length_int_max():
    # The reference accepts views up to int.MaxValue elements
    # (RadixSortExtensions.cs:1195-1199, ScanExtensions.cs:675-678): every
    # primitive at exactly 2^31 - 1 elements, checked by totals and structure.
    import torch
    n = (1 << 31) - 1
    dev = "cuda:0"
    note("maximum length: 2^31 - 1 uint8 samples / keys")
    idx = torch.arange(n, device=dev, dtype=torch.int32)
    samples = ((idx * 37) ^ (idx >> 9)).to(torch.uint8)     # every byte value, uneven counts
    del idx
    # histogram: totals against chunked bincounts
    counts = torch.zeros(256, dtype=torch.int64, device=dev)
    for lo in range(0, n, 1 << 28):
        counts += torch.bincount(samples[lo: lo + (1 << 28)].to(torch.int64), minlength=256)
    bins = D.zeros(256, np.int64)
    capi.histogram(wrap(samples, np.uint8), bins)
    torch.cuda.synchronize()
    assert np.array_equal(bins.numpy(), counts.cpu().numpy())
    # sort of the same bytes: output = each value repeated count times
    keys = samples.clone()
    capi.radix_sort_keys(wrap(keys, np.uint8))
    torch.cuda.synchronize()
    starts = torch.cumsum(counts, 0) - counts
    for v in (0, 1, 127, 128, 255):
        s, c = int(starts[v].item()), int(counts[v].item())
        assert bool((keys[s: s + c] == v).all().item()), v
    assert bool((keys[1:] >= keys[:-1]).all().item())
    del keys, samples
    note("maximum length: 2^31 - 1 int32 scan and reduce")
    x = (torch.arange(n, device=dev, dtype=torch.int32) & 7) - 3      # -3 .. 4
    out = torch.empty_like(x)
    capi.scan(wrap(x, np.int32), wrap(out, np.int32), kind=capi.SCAN_INCLUSIVE)
    total = D.zeros(1, np.int32)
    capi.reduce(wrap(x, np.int32), total)
    torch.cuda.synchronize()
    # x has period 8 with sum 4: closed form for the inclusive scan at any index
    probe = torch.tensor([0, 1, 7, 8, 12345, (1 << 30) + 3, n - 2, n - 1], device=dev, dtype=torch.int64)
    pre = torch.tensor([-3, -5, -6, -6, -5, -3, 0, 4], device=dev, dtype=torch.int64)
    closed = (probe // 8) * 4 + pre[probe % 8]
    assert bool((out[probe].to(torch.int64) == closed).all().item())
    assert bool(((out[1:] - out[:-1]) == x[1:]).all().item())
    assert int(total.numpy()[0]) == int(closed[-1].item())
