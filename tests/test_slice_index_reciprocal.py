"""The device code finds the heap slice of an offset d without dividing: with S = slice size in units of
2 MiB and magic = floor(2^40 / S) + 1, slice = ((d >> 21) * magic) >> 40 (nvshmemi_amd_slice_offset,
include/nvshmem_amd/device/nvshmemi_device.h; the role of the reference's peer_heap_base_p2p[] lookup,
src/include/non_abi/device/common/nvshmemi_common_device.cuh:493-498).  Checked here against integer
division for every heap the runtime accepts: slice sizes that are multiples of 2 MiB, whole heap at most 512 GiB."""
import numpy as np


def _magic(slice_units):
    return (1 << 40) // slice_units + 1


def _slice(d, magic):
    return (((d >> 21) & 0xFFFFFFFF) * magic) >> 40


def test_reciprocal_slice_index_matches_division_at_every_slice_boundary():
    rng = np.random.default_rng(5)
    sizes = [1, 2, 3, 5, 7, 8, 9, 56, 511, 512, 513, 520, 3127, 1 << 12, (1 << 12) + 1, 65535, 1 << 16, (1 << 17) - 1, 1 << 17]
    sizes += [int(x) for x in rng.integers(1, 1 << 17, 300)]
    for units in sizes:                                     # slice size = units x 2 MiB
        magic, size = _magic(units), units << 21
        max_pes = min(64, (1 << 39) // size)
        for pe in range(max_pes + 1):                       # one slice beyond the last PE as well
            lo, hi = pe * size, (pe + 1) * size
            for d in (lo, lo + 1, lo + (1 << 21) - 1, lo + (1 << 21), (lo + hi) // 2, hi - (1 << 21), hi - 1):
                assert _slice(d, magic) == d // size, (units, pe, d)


def test_reciprocal_slice_index_matches_division_on_random_offsets():
    rng = np.random.default_rng(6)
    for _ in range(20000):
        units = int(rng.integers(1, 1 << 18))
        size = units << 21
        npes = max(1, min(64, (1 << 39) // size))
        d = int(rng.integers(0, npes * size))
        assert _slice(d, _magic(units)) == d // size, (units, d)


def test_the_bound_is_needed():
    # beyond the 512 GiB the runtime accepts the 40-bit reciprocal does go wrong: the check in
    # nvshmemx_amd_init is not decoration
    units = (1 << 18) - 1
    size = units << 21
    bad = 0
    for pe in range(1 << 10, (1 << 10) + 4096):
        d = (pe + 1) * size - 1
        bad += _slice(d, _magic(units)) != d // size
    assert bad > 0
