"""Orders of the wide kernel's units (sparse24_wide_kernel's first lines, restated): every order gives each
(tile, column group) to exactly one workgroup of the grid the host launches, and no workgroup looks at a tile past the
host's bound.  The grid sizes are the library's (triteia_hip_wide_grid_units)."""
import collections

import pytest

from triteia_amd.python.capi import _ffi


def unit_of(u, cgs, rows, order):
    """(tile, column group) of workgroup u, or None where the kernel returns before it reads a tile."""
    cg_pad = (cgs + 7) // 8 * 8
    grp, i = divmod(u, cg_pad)
    if order == 2:
        grp, cg = divmod(u, cgs)
        if grp >= rows:
            return None
    elif order == 3:
        pad = cg_pad - cgs
        R = (cgs + pad - 1) // pad
        sg, row = divmod(grp, R)
        c = (i & 7) * (cg_pad >> 3) + (i >> 3)
        if c < cgs:
            grp, cg = sg * (R + 1) + row, c
        else:
            grp, cg = sg * (R + 1) + R, row * pad + (c - cgs)
        if grp >= rows:
            return None
    else:
        cg = (i & 7) * (cg_pad >> 3) + (i >> 3) if order else i
    if cg >= cgs:
        return None
    return grp, cg


def block_unit_of(u, cgs, rows_live, xc):
    """Order 4: XCD u % 8 takes block (u % 8) % n of the column groups and block (u % 8) // n of the live tiles."""
    cg_pad = (cgs + 7) // 8 * 8
    n_cgb = cg_pad // xc
    tbs = 8 // n_cgb
    tpb = (rows_live + tbs - 1) // tbs
    xcd, slot = u & 7, u >> 3
    cg = (xcd % n_cgb) * xc + slot % xc
    tslot = slot // xc
    grp = (xcd // n_cgb) * tpb + tslot
    if tslot >= tpb or grp >= rows_live or cg >= cgs:
        return None
    return grp, cg


def test_blocks_per_xcd_give_every_unit_once():
    """The grid is sized on the host's bound of tiles; the device cuts the blocks of tiles from the live count."""
    lib = _ffi.lib()
    for cgs in range(1, 41):
        cg_pad = (cgs + 7) // 8 * 8
        m = 512 * cgs
        sizes = [xc for xc in range(1, cg_pad + 1) if cg_pad % xc == 0 and cg_pad // xc <= 8 and 8 % (cg_pad // xc) == 0]
        assert cg_pad // 8 in sizes and cg_pad in sizes
        for xc in range(1, cg_pad + 1):
            if xc not in sizes:
                assert lib.triteia_hip_wide_block_grid_units(5, m, xc) == -1
        for xc in sizes:
            for rows in list(range(1, 20)) + [127, 129, 500]:
                grid = lib.triteia_hip_wide_block_grid_units(rows, m, xc)
                assert grid > 0 and grid % 8 == 0
                for rows_live in {rows, max(1, rows // 2), max(1, rows - 1), 1}:
                    seen = collections.Counter()
                    per_xcd = collections.defaultdict(set)
                    for u in range(grid):
                        t = block_unit_of(u, cgs, rows_live, xc)
                        if t is not None:
                            seen[t] += 1
                            per_xcd[u % 8].add(t[1])
                    assert len(seen) == rows_live * cgs and set(seen.values()) == {1}, (cgs, xc, rows, rows_live)
                    assert all(len(v) <= xc for v in per_xcd.values())


@pytest.mark.parametrize("order", [0, 1, 2, 3])
def test_every_unit_once_and_none_past_the_bound(order):
    lib = _ffi.lib()
    for cgs in range(1, 41):
        if order == 3 and cgs % 8 == 0:
            continue    # no padding: the host never asks for this order
        m = 512 * cgs
        for rows in list(range(1, 40)) + [127, 128, 129, 1000]:
            grid = lib.triteia_hip_wide_grid_units(rows, m, order)
            seen = collections.Counter()
            for u in range(grid):
                t = unit_of(u, cgs, rows, order)
                if t is not None:
                    assert 0 <= t[0] < rows, (order, cgs, rows, u, t)
                    seen[t] += 1
            assert len(seen) == rows * cgs and set(seen.values()) == {1}, (order, cgs, rows)


def test_the_idle_slots_balance_the_xcds():
    lib = _ffi.lib()
    for cgs, rows in ((28, 18), (27, 18), (22, 27), (12, 20)):
        loads = {}
        for order in (1, 3):
            load = [0] * 8
            for u in range(lib.triteia_hip_wide_grid_units(rows, 512 * cgs, order)):
                if unit_of(u, cgs, rows, order) is not None:
                    load[u % 8] += 1
            loads[order] = load
        assert max(loads[3]) < max(loads[1]), (cgs, rows, loads)
        assert lib.triteia_hip_wide_unit_order(512 * cgs) == (3 if (cgs + 7) // 8 * 8 - cgs >= 3 else 1)


def streaming_unit_of(u, n_groups, col_units, order):
    """(group, column unit) of workgroup u of sparse24_grouped_kernel, or None for a padding slot (the kernel's first
    lines, restated): order 1 gives every XCD (u % 8) a run of column units of every group, order 5 whole groups."""
    cu_pad = (col_units + 7) // 8 * 8
    grp, i = divmod(u, cu_pad)
    cu = (i & 7) * (cu_pad >> 3) + (i >> 3)
    if order == 5:
        gpx = n_groups >> 3
        if u < 8 * gpx * cu_pad:
            xcd, s = u & 7, u >> 3
            grp, cu = xcd * gpx + s // cu_pad, s % cu_pad
    return (grp, cu) if cu < col_units else None


def test_whole_groups_per_xcd_in_the_streaming_kernel():
    for n_groups in range(8, 41):
        for col_units in (1, 2, 7, 8, 32, 43, 86, 224):
            cu_pad = (col_units + 7) // 8 * 8
            seen = collections.Counter()
            groups_of_xcd = collections.defaultdict(set)
            for u in range(n_groups * cu_pad):
                t = streaming_unit_of(u, n_groups, col_units, 5)
                if t is not None:
                    seen[t] += 1
                    if t[0] < (n_groups >> 3) * 8:
                        groups_of_xcd[u % 8].add(t[0])
            assert len(seen) == n_groups * col_units and set(seen.values()) == {1}, (n_groups, col_units)
            # the groups that fill the XCDs evenly go whole to one XCD each, n_groups // 8 per XCD
            assert all(len(v) == n_groups >> 3 for v in groups_of_xcd.values())
            assert len(set().union(*groups_of_xcd.values())) == (n_groups >> 3) * 8
