"""The slab convolution's host-side sizing against a brute-force walk over every window and tap.

The kernel keeps, per block, the input positions [lo, hi] of one flattened input plane in LDS, lo / hi being the
smallest window origin and the largest origin plus the last tap's offset over the block's windows (clamped to the
plane).  The host sizes the LDS for the longest such run from the ends of each block and of the output rows inside
it only.  Here every window of every block is visited: the run must hold every tap that lies inside the input, and
the plan's capacity must equal the longest run exactly (the kernel's own clamp to the capacity then never acts).
No device is touched.
"""
import itertools

import numpy as np
import pytest

from nnabla_amd import kernels


def brute_force(in_sp, kernel, pad, stride, dil, tile_rows):
    nd = len(in_sp)
    in3 = [1] * (3 - nd) + list(in_sp)
    k3 = [1] * (3 - nd) + list(kernel)
    p3 = [0] * (3 - nd) + list(pad)
    s3 = [1] * (3 - nd) + list(stride)
    d3 = [1] * (3 - nd) + list(dil)
    out3 = [(in3[i] + 2 * p3[i] - (d3[i] * (k3[i] - 1) + 1)) // s3[i] + 1 for i in range(3)]
    plane = in3[0] * in3[1] * in3[2]
    n_out = out3[0] * out3[1] * out3[2]
    o = np.arange(n_out)
    o2, o1, o0 = o % out3[2], (o // out3[2]) % out3[1], o // (out3[2] * out3[1])
    b = [o0 * s3[0] - p3[0], o1 * s3[1] - p3[1], o2 * s3[2] - p3[2]]
    origin = (b[0] * in3[1] + b[1]) * in3[2] + b[2]
    last = ((k3[0] - 1) * d3[0] * in3[1] + (k3[1] - 1) * d3[1]) * in3[2] + (k3[2] - 1) * d3[2]
    longest, uncovered = 1, 0
    tiles = -(-n_out // tile_rows)
    for t in range(tiles):
        sel = slice(t * tile_rows, min((t + 1) * tile_rows, n_out))
        lo = int(np.clip(origin[sel].min(), 0, plane - 1))
        hi = int(np.clip(origin[sel].max() + last, 0, plane - 1))
        longest = max(longest, hi - lo + 1)
        # every tap of every window of the tile that lies inside the input
        for t0, t1, t2 in itertools.product(range(k3[0]), range(k3[1]), range(k3[2])):
            c = [b[0][sel] + t0 * d3[0], b[1][sel] + t1 * d3[1], b[2][sel] + t2 * d3[2]]
            inside = np.ones(c[0].shape, bool)
            for i in range(3):
                inside &= (c[i] >= 0) & (c[i] < in3[i])
            pos = (c[0] * in3[1] + c[1]) * in3[2] + c[2]
            uncovered += int(((pos[inside] < lo) | (pos[inside] > hi)).sum())
    return out3, tiles, longest, uncovered


def geometries():
    rng = np.random.RandomState(20240)
    fixed = [
        ((14, 14), (3, 3), (1, 1), (1, 1), (1, 1)), ((56, 56), (3, 3), (1, 1), (1, 1), (1, 1)),
        ((28, 28), (3, 3), (1, 1), (2, 2), (1, 1)), ((7, 7), (3, 3), (1, 1), (1, 1), (1, 1)),
        ((5, 70), (3, 3), (1, 1), (1, 1), (1, 1)), ((6, 6), (1, 1), (0, 0), (1, 1), (1, 1)),
        ((9, 11), (3, 2), (2, 0), (1, 2), (2, 1)), ((40,), (5,), (2,), (1,), (1,)), ((33,), (3,), (0,), (2,), (3,)),
        ((4, 6, 5), (2, 3, 2), (1, 1, 0), (1, 1, 1), (1, 1, 1)), ((3, 9, 9), (3, 3, 3), (1, 1, 1), (1, 2, 1), (1, 1, 2)),
        ((14, 14), (3, 3), (4, 4), (1, 1), (1, 1)),  # padding wider than the kernel: windows wholly outside
    ]
    for g in fixed:
        yield g
    for _ in range(300):
        nd = int(rng.randint(1, 4))
        in_sp = tuple(int(v) for v in rng.randint(1, [9, 20, 40][3 - nd:][0] + 1, size=nd))
        in_sp = tuple(max(v, 1) for v in in_sp)
        kernel = tuple(int(v) for v in rng.randint(1, 4, size=nd))
        dil = tuple(int(v) for v in rng.randint(1, 3, size=nd))
        stride = tuple(int(v) for v in rng.randint(1, 4, size=nd))
        pad = tuple(int(v) for v in rng.randint(0, 4, size=nd))
        if any(in_sp[i] + 2 * pad[i] < dil[i] * (kernel[i] - 1) + 1 for i in range(nd)):
            continue
        yield in_sp, kernel, pad, stride, dil


def test_the_plan_holds_every_tap_and_is_tight():
    planned = 0
    for in_sp, kernel, pad, stride, dil in geometries():
        for C in (32, 96):
            plan = kernels.binary_convolution_slab_plan(2, C, in_sp, 64, kernel, pad, stride, dil, 1)
            if plan is None:
                continue
            planned += 1
            out3, tiles, longest, uncovered = brute_force(in_sp, kernel, pad, stride, dil, plan["tile_rows"])
            what = "in %s k %s pad %s stride %s dil %s C %d" % (in_sp, kernel, pad, stride, dil, C)
            assert plan["tile_rows"] <= 32, what
            assert plan["tiles_per_sample"] == tiles, what
            assert uncovered == 0, what
            assert plan["cap"] == longest, what
            cgp = -(-C // 32) * 32
            assert (plan["cap"] + 1) * (4 * cgp + 16) <= plan["lds_bytes"] <= 156 * 1024, what
    assert planned >= 300


@pytest.mark.parametrize("C,in_sp,expected", [
    (8, (14, 14), False),      # too few input channels per group
    (40, (14, 14), False),     # 40 channels padded to 64: more than a third wasted
    (256, (14, 14), True),
    (1024, (56, 56), False),   # the positions under 32 windows do not fit the LDS
])
def test_which_geometries_take_the_form(C, in_sp, expected):
    plan = kernels.binary_convolution_slab_plan(1, C, in_sp, 64, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    assert (plan is not None) == expected


def test_whole_rows_of_the_output_map_per_block():
    # 14 x 14 outputs: two rows of 14 per block, seven blocks per sample
    plan = kernels.binary_convolution_slab_plan(32, 256, (14, 14), 256, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    assert plan["tile_rows"] == 28 and plan["tiles_per_sample"] == 7
    # the run: two output rows' windows span four input rows, plus the position before the first row's first window
    # (origin one column to the left) and the one after the last window's last tap
    assert plan["cap"] == 4 * 14 + 2
