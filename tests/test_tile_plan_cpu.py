"""The geometry search of the persistent recurrences (haste_hip_plan_tiles), swept on the host
over hidden sizes, batch sizes and device shapes: whatever it finds must be a geometry the
kernels can run."""
import ctypes

import pytest

from haste_amd import lib as hlib

DEVICES = [(256, 8), (256, 0), (128, 4), (304, 8), (64, 1)]
BATCHES = [1, 3, 4, 8, 9, 16, 31, 32, 64, 100, 128, 200, 256, 512]


def _plan(lib, cus, xcds, gates, N, H):
    out = (ctypes.c_int * 16)()
    rc = lib.haste_hip_plan_tiles(cus, xcds, gates, N, H, out)
    assert rc == 0
    return list(out[:8]), list(out[8:])


@pytest.mark.parametrize("cus,xcds", DEVICES)
@pytest.mark.parametrize("gates", [3, 4])
def test_every_geometry_found_is_one_the_kernels_can_run(cus, xcds, gates):
    lib = hlib.load()
    lib.haste_hip_plan_tiles.restype = ctypes.c_int
    sizes = list(range(16, 4097, 16)) + [1, 5, 37, 100, 300, 500, 1001, 1300, 2049]
    resident = 0
    for H in sizes:
        for N in BATCHES:
            for which, plan in zip(("forward", "backward"), _plan(lib, cus, xcds, gates, N, H)):
                found, nb, hs, ct, gx, gy, reg, groups = plan
                where = (which, cus, xcds, gates, N, H, plan)
                if not found:
                    assert plan == [0] * 8, where
                    continue
                assert nb in (4, 8, 16, 32, 64), where
                if which == "forward":  # the gate columns of the workgroup's units fit its slice
                    assert hs in (4, 8, 16) and gates * hs <= 16 * ct, where
                assert gx == -(-H // hs) and gy == -(-N // nb), where
                # one workgroup per CU, all on the chip at once
                assert gx * gy <= cus, where
                # part of the slice in registers: tall tiles only, whole batches of 8 groups, and
                # some of the slice stays in LDS
                if reg:
                    resident += 1
                    assert nb >= 16 and reg % 8 == 0 and 0 < reg < groups, where
    if cus >= 256:
        assert resident > 0  # the sweep reaches the register-resident range


def test_plan_tiles_refuses_bad_arguments():
    lib = hlib.load()
    lib.haste_hip_plan_tiles.restype = ctypes.c_int
    out = (ctypes.c_int * 16)()
    assert lib.haste_hip_plan_tiles(256, 8, 5, 4, 64, out) != 0
    assert lib.haste_hip_plan_tiles(256, 8, 4, 0, 64, out) != 0
    assert lib.haste_hip_plan_tiles(256, 8, 4, 4, 64, None) != 0
    assert lib.haste_hip_plan_tiles(0, 8, 4, 4, 64, out) != 0
