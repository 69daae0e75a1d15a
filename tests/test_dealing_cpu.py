"""The dealing of work items to the persistent workgroups, enumerated on the host with the kernels' own
code (intra_model_deal): whatever the grid and the workgroup size, every row block that exists is
dealt exactly once - also where the heavy text row blocks of image gather0 stand for several rounds
of their workgroups - and no workgroup count changes which row blocks exist."""
import numpy as np
import pytest

from intra_amd import _lib

LLM, IMAGE = 0, 1
SCATTER, GATHER1, GATHER0, WINDOW = 0, 1, 4, 4


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def deal(lib, domain, pattern, B, S, H, Hkv, arg0, arg1, waves, grid):
    plan = _lib.IntraPlan()
    plan_fn = lib.intra_plan
    assert plan_fn(domain, pattern, B, S, H, Hkv, arg0, arg1, plan) == 0, _lib.last_error()
    n = plan.work_items * (2 if waves == 4 and plan.waves == 8 else 1) * 2  # room for either shape
    visits = np.zeros(n, dtype=np.uint8)
    rc = lib.intra_model_deal(domain, pattern, B, S, H, Hkv, arg0, arg1, waves, grid, visits.ctypes.data, n)
    return rc, visits


@pytest.mark.parametrize("waves", [8, 4])
@pytest.mark.parametrize("width,B,H", [(64, 1, 24), (128, 1, 24), (128, 2, 24), (32, 1, 3), (96, 1, 5), (128, 1, 40)])
def test_image_gather0_every_row_block_once(lib, width, B, H, waves):
    S = 512 + width * width
    rc, base = deal(lib, IMAGE, GATHER0, B, S, H, H, width, 512, waves, 8)
    assert rc == 0, _lib.last_error()
    assert base.max() == 1 and base.sum() > 0
    for grid in (16, 64, 256, 512, 1024):
        rc, visits = deal(lib, IMAGE, GATHER0, B, S, H, H, width, 512, waves, grid)
        if rc != 0:
            assert "grid" in _lib.last_error()  # more workgroups than row blocks
            continue
        assert np.array_equal(visits, base), (width, B, H, waves, grid)


@pytest.mark.parametrize("waves", [8, 4])
def test_other_patterns_every_row_block_once(lib, waves):
    cases = [(LLM, SCATTER, 1, 8192, 32, 8, 8, 0), (LLM, GATHER1, 2, 4100, 8, 2, 8, 0), (LLM, WINDOW, 1, 8192, 32, 8, 8, 576),
             (IMAGE, SCATTER, 1, 4608, 24, 24, 64, 512), (IMAGE, SCATTER, 1, 16896, 24, 24, 128, 512)]
    for case in cases:
        rc, base = deal(lib, *case, waves, 8)
        assert rc == 0, _lib.last_error()
        assert base.max() == 1 and base.sum() > 0
        for grid in (64, 256, 512):
            rc, visits = deal(lib, *case, waves, grid)
            if rc != 0:
                assert "grid" in _lib.last_error()
                continue
            assert np.array_equal(visits, base), (case, waves, grid)


def test_plan_names_the_half_size_workgroups_for_image_gather0(lib):
    plan = _lib.IntraPlan()
    assert lib.intra_plan(IMAGE, GATHER0, 1, 16896, 24, 24, 128, 512, plan) == 0
    assert plan.waves == 4 and plan.pos_per_block == 128 and plan.lds_bytes < 80 * 1024
    assert lib.intra_plan(IMAGE, SCATTER, 1, 16896, 24, 24, 128, 512, plan) == 0
    assert plan.waves == 8 and plan.pos_per_block == 256
