"""The oracle against the committed golden vectors of configuration 0 (tests/golden/config0.npz,
written by tests/golden/make_golden.py) on the scene stored with them.  Hit sets, counters and ray
distances must reproduce exactly; colours and gradients pass through libm's expf, whose last bit
may depend on the CPU model, and get a tolerance far below the parity gates."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden  # noqa: E402

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config0.npz")


@pytest.fixture(scope="module")
def golden():
    return dict(np.load(GOLDEN))


def test_oracle_reproduces_golden_vectors(orc, golden):
    got = make_golden.compute(make_golden.scene_of(golden))
    assert sorted(got) == sorted(golden)
    assert np.abs(got["image"] - golden["image"]).max() <= 1e-6
    for k in ("seg_ray", "seg_lo", "seg_hi", "seg_off", "seg_ids", "fh_ray", "fh_lo", "fh_hi", "fh_t",
              "stats_hit_pairs", "stats_slabs", "stats_empty_slabs", "stats_rays_hit"):
        np.testing.assert_array_equal(got[k], golden[k], err_msg=k)
    for k in ("d_positions", "d_scales", "d_quaternions", "d_densities", "d_color_features"):
        scale = np.abs(golden[k]).max()
        assert np.abs(got[k] - golden[k]).max() <= 1e-6 * scale, k


def test_golden_vectors_are_not_trivial(golden):
    assert golden["image"].shape == (128 * 128, 3) and 0.05 < golden["image"].std()
    assert golden["stats_hit_pairs"] > 100000 and golden["stats_rays_hit"] > 5000
    assert len(golden["seg_ray"]) > 1000 and np.diff(golden["seg_off"]).max() >= 4
    assert (golden["fh_t"] >= 0).sum() > 300 and (golden["fh_t"] < 0).sum() > 300
    for k in ("d_positions", "d_scales", "d_quaternions", "d_densities", "d_color_features"):
        assert np.isfinite(golden[k]).all() and np.count_nonzero(golden[k]) > golden[k].size // 4, k
