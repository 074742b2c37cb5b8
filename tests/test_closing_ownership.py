"""Host-side statement of the rule by which the depthwise kernel that finishes its producer's open
activation (dc_expand_depthwise) commits the producer's cached state: every lane group -- one per
OUTPUT pixel of the 3x3, padding-1 depthwise layer -- commits the input pixels it owns, with stride 1
its centre pixel, with stride 2 the 2 x 2 block at twice its output coordinates.  For the commit to
happen exactly once per input pixel, every input pixel has to be owned by exactly one group, and
for the group to know the pixel's keep decision the pixel has to lie in the group's own window, at
tap (1 + dy, 1 + dx).  Checked here for all map sizes up to 24 x 24.  No GPU involved."""
import itertools

import numpy as np
import pytest


def _out(n, stride):
    return (n + 2 - 3) // stride + 1  # kernel 3, padding 1


@pytest.mark.parametrize("stride", [1, 2])
def test_every_input_pixel_is_owned_once_and_seen_by_its_owner(stride):
    for Hi, Wi in itertools.product(range(1, 25), range(1, 25)):
        Ho, Wo = _out(Hi, stride), _out(Wi, stride)
        assert stride * Ho >= Hi and stride * Wo >= Wi  # what the host checks before it takes the form
        owners = np.zeros((Hi, Wi), dtype=np.int32)
        blocks = [(0, 0)] if stride == 1 else [(0, 0), (0, 1), (1, 0), (1, 1)]
        for oy, ox in itertools.product(range(Ho), range(Wo)):
            for dy, dx in blocks:
                iy, ix = oy * stride + dy, ox * stride + dx
                if iy >= Hi or ix >= Wi:  # cut by the map's edge: the tap is out of bounds and never set
                    continue
                owners[iy, ix] += 1
                # the owned pixel is tap (1 + dy, 1 + dx) of the owner's window
                ky, kx = 1 + dy, 1 + dx
                assert (oy * stride - 1 + ky, ox * stride - 1 + kx) == (iy, ix)
                assert ky * 3 + kx in ((4,) if stride == 1 else (4, 5, 7, 8))
        assert (owners == 1).all(), (Hi, Wi, stride)
