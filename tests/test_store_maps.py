"""Host-side emulation of the store gates and address arithmetic with which the pointwise kernels
that end an OPEN activation write their two results (the activated difference D and the
candidate T): every element of every updated pixel is written exactly once, nothing else is
touched, also in a ragged last tile (pixel count not a multiple of 16) whose surplus lanes
shadow the last pixel.  Two forms are emulated: the per-lane 8-byte store of the MFMA
accumulator layout (lane (l16, kq) holds channels tile * 16 + kq * 4 .. + 3 of pixel l16,
gated by bit l16 of the tile's update mask) and the staged form that replaced it (pixel rows
in LDS, 16-byte pieces assigned to lanes by a flat index).  No GPU involved."""
import itertools

import numpy as np
import pytest

WAVE = 64
NW = 8  # wavefronts per workgroup of pw_pair_kernel


def _tile_mask(P, pbase, rng, density):
    """Update bits of the 16 pixel slots of a tile: only pixels below P can be set."""
    bits = 0
    for r in range(16):
        if pbase + r < P and rng.random() < density:
            bits |= 1 << r
    return bits


def _per_lane_stores(P, Ce, pbase, bo, grid_y, ct2):
    """(pixel, channel) elements written by the accumulator-layout epilogue of one pixel tile."""
    hits = np.zeros((P, Ce), dtype=np.int32)
    ce_tiles = (Ce + 15) // 16
    for by, wave, j, lane in itertools.product(range(grid_y), range(NW), range(ct2), range(WAVE)):
        l16, kq = lane & 15, lane >> 4
        tile = (by * NW + wave) * ct2 + j
        if tile >= ce_tiles:       # surplus tiles shadow the last one and store nothing
            continue
        co = tile * 16 + kq * 4
        if co >= Ce or not (bo >> l16) & 1:
            continue
        pix = pbase + l16
        assert pix < P, "a set bit belongs to a pixel of the map"
        hits[pix, co:co + 4] += 1
    return hits


def _staged_stores(P, Ce, pbase, bo, grid_y, ct2):
    """The same for the staged epilogue: rows of NW * ct2 * 16 channels per workgroup, 16-byte pieces."""
    hits = np.zeros((2, P, Ce), dtype=np.int32)
    per_row = NW * ct2 * 2
    for by in range(grid_y):
        c0 = by * NW * ct2 * 16
        for tid in range(NW * WAVE):
            for c in range(tid, 2 * 16 * per_row, NW * WAVE):
                which, rr = divmod(c, 16 * per_row)
                r, cc = divmod(rr, per_row)
                ch = c0 + cc * 8
                if ch >= Ce or not (bo >> r) & 1:
                    continue
                assert pbase + r < P
                hits[which, pbase + r, ch:ch + 8] += 1
    return hits


@pytest.mark.parametrize("P,Ce", [(196, 384), (196, 576), (49, 960), (200, 192), (16, 64), (17, 96), (1, 32)])
@pytest.mark.parametrize("density", [0.05, 0.5, 1.0])
def test_open_activation_store_maps_cover_every_updated_element_once(P, Ce, density):
    rng = np.random.default_rng(P * 1000 + Ce)
    ct2 = 1
    ce_tiles = (Ce + 15) // 16
    grid_y = (ce_tiles + NW * ct2 - 1) // (NW * ct2)
    want = np.zeros((P, Ce), dtype=np.int32)
    lane_hits = np.zeros((P, Ce), dtype=np.int32)
    staged_hits = np.zeros((2, P, Ce), dtype=np.int32)
    for pbase in range(0, P, 16):
        bo = _tile_mask(P, pbase, rng, density)
        if pbase + 16 > P:  # the ragged tile: make sure its pixels take part
            bo |= 1 << ((P - 1) - pbase)
        for r in range(16):
            if (bo >> r) & 1:
                want[pbase + r, :] = 1
        lane_hits += _per_lane_stores(P, Ce, pbase, bo, grid_y, ct2)
        staged_hits += _staged_stores(P, Ce, pbase, bo, grid_y, ct2)
    assert np.array_equal(lane_hits, want)
    assert np.array_equal(staged_hits[0], want) and np.array_equal(staged_hits[1], want)


def test_ragged_tile_of_the_recorded_failure():
    """The one recorded loss (196 pixels, 384 channels, pixel 194 = slot 2 of the last tile, channel
    tile 14, quarters 1..3): both maps address those twelve elements exactly once."""
    P, Ce, pbase = 196, 384, 192
    bo = 0b0100
    lane = _per_lane_stores(P, Ce, pbase, bo, 3, 1)
    staged = _staged_stores(P, Ce, pbase, bo, 3, 1)
    assert lane[194].tolist() == [1] * Ce and staged[0, 194].tolist() == [1] * Ce
    assert lane.sum() == Ce and staged.sum() == 2 * Ce
    assert lane[194, 14 * 16 + 4:14 * 16 + 16].tolist() == [1] * 12
