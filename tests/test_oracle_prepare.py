"""The checker's forward map of the prepared (gfx950 operand order) image: hand-worked coordinates
of every region, bijection, one rank and four."""
import numpy as np
import pytest

import b1_oracle as O

IMAGE = 3342336
GATE, GATE_S, UP, UP_S, DOWN, DOWN_S = 0, 1048576, 1114112, 2162688, 2228224, 3276800


def images(n, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, 256, IMAGE, dtype=np.uint8) for _ in range(n)]


def test_hand_worked_coordinates_one_rank():
    img = images(1, 3)
    p = O.prepared_g950(img)
    assert p.size == IMAGE  # a permutation of the canonical image
    i = img[0]
    # cell = (((set of eight blocks * k-steps + k-step) * 8 + place in the set) * 4 + tile) * 64 + lane
    # up row 37, k-block 9 (k 288..319): column block 1 = set 0 place 1, k-step 2, tile 0 + 2, lane 16 * 1 + 5
    cell = (((0 * 32 + 2) * 8 + 1) * 4 + 2) * 64 + 21
    assert np.array_equal(p[cell * 16:cell * 16 + 16], i[UP + 37 * 2048 + 9 * 16:UP + 37 * 2048 + 10 * 16])
    # gate row 500, k-block 127: column block 15 = set 1 place 7, k-step 31, tile 1, lane 16 * 3 + 4
    cell = (((1 * 32 + 31) * 8 + 7) * 4 + 1) * 64 + 52
    assert np.array_equal(p[cell * 16:cell * 16 + 16], i[GATE + 500 * 2048 + 127 * 16:GATE + 500 * 2048 + 128 * 16])
    # gate row 500, scale of k-block 127: k-step 31 = quad 7 byte 3
    s13 = 512 * 4096
    assert p[s13 + (((15 * 8 + 7) * 4 + 1) * 64 + 52) * 4 + 3] == i[GATE_S + 500 * 128 + 127]
    # up row 0, scale of k-block 6: k-step 1 = quad 0 byte 1, lane 16 * 2
    assert p[s13 + ((0 * 4 + 2) * 64 + 32) * 4 + 1] == i[UP_S + 6]
    # down row 4095, k-block 13 (of 16): output block 63 = set 7 place 7, k-step 3 (of 4), tile 3, lane 16 * 1 + 15
    w2 = s13 + 512 * 256
    cell = (((7 * 4 + 3) * 8 + 7) * 4 + 3) * 64 + 31
    assert np.array_equal(p[w2 + cell * 16:w2 + cell * 16 + 16], i[DOWN + 4095 * 256 + 13 * 16:DOWN + 4095 * 256 + 14 * 16])
    # down row 70, scale of k-block 5: output block 1, the only quad, tile 0, lane 16 * 1 + 6, byte 1
    s2 = w2 + 512 * 2048
    assert p[s2 + ((1 * 4 + 0) * 64 + 22) * 4 + 1] == i[DOWN_S + 70 * 16 + 5]


def test_hand_worked_coordinates_four_ranks():
    img = images(4, 4)
    p = O.prepared_g950(img)
    assert p.size == 4 * IMAGE
    # gate column 1300 = rank 2 row 276, k-block 40: column block 40 = set 5 place 0, k-step 10, tile 1, lane 4
    cell = (((5 * 32 + 10) * 8 + 0) * 4 + 1) * 64 + 4
    assert np.array_equal(p[cell * 16:cell * 16 + 16], img[2][GATE + 276 * 2048 + 40 * 16:GATE + 276 * 2048 + 41 * 16])
    # down row 129, K block 3 * 16 + 7 = 55 (rank 3's block 7): output block 2 = set 0 place 2, k-step 13 of 16, tile 0, lane 16 * 3 + 1
    s13 = 2048 * 4096
    w2 = s13 + 2048 * 256
    cell = (((0 * 16 + 13) * 8 + 2) * 4 + 0) * 64 + 49
    assert np.array_equal(p[w2 + cell * 16:w2 + cell * 16 + 16], img[3][DOWN + 129 * 256 + 7 * 16:DOWN + 129 * 256 + 8 * 16])
    # its scale: k-step 13 = quad 3 byte 1
    s2 = w2 + 2048 * 2048
    assert p[s2 + (((2 * 4 + 3) * 4 + 0) * 64 + 49) * 4 + 1] == img[3][DOWN_S + 129 * 16 + 7]


@pytest.mark.parametrize("ranks", [1, 4])
def test_bijection_keeps_every_byte(ranks):
    img = images(ranks, 5 + ranks)
    p = O.prepared_g950(img)  # raises when a destination is hit twice or never
    assert np.array_equal(np.bincount(p, minlength=256), sum(np.bincount(i, minlength=256) for i in img))
