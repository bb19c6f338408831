"""Pins of oracle/shuffle.py. The oracle follows the reference's index arithmetic; here the same
layouts are stated a second, independent way, as a reshape into tile coordinates followed by an
axis permutation (the form AITER publishes: ``shuffle_weight(x, (16, 16))`` =
``x.view(-1, N/16, 16, K/32, 2, 16).permute(0, 1, 3, 4, 2, 5)`` and ``e8m0_shuffle`` =
``s.view(M/32, 2, 16, N/8, 2, 4).permute(0, 3, 5, 2, 4, 1)``), plus offsets worked out by hand and
the bijection property. A swapped pair of axes or a wrong stride fails each of them."""

import numpy as np
import pytest

from oracle import shuffle as S


@pytest.mark.parametrize("rows,row_bytes", [(16, 32), (32, 64), (48, 160), (256, 512)])
def test_codes_match_axis_permutation(rows, row_bytes):
    x = np.random.default_rng(rows + row_bytes).integers(0, 256, (rows, row_bytes), dtype=np.uint8)
    want = x.reshape(rows // 16, 16, row_bytes // 32, 2, 16).transpose(0, 2, 3, 1, 4).reshape(rows, row_bytes)
    got = S.shuffle_codes(x)
    assert np.array_equal(got, want)
    assert np.array_equal(S.unshuffle_codes(got), x)


def test_codes_hand_offsets():
    off = S.shuffled_code_offsets(32, 64)
    assert off[0, 0] == 0 and off[0, 15] == 15
    assert off[1, 0] == 16            # next row of the same half-tile: 16 bytes on
    assert off[0, 16] == 256          # second half of the 32-byte block: after 16 rows x 16 bytes
    assert off[0, 32] == 512          # next 32-byte block of the band
    assert off[16, 0] == 16 * 64      # next band of 16 rows
    assert off[17, 40] == 1024 + 512 + 16 + 8
    assert sorted(off.ravel().tolist()) == list(range(32 * 64))


@pytest.mark.parametrize("M,N", [(32, 8), (64, 16), (256, 8), (100, 5), (300, 12), (1, 1)])
def test_scale_matches_axis_permutation(M, N):
    s = np.random.default_rng(M * 31 + N).integers(1, 256, (M, N), dtype=np.uint8)
    Mp, Np = S.scale_pad_shape(M, N)
    assert Mp % 256 == 0 and Np % 8 == 0 and 0 <= Mp - M < 256 and 0 <= Np - N < 8
    padded = np.zeros((Mp, Np), dtype=np.uint8)
    padded[:M, :N] = s
    want = padded.reshape(Mp // 32, 2, 16, Np // 8, 2, 4).transpose(0, 3, 5, 2, 4, 1).reshape(Mp, Np)
    got = S.shuffle_scale(s)
    assert got.shape == (Mp, Np) and np.array_equal(got, want)
    assert np.array_equal(S.unshuffle_scale(got, M, N), s)


def test_scale_hand_offsets():
    off = S.shuffled_scale_offsets(64, 16, 16)
    assert off[0, 0] == 0
    assert off[16, 0] == 1            # the row 16 further down is the neighbouring byte
    assert off[0, 4] == 2             # then the column 4 further right
    assert off[1, 0] == 4             # the next row starts the next 4-byte word
    assert off[0, 1] == 64            # the next column: after 16 rows x 4 bytes
    assert off[0, 8] == 256           # next 32 x 8 tile to the right
    assert off[32, 0] == 2 * 256      # next band of 32 rows: N_pad / 8 = 2 tiles further
    assert off[50, 13] == 1 * 512 + 1 * 256 + 1 * 64 + 2 * 4 + 1 * 2 + 1
    assert sorted(off.ravel().tolist()) == list(range(64 * 16))
