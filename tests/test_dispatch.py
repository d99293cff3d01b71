"""Choices that the product dispatcher makes on the host (no GPU needed)."""
from spite_amd.parts.linear import grouped_tile_shape


def test_tile_shape_follows_the_expected_number_of_row_tiles():
    # 2048 tokens over 16 experts: groups of 128 +- 11 rows, half of them past one tile of 128
    assert grouped_tile_shape(2048, 16, 1) == 3
    # groups of about 64 rows fit one tile of either kind: the cheaper tile
    assert grouped_tile_shape(1024, 16, 1) == 1
    # a short prompt: a few rows a group, the small tile that streams the weights faster
    assert grouped_tile_shape(256, 16, 1) == 4 and grouped_tile_shape(96, 16, 1) == 4
    # ... unless the group that takes every row would need many of the small tiles
    assert grouped_tile_shape(512, 16, 1) == 1
    # many near-empty groups
    assert grouped_tile_shape(2048, 128, 1) == 1
    # groups of about 200 rows need two tiles of either kind
    assert grouped_tile_shape(3200, 16, 1) == 1
    # nothing to spread
    assert grouped_tile_shape(0, 16, 1) == 1 and grouped_tile_shape(100, 0) == 1
