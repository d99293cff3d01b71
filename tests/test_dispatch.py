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


def test_tile_shape_by_the_rounds_its_tiles_make():
    # the eight products measured at 2,048 tokens on 256 compute units: (experts, column tiles) -> the faster tile
    for E, cols, want in ((16, 32, 3), (16, 10, 1), (8, 32, 3), (8, 8, 3), (8, 12, 1), (8, 56, 1)):
        assert grouped_tile_shape(2048, E, 1, col_tiles=cols, cus=256) == want, (E, cols)
    # a short prompt still takes the small tile, whatever the columns
    assert grouped_tile_shape(256, 16, 1, col_tiles=10, cus=256) == 4


def test_runs_of_a_split_product_are_never_empty():
    from spite_amd.csrc.hipops import tiled_k_runs
    for M in (65, 100, 256, 700, 2048):
        for N in (16, 512, 5120, 7168, 202048):
            for K in (64, 192, 320, 1024, 5120, 8192):
                runs, steps = tiled_k_runs(M, N, K), K // 64
                assert 1 <= runs <= 8
                if runs > 1:
                    per = -(-steps // runs)
                    assert per * (runs - 1) < steps and per >= 4 and -(-M // 128) * -(-N // 512) < 128


def test_the_benchmark_counts_what_a_query_can_see():
    import importlib.util
    import os
    from spite_amd.config import read_config
    spec = importlib.util.spec_from_file_location("bench", os.path.join(os.path.dirname(os.path.dirname(__file__)), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    # pairs of (query, key) of a portion, against a count by hand: layers that rotate read their chunk or window
    for kind in ("chunk", "window"):
        for T, past, span in ((5, 0, 64), (7, 9, 64), (6, 0, 4), (10, 13, 8), (3, 7, 8), (20, 30, 16)):
            cfg = dict(bench.TINY, num_hidden_layers=4, no_rope_layers=[1, 1, 0, 1], attention_chunk_size=span,
                       attention_local_kind=kind)
            sizes = bench.Sizes(read_config(cfg)[1], 2)
            first = (lambda p: (p // span) * span) if kind == "chunk" else (lambda p: max(p - span + 1, 0))
            local = sum(1 for p in range(past, past + T) for j in range(p + 1) if j >= first(p))
            full = sum(p + 1 for p in range(past, past + T))
            assert sizes.pairs(T, past) == 3 * local + full, (kind, T, past, span)
    sizes = bench.Sizes(read_config(dict(bench.SCOUT, no_rope_layers=None))[1], 2)
    # more context costs more bytes on every layer below a chunk, only on every fourth above it
    a, b = sizes.decode_bytes(8, 4096, 6.4), sizes.decode_bytes(8, 4097, 6.4)
    c, d = sizes.decode_bytes(8, 32768, 6.4), sizes.decode_bytes(8, 32769, 6.4)
    kv_token = 2 * 8 * 128 * 2
    assert b - a == 8 * 48 * kv_token and d - c == 8 * 48 * kv_token
    assert sizes.decode_bytes(8, 8192, 6.4) < sizes.decode_bytes(8, 8191, 6.4)   # a new chunk begins
    assert len(sizes.full_layers) == 12 and sizes.n_moe == 48
