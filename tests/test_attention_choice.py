"""How the tile attention kernel's launch is chosen (no GPU needed): the choices that were measured, and what every
choice must satisfy for the kernel to be right."""
import random

import numpy as np

from inferflux_amd.kernels.attention import TILE_MAX_SPLITS, choose_tiling, tile_order

ROWS_OF = lambda qt: 64 * qt          # head size 128


def test_head_size_128_gets_the_choices_that_were_fastest():
    """Tiles of 64 rows / of 128 rows (the kernel that loads straight into LDS), in us, each with its best splits."""
    cases = [  # rows of the portion, keys it sees, query heads -> (tiling, key splits)
        ([512], 512, 28, (1, 1)),        # 20 / 24
        ([1024], 1024, 28, (2, 1)),      # 37 / 30
        ([2048], 2048, 28, (2, 1)),      # 77 / 58
        ([8192], 8192, 28, (2, 1)),      # 865 / 533
        ([512], 1024, 28, (2, 1)),       # 34 / 27
        ([512], 2048, 28, (2, 1)),       # 62 / 47 (55 in four splits)
        ([512], 2048, 16, (2, 4)),       # 47 / 41 in four splits (47 whole)
        ([512], 4096, 28, (2, 4)),       # 96 / 69 (85 whole)
        ([256], 4096, 28, (2, 8)),       # 59 / 45 (84 whole)
        ([1024], 4096, 28, (2, 1)),      # 141 / 93 (117 in two splits)
        ([1024], 8192, 28, (2, 1)),      # 258 / 176 (174 in four splits)
        ([512], 8192, 28, (2, 4)),       # 151 / 99 (164 whole)
        ([128], 4096, 28, (2, 8)),       # 41 / 34 (83 whole)
        ([128], 8192, 28, (2, 16)),      # 56 / 40
        ([2048], 8192, 28, (2, 1)),      # 436 / 226
        ([2048], 4096, 16, (2, 1)),      # 131 / 93
        ([2048], 8192, 40, (2, 1)),      # 586 / 372
        ([130], 130, 28, (1, 1)),
        ([70] * 16, 70, 28, (1, 1)),     # sixteen short prompts: tall tiles would be half empty
    ]
    for rows, longest, heads, want in cases:
        qt, splits, chunk = choose_tiling(rows, [longest] * len(rows), heads, ROWS_OF, tall_direct=True)
        assert (qt, splits) == want, (rows, longest, heads, qt, splits, chunk)
    qt, splits, _ = choose_tiling([64], [4096], 28, ROWS_OF, tall_direct=True)        # a half-empty tall tile: 26 us, this 30
    assert qt == 1 and splits >= 8


def test_other_head_sizes_get_the_choices_measured_with_two_query_tiles_per_wave():
    cases = [  # rows of the portion, keys it sees, query heads -> (query tiles per wave, key splits)
        ([512], 1024, 28, (1, 1)),      # 34 us whole against 40 in two splits
        ([512], 1024, 16, (1, 4)),      # half as many workgroups: 29 us in four splits against 33
        ([512], 2048, 28, (2, 4)),
        ([256], 4096, 28, (2, 8)),
        ([1024], 4096, 28, (2, 2)),
        ([1024], 8192, 28, (2, 2)),
        ([512], 8192, 28, (2, 4)),
        ([2048], 2048, 28, (1, 1)),     # a short causal prompt: 75 us against 81 with two tiles per wave
        ([2048], 2048, 16, (1, 1)),
        ([4096], 4096, 28, (2, 1)),
        ([2048], 4096, 28, (2, 1)),     # 158 us against 218 with one tile per wave
        ([2048], 8192, 28, (2, 1)),
        ([8192], 8192, 28, (2, 1)),
        ([2048], 2048, 40, (2, 1)),
        ([130], 130, 28, (1, 1)),
        ([100] * 16, 100, 28, (1, 1)),
    ]
    for rows, longest, heads, want in cases:
        qt, splits, chunk = choose_tiling(rows, [longest] * len(rows), heads, ROWS_OF)
        assert (qt, splits) == want, (rows, longest, heads, qt, splits, chunk)


def test_a_short_portion_does_not_take_half_empty_tall_tiles():
    qt, splits, chunk = choose_tiling([64], [8256], 28, ROWS_OF)
    assert qt == 1 and splits > 8


def test_every_choice_covers_its_keys_in_splits_the_kernel_takes():
    rng = random.Random(5)
    for _ in range(3000):
        rows = [rng.randint(16, rng.choice([40, 300, 3000])) for _ in range(rng.randint(1, 6))]
        longest = max(rows) + rng.choice([0, rng.randint(0, 500), rng.randint(0, 40000)])
        heads = rng.choice([1, 2, 5, 16, 28, 40, 64])
        qt, splits, chunk = choose_tiling(rows, [r + rng.randint(0, longest - r) for r in rows[:-1]] + [longest], heads, ROWS_OF,
                                          tall_direct=rng.random() < 0.5)
        assert qt in (1, 2) and 1 <= splits <= TILE_MAX_SPLITS
        if splits > 1:
            assert chunk % 64 == 0 and splits * chunk >= longest > (splits - 1) * chunk
        else:
            assert chunk == 0


def _walks(first, last, window, splits, chunk):
    """Key tiles each (tile, split) walks, written out from the kernel's loop bounds."""
    out = []
    for f, l in zip(first, last):
        row = []
        for s in range(splits):
            lo = max(f - window + 1, 0) if window else 0
            hi = l
            if splits > 1:
                lo, hi = max(lo, s * chunk), min(hi, (s + 1) * chunk - 1)
            j0, n = lo // 64 * 64, 0
            while j0 <= hi:
                n, j0 = n + 1, j0 + 64
            row.append(n)
        out.append(row)
    return out


def test_the_order_names_every_work_item_once_and_balances_the_units():
    rng = random.Random(9)
    for trial in range(200):
        n_tiles, heads = rng.randint(1, 40), rng.choice([1, 4, 16, 28])
        rows = rng.choice([64, 128])
        start = rng.randint(0, 3000)
        first = [start + rows * t for t in range(n_tiles)]
        last = [f + rng.randint(1, rows) - 1 for f in first]
        window = rng.choice([None, None, 100, 1000])
        splits = rng.choice([1, 1, 2, 5])
        chunk = -(-(last[-1] + 1) // splits + 63) // 64 * 64 if splits > 1 else 0
        period = rng.choice([2, 3, 32])
        order = tile_order(first, last, heads, window, splits, chunk, period)
        n_items = n_tiles * heads * splits
        assert order.dtype == np.int32 and order.shape[0] % 8 == 0 and order.shape[0] // 8 <= n_items
        assert sorted(order[order >= 0].tolist()) == list(range(n_items))
        assert set(order[order < 0].tolist()) <= {-1}
    # a causal prompt of 2,048 rows in tiles of 64, 28 heads: the compute units' first three workgroups (unit = place
    # modulo 32 within an XCD) walk 50-61 key tiles together on every unit, where longest first head by head gave 3 to 96
    first = [64 * t for t in range(32)]
    last = [f + 63 for f in first]
    order = tile_order(first, last, 28, None, 1, 0).reshape(8, -1)
    walks = _walks(first, last, None, 1, 0)
    sums = []
    for x in range(8):
        unit = [0] * 32
        for i, w in enumerate(order[x][:96]):
            if w >= 0:
                unit[i % 32] += walks[31 - w % 32][0]
        sums += unit
        # an XCD's workgroups read the keys of few kv heads (7 query heads each)
        assert len({int(w) // 32 // 7 for w in order[x] if w >= 0}) <= 2
    assert min(sums) >= 48 and max(sums) <= 62, (min(sums), max(sums))


def test_library_products_are_cut_only_where_slices_fill_the_chip_and_stay_long():
    from inferflux_amd.kernels.ops import library_k_slices as f
    assert [f(M, 3584, 18944) for M in (129, 512, 1024, 2048, 4096)] == [8, 8, 4, 2, 1]     # down of the 7B shape
    assert all(f(M, 3584, 3584) == 1 and f(M, 4608, 3584) == 1 for M in (129, 512, 2048))  # o, q/k/v: K too short to cut
    assert f(512, 37888, 3584) == 1 and f(512, 152064, 3584) == 1                           # tall weights fill the chip as they are
    assert f(512, 2048, 11008) == 4 and f(512, 8192, 29568) == 4                            # down of the 3B and 72B shapes
    assert f(512, 3584, 18944 + 8) == 1                                                     # slices must be multiples of 8 k-values
    for M in (130, 777, 3000):
        for N in (64, 1000, 5120):
            for K in (2048, 4096, 10000, 65536):
                S = f(M, N, K)
                assert S in (1, 2, 4, 8) and K % S == 0 and (S == 1 or (K // S >= 2048 and (K // S) % 8 == 0))


def test_row_launch_shape():
    """Launches with (row, kv head) pairs enough to fill the chip take a pair whole in one workgroup, with about one
    round of 2,048 waves; fewer pairs are cut into splits that reach past the longest request."""
    from inferflux_amd.kernels.attention import ROW_MAX_SPLITS, row_launch_shape
    assert row_launch_shape(64, 4, 4096) == (0, 8, 1)
    assert row_launch_shape(48, 4, 4096) == (0, 8, 1)
    assert row_launch_shape(96, 4, 4096) == (0, 4, 1)
    assert row_launch_shape(128, 4, 4096) == (0, 4, 1)
    assert row_launch_shape(256, 4, 4096) == (0, 2, 1)
    assert row_launch_shape(600, 4, 4096) == (0, 1, 1)
    assert row_launch_shape(64, 4, 4096, max_waves=4) == (0, 4, 1)      # what the kernel's LDS allows at these head counts
    assert row_launch_shape(64, 2, 4096)[1] == 0                        # 128 pairs: splits
    assert row_launch_shape(1, 4, 4096) == (64, 0, 64) and row_launch_shape(1, 4, 32768) == (128, 0, 256)   # one request: many short splits
    assert row_launch_shape(16, 4, 4096) == (128, 0, 32) and row_launch_shape(32, 4, 4096) == (256, 0, 16)
    for rows, kv_heads, bound in [(1, 4, 4096), (8, 4, 4096), (32, 4, 4096), (1, 1, 131072), (8, 8, 32768), (47, 4, 1024)]:
        chunk, waves, splits = row_launch_shape(rows, kv_heads, bound)
        assert waves == 0 and chunk % 32 == 0 and chunk >= 64
        assert splits * chunk >= bound > (splits - 1) * chunk and splits <= ROW_MAX_SPLITS
