"""How the tile attention kernel's launch is chosen (no GPU needed): the choices that were measured, and what every
choice must satisfy for the kernel to be right."""
import random

from inferflux_amd.kernels.attention import TILE_MAX_SPLITS, choose_tiling

ROWS_OF = lambda qt: 64 * qt          # head size 128


def test_the_measured_cases_get_the_choice_that_was_fastest():
    cases = [  # rows of the portion, keys it sees, query heads -> (query tiles per wave, key splits)
        ([512], 1024, 28, (1, 1)),      # 34 us whole against 40 in two splits
        ([512], 1024, 16, (1, 4)),      # half as many workgroups: 29 us in four splits against 33
        ([512], 2048, 28, (2, 4)),
        ([256], 4096, 28, (2, 8)),
        ([1024], 4096, 28, (2, 2)),
        ([1024], 8192, 28, (2, 2)),
        ([512], 8192, 28, (2, 4)),
        ([2048], 4096, 28, (2, 1)),     # 185 us against 236 with one tile per wave
        ([2048], 8192, 28, (2, 1)),
        ([8192], 8192, 28, (2, 1)),
        ([2048], 2048, 40, (2, 1)),
        ([130], 130, 28, (1, 1)),
        ([100] * 16, 100, 28, (1, 1)),
    ]
    for rows, longest, heads, want in cases:
        qt, splits, chunk = choose_tiling(rows, longest, heads, ROWS_OF)
        assert (qt, splits) == want, (rows, longest, heads, qt, splits, chunk)


def test_a_short_portion_does_not_take_half_empty_tall_tiles():
    qt, splits, chunk = choose_tiling([64], 8256, 28, ROWS_OF)
    assert qt == 1 and splits > 8


def test_every_choice_covers_its_keys_in_splits_the_kernel_takes():
    rng = random.Random(5)
    for _ in range(3000):
        rows = [rng.randint(16, rng.choice([40, 300, 3000])) for _ in range(rng.randint(1, 6))]
        longest = max(rows) + rng.choice([0, rng.randint(0, 500), rng.randint(0, 40000)])
        heads = rng.choice([1, 2, 5, 16, 28, 40, 64])
        qt, splits, chunk = choose_tiling(rows, longest, heads, ROWS_OF)
        assert qt in (1, 2) and 1 <= splits <= TILE_MAX_SPLITS
        if splits > 1:
            assert chunk % 64 == 0 and splits * chunk >= longest > (splits - 1) * chunk
        else:
            assert chunk == 0
