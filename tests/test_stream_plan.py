"""The host-side plan of the weight-streaming product: which arrangement of a block's waves, how many runs of k and
how many blocks along the columns a product gets. No GPU is touched."""

import random

from mini_engine_amd.ops.kernels import stream_plan, stream_splits


def check(rows, n, k, gated, splits, units):
    tiles_per_block, runs, grid = stream_plan(rows, n, k, gated, splits, units=units)
    assert tiles_per_block in (1, 2, 4, 8) and runs == splits and grid >= 1
    assert grid >= -(-n // (16 * tiles_per_block))  # every column has a block
    assert -(-(-(-n // 4)) // grid) * 4 <= 16 * tiles_per_block  # no block has more columns than its waves take
    assert grid <= max(-(-n // (16 * tiles_per_block)) * 4 // 3, 1) + 1  # at most a third more blocks than tiles need
    return tiles_per_block, runs, grid


def test_random_products_on_any_number_of_compute_units():
    rng = random.Random(1)
    for _ in range(3000):
        rows = rng.choice([1, 2, 8, 16, 17, 32, 33, 64, 65, 128, 256])
        n = rng.choice([4, 16, 40, 100, 1000, 1024, 3072, 4096, 5003, 5120, 12288, 25600, 151936, rng.randint(1, 30000)])
        k = 8 * rng.randint(1, 4000)
        units = rng.choice([1, 8, 64, 104, 228, 256, 304])
        gated = rng.random() < 0.3
        splits = 1
        if not gated and rng.random() < 0.6:
            splits = stream_splits(n, k, rows=rows, units=units)
            steps = -(-k // 128)
            assert 1 <= splits <= 16 and -(-steps // -(-steps // splits)) == splits  # whole steps, no empty run
            assert splits == 1 or steps // splits >= 3  # runs of about four steps and more
        check(rows, n, k, gated, splits, units)


def test_the_measured_shapes_get_what_was_measured_best():
    """256 compute units; (rows, columns, k) of the layer shapes the rules were measured on."""
    assert check(1, 6144, 4096, False, 1, 256) == (2, 1, 256)        # 384 tiles of 16 columns on 256 blocks of 24
    assert check(1, 25600, 5120, True, 1, 256) == (4, 1, 512)        # 400 blocks' worth of columns on 512 blocks of 50
    assert check(8, 12288, 4096, True, 1, 256) == (2, 1, 512)
    assert stream_splits(4096, 12288, units=256) == 4 and check(1, 4096, 12288, False, 4, 256) == (4, 4, 64)
    assert stream_splits(5120, 25600, units=256) == 3 and check(16, 5120, 25600, False, 3, 256) == (4, 3, 85)
    assert stream_splits(1024, 3072, units=256) == 6 and check(8, 1024, 3072, False, 6, 256) == (2, 6, 42)
    assert stream_splits(5120, 25600, rows=64, units=256) == 6 and check(64, 5120, 25600, False, 6, 256) == (8, 6, 42)
    assert check(64, 10240, 5120, False, 1, 256) == (4, 1, 160)      # many rows: wide blocks before whole rounds
    assert check(100, 3072, 1024, True, 1, 256) == (2, 1, 128)       # two groups of 64 rows: 256 blocks
    assert check(130, 3072, 1024, True, 1, 256) == (4, 1, 48)        # three groups: wider blocks give enough
