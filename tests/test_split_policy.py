"""The policy that splits the K range of residual-writing products (no GPU needed)."""

from burn_transformers_amd.parts.base import split_count


def slices(k, splits):
    chunks = (k + 31) // 32
    per = (chunks + splits - 1) // splits
    return [min(per, max(0, chunks - i * per)) for i in range(splits)]


def test_many_rows_never_split():
    assert split_count(65, 1600, 6400) == 1
    assert split_count(2048, 1600, 1600) == 1


def test_every_slice_has_work_and_is_not_thin():
    for rows in (1, 8, 16, 17, 64):
        for columns in (16, 64, 96, 517, 1600, 50257):
            for k in (8, 64, 96, 320, 1600, 1608, 6400, 20480):
                for units in (64, 256, 304):
                    splits = split_count(rows, columns, k, units)
                    assert 1 <= splits <= 8
                    parts = slices(k, splits)
                    assert all(p > 0 for p in parts), (rows, columns, k, units, parts)
                    if splits > 1:
                        assert parts[0] >= 4


def test_choices_at_measured_sizes():
    # 100 tiles of 16 columns on 256 compute units: measured best are 2 splits for K 1600, 5 for K 6400
    assert split_count(8, 1600, 1600) == 2
    assert split_count(8, 1600, 6400) == 5
    # wide outputs fill the compute units on their own
    assert split_count(8, 50257, 1600) == 1
    # beyond 16 rows a work-group owns 32 columns, so there are half as many tiles to spread
    assert split_count(64, 1600, 6400) >= split_count(8, 1600, 6400)
