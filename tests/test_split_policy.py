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
    # every slice is read again by the norm behind the product: K = 1,024 is not cut into eight slices of
    # four chunks where four of eight do nearly as well (a step of 17 rows at width 1,024 was 2 % slower)
    assert split_count(17, 1024, 1024) == 4


def test_a_folded_norm_is_worth_it_by_rows_and_width():
    """Up to eight rows at every width the kernel takes; nine to sixteen rows only where a wave's two
    rows are short (measured at widths 768, 1,024 and 1,600)."""
    from burn_transformers_amd.kernels.library import Normalized
    assert all(Normalized.worth_it(8, width) for width in (768, 1024, 1600, 2048))
    assert Normalized.worth_it(16, 768) and Normalized.worth_it(9, 1024) and Normalized.worth_it(16, 1024)
    assert not Normalized.worth_it(9, 1600) and not Normalized.worth_it(16, 1280)
    assert not Normalized.worth_it(17, 768) and not Normalized.worth_it(4, 4096) and not Normalized.worth_it(4, 772)


# --- the runs a decode step's keys are cut into, and the classes of context ---------------------

def _runs(monkeypatch, n_seqs, context_limit, kv_heads=25, head_dim=64, bf16=True, window=0, decode=True, units=256):
    from types import SimpleNamespace
    from burn_transformers_amd.parts import attention
    monkeypatch.setattr(attention, "compute_units", lambda device: units)
    mixer = SimpleNamespace(kv_heads=kv_heads, head_dim=head_dim, window=window)
    step = SimpleNamespace(decode=decode, context_limit=context_limit, dtype_is_bf16=bf16, n_seqs=n_seqs)
    return attention.CausalSelfAttention.decode_runs(mixer, step, "cuda:0")


def _prompt_runs(monkeypatch, capacity, n_seqs, context_limit, heads=25, head_dim=64, bf16=True, window=0, units=256):
    from types import SimpleNamespace
    from burn_transformers_amd.parts import attention
    monkeypatch.setattr(attention, "compute_units", lambda device: units)
    mixer = SimpleNamespace(heads=heads, head_dim=head_dim, window=window, plain_only=False)
    step = SimpleNamespace(decode=False, context_limit=context_limit, dtype_is_bf16=bf16, n_seqs=n_seqs,
                           token_capacity=capacity)
    return attention.CausalSelfAttention.prompt_runs(mixer, step, "cuda:0")


def test_prompt_runs_for_chunks_behind_long_contexts(monkeypatch):
    """A chunk of a prompt has few tiles of 128 queries: their keys are cut into runs until the
    work-groups fill the chip, each run at least 8 blocks of keys per 256 tokens of the step, none
    while the class of context is 1,024 tokens or less, and only where the kernel that takes runs
    is the one that runs (bfloat16, heads of 64, no window)."""
    assert _prompt_runs(monkeypatch, 256, 1, 1024) == 1
    assert _prompt_runs(monkeypatch, 256, 1, 2048) == 4            # 32 blocks in runs of 8
    assert _prompt_runs(monkeypatch, 256, 1, 4096) == 5            # 2 tiles x 25 heads x 5 = 250 work-groups
    assert _prompt_runs(monkeypatch, 256, 1, 8192) == 5
    assert _prompt_runs(monkeypatch, 128, 1, 8192) == 8            # never more than eight
    assert _prompt_runs(monkeypatch, 512, 2, 2048) == 2            # 5 tiles x 25 heads: two runs fit the chip, 16 blocks each
    assert _prompt_runs(monkeypatch, 512, 2, 4096) == 2
    assert _prompt_runs(monkeypatch, 1024, 1, 2048) == 1           # 8 blocks per 256 tokens: 32 a run here
    assert _prompt_runs(monkeypatch, 2048, 1, 8192) == 1           # 16 tiles x 25 heads fill the chip already
    assert _prompt_runs(monkeypatch, 256, 1, 8192, bf16=False) == 1
    assert _prompt_runs(monkeypatch, 256, 1, 8192, head_dim=32) == 1
    assert _prompt_runs(monkeypatch, 256, 1, 8192, window=512) == 1
    assert _prompt_runs(monkeypatch, 256, 1, 8192, heads=4) == 8   # few heads: the runs are what fills the chip


def test_decode_runs_at_measured_sizes(monkeypatch):
    # 25 heads of 64: bfloat16 is not cut at 1,024 keys, and best with 4 / 8 runs at 2,048 / 4,096
    assert _runs(monkeypatch, 1, 1024) == 1
    assert _runs(monkeypatch, 1, 2048) == 4
    assert _runs(monkeypatch, 1, 4096) == 8
    assert _runs(monkeypatch, 1, 8192) == 10           # no more work-groups than compute units
    assert _runs(monkeypatch, 4, 8192) == 2
    assert _runs(monkeypatch, 8, 8192) == 1            # 200 pairs of sequence and head fill the chip
    assert _runs(monkeypatch, 64, 8192) == 1
    # float32 holds twice the bytes per key
    assert _runs(monkeypatch, 1, 1024, bf16=False) == 4
    assert _runs(monkeypatch, 8, 1024, bf16=False) == 1
    # a window bounds the keys a query reads; steps with prompt tokens are never cut
    assert _runs(monkeypatch, 1, 8192, window=512) == 1
    assert _runs(monkeypatch, 1, 8192, decode=False) == 1


def test_context_classes():
    from burn_transformers_amd.engine.step import StepPlan, context_limit
    assert [context_limit(n) for n in (1, 1024, 1025, 2048, 2049, 5000)] == [1024, 1024, 2048, 2048, 4096, 8192]
    plan = StepPlan([0, 1], [10, 3000], [1, 1], [5, 6], [0, 1], [[[0], list(range(47))]], 128)
    assert plan.context_limit == 4096 and plan.decode
    # never more than a sequence can hold (3 blocks of 64 tokens here)
    assert StepPlan([0], [100], [1], [5], [0], [[[0, 1]]], 3).context_limit == 192


def test_whether_a_graph_pays_is_decided_by_the_median_of_the_measured_steps():
    """``engine.launch_bound``: the GPU is the limit (no graph) when its time for a step stands
    clearly above the host's time for walking the step's launch list; one odd sample of three
    changes nothing."""
    from burn_transformers_amd.engine.engine import launch_bound
    host_bound = (1.00e-3, 0.98e-3)       # the GPU waited for every launch: both times about equal
    gpu_bound = (1.70e-3, 1.30e-3)        # the kernels outlast their launches
    assert launch_bound([gpu_bound] * 3) is True
    assert launch_bound([host_bound] * 3) is False
    assert launch_bound([gpu_bound, host_bound, gpu_bound]) is True
    assert launch_bound([host_bound, (9e-3, 1e-3), host_bound]) is False      # a first use, a clock still rising
    assert launch_bound([gpu_bound, (1e-3, 9e-3), gpu_bound]) is True         # the host was interrupted once
    assert launch_bound([(1.05e-3, 1e-3)]) is False and launch_bound([(1.2e-3, 1e-3)]) is True
    assert launch_bound([(1e-3, 0.0)]) is True                                # never a division by zero


def test_products_of_short_prompts_and_how_they_cut_k():
    """``deep_form_rows`` / ``deep_split_count``: 65 to 256 rows with K a multiple of 64 go to the
    tile kernel's deep forms, up to 512 where slices of K may stay pending and up to 384 where keys and
    values are scattered into the cache (the vendor's library would need a copy behind it); a residual-writing one
    cuts K so that every work-group has a compute unit, or at most two share one, into at most four
    slices of at least four tiles of K."""
    from burn_transformers_amd.kernels.library import deep_form_rows, deep_split_count
    assert not deep_form_rows(64, 1600, 1600, 4800) and deep_form_rows(65, 1600, 1600, 4800)
    assert deep_form_rows(256, 1600, 1600, 4800) and not deep_form_rows(257, 1600, 1600, 4800)
    assert deep_form_rows(512, 1600, 1600, 1600, sliced=True) and not deep_form_rows(513, 1600, 1600, 1600, sliced=True)
    assert deep_form_rows(384, 1600, 1600, 4800, scatters=True) and not deep_form_rows(385, 1600, 1600, 4800, scatters=True)
    assert not deep_form_rows(128, 1608, 1608, 4800)            # K in tiles of 64
    assert not deep_form_rows(128, 64, 1 << 25, 64)             # operands addressed with 32 bits
    assert deep_split_count(128, 1600, 1600) == 4 and deep_split_count(128, 1600, 6400) == 4
    assert deep_split_count(192, 1600, 1600) == 3 and deep_split_count(192, 1600, 6400) == 3
    assert deep_split_count(256, 1600, 1600) == 2 and deep_split_count(256, 1600, 6400) == 2
    assert deep_split_count(384, 1600, 6400) == 3 and deep_split_count(512, 1600, 6400) == 2     # two work-groups a unit
    assert deep_split_count(128, 768, 768) == 3                 # 12 tiles of K: three slices of four
    assert deep_split_count(100, 64, 64) == 1 and deep_split_count(100, 64, 256) == 1   # K too short to cut
    assert deep_split_count(512, 6400, 1600) == 1               # tiles enough without a cut
    assert deep_split_count(64, 1600, 1600) == 1 and deep_split_count(513, 1600, 1600) == 1
    for rows in (65, 100, 128, 200, 256, 300, 512):
        for columns in (64, 768, 1024, 1600, 50257):
            for k in (64, 128, 768, 1024, 1600, 6400):
                splits = deep_split_count(rows, columns, k)
                assert 1 <= splits <= 4 and (splits == 1 or (k // 64) // splits >= 4)
