"""Launch plans are plain functions of sizes; whatever they return must be something the kernels take."""

import numpy as np

from paged_llm_amd.csrc import ops


def test_attention_plan_always_returns_a_launch_the_kernels_take():
    rng = np.random.default_rng(7)
    lds = 160 * 1024
    for _ in range(3000):
        seqs = int(rng.choice([1, 2, 3, 7, 8, 16, 33, 64, 100, 256, 1000]))
        kv_heads = int(rng.choice([1, 2, 4, 8, 16]))
        group = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
        max_q = int(rng.choice([1, 1, 1, 2, 3, 8, 17, 64, 500]))
        max_k = max(max_q, int(rng.choice([1, 15, 64, 65, 200, 256, 1000, 2048, 2049, 8192, 100000])))
        d = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256]))
        waves, size, parts = ops.attention_plan(seqs, kv_heads, max_q, max_k, group, d, lds)
        what = f"plan({seqs}, {kv_heads}, {max_q}, {max_k}, {group}, {d}) = {(waves, size, parts)}"
        assert waves in (1, 4, 8), what
        assert size % 64 == 0 and size >= 0 and parts >= 1, what
        if size == 0:
            assert parts == 1, what
        else:
            assert parts > 1 and (parts - 1) * size < max_k <= parts * size, what     # the partitions cover the keys, none is empty
            assert kv_heads * parts <= 65535, what                                  # a grid dimension
        if max_q * group > 64:
            assert (waves, size, parts) == (1, 0, 1), what                          # prompt portions: the other kernel
        if waves > 1:
            ncb = 1 if max_q * group <= 16 else (2 if max_q * group <= 32 else 4)
            assert ops._merge_lds_bytes(ncb, waves, d) <= lds, what


def test_attention_plan_depends_on_sizes_only():
    a = ops.attention_plan(8, 4, 1, 2048, 8, 64, 160 * 1024)
    assert a == ops.attention_plan(8, 4, 1, 2048, 8, 64, 160 * 1024) == (4, 256, 8)


def test_graph_batch_sizes_cover_every_batch_with_at_most_half_as_many_rows_again():
    from paged_llm_amd.engine.runner import ModelRunner
    sizes = [ModelRunner._bucket(n) for n in range(1, 600)]
    assert all(b >= n and 2 * b <= 3 * n + 1 for n, b in zip(range(1, 600), sizes))      # never fewer rows, at most half again
    assert sizes == sorted(sizes)
    assert len(set(sizes)) <= 24                                                       # few graphs for a batch that shrinks one by one
    assert [ModelRunner._bucket(n) for n in (1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 64, 65)] == [1, 2, 3, 4, 6, 6, 8, 8, 12, 16, 64, 96]


def test_ranges_of_the_inner_dimension_are_never_empty():
    """The products' plans cut K into ranges of equal numbers of stages; whatever the sizes, no range is left empty
    (a matrix of 2048 x 5632 at 150 rows once asked for 16 ranges of 6 of its 88 stages)."""
    from paged_llm_amd.csrc import ops
    for rows in (17, 64, 100, 128, 129, 150, 160, 161, 264, 320, 400, 512, 640):
        for n, k in ((2048, 2048), (2048, 5632), (2560, 2048), (4096, 4096), (96, 992), (2048, 14336), (32, 32)):
            for cus in (256, 304, 64):
                ranges, stages = ops.tile_linear_plan(rows, n, k, cus), -(-k // 64)
                assert ranges == 1 or -(-stages // ranges) * (ranges - 1) < stages, (rows, n, k, ranges)
                _, ranges = ops.stream_linear_plan(rows, n, k, cus)
                stages = -(-k // 256)
                assert ranges == 1 or -(-stages // ranges) * (ranges - 1) < stages, (rows, n, k, ranges)


def test_streaming_product_plans_by_sizes():
    from paged_llm_amd.csrc import ops
    plan, cus = ops.stream_linear_plan, 256
    assert plan(64, 2048, 5632, cus) == (2, 4)                # 64 blocks of 32 weight rows x 4 ranges: a workgroup per compute unit
    assert plan(64, 2048, 2048, cus) == (2, 4) and plan(64, 2560, 2048, cus) == (2, 3)
    assert plan(64, 4096, 14336, cus) == (4, 4)               # long K, few rows: four blocks, fewer reads of the rows
    assert plan(128, 4096, 14336, cus) == (2, 2)
    assert plan(64, 2048, 2048, cus, partial=False) == (1, 1) and plan(64, 6144, 4096, cus, partial=False) == (2, 1)
    assert ops.gated_blocks_per_workgroup(5632, cus) == 3 and ops.gated_blocks_per_workgroup(14336, cus) == 4
    assert ops.gated_blocks_per_workgroup(8192, cus) == 4     # 1024 blocks: 342 workgroups of three would need a second round
