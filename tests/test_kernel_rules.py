"""The host-side rules that pick a kernel form (pure functions of the sizes), on the CPU."""
import torch

from mini_engine_amd.kernels import ops


def test_decode_partitions_cover_the_context():
    for S, Hq, Hkv, ctx in ((1, 16, 8, 2048), (8, 16, 8, 2048), (64, 16, 8, 2304), (1, 32, 8, 100), (3, 6, 2, 130000),
                            (256, 64, 8, 1), (1, 4, 4, 129), (24, 16, 8, 2070), (40, 16, 8, 3000), (95, 16, 8, 2048)):
        part, parts = ops.decode_partitions(S, Hq, Hkv, ctx)
        assert part % 32 == 0 and part >= 128 and (parts <= 64 or part * 64 >= ctx)
        assert part * parts >= ctx and part * (parts - 1) < ctx
    # fewer (request, head block) pairs than compute units: the size that the reckoning of the launch's time puts
    # first. 8 requests of 2,048 keys: 8 partitions of 256 keys are two workgroups to every compute unit, a few keys
    # more and 11 of 192 (704 workgroups, all at once: 18.4 us where 1,088 of 128 keys took 20.5); longer contexts in
    # one round of larger partitions (8 of 8,200 keys: 12 of 704, 48 us where 17 of 512 took 52)
    assert ops.decode_partitions(8, 16, 8, 2048) == (256, 8) and ops.decode_partitions(8, 16, 8, 2070) == (192, 11)
    assert ops.decode_partitions(16, 16, 8, 2070) == (352, 6) and ops.decode_partitions(12, 16, 8, 2070) == (416, 5)
    assert ops.decode_partitions(8, 16, 8, 4100) == (352, 12) and ops.decode_partitions(8, 16, 8, 8200) == (704, 12)
    assert ops.decode_partitions(1, 16, 8, 2048) == (128, 16) and ops.decode_partitions(4, 16, 8, 2070) == (128, 17)
    assert ops.decode_partitions(24, 16, 8, 2070) == (544, 4) and ops.decode_partitions(48, 16, 8, 2070, even=True) == (512, 5)
    assert all(8 * S * ops.decode_partitions(S, 16, 8, 2070)[1] <= 768 for S in (1, 2, 3, 5, 8, 11, 16, 24, 31))
    # the reckoning itself: a round more costs, a partition of a block more to a wave costs, and what counts of the
    # workgroups is how many the busiest compute unit has
    cost = ops._decode_partition_cost
    assert cost(64, 2070, 128) > cost(64, 2070, 192) < cost(64, 2070, 256) and cost(64, 2048, 256) < cost(64, 2048, 192)
    assert cost(64, 8200, 704) < cost(64, 8200, 512) and cost(8, 2048, 128) < cost(8, 2048, 256)
    # never more than 64 partitions; a partition holds at most 2,048 keys while 64 partitions cover the context
    assert ops.decode_partitions(8, 16, 8, 32768) == (1024, 32) and ops.decode_partitions(1, 16, 8, 70000) == (1152, 61)
    assert ops.decode_partitions(128, 16, 8, 16384) == (2048, 8) and ops.decode_partitions(256, 16, 8, 8192) == (2048, 4)
    assert ops.decode_partitions(3, 6, 2, 130000) == (2048, 64) and ops.decode_partitions(4, 16, 8, 1 << 20) == (16384, 64)
    # 768 workgroups without a split: contexts up to 4,096 keys stay whole
    assert ops.decode_partitions(256, 16, 8, 2048) == (2048, 1) and ops.decode_partitions(96, 16, 8, 2048) == (2048, 1)
    assert ops.decode_partitions(95, 16, 8, 2048)[1] > 1 and ops.decode_partitions(97, 16, 8, 2049)[1] > 1 and ops.decode_partitions(256, 16, 8, 4097)[1] > 1
    # equally long contexts: whole from 192 workgroups on if they fill the compute units evenly, up to 8,192 keys
    assert ops.decode_partitions(32, 16, 8, 2048, even=True) == (2048, 1) and ops.decode_partitions(64, 32, 8, 8192, even=True) == (8192, 1)
    assert ops.decode_partitions(24, 16, 8, 2048, even=True)[1] > 1 and ops.decode_partitions(64, 16, 8, 8193, even=True)[1] > 1
    assert ops.decode_partitions(64, 16, 8, 2048, even=False)[1] > 1


def test_prefill_segments_cover_the_span_and_hold_512_keys_or_more():
    assert ops.prefill_segments(8192, 0, 8192, 16) == (0, 1)          # workgroups enough: left whole
    assert ops.prefill_segments(900, 0, 4, 16) == (0, 1)              # short span: left whole
    for ctx, window, tokens, heads in ((8192, 0, 256, 16), (32768, 0, 64, 16), (40000, 0, 2, 32), (5000, 3000, 8, 4),
                                       (2048, 0, 2048, 16), (4096, 0, 4096, 16), (1900, 0, 4, 16), (1536, 0, 1536, 16),
                                       (4096, 0, 1024, 16), (2048, 0, 512, 16)):
        seg, most = ops.prefill_segments(ctx, window, tokens, heads)
        span = min(ctx, window + 256) if window else ctx
        wide_portion = ops.prefill_col_tiles(ctx, window, tokens, heads) == 2 and tokens * heads < 32768
        assert seg >= (512 if span <= 4096 or wide_portion else 1024) and seg % 32 == 0 and (most - 1) * seg >= span
        assert tokens * heads * most * 130 * 4 <= 1 << 28
    assert ops.prefill_segments(2048, 0, 2048, 16)[0] == 704          # a prompt from its beginning: thirds
    # a later portion over a long context runs with two column tiles per wave and segments of 512-1,024 keys that give
    # about 512 workgroups; a short context, or few tokens, stays with one column tile
    assert ops.prefill_col_tiles(4096, 0, 1024, 16) == 2 and ops.prefill_segments(4096, 0, 1024, 16)[0] == 1024
    assert ops.prefill_col_tiles(8192, 0, 256, 16) == 2 and ops.prefill_segments(8192, 0, 256, 16)[0] == 512
    assert ops.prefill_col_tiles(2048, 0, 512, 16) == 1 and ops.prefill_col_tiles(8192, 0, 128, 16) == 1
    assert ops.prefill_col_tiles(8192, 0, 2048, 16) == 2 and ops.prefill_segments(8192, 0, 2048, 16)[0] == 4096
    assert ops.prefill_col_tiles(8192, 0, 512, 2, D=256) == 1          # head sizes beyond 128: one column tile
    assert ops.prefill_segments(8192, 512, 64, 16) == (0, 1)          # a window bounds the span
    assert ops.prefill_segments(1 << 20, 0, 8192, 64)[1] <= 3         # the partial results stay under 256 MB


def test_a_few_hundred_rows_over_small_weights_go_to_the_own_product():
    assert ops.mid_takes(128, 4096, 1024, False) == 1 and ops.mid_takes(256, 6144, 1024, False) == 1
    assert ops.mid_takes(257, 6144, 1024, False) == 0                   # more rows: the library's larger tiles
    assert ops.mid_takes(32, 4096, 1024, False) == 0                    # few rows: the skinny kernels
    assert ops.mid_takes(128, 1024, 2048, True) == 4 and ops.mid_takes(512, 1024, 3072, True) == 4
    assert ops.mid_takes(64, 1024, 2048, True) == 8 and ops.mid_takes(64, 1024, 3072, True) == 8       # one tile of rows: 128 workgroups
    assert ops.mid_takes(513, 1024, 3072, True) == 0 and ops.mid_takes(128, 1024, 2048, False) == 1
    assert ops.mid_takes(128, 4096, 1024, True) == 1                    # many features: no slices of K
    assert ops.mid_takes(128, 12288, 2048, False) == 0                  # beyond 8 M weight elements
    assert ops.mid_takes(128, 4096, 1000, False) == 0                   # K no multiple of 64


def test_gate_up_gates_in_its_epilogue_for_few_rows_and_for_a_few_hundred_over_small_weights():
    w = torch.empty(6144, 1024, dtype=torch.bfloat16)
    assert all(ops.gated_linear_rows(m, w) for m in (1, 8, 16, 17, 32, 33, 64, 256))
    assert not any(ops.gated_linear_rows(m, w) for m in (257, 2048))           # a kernel of its own
    assert not ops.gated_linear_rows(24, torch.empty(12288, 2048, dtype=torch.bfloat16))     # 17-32 rows: only over small weights
    assert not ops.gated_linear_rows(128, torch.empty(12288, 2048, dtype=torch.bfloat16))    # the library's product
    assert not ops.gated_linear_rows(128, torch.empty(6144, 1024))                            # float32


def test_three_waves_per_simd_only_for_large_launches_from_a_prompts_beginning():
    assert ops.prefill_waves(16384, 16384, 1, 16, 8, 2, 1) == 3         # one prompt of 16,384 tokens: 257 tiles x 8 kv heads
    assert ops.prefill_waves(8192, 8192, 1, 16, 8, 2, 1) == 2           # ... of 8,192: 1,032 workgroups, better with two
    assert ops.prefill_waves(2048, 16384, 8, 16, 8, 2, 1) == 3          # eight prompts of 2,048 tokens
    assert ops.prefill_waves(4200, 4200, 1, 64, 8, 2, 1) == 3           # 16 tokens to a tile at a group of 8
    assert ops.prefill_waves(1024, 18000, 32, 16, 8, 2, 1) == 3         # ragged prompts: the longest under twice the mean
    assert ops.prefill_waves(16384, 4096, 1, 64, 8, 2, 1) == 2          # a portion over a long prefix
    assert ops.prefill_waves(16384, 16384, 1, 16, 8, 2, 3) == 2         # tiles cut into segments
    assert ops.prefill_waves(16384, 16384, 1, 16, 8, 1, 1) == 2         # one column tile per wave
    assert ops.prefill_waves(0, 16384, 1, 16, 8, 2, 1) == 2             # no bound on the contexts known


def test_ksplit_keeps_512_of_k_per_split_and_fills_the_gpu():
    assert ops.choose_ksplit(8, 4096, 1024) == 1                       # 256 feature tiles already
    assert ops.choose_ksplit(8, 4096, 12288) == 1                      # 256 tiles over a long K: even, left whole
    assert ops.choose_ksplit(1, 5120, 8192) == 4                       # 320 tiles load the compute units unevenly
    assert ops.choose_ksplit(8, 5120, 25600) == 4
    assert ops.choose_ksplit(64, 5120, 25600) == 1                     # many rows: left to the library
    assert ops.choose_ksplit(8, 6144, 1024) == 1                       # uneven but short: left whole
    for M, N, K in ((8, 1024, 2048), (1, 1024, 3072), (16, 80, 224), (8, 1024, 256)):
        ks = ops.choose_ksplit(M, N, K)
        assert 1 <= ks <= 8 and (ks == 1 or K // ks >= 512)


def test_large_weights_with_several_rows_go_to_the_library():
    assert not ops.library_streams_better(1, 24576, 4096)              # one row: the skinny kernel
    assert not ops.library_streams_better(2, 24576, 4096)              # two rows: still level
    assert not ops.library_streams_better(16, 24576, 4096)             # up to 16 rows the skinny kernel's wide loads are ahead
    assert ops.library_streams_better(17, 24576, 4096)
    assert not ops.library_streams_better(10, 51200, 5120) and ops.library_streams_better(11, 51200, 5120)   # a longer K: up to 10
    assert ops.library_streams_better(8, 24576, 4000)                  # K no multiple of 128: no wide loads, the library from 4 rows
    assert not ops.library_streams_better(8, 4096, 4096)               # below the size threshold
    assert not ops.library_streams_better(8, 5120, 25600)              # very long K: the library's choice is poor
    assert not ops.library_streams_better(16, 6144, 1024)


def test_skinny_kernel_takes_few_rows():
    assert ops.skinny_takes(32, 6144, 1024) and not ops.skinny_takes(33, 6144, 1024)
    assert ops.skinny_takes(64, 4096, 1024) and not ops.skinny_takes(65, 4096, 1024)
    assert ops.skinny_takes(1, 151936, 1024) and ops.skinny_takes(12, 151936, 4096)      # the head: up to 12 rows with the wide loads
    assert not ops.skinny_takes(13, 151936, 1024) and not ops.skinny_takes(1, 151936, 1000)  # ... else the library
    assert ops.skinny_takes(10, 151936, 5120) and not ops.skinny_takes(11, 151936, 5120)  # a longer K: up to 10
    assert ops.skinny_takes(16, 24576, 4096) and not ops.skinny_takes(17, 24576, 4096)   # large weights: as far as the wide loads go


def test_rows_kernel_reads_wide_with_few_rows_and_many_workgroups():
    assert ops.rows_wide(24, 4096, 8) == 1 and ops.rows_wide(32, 5120, 8) == 1
    assert ops.rows_wide(33, 4096, 8) == 0 and ops.rows_wide(24, 6144, 1) == 0 and ops.rows_wide(24, 4096, 4) == 0


def test_rows_kernel_takes_many_rows_over_large_weights():
    assert ops.rows_takes(24, 4096, 4096) and not ops.rows_takes(64, 4096, 4096)     # above 32 rows only over a long K
    assert ops.rows_takes(32, 4096, 12288) and ops.rows_takes(32, 5120, 8192) and not ops.rows_takes(64, 5120, 8192)
    assert not ops.rows_takes(64, 4096, 12288)       # from 33 rows the library's slices of K take these weights
    assert ops.rows_takes(64, 1400, 12296)           # ... unless K has no equal slices of a multiple of 8
    assert not ops.rows_takes(8, 5120, 25600) and not ops.rows_takes(4, 5120, 25600)   # few rows: the skinny kernel's wide loads
    assert ops.rows_takes(8, 5120, 25608)                                              # ... unless K is no multiple of 128
    assert not ops.rows_takes(8, 4096, 12288) and not ops.rows_takes(64, 1024, 3072) and not ops.rows_takes(65, 5120, 25600)
    for K in (4096, 4104, 9728, 12288, 25600):
        ks, chunks = ops.rows_ksplit(K), -(-K // 512)
        assert 1 <= ks <= 8 and (ks - 1) * -(-chunks // ks) < chunks



def test_library_slices_of_k_for_o_and_down_at_many_rows():
    assert ops.library_splits(32, 4096, 12288) == 1 and ops.library_splits(33, 4096, 12288) == 8
    assert ops.library_splits(256, 5120, 25600) == 8 and ops.library_splits(257, 5120, 25600) == 4
    assert ops.library_splits(512, 5120, 8192) == 4 and ops.library_splits(1024, 5120, 8192) == 2
    assert ops.library_splits(1025, 5120, 8192) == 1
    assert ops.library_splits(128, 1024, 3072) == 1 and ops.library_splits(128, 2048, 8192) == 8   # 10 M elements or more
    assert ops.library_splits(64, 1400, 12296) == 1      # 12296 = 8 x 1537: no two equal slices of a multiple of 8
    assert ops.library_splits(64, 4096, 4096 + 32) == 4  # 4128 = 4 x 1032
    for M, N, K in ((100, 4096, 4096), (300, 5120, 17408), (100, 2560, 9728)):
        s = ops.library_splits(M, N, K)
        assert s > 1 and K % (8 * s) == 0 and K // s >= 512


def test_requests_stay_on_one_xcd_only_when_their_contexts_are_equally_long():
    assert ops.decode_contexts_even(8, 2048, 2048) and ops.decode_contexts_even(64, 2000, 2100)
    assert not ops.decode_contexts_even(64, 1900, 2100) and not ops.decode_contexts_even(256, 100, 2048)
    assert not ops.decode_contexts_even(7, 2048, 2048)          # fewer requests than XCDs: spread
    assert not ops.decode_contexts_even(8, 0, 0)                # unknown


def test_rules_at_the_layer_sizes_between_the_measured_ones():
    """What was corrected after the products of the 1.7B (2048 / 6144), 4B (2560 / 9728) and 14B (5120 / 17408) layer sizes
    were timed beside every other kernel: each line is a place where the rule had picked the slower one."""
    # down at the 1.7B sizes (12.6 M elements): the library's slices of K from 33 rows (64 rows: 16.9 -> 9.0 us), the rows
    # kernel at 17-32 (32 rows: 11.0 -> 9.1)
    assert ops.library_splits(64, 2048, 6144) == 8 and ops.library_splits(512, 2048, 6144) == 4
    assert ops.rows_takes(32, 2048, 6144) and not ops.rows_takes(64, 2048, 6144)
    # o at the 4B sizes (10.5 M elements over a K of 4,096): slices only from 128 rows, the plain call below (64 rows: 17.1
    # -> 11.5 us), and no skinny split beyond 32 rows over a weight this large
    assert ops.library_splits(64, 2560, 4096) == 1 and ops.library_splits(128, 2560, 4096) == 8
    assert ops.rows_takes(32, 2560, 4096) and not ops.rows_takes(48, 2560, 4096)
    # down at the 4B sizes (2560 features over a K of 9,728): the rows kernel at 33-64 rows, where the library's slices take
    # 48 us and its plain call 29 (64 rows: -> 21 us); the slices again beyond
    assert ops.rows_takes(64, 2560, 9728) and ops.library_splits(64, 2560, 9728) == 1 and ops.library_splits(128, 2560, 9728) == 8
    # ... and ahead of both, with the norm that adds the slices counted in: the tiled kernel in 8 slices (64 rows: 24.7 ->
    # 21.3 us) and in 4 at 128 rows (35.1 -> 31.5); o at the 8B sizes likewise up to 128 rows (64 rows: 17.2 -> 14.3), at
    # the 14B sizes up to 64; down at the 8B and 14B sizes stays with the library's slices
    assert ops.mid_takes(64, 2560, 9728, True) == 4 and ops.mid_takes(128, 2560, 9728, True) == 2 and ops.mid_takes(256, 2560, 9728, True) == 0
    assert ops.mid_takes(64, 4096, 4096, True) == 4 and ops.mid_takes(128, 4096, 4096, True) == 2 and ops.mid_takes(256, 4096, 4096, True) == 0
    assert ops.mid_takes(64, 5120, 5120, True) == 0 and ops.mid_takes(64, 4096, 12288, True) == 0 and ops.mid_takes(64, 5120, 17408, True) == 0
    assert ops.mid_takes(64, 2048, 6144, True) == 8 and ops.mid_takes(128, 2560, 4096, True) == 2 and ops.mid_takes(256, 2560, 4096, True) == 2
    # over these larger weights from 17 rows on (24 rows, 2560 x 9728: 20.3 -> 17.6 us); the small ones keep the skinny split there
    assert ops.mid_takes(24, 2560, 9728, True) == 4 and ops.mid_takes(24, 2048, 6144, True) == 8 and ops.mid_takes(24, 4096, 4096, True) == 4
    assert ops.mid_takes(24, 1024, 2048, True) == 0 and ops.mid_takes(32, 2048, 2048, True) == 0 and ops.mid_takes(16, 2560, 9728, True) == 0
    assert all(ops.mid_takes(M, N, K, False) == 0 for M, N, K in ((64, 2560, 9728), (64, 4096, 4096), (64, 2048, 6144)))
    assert not ops.rows_has_few_features(64, 5120, 17408) and ops.library_splits(64, 5120, 17408) == 8     # 14B: stays with the slices
    # qkv at the 4B sizes (15.7 M elements): the library from 17 rows (32 rows: 18.8 -> 10.4 us), the skinny kernel's wide loads below
    assert ops.library_streams_better(32, 6144, 2560) and not ops.library_streams_better(16, 6144, 2560)
    assert not ops.skinny_takes(32, 6144, 2560) and ops.skinny_takes(16, 6144, 2560)
    # qkv at the 1.7B sizes (8.4 M elements) at 64 rows: the library's tiles, not the tiled kernel for small weights (12.2 -> 9.8 us);
    # from 128 rows the two are level and the own kernel stays
    assert ops.mid_takes(64, 4096, 2048, False) == 0 and ops.mid_takes(128, 4096, 2048, False) == 1
    assert ops.mid_takes(64, 4096, 1024, False) == 1                     # the 0.6B sizes keep theirs
    # o at the 1.7B sizes at 33-64 rows: the tiled kernel's four slices of K, not the skinny split (64 rows: 7.9 -> 5.9 us);
    # beyond 1,024 features only up to 256 rows (512 rows: 13.1 -> 11.7 with the library), and there in two slices
    # (128 tiles: 256 workgroups)
    assert ops.mid_takes(64, 2048, 2048, True) == 4 and ops.mid_takes(256, 2048, 2048, True) == 2
    assert ops.mid_takes(512, 2048, 2048, True) == 0 and ops.mid_takes(512, 1024, 2048, True) == 4


def test_slices_of_the_tiled_kernel_fit_what_the_kernel_and_the_norm_take():
    """Whatever sizes come: the slices that `mid_slices` names leave no slice without steps (the kernel refuses that),
    are at most the 8 partial sums that the norm kernel adds, and only K in whole steps of 64 is sliced."""
    import random
    rng = random.Random(5)
    seen = set()
    for _ in range(20000):
        M, N, K = rng.randint(1, 700), 4 * rng.randint(1, 1600), 64 * rng.randint(1, 300)
        if rng.random() < 0.2:
            K += rng.choice([8, 16, 32])
        slices = ops.mid_slices(M, N, K)
        seen.add(slices)
        assert slices in (1, 2, 4, 8)
        if slices > 1:
            steps = K // 64
            per = -(-steps // slices)
            assert K % 64 == 0 and M > 16 and (slices - 1) * per < steps and N * K <= ops.MID_SLICES_MAX_WEIGHT
            assert ops.mid_takes(M, N, K, True) == slices and ops.mid_takes(M, N, K, False) in (0, 1)
    assert seen == {1, 2, 4, 8}


def test_decode_partitions_always_fit_the_kernel():
    """Whatever batch, heads and context come: partitions of a multiple of 32 keys, at least 128, that cover the
    context without an empty last one, and at most the 64 that the merge takes unless even 64 of the largest size on
    the list do not cover the context (then partitions of up to 16,384 keys, still 64)."""
    import random
    rng = random.Random(11)
    for _ in range(20000):
        Hkv = rng.choice([1, 2, 4, 8, 16])
        Hq = Hkv * rng.choice([1, 2, 4, 5, 8, 20])
        S = rng.choice([1, 2, 3, 5, 8, 13, 24, 31, 32, 64, 100, 300])
        ctx = rng.choice([1, 17, 128, 129, 700, 2048, 2070, 5000, 33000, 140000, 1 << 20])
        even = rng.random() < 0.5
        part, parts = ops.decode_partitions(S, Hq, Hkv, ctx, even)
        assert part % 32 == 0 and part >= 128 and parts >= 1, (S, Hq, Hkv, ctx, even, part, parts)
        assert part * parts >= ctx and part * (parts - 1) < ctx, (S, Hq, Hkv, ctx, even, part, parts)
        assert parts <= 64, (S, Hq, Hkv, ctx, even, part, parts)
