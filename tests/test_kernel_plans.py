"""The host-side plans of the attention kernels stay inside what the kernels take (no GPU needed)."""

import pathlib
import re

import pytest

from conftest import ROOT


def test_key_shares_never_exceed_what_the_merge_takes():
    from tie_amd import kernels

    header = (pathlib.Path(ROOT) / "tiny-inference-engine_amd" / "csrc" / "attention_merge.h").read_text()
    assert int(re.search(r"#define\s+MERGE_MAX_SPLITS\s+(\d+)", header).group(1)) == kernels.MAX_KEY_SPLITS
    contexts = [1, 100, 1024, 4096, 32768, 40960, 65536, 131072, 1 << 20]
    for seqs in (1, 2, 3, 4, 7, 8, 64, 256):
        for kv_heads in (1, 2, 4, 8, 16):
            for context in contexts:
                for block_size in (4, 8, 16, 64):
                    n = kernels.decode_splits(seqs, kv_heads, context, block_size)
                    assert 1 <= n <= kernels.MAX_KEY_SPLITS, (seqs, kv_heads, context, block_size, n)
    # the cases that used to ask for more than the kernel takes
    assert kernels.decode_splits(1, 4, 65536, 8) == kernels.MAX_KEY_SPLITS
    assert kernels.decode_splits(1, 2, 81920, 8) == kernels.MAX_KEY_SPLITS
    assert kernels.decode_splits(1, 1, 65536, 16) == kernels.MAX_KEY_SPLITS
    # about 512 waves in shares of at least 128 keys where a wave keeps several tiles in flight
    assert kernels.decode_splits(8, 8, 4096) == 8 and kernels.decode_splits(64, 8, 4096) == 1
    assert kernels.decode_splits(31, 8, 4096) == 3 and kernels.decode_splits(32, 8, 4096) == 1 and kernels.decode_splits(48, 8, 4096) == 2
    assert kernels.decode_splits(1, 8, 4096) == 32 and kernels.decode_splits(1, 8, 200) == 1
    # where 512 waves would not spread evenly over 256 compute units, the count up to twice as large that does
    assert kernels.decode_splits(24, 8, 4096) == 4 and kernels.decode_splits(40, 8, 4096) == 3      # 768 and 960 waves
    assert kernels.decode_splits(12, 8, 4096) == 8 and kernels.decode_splits(20, 8, 4096) == 6      # 768 and 960
    assert kernels.decode_splits(24, 8, 300) == 2 and kernels.decode_splits(56, 8, 4096) == 2       # short shares; 1344 are too many
    # whatever the batch: between the count for 512 waves and twice that, more shares than that count only where
    # the GPU holds all their waves at once, and shares of at least 128 keys
    for seqs in range(1, 130):
        for kv_heads in (1, 2, 4, 8):
            for context in (200, 1024, 4096, 40000):
                n = kernels.decode_splits(seqs, kv_heads, context)
                pairs = seqs * kv_heads
                first = min(-(-512 // pairs), max(1, context // 128), kernels.MAX_KEY_SPLITS)
                assert (n == 1 and pairs == 256) or first <= n <= 2 * first, (seqs, kv_heads, context, n)
                assert n == 1 or context // n >= 64, (seqs, kv_heads, context, n)
                assert n <= first or pairs * n <= 1024, (seqs, kv_heads, context, n)
    for items in (1, 2, 5, 40, 300):
        for kv_heads in (1, 2, 8):
            for group in (1, 3, 4, 8, 16):
                for context in contexts:
                    n = kernels.prefill_splits(items, kv_heads, group, context, 64 * items)
                    assert 1 <= n <= kernels.MAX_KEY_SPLITS, (items, kv_heads, group, context, n)


def test_sizes_no_kernel_takes_are_refused_when_the_model_is_built():
    from tie_amd.config.qwen3 import Qwen3Config
    from tie_amd.errors import InvalidArgument
    from tie_amd.models import Model
    from tie_amd.models.qwen3 import build_qwen3_spec
    from conftest import TINY_A

    with pytest.raises(InvalidArgument, match="head_dim 520"):
        Model(build_qwen3_spec(Qwen3Config.from_json(dict(TINY_A, head_dim=520))))
    Model(build_qwen3_spec(Qwen3Config.from_json(dict(TINY_A, head_dim=512))))


def test_the_cache_has_a_precision_of_its_own_where_a_kernel_takes_the_pair():
    """float32 arithmetic runs over float32, bfloat16 or float16 pages (the reference's KVCacheConfig.dtype,
    src/kv/paged_kv_cache.h:18-25); the matrix-core kernels read bfloat16 pages only. What no kernel takes is
    refused when the engine is made, by name, before any weight is read."""
    from tie_amd import kernels
    from tie_amd.api import create_engine
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.errors import InvalidArgument

    assert kernels.cache_dtype_for("float32") == "float32" and kernels.cache_dtype_for("bfloat16") == "bfloat16"
    assert kernels.cache_dtype_for("float32", "bf16") == "bfloat16"
    assert kernels.cache_dtype_for("float32", "float16") == "float16"
    assert kernels.cache_dtype_for("bfloat16", "bfloat16") == "bfloat16"
    for mode, asked, words in (("bfloat16", "float32", "bfloat16 arithmetic over a float32 cache"),
                               ("bfloat16", "float16", "bfloat16 arithmetic over a float16 cache"),
                               ("float32", "int8", "float32, bfloat16 or float16")):
        with pytest.raises(InvalidArgument, match=words):
            kernels.cache_dtype_for(mode, asked)
    # the folder does not exist: the refusal comes first
    with pytest.raises(InvalidArgument, match="over a float32 cache"):
        create_engine("/nonexistent/model", dtype="bfloat16", kv_dtype="float32")
    with pytest.raises(InvalidArgument, match="over a float16 cache"):
        TraceReplayer.from_folder("/nonexistent/model", "bfloat16", 64, kv_dtype="float16")


def test_cache_pages_are_sized_by_the_cache_dtype():
    from tie_amd.cache.manager import CacheManager
    from tie_amd.config.qwen3 import Qwen3Config
    from tie_amd.errors import InvalidArgument
    from tie_amd.models import Model
    from tie_amd.models.qwen3 import build_qwen3_spec
    from conftest import TINY_A

    plan = Model(build_qwen3_spec(Qwen3Config.from_json(TINY_A))).cache_plan
    sizes = {d: CacheManager(plan, block_size=4, num_blocks=8, dtype=d).bytes_per_block
             for d in ("float32", "bfloat16", "float16")}
    assert sizes["float32"] == 2 * sizes["bfloat16"] == 2 * sizes["float16"] == 2 * 2 * 2 * 4 * 16 * 4
    with pytest.raises(InvalidArgument, match="int8"):
        CacheManager(plan, block_size=4, num_blocks=8, dtype="int8")


TILE_ROWS_COLS = {4: (256, 256), 5: (256, 128), 6: (128, 256), 7: (128, 128), 10: (256, 192)}


def test_the_tiled_product_plans_by_rounds_of_workgroups():
    """Above 128 rows the tile and the ranges of K come from an estimate of the time; these are the measured choices."""
    from tie_amd import kernels

    qkv, o, gate_up, down = (6144, 4096), (4096, 4096), (24576, 4096), (4096, 12288)    # [N, K] of an 8B layer
    # 2048 rows, the prefill step that is measured: 256 x 256 tiles; O alone is too narrow for them and stays whole;
    # QKV's 6144 columns in tiles of 192 make 256 workgroups where tiles of 256 leave a quarter of the compute
    # units idle (88 against 93 us)
    assert (kernels.gemm_tile(2048, *qkv, True), kernels.gemm_splits(2048, *qkv, True)) == (10, 1)
    assert (kernels.gemm_tile(2048, *o, True), kernels.gemm_splits(2048, *o, True)) == (6, 1)
    assert kernels.gemm_tile(2048, *gate_up, True, 1) == 4
    assert (kernels.gemm_tile(2048, *down, True), kernels.gemm_splits(2048, *down, True)) == (4, 2)
    assert kernels.gemm_splits(1024, *down, True) == 4
    # 768 rows: two ranges of 256 x 128 tiles would be 288 workgroups, a second round for 32 of them
    tile, ranges = kernels.gemm_tile(768, *qkv, True), kernels.gemm_splits(768, *qkv, True)
    rows, cols = TILE_ROWS_COLS[tile]
    assert -(-768 // rows) * -(-6144 // cols) * ranges <= 256
    # every plan: a tile that loads straight into LDS, 1 to 8 ranges, none shorter than 512 of K
    for N, K in (qkv, o, down, (2048, 2048), (10240, 5120), (5120, 25600)):
        for M in range(129, 2300, 61):
            ranges = kernels.gemm_splits(M, N, K, True)
            assert ranges in (1, 2, 4, 8) and (ranges == 1 or K // ranges >= 512), (M, N, K, ranges)
            assert kernels.gemm_tile(M, N, K, True) in TILE_ROWS_COLS
            assert kernels.gemm_tile(M, N, K, True, 1) in TILE_ROWS_COLS
    # 65 to 128 rows: the weights are read once, and one round of workgroups should fill the compute units.
    # 8B gate/up on 128 x 128 tiles (192 workgroups; 96 of 128 x 256 took 82 us against 61), the 1.7B's on
    # 64 x 128 (192), the 32B's on 128 x 256 (200); the 32B's QKV in 4 ranges (160 workgroups; 8 are two rounds)
    assert kernels.gemm_tile(128, *gate_up, True, 1) == 7 and kernels.gemm_tile(80, *gate_up, True, 1) == 7
    assert kernels.gemm_tile(96, 12288, 2048, True, 1) == 9 and kernels.gemm_tile(128, 51200, 5120, True, 1) == 6
    assert (kernels.gemm_tile(128, 10240, 5120, True), kernels.gemm_splits(128, 10240, 5120, True)) == (6, 4)
    assert (kernels.gemm_tile(128, 4096, 2048, True), kernels.gemm_splits(128, 4096, 2048, True)) == (9, 4)
    assert (kernels.gemm_tile(128, *down, True), kernels.gemm_splits(128, *down, True)) == (7, 8)
    for N, K in (qkv, o, down, (2048, 2048), (10240, 5120), (5120, 25600), (2048, 6144)):
        for M in range(65, 129, 9):
            ranges = kernels.gemm_splits(M, N, K, True)
            assert ranges in (1, 2, 4, 8) and (ranges == 1 or K // ranges >= 512), (M, N, K, ranges)
            assert kernels.gemm_tile(M, N, K, True) in (6, 7, 8, 9) and kernels.gemm_tile(M, N, K, True, 1) in (6, 7, 8, 9)
    # shapes the straight-to-LDS tiles do not take keep the older tiles and their rule
    assert kernels.gemm_splits(300, 200, 1000) == 2 and kernels.gemm_tile(300, 200, 1000) == 1
    assert kernels.gemm_splits(128, 4096, 4096) == 8 and kernels.gemm_splits(128, 4096, 256) == 1


def test_the_prefill_attention_kernel_refuses_caches_it_cannot_address():
    """Its addresses are 32-bit counts of 8 bytes, a page's number times the page's size by a 24-bit multiply."""
    import torch
    from tie_amd import kernels

    def plane(pages, kv_heads, block, dim):
        return torch.empty((pages, kv_heads, block, dim), dtype=torch.bfloat16, device="meta")

    assert kernels.prefill_addressable(plane(300_000, 8, 16, 128))          # 9.8 GB: a long cache of an 8B model
    assert kernels.prefill_addressable(plane((1 << 20) - 1, 8, 16, 128))    # just under 32 GB
    assert not kernels.prefill_addressable(plane(1 << 20, 8, 16, 128))      # 32 GB
    assert not kernels.prefill_addressable(plane(4, 64, 4096, 256))         # a page of 128 MB
    assert not kernels.prefill_addressable(plane(1 << 24, 1, 4, 16))        # 2^24 pages


def test_the_decode_products_plan_for_17_to_64_rows():
    """Which kernel, how many tiles a workgroup and how many ranges of K come from one score (what x costs beside
    the weights, the planes, how full the compute units are), not from a table of shapes: its choices on the shapes
    it was measured on, and what must hold on any shape."""
    from tie_amd import kernels

    # 8B QKV at 24 rows: x through LDS, three tiles a workgroup, two ranges: 256 workgroups, one a compute unit
    # (15.1 us with the kernel that adds the planes; six tiles in four ranges, the same 256 workgroups: 17.1)
    assert kernels.few_rows_plan(24, 6144, 4096) == (True, 3, 2)
    # a gate/up of 16384 x 3072: 1024 tiles are 342 workgroups of three or 171 of six, a round and a third or two
    # thirds of one; x from memory in workgroups of four tiles fills one round exactly (20.6 against 22.4 and 24.7 us)
    assert kernels.few_rows_plan(24, 16384, 3072, True) == (False, 4, 1)
    # a gate/up of 34816 x 5120: eight tiles a workgroup would be 272 workgroups, a second round for 16 of them
    assert kernels.few_rows_plan(32, 34816, 5120, True) == (True, 3, 1)
    # up to 16 rows the shape alone decides
    assert kernels.few_rows_plan(16, 6144, 4096) == (False, 0, kernels.skinny_splits(6144, 4096))
    for N, K in ((6144, 4096), (4096, 12288), (5120, 3072), (2560, 9728), (1024, 2048), (8192, 28672), (10240, 5120)):
        for M in (17, 24, 32, 33, 48, 64):
            shares_x, tiles, splits = kernels.few_rows_plan(M, N, K)
            assert splits in (1, 2, 4, 8) and tiles in ((3, 6, 8) if shares_x else (1, 2, 3, 4)), (M, N, K)
            if shares_x:      # whole chunks of four k-blocks a wave, ranges of at least 1024 of K
                assert (K // 32) % (16 * splits) == 0 and (splits == 1 or K // splits >= 1024), (M, N, K, splits)
            assert kernels.few_rows_plan(M, N, K, True)[2] == 1                      # a gated product is never cut
    # the tiled product with 64-row tiles: the 32B shape's QKV in two ranges of 64 x 128 tiles (160 workgroups), not
    # eight of 64 x 256 (320: a second round for 64 of them, 1.7 times the time); a tile is the same whether the
    # plan is asked for the ranges too or handed them back
    assert (kernels.gemm_tile(64, 10240, 5120, True), kernels.gemm_splits(64, 10240, 5120, True)) == (9, 2)
    for N, K in ((6144, 4096), (4096, 12288), (10240, 5120), (8192, 8192), (1024, 2048), (5120, 25600)):
        for M in (40, 64):
            ranges = kernels.gemm_splits(M, N, K, True)
            assert ranges in (1, 2, 4, 8) and (ranges == 1 or K // ranges >= 512)
            assert kernels.gemm_tile(M, N, K, True) == kernels.gemm_tile(M, N, K, True, ranges) in (8, 9)
    assert kernels.gemm_tile(64, 51200, 5120, True, 1) == 8 and kernels.gemm_tile(64, 151936, 4096, True, 1) == 8


def test_shares_of_one_length_are_planned_for_sequences_of_very_different_lengths():
    import random

    from tie_amd import kernels

    rng = random.Random(0)
    assert kernels.decode_share_plan([2048] * 32, 8, 4096) == (kernels.decode_splits(32, 8, 4096), 0)
    assert kernels.decode_share_plan([4000, 3900, 4096] * 11, 8, 4096)[1] == 0          # about one length
    assert kernels.decode_share_plan([100, 4000], 8, 4096) == (kernels.decode_splits(2, 8, 4096), 0)   # many shares anyway
    assert kernels.decode_share_plan([32768] + [1024] * 7, 8, 32768) == (64, 21)          # one long sequence among short ones
    assert kernels.decode_share_plan([32768] * 8, 8, 32768)[1] == 0
    assert kernels.decode_share_plan([100, 4000] * 16, 8, 4096, block_size=8)[1] == 0     # the other kernel
    planned = 0
    for S, kvh, ctx in ((32, 8, 4096), (64, 8, 4096), (16, 8, 4096), (40, 4, 16384), (24, 8, 2048)):
        for i in range(20):
            lens = [rng.randint(20, ctx) for _ in range(S)] if i % 2 else [ctx] * 2 + [rng.randint(20, ctx // 6) for _ in range(S - 2)]
            shares, length = kernels.decode_share_plan(lens, kvh, ctx)
            equal = kernels.decode_splits(S, kvh, ctx)
            if length == 0:
                assert shares == equal
                continue
            tiles = [(n - 1) // 32 + 1 for n in lens]
            planned += 1
            assert shares >= equal and shares * length >= max(tiles) and length >= 4
            assert kvh * sum(-(-t // length) for t in tiles) <= (512 if S * kvh <= 128 else 768 if S * kvh <= 256 else 1024)
            before = -(-max(tiles) // equal)
            assert 2 * length <= before if equal <= 3 else 4 * length < before
    assert planned >= 20
    # a window bounds what a sequence shows: sequences far longer than the window are all of one length
    assert kernels.decode_share_plan([300, 4000] * 16, 8, 4096, window=256)[1] == 0
