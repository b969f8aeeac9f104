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
                n = kernels.decode_splits(seqs, kv_heads, context)
                assert 1 <= n <= kernels.MAX_KEY_SPLITS, (seqs, kv_heads, context, n)
    # the cases that used to ask for more than the kernel takes
    assert kernels.decode_splits(1, 4, 65536) == kernels.MAX_KEY_SPLITS
    assert kernels.decode_splits(1, 2, 81920) == kernels.MAX_KEY_SPLITS
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


def test_a_float16_cache_is_refused_when_it_is_made():
    from tie_amd.cache.manager import CacheManager
    from tie_amd.cache.spec import plan_cache
    from tie_amd.errors import InvalidArgument
    from tie_amd.config.qwen3 import Qwen3Config
    from tie_amd.models import Model
    from tie_amd.models.qwen3 import build_qwen3_spec
    from conftest import TINY_A

    model = Model(build_qwen3_spec(Qwen3Config.from_json(TINY_A)))
    with pytest.raises(InvalidArgument, match="float16"):
        CacheManager(model.cache_plan, block_size=4, num_blocks=8, dtype="float16")
