"""Configurations at the edges of what the kernels take, end to end against the plain implementation.

Widths that are no multiple of 8 or 16, one to seventeen query heads per KV head, head sizes from
16 to 256 and one (24) that the matrix-core kernels refuse and the generic ones take, vocabularies
that are no power of two, feed-forward widths that rule the fused gate/up product out. Every
configuration runs whole requests and a mixed trace (portions beside decoded tokens, pages used
again) in float32 and in bfloat16.
"""

import pytest
import torch

import plain_qwen3 as plain
import tolerances
import trace_helpers as th
from conftest import load_plain_weights

pytestmark = pytest.mark.gpu

TOLERANCE = {"float32": tolerances.FLOAT32, "bfloat16": tolerances.BFLOAT16["edge shapes"]}


def config(layers, hidden, heads, kv_heads, head_dim, inter, vocab, theta=10000.0, eps=1e-6, tied=False, max_pos=512):
    return {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": layers,
            "hidden_size": hidden, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
            "head_dim": head_dim, "intermediate_size": inter, "vocab_size": vocab, "rope_theta": theta,
            "rms_norm_eps": eps, "tie_word_embeddings": tied, "max_position_embeddings": max_pos}


# name -> (configuration, block size, request lengths)
SHAPES = {
    "three_per_group_dh48": (config(2, 72, 3, 1, 48, 56, 101, tied=True), 8, [1, 37, 70, 130]),
    "width100_dh80_ungrouped": (config(1, 100, 5, 5, 80, 60, 37, theta=5e5, eps=1e-5), 16, [2, 45, 66, 131]),
    "seventeen_per_group_dh16": (config(2, 136, 17, 1, 16, 88, 1000), 4, [3, 33, 65, 100]),
    "dh128_long": (config(1, 128, 8, 2, 128, 256, 500, theta=1e6), 16, [5, 64, 129, 300]),
    "dh24_generic_attention": (config(2, 48, 4, 4, 24, 40, 77, tied=True), 4, [4, 31, 64, 90]),
    "dh256": (config(1, 64, 2, 1, 256, 96, 130), 32, [1, 50, 64, 140]),
    "dh96_dh112": (config(1, 88, 6, 3, 96, 104, 211), 8, [7, 70, 129]),
    "block_of_12": (config(1, 64, 4, 2, 32, 72, 90), 12, [5, 40, 100]),       # no power of two: generic attention
    # five and eight query heads a KV head (the 14B and 32B models' grouping): the prefill kernel takes a group in two
    # passes of four heads, the decode kernel's matrix columns hold five or eight of sixteen
    "five_per_group_dh128": (config(2, 160, 10, 2, 128, 224, 300, theta=1e6), 16, [3, 40, 129, 200]),
    "eight_per_group_dh64": (config(1, 128, 16, 2, 64, 160, 257), 16, [6, 65, 130]),
}


@pytest.fixture(scope="module")
def shape_folders(tmp_path_factory):
    from tie_amd.weights.random_init import write_random_model

    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            folder = tmp_path_factory.mktemp(f"shape_{name}_{dtype}")
            write_random_model(folder, SHAPES[name][0], seed=31 + len(made), dtype=dtype)
            made[(name, dtype)] = str(folder)
        return made[(name, dtype)]

    return get


def compare(got, want, dtype, label):
    worst = 0.0
    for rid, ref in want.items():
        mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - ref).abs().amax(dim=1) / ref.abs().max()
        bad = err > TOLERANCE[dtype]
        assert not bool(bad.any()), (f"{label}: request {rid} first differs at position {int(torch.argmax(bad.float()))} "
                                     f"(relative error {float(err.max()):.3e}, allowed {TOLERANCE[dtype]:.0e})")
        worst = max(worst, float(err.max()))
    print(f"[observed] {label}: {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_shape_whole_and_mixed(shape_folders, name, dtype):
    from tie_amd.engine.replay import TraceReplayer

    cfg, block_size, lengths = SHAPES[name]
    folder = shape_folders(name, dtype)
    requests = th.make_requests(cfg["vocab_size"], lengths, seed=7)
    weights = load_plain_weights(folder)
    want = {rid: plain.forward(weights, cfg, toks).float() for rid, toks in requests.items()}

    biggest = max(th.round64(len(t)) for t in requests.values())
    got = th.collect(TraceReplayer.from_folder(folder, dtype, biggest, block_size=block_size), th.whole(requests))
    compare(got, want, dtype, f"{name}/{dtype}/whole")

    steps, peak = th.mixed(requests, max_live=4, seed=11)
    rep = TraceReplayer.from_folder(folder, dtype, peak, block_size=block_size)
    got = th.collect(rep, steps)
    assert rep.cache.num_free() == rep.cache.num_blocks
    compare(got, want, dtype, f"{name}/{dtype}/mixed")
