"""The serving-size widths (a Qwen3-8B config.json with one layer): the bfloat16 kernels against the float32 ones.

The tiny configurations cannot show what only large shapes do: grids of thousands of workgroups,
offsets beyond 2^31 bytes, a vocabulary of 151936, the 256 x 256 matrix-product tile, key splits,
planes of partial sums. The two paths share no matrix-product or attention kernel, so their
agreement at this size checks the indexing of both. Both paths are compared with the plain
implementation at small sizes elsewhere.
"""

import pytest
import torch

import trace_helpers as th

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 1, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "intermediate_size": 12288, "vocab_size": 151936, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 4096,
}


def test_serving_widths_bfloat16_against_float32():
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.models import expected_tensors_for_config, load_model_from_tensors
    from tie_amd.weights.random_init import random_tensors

    specs = [s for s in expected_tensors_for_config(WIDE) if not s.optional]
    tensors = dict(random_tensors(specs, 5, torch.bfloat16, device="cuda"))
    requests = th.make_requests(WIDE["vocab_size"], [700, 130, 40, 300], seed=3)
    # the largest token ids, so that the last rows of the embedding and of the head are used
    requests["r0"][:3] = [WIDE["vocab_size"] - 1, 0, WIDE["vocab_size"] - 2]

    def run(dtype, steps, max_tokens):
        model = load_model_from_tensors(WIDE, tensors, dtype, "cuda:0")
        got = th.collect(TraceReplayer(model, max_tokens, block_size=16), steps)
        del model
        torch.cuda.empty_cache()
        return got

    # one prompt of the size the prefill is measured at, ragged against every tile (2100 = 8 x 256 + 52 rows):
    # a few of its positions are compared, the last among them
    long_prompt = th.make_requests(WIDE["vocab_size"], [2100], seed=4)["r0"]
    long_steps = [{"step": 0, "entries": [{"id": "long", "tokens": long_prompt, "want": [0, 255, 256, 1023, 2047, 2099]}],
                   "end": ["long"]}]
    want_long = run("float32", long_steps, th.round64(2100))["long"]
    got_long = run("bfloat16", long_steps, th.round64(2100))["long"]
    for position, ref in want_long.items():
        err = float((got_long[position] - ref).abs().max() / ref.abs().max())
        assert torch.isfinite(got_long[position]).all() and err < 3e-2, f"long prompt, position {position}: {err:.3e}"

    biggest = max(th.round64(len(t)) for t in requests.values())
    want = run("float32", th.whole(requests), biggest)
    steps, peak = th.mixed(requests, max_live=4, seed=5, tail=40)     # long runs of decoded tokens, portions beside them
    for label, got in (("whole", run("bfloat16", th.whole(requests), biggest)),
                       ("mixed", run("bfloat16", steps, peak))):
        for rid, toks in requests.items():
            ref = torch.stack([want[rid][p] for p in range(len(toks))])
            mine = torch.stack([got[rid][p] for p in range(len(toks))])
            assert torch.isfinite(mine).all()
            err = float(((mine - ref).abs().amax(dim=1) / ref.abs().max()).max())
            assert err < 3e-2, f"{label}: request {rid} differs by {err:.3e} of the largest logit"
            # and the two paths agree on most greedy choices (near-ties may flip between precisions)
            agree = float((mine.argmax(dim=1) == ref.argmax(dim=1)).float().mean())
            assert agree > 0.9, f"{label}: request {rid}: only {agree:.2f} of the argmax tokens agree"
