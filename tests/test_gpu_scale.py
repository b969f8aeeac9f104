"""The serving-size widths against the plain implementation, in float32 and in bfloat16.

A Qwen3-8B config.json (hidden 4096, 32 query heads over 8 KV heads of 128, feed-forward 12288, vocabulary
151936, untied head) with 2 of its 36 layers: the widths are the real ones, the depth is cut so that the
plain implementation (float64, on the CPU) stays affordable. The tiny configurations cannot show what only
these shapes do: grids of thousands of workgroups, offsets beyond 2^31 bytes, the 256 x 256 matrix-product
tiles over packed weights, planes of partial sums, dozens of key shares in decode attention.

The weights are drawn once and rounded to bfloat16; the float32 engine and the plain implementation read
those same values widened, so one plain result serves both comparisons: float32 within 1e-4 of the largest
logit, bfloat16 within 2.5e-2 (tests/tolerances.py), in every way of cutting the work (the reference's own test of this:
``tests/model/test_qwen3_forward.cpp:60-87``), and the stream after every layer (``:143-187``).
"""

import pytest
import torch

import plain_qwen3 as plain
import tolerances
import trace_helpers as th

pytestmark = pytest.mark.gpu

LAYERS_RUN, LAYERS_OF_THE_MODEL = 2, 36
WIDE = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": LAYERS_RUN, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "intermediate_size": 12288, "vocab_size": 151936, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 4096,
}
TOLERANCE = {"float32": tolerances.FLOAT32, "bfloat16": tolerances.BFLOAT16["serving widths"]}
LONG_ROWS = [0, 255, 256, 1023, 2047, 2099]


@pytest.fixture(scope="module")
def wide():
    """Weights on the GPU (bfloat16 values), the requests, and the plain implementation's results."""
    from tie_amd.models import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    specs = [s for s in expected_tensors_for_config(WIDE) if not s.optional]
    tensors = dict(random_tensors(specs, 5, torch.bfloat16, device="cuda"))
    host = {name: t.cpu() for name, t in tensors.items()}          # bfloat16; each product widens its operands
    requests = th.make_requests(WIDE["vocab_size"], [130, 40, 97, 64], seed=3)
    # the largest token ids, so that the last rows of the embedding and of the head are used
    requests["r0"][:3] = [WIDE["vocab_size"] - 1, 0, WIDE["vocab_size"] - 2]
    want, hidden = {}, {}
    for rid, toks in requests.items():
        hidden[rid] = []
        want[rid] = plain.forward(host, WIDE, toks, hidden_states=hidden[rid]).float()
        hidden[rid] = [h.float() for h in hidden[rid]]
    # one prompt of the size the prefill is measured at, ragged against every tile (2100 = 8 x 256 + 52 rows)
    long_prompt = th.make_requests(WIDE["vocab_size"], [2100], seed=4)["r0"]
    want_long = plain.forward(host, WIDE, long_prompt, rows=LONG_ROWS).float()
    yield dict(tensors=tensors, requests=requests, want=want, hidden=hidden, long_prompt=long_prompt,
               want_long=want_long)
    tensors.clear()
    torch.cuda.empty_cache()


def load(wide, dtype):
    from tie_amd.models import load_model_from_tensors

    tensors = wide["tensors"]
    if dtype == "float32":
        tensors = {name: t.float() for name, t in tensors.items()}
    return load_model_from_tensors(WIDE, tensors, dtype, "cuda:0")


def check(got, want, dtype, label):
    for rid, ref in want.items():
        rows = got[rid]
        assert sorted(rows) == list(range(ref.shape[0])), f"{label}: request {rid} misses positions"
        mine = torch.stack([rows[p] for p in range(ref.shape[0])])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - ref).abs().amax(dim=1) / ref.abs().max()
        over = err > TOLERANCE[dtype]
        assert not bool(over.any()), (f"{label}: request {rid} first differs at position {int(torch.argmax(over.float()))} "
                                      f"(relative error {float(err[over][0]):.3e}, allowed {TOLERANCE[dtype]:.0e})")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_serving_widths_against_the_plain_implementation_in_every_way_of_cutting(wide, dtype):
    from tie_amd.engine.replay import TraceReplayer

    model = load(wide, dtype)
    requests, want = wide["requests"], wide["want"]
    biggest = max(th.round64(len(t)) for t in requests.values())

    # whole prompts, with the stream after every layer against the plain implementation's
    seen = {}
    model.layer_hook = lambda index, x: seen.setdefault(index, []).append(x.float().cpu())
    got = th.collect(TraceReplayer(model, biggest, block_size=16), th.whole(requests))
    model.layer_hook = None
    check(got, want, dtype, f"{dtype}/whole")
    for n, rid in enumerate(requests):
        for layer in range(LAYERS_RUN):
            mine, ref = seen[layer][n], wide["hidden"][rid][layer]
            err = float((mine - ref).abs().max() / ref.abs().max())
            assert err <= TOLERANCE[dtype], f"{dtype}: stream after layer {layer} of request {rid} differs by {err:.3e}"

    check(th.collect(TraceReplayer(model, biggest, block_size=16), th.prefill_then_decode(requests)), want, dtype,
          f"{dtype}/prefill+decode")
    check(th.collect(TraceReplayer(model, biggest, block_size=16), th.portions(requests)), want, dtype,
          f"{dtype}/portions")
    steps, peak = th.mixed(requests, max_live=4, seed=5, tail=40)     # long runs of decoded tokens, portions beside them
    replayer = TraceReplayer(model, peak, block_size=16)
    check(th.collect(replayer, steps), want, dtype, f"{dtype}/mixed")
    assert replayer.cache.num_free() == replayer.cache.num_blocks
    # the same requests once more through a pool that holds two of them: the second pair gets the first pair's pages
    few, peak_few = th.mixed(requests, max_live=2, seed=6, tail=40)
    replayer = TraceReplayer(model, peak_few, block_size=16)
    check(th.collect(replayer, few), want, dtype, f"{dtype}/mixed, pages used again")
    assert replayer.cache.num_free() == replayer.cache.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_serving_widths_a_long_prompt_whole_and_in_portions(wide, dtype):
    from tie_amd.engine.replay import TraceReplayer

    model = load(wide, dtype)
    prompt, want = wide["long_prompt"], wide["want_long"]

    def rows_of(steps):
        got = th.collect(TraceReplayer(model, th.round64(len(prompt)), block_size=16), steps)["long"]
        return torch.stack([got[p] for p in LONG_ROWS])

    whole = [{"step": 0, "entries": [{"id": "long", "tokens": prompt, "want": LONG_ROWS}], "end": ["long"]}]
    cuts = [0, 512, 1024, 1100, 2048, 2098, 2100]                     # portions of 512 and ragged ones, down to two tokens
    portions = []
    for a, b in zip(cuts[:-1], cuts[1:]):
        portions.append({"step": len(portions), "entries": [{"id": "long", "tokens": prompt[a:b],
                                                              "want": [p - a for p in LONG_ROWS if a <= p < b]}], "end": []})
    portions[-1]["end"] = ["long"]
    for label, steps in (("whole", whole), ("portions", portions)):
        mine = rows_of(steps)
        assert torch.isfinite(mine).all()
        err = (mine - want).abs().amax(dim=1) / want.abs().max()
        assert float(err.max()) <= TOLERANCE[dtype], (f"{dtype}, long prompt {label}: positions {LONG_ROWS} differ by "
                                                      f"{[f'{float(e):.2e}' for e in err]}")


def test_serving_widths_a_corrupted_page_is_caught(wide):
    """The bfloat16 bound against a real fault at these widths, where attention averages over keys of small
    random projections: one page of 16 keys (or values) of one layer overwritten with another page's after the
    prefill, then one token decoded. The first layer's fault moves the logits by half their size; the last
    layer's by less, and still by more than the bound."""
    from tie_amd.engine.replay import TraceReplayer

    model = load(wide, "bfloat16")
    tokens, want = wide["requests"]["r0"], wide["want"]["r0"][-1]
    bound = TOLERANCE["bfloat16"]

    def last_row_error(layer=None, plane=0):
        rep = TraceReplayer(model, th.round64(len(tokens)), block_size=16)
        rep.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:-1], "want": []}], "end": []})
        if layer is not None:
            table = rep.requests["a"].tables[0]
            pages = rep.cache.kv[0]
            pages[layer, plane, table[3]] = pages[layer, plane, table[5]].clone()
        logits = rep.run_step({"step": 1, "entries": [{"id": "a", "tokens": tokens[-1:], "want": [0]}], "end": ["a"]})
        return float((logits[0].float().cpu() - want).abs().max() / want.abs().max())

    assert last_row_error() < bound / 2
    seen = {(layer, what): last_row_error(layer, plane)
            for layer in range(LAYERS_RUN) for plane, what in ((0, "keys"), (1, "values"))}
    print(f"[observed] serving widths: a corrupted page moves the last row by {seen} (bound {bound})")
    assert min(seen.values()) > 1.25 * bound and seen[(0, "keys")] > 10 * bound, f"a wrong page passes under the bound: {seen}"
