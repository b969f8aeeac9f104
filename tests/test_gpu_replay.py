"""The engine against the plain implementation under every way of cutting the work.

Each request alone and whole; most of it in one step and the last 32 tokens one by one; in
portions of changing size down to two tokens; and mixed, up to four live requests, portions
of some beside decoded tokens of others, in a pool so small that pages are used again -
in float32 and in bfloat16, for two tiny configurations that differ in every size.
"""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import tolerances
import trace_helpers as th
from conftest import BLOCK_SIZE, ROOT, TINY, load_plain_weights

pytestmark = pytest.mark.gpu

# max |engine - plain| / max |plain| over a request's logits: float32, and bfloat16 by fixture (the label of every
# check begins with the fixture's letter)
TOLERANCE = {"float32": tolerances.FLOAT32, "A": tolerances.BFLOAT16["tiny A"], "B": tolerances.BFLOAT16["tiny B"]}
LENGTHS = {"A": [5, 11, 17, 40, 64, 33], "B": [1, 23, 40, 64, 90, 37]}


def reference_logits(folder, cfg, requests):
    weights = load_plain_weights(folder)
    return {rid: plain.forward(weights, cfg, toks).float() for rid, toks in requests.items()}


def check(got, want, dtype, label, tolerance=None):
    worst = 0.0
    if tolerance is None:
        tolerance = TOLERANCE["float32"] if dtype == "float32" else TOLERANCE[label[0]]
    for rid, ref in want.items():
        rows = got[rid]
        assert sorted(rows) == list(range(ref.shape[0])), f"{label}: request {rid} misses positions"
        mine = torch.stack([rows[p] for p in range(ref.shape[0])])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - ref).abs().amax(dim=1) / ref.abs().max()
        bad = int(torch.argmax((err > tolerance).float())) if bool((err > tolerance).any()) else -1
        assert bad < 0, (f"{label}: request {rid} first differs at position {bad} "
                         f"(relative error {float(err[bad]):.3e}, allowed {tolerance:.0e})")
        worst = max(worst, float(err.max()))
    print(f"[observed] {label}: {worst:.3e}")
    return worst


@pytest.fixture(scope="module")
def folders(model_folders, model_folders_bf16):
    return {"float32": model_folders, "bfloat16": model_folders_bf16}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_all_ways_of_cutting(folders, name, dtype):
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders[dtype][name]
    requests = th.make_requests(cfg["vocab_size"], LENGTHS[name], seed=5)
    want = reference_logits(folder, cfg, requests)
    bs = BLOCK_SIZE[name]
    biggest = max(th.round64(len(t)) for t in requests.values())

    def replayer(max_tokens):
        return TraceReplayer.from_folder(folder, dtype, max_tokens, block_size=bs)

    results = {}
    results["whole"] = th.collect(replayer(biggest), th.whole(requests))
    results["prefill+decode"] = th.collect(replayer(biggest), th.prefill_then_decode(requests))
    results["portions"] = th.collect(replayer(biggest), th.portions(requests))
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    assert max(len(s["entries"]) for s in steps) >= 3
    rep = replayer(peak)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.num_free() == rep.cache.num_blocks          # every page came back
    for label, got in results.items():
        check(got, want, dtype, f"{name}/{dtype}/{label}")
    # the ways of cutting agree with each other far more closely than with the reference in bf16
    if dtype == "float32":
        for label in ("prefill+decode", "portions", "mixed"):
            for rid in requests:
                a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
                b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
                assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


# float32 arithmetic over a narrower cache: the reference pins its own such pair (F32 activations, F16 cache) at
# 3e-3 (tests/backend/test_paged_attention.cpp:70-103); bfloat16 keeps 3 bits fewer than float16.
NARROW_CACHE_TOLERANCE = {"float16": 3e-3, "bfloat16": 3e-3}


@pytest.mark.parametrize("kv_dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_arithmetic_over_a_narrower_cache(folders, name, kv_dtype):
    """The cache's precision is its own knob (src/kv/paged_kv_cache.h:18-25; the reference's default run is
    float32 activations over a 16-bit cache): float32 weights and arithmetic, keys and values rounded once as
    they are written. All four ways of cutting against the plain implementation; they agree with each other
    as closely as in pure float32, since every key is rounded the same way whichever step wrote it."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["float32"][name]
    requests = th.make_requests(cfg["vocab_size"], LENGTHS[name], seed=5)
    want = reference_logits(folder, cfg, requests)
    bs = BLOCK_SIZE[name]
    biggest = max(th.round64(len(t)) for t in requests.values())
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    traces = {"whole": (th.whole(requests), biggest), "prefill+decode": (th.prefill_then_decode(requests), biggest),
              "portions": (th.portions(requests), biggest), "mixed": (steps, peak)}
    results, worst = {}, 0.0
    for label, (trace, pool) in traces.items():
        rep = TraceReplayer.from_folder(folder, "float32", pool, block_size=bs, kv_dtype=kv_dtype)
        assert rep.cache.dtype == kv_dtype and rep.cache.kv[0].dtype == getattr(torch, kv_dtype)
        assert rep.model.mode == "float32"
        results[label] = th.collect(rep, trace)
        assert rep.cache.num_free() == rep.cache.num_blocks
        worst = max(worst, check(results[label], want, "float32", f"{name}/float32 over {kv_dtype}/{label}",
                                 tolerance=tolerances.NARROW_CACHE[kv_dtype]))
    print(f"[observed] {name} float32 over {kv_dtype}: worst relative error {worst:.3e}")
    assert worst > 1e-6, "the cache rounded nothing: is it float32 after all?"
    for label in ("prefill+decode", "portions", "mixed"):
        for rid in requests:
            a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
            b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
            assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


@pytest.mark.parametrize("name", ["A", "B"])
def test_single_rows_beside_portions_on_either_attention_kernel(folders, name, monkeypatch):
    """In a mixed step a few single decoded rows run in the prefill attention kernel beside the portions, many in
    the decode kernel: the mixed trace through both ways (the traces above only meet the first)."""
    from tie_amd import kernels
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["bfloat16"][name]
    requests = th.make_requests(cfg["vocab_size"], LENGTHS[name], seed=6)
    want = reference_logits(folder, cfg, requests)
    steps, peak = th.mixed(requests, max_live=4, seed=4)
    assert any(sum(len(e["tokens"]) == 1 for e in s["entries"]) and any(len(e["tokens"]) > 1 for e in s["entries"])
               for s in steps), "no step mixes single rows with a portion"
    got = {}
    for ride_along in (kernels.SINGLE_ROWS_RIDE_ALONG, 0):
        monkeypatch.setattr(kernels, "SINGLE_ROWS_RIDE_ALONG", ride_along)
        got[ride_along] = th.collect(TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=BLOCK_SIZE[name]), steps)
        check(got[ride_along], want, "bfloat16", f"{name}/bfloat16/mixed, single rows riding along up to {ride_along}")


@pytest.mark.parametrize("block_size", [32, 64])
def test_pages_of_32_and_64_positions(folders, block_size):
    """Configuration B in bfloat16 over larger pages (a page then holds several blocks of 16 keys, which the
    attention kernels that load by such blocks must find inside it): mixed steps and decoding against the plain
    implementation, pages counted in the replayer's own page size."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["bfloat16"]["B"]
    requests = th.make_requests(cfg["vocab_size"], [130, 23, 70, 64, 97, 33], seed=12)
    want = reference_logits(folder, cfg, requests)
    steps, peak = th.mixed(requests, max_live=4, seed=7)
    rep = TraceReplayer.from_folder(folder, "bfloat16", 2 * peak, block_size=block_size)
    got = th.collect(rep, steps)
    assert rep.cache.num_free() == rep.cache.num_blocks
    check(got, want, "bfloat16", f"B/bfloat16/mixed, pages of {block_size}")
    tail = th.collect(TraceReplayer.from_folder(folder, "bfloat16", 2 * peak, block_size=block_size),
                      th.prefill_then_decode(requests))
    check(tail, want, "bfloat16", f"B/bfloat16/prefill+decode, pages of {block_size}")


@pytest.mark.parametrize("use_graphs", [False, True])
def test_decode_steps_with_and_without_the_attention_kernel_that_prepares(folders, monkeypatch, use_graphs):
    """Steps of single decoded tokens run on the attention kernel that makes its own queries and newest keys
    (heads of 32, pages of 16: configuration B); switched off, the q/k kernel runs before the decode attention.
    Both against the plain implementation, the last 32 tokens of every request decoded one by one, and the
    keys and values the first way left in the cache serve the second way's later steps just as well."""
    import tie_amd.parts.attention as attention_part
    from tie_amd import kernels
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["bfloat16"]["B"]
    requests = th.make_requests(cfg["vocab_size"], LENGTHS["B"], seed=9)
    want = reference_logits(folder, cfg, requests)
    steps = th.prefill_then_decode(requests)
    biggest = max(th.round64(len(t)) for t in requests.values())
    calls = {"prepared": 0}
    prepared = kernels.paged_attention_prepared

    def counted(*args, **kwargs):
        calls["prepared"] += 1
        return prepared(*args, **kwargs)

    monkeypatch.setattr(attention_part.kernels, "paged_attention_prepared", counted)
    on = th.collect(TraceReplayer.from_folder(folder, "bfloat16", biggest, block_size=16, use_graphs=use_graphs), steps)
    assert calls["prepared"] > 0, "no decode step took the kernel that prepares its own queries"
    check(on, want, "bfloat16", "B/bfloat16/decode steps on the kernel that prepares")
    monkeypatch.setattr(attention_part.kernels, "decode_attention_prepares", lambda *a, **k: False)
    before = calls["prepared"]
    off = th.collect(TraceReplayer.from_folder(folder, "bfloat16", biggest, block_size=16, use_graphs=use_graphs), steps)
    assert calls["prepared"] == before
    check(off, want, "bfloat16", "B/bfloat16/decode steps on the q/k kernel and the decode attention")
    for rid in requests:
        a = torch.stack([on[rid][p] for p in sorted(on[rid])])
        b = torch.stack([off[rid][p] for p in sorted(off[rid])])
        assert float((a - b).abs().max() / b.abs().max()) < 2e-2, f"request {rid}: the two ways differ by more than rounding"


# Every width a multiple of 32 and none under 96, so that every projection is stored in the decode product's
# packed layout: only such products take the norms' work (tiny A and B keep some or all of theirs unpacked).
PACKED_WIDTHS = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 160, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 224, "vocab_size": 300, "rope_theta": 50000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 128,
}


def test_steps_of_a_few_rows_leave_the_norms_to_the_products(tmp_path, monkeypatch):
    """In steps of a few rows (how few is a measured rule by the weight's shape) the product that ends a sub-layer
    adds to the stream and prepares the next norm in its epilogue, and the products behind that norm apply its
    1 / rms: no norm kernel runs between the layers' parts. Both ways against the plain implementation, through decoding, small portions and mixed steps; the norm
    kernels that still run are the first layer's first (nothing precedes it) and the head's."""
    from tie_amd import kernels
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.random_init import write_random_model

    cfg = PACKED_WIDTHS
    folder = str(tmp_path)
    write_random_model(folder, cfg, seed=31, dtype="bfloat16")
    requests = th.make_requests(cfg["vocab_size"], [5, 11, 17, 40, 64, 33], seed=15)
    want = reference_logits(folder, cfg, requests)
    layers = cfg["num_hidden_layers"]
    few_rows = kernels.norm_epilogue_rows(cfg["hidden_size"], cfg["intermediate_size"])   # of the product that ends a layer
    assert 2 <= few_rows == kernels.norm_epilogue_rows(cfg["hidden_size"], 4 * 32) <= kernels.NORM_EPILOGUE_ROWS
    calls = []
    for fn in ("rms_norm", "add_partials"):
        real = getattr(kernels, fn)
        monkeypatch.setattr(kernels, fn, lambda *a, _real=real, _fn=fn, **k: (calls.append(_fn), _real(*a, **k))[1])
    steps, peak = th.mixed(requests, max_live=4, seed=9, sizes=(31, 7, 2, 18, 3, 2, 9))
    got = {}
    for in_products in (True, False):
        monkeypatch.setattr(kernels, "NORMS_IN_PRODUCTS", in_products)
        rep = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=16, use_graphs=False)
        norm_kernels = {}
        real_step = rep.run_step

        def counted(step, _real=real_step, _seen=norm_kernels):
            del calls[:]
            out = _real(step)
            rows = sum(len(e["tokens"]) for e in step["entries"])
            _seen.setdefault(rows <= few_rows, []).append(len(calls))
            return out

        rep.run_step = counted
        got[in_products] = th.collect(rep, steps)
        check(got[in_products], want, "bfloat16", f"packed widths/mixed, norms in the products: {in_products}",
              tolerance=tolerances.BFLOAT16["packed widths"])
        assert norm_kernels[True] and norm_kernels[False], "the trace needs steps of few rows and of many"
        if in_products:
            assert max(norm_kernels[True]) <= 3, f"steps of few rows launched {norm_kernels[True]} norm kernels"
        else:
            assert min(norm_kernels[True]) >= 2 * layers
        assert min(norm_kernels[False]) >= 2 * layers          # steps of many rows: every norm a kernel
    for rid in requests:
        a = torch.stack([got[True][rid][p] for p in sorted(got[True][rid])])
        b = torch.stack([got[False][rid][p] for p in sorted(got[False][rid])])
        assert float((a - b).abs().max() / b.abs().max()) < 1e-2, f"request {rid}: the two ways differ by more than rounding"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("use_graphs", [False, True])
def test_layers_of_one_shape_run_from_one_layers_launch_list(tmp_path, dtype, use_graphs):
    """With four or more layers alike, only the first three run the parts' code in a step; the others run the
    same launches with their own weights and cache planes. Every logit must be the very bits of a run in which
    every layer runs its own code, through portions, mixed steps and decoding (recorded into graphs or not)."""
    from conftest import TINY_B
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.random_init import write_random_model

    cfg = dict(TINY_B, num_hidden_layers=7)
    folder = tmp_path / "seven_layers"
    write_random_model(folder, cfg, seed=31, dtype=dtype)
    requests = th.make_requests(cfg["vocab_size"], [150, 37, 90, 64, 121], seed=8)
    want = reference_logits(folder, cfg, requests)
    steps, peak = th.mixed(requests, max_live=4, seed=5)
    got = {}
    for replay in (True, False):
        rep = TraceReplayer.from_folder(folder, dtype, peak, block_size=16, use_graphs=use_graphs)
        rep.model.replay_layers = replay
        assert rep.model._alike == {0: 7}
        got[replay] = th.collect(rep, steps)
        assert (rep.model.layers_replayed > 0) == replay
        assert rep.cache.num_free() == rep.cache.num_blocks
    check(got[True], want, dtype, f"B with seven layers alike/{dtype}")
    for rid in requests:
        for position, row in got[True][rid].items():
            assert torch.equal(row, got[False][rid][position]), f"request {rid}, position {position}"


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_corrupted_page_is_caught(folders, name):
    """The bound the bfloat16 checks use must not be so wide that a wrong page of the cache passes under it. A
    request is prefilled, ONE page of ONE layer's keys (then, in another run, values) is overwritten with the
    page after it, and the last token is decoded: its logits must miss the plain implementation's by more than
    the bound, in every layer; the clean run of the same steps stays well within it. (Swapping two entries of the
    block table is no such fault: keys and values move together, and attention does not care in which order it
    meets them.)"""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["bfloat16"][name]
    tokens = th.make_requests(cfg["vocab_size"], LENGTHS[name], seed=5)["r4"]
    want = plain.forward(load_plain_weights(folder), cfg, tokens, rows=[len(tokens) - 1]).float()[0]
    bound = TOLERANCE[name]

    def last_row_error(layer=None, plane=0):
        rep = TraceReplayer.from_folder(folder, "bfloat16", th.round64(len(tokens)), block_size=BLOCK_SIZE[name])
        rep.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:-1], "want": []}], "end": []})
        if layer is not None:
            table = rep.requests["a"].tables[0]
            pages = rep.cache.kv[0]                    # [layer, keys | values, page, kv head, ...]
            pages[layer, plane, table[1]] = pages[layer, plane, table[2]].clone()
        logits = rep.run_step({"step": 1, "entries": [{"id": "a", "tokens": tokens[-1:], "want": [0]}], "end": ["a"]})
        return float((logits[0].float().cpu() - want).abs().max() / want.abs().max())

    assert last_row_error() < bound / 2
    seen = {}
    for layer in range(cfg["num_hidden_layers"]):
        for plane, what in ((0, "keys"), (1, "values")):
            seen[(layer, what)] = last_row_error(layer, plane)
    print(f"[observed] {name}: a corrupted page moves the last row by {seen} (bound {bound})")
    first_layer = max(seen[(0, "keys")], seen[(0, "values")])
    assert seen[(0, "keys")] > 1.25 * bound and first_layer > 2 * bound, f"a wrong page passes under the bound: {seen}"


def test_pages_are_used_again(folders):
    """A pool of exactly one request's pages serves request after request."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["float32"]["A"]
    requests = th.make_requests(cfg["vocab_size"], [60, 64, 50, 61], seed=9)
    want = reference_logits(folder, cfg, requests)
    rep = TraceReplayer.from_folder(folder, "float32", 64, block_size=4)
    got = th.collect(rep, th.portions(requests, sizes=(9, 2, 30, 5)))
    check(got, want, "float32", "A/reuse")


def test_trace_run_program(folders, tmp_path):
    """The program itself: JSON lines in, .f32 files and 'done' lines out."""
    folder, cfg = folders["float32"]["B"]
    requests = th.make_requests(cfg["vocab_size"], [23, 40], seed=2)
    steps, peak = th.mixed(requests, max_live=2, seed=1)
    steps.append({"step": len(steps), "entries": [{"id": "late", "tokens": [1, 2, 3], "want": []}], "end": ["late"]})
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", folder, "--dtype", "float32",
         "--out", str(out), "--max-tokens", str(peak + 64)],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    assert not (out / f"{steps[-1]['step']}.f32").exists()        # nothing was wanted in the last step
    want = reference_logits(folder, cfg, requests)
    position = {}
    for s in steps[:-1]:
        data = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
        r = 0
        for e in s["entries"]:
            start = position.get(e["id"], 0)
            for w in e["want"]:
                ref = want[e["id"]][start + w]
                assert float(np.abs(data[r] - ref.numpy()).max() / ref.abs().max()) < 1e-4
                r += 1
            position[e["id"]] = start + len(e["tokens"])
        assert r == data.shape[0]


def test_recorded_decode_steps_replay_to_the_eager_result(folders):
    """Decode steps replayed from a HIP graph give bit for bit what eager launches give, replay after
    replay, with other steps (prompt portions, other batch shapes) and synchronisations in between."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders["bfloat16"]["B"]
    requests = th.make_requests(cfg["vocab_size"], [70, 45, 52], seed=12)
    steps, peak = th.mixed(requests, max_live=3, seed=4, tail=24)
    eager = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=16, use_graphs=False)
    graphs = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=16, use_graphs=True)
    for step in steps:
        a = eager.run_step(step)
        b = graphs.run_step(step)
        torch.cuda.synchronize()
        assert (a is None) == (b is None)
        if a is not None:
            assert torch.equal(a, b), f"step {step['step']} differs between eager launches and the replayed graph"
    assert graphs.runner.graph_replays >= 10 and eager.runner.graph_replays == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_more_sequences_decode_together_than_the_decode_product_takes(folders, dtype):
    """Eighty requests decode side by side: above 64 rows a step's products run on the tiled kernels
    (over packed weights, in ranges of K), also inside the recorded graphs that later steps replay."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders[dtype]["B"]
    requests = th.make_requests(cfg["vocab_size"], [9 + i % 7 for i in range(80)], seed=77)
    want = reference_logits(folder, cfg, requests)
    tail = 6
    steps = []
    ids = list(requests)
    for at in range(0, len(ids), 16):                     # prompts, sixteen requests a step
        steps.append({"step": len(steps), "end": [], "entries": [
            {"id": r, "tokens": requests[r][:-tail], "want": list(range(len(requests[r]) - tail))} for r in ids[at:at + 16]]})
    for t in range(tail, 0, -1):                          # then one token each, all eighty together
        steps.append({"step": len(steps), "end": ids if t == 1 else [], "entries": [
            {"id": r, "tokens": [requests[r][-t]], "want": [0]} for r in ids]})
    replayer = TraceReplayer.from_folder(folder, dtype, 80 * 64, block_size=16)
    got = th.collect(replayer, steps)
    check(got, want, dtype, f"B/{dtype}/eighty together")
    if dtype == "bfloat16":
        assert replayer.runner.graph_replays >= tail - 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """A short prompt, then every further token one by one, up to the model's context."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders[dtype]["B"]
    requests = th.make_requests(cfg["vocab_size"], [250], seed=31)
    want = reference_logits(folder, cfg, requests)
    got = th.collect(TraceReplayer.from_folder(folder, dtype, 256, block_size=16),
                     th.prefill_then_decode(requests, tail=243))
    check(got, want, dtype, f"B/{dtype}/long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_the_first_tokens_of_a_sequence(folders, name, dtype):
    """Position 0 alone, the first few positions one by one, and prompts of one, two and three tokens."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg = folders[dtype][name]
    requests = th.make_requests(cfg["vocab_size"], [1, 2, 3, 6], seed=33)
    want = reference_logits(folder, cfg, requests)
    rep = lambda: TraceReplayer.from_folder(folder, dtype, 256, block_size=BLOCK_SIZE[name])
    check(th.collect(rep(), th.whole(requests)), want, dtype, f"{name}/{dtype}/first tokens whole")
    check(th.collect(rep(), th.prefill_then_decode(requests, tail=32)), want, dtype, f"{name}/{dtype}/first tokens one by one")
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:1], "want": [0]} for rid, toks in requests.items()], "end": ["r0"]}]
    for i in range(1, 6):
        entries = [{"id": rid, "tokens": [toks[i]], "want": [0]} for rid, toks in requests.items() if len(toks) > i]
        steps.append({"step": i, "entries": entries, "end": [rid for rid, toks in requests.items() if len(toks) == i + 1]})
    check(th.collect(rep(), steps), want, dtype, f"{name}/{dtype}/first tokens together")
