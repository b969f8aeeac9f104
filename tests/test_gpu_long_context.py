"""Decoding where serving runs it: contexts of thousands of keys, across the buckets a decode step is planned in.

A decode step's grid (the shares a sequence's keys are cut into) and its recorded HIP graph are chosen by the
longest context of the step, in buckets of 1024, 2048, 4096, ... keys. The tiny configurations stop at 256
positions and never leave the first bucket; here three, then four requests decode side by side while the longest
crosses 1024, 2048 and 4096 keys, so that

* a new graph is recorded at every boundary and replayed on both sides of it,
* one recording serves sequences of very different lengths (300 keys beside 4000),
* the decode attention runs with dozens of shares, on the kernel that prepares its own queries and on the one
  behind the q/k kernel,

and every decoded row is compared with the plain implementation (the reference's own equivalence of whole
prompts and token-by-token decoding, tests/model/test_qwen3_forward.cpp:60-87, at the lengths it never reaches).

Random projections of width 0.02 make attention an average over thousands of keys, under which a lost tile of
32 keys would move the logits by less than bfloat16 rounding does. The q and k norm weights of these models are
therefore scaled up so that scores spread over several units and a few dozen keys carry a row's weight: which
they are differs from row to row, and losing any stretch of keys shows. ``test_a_far_page_matters`` holds the
bound against exactly that.
"""

import pytest
import torch

import plain_qwen3 as plain
import trace_helpers as th
from conftest import load_plain_weights

pytestmark = pytest.mark.gpu

CONFIGS = {
    # two layers, four query heads over two KV heads of 128 (the serving head size)
    "heads of 128": {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2,
                     "hidden_size": 128, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128,
                     "intermediate_size": 256, "vocab_size": 512, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
                     "tie_word_embeddings": False, "max_position_embeddings": 4608},
    # one layer, six query heads over two KV heads of 32: three heads a group, another head size
    "heads of 32": {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 1,
                    "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32,
                    "intermediate_size": 160, "vocab_size": 384, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
                    "tie_word_embeddings": True, "max_position_embeddings": 4608},
}
QK_SCALE = 1.6           # q_norm and k_norm weights are multiplied by this: scores spread 2.5 times wider
# max |engine - plain| / max |plain| over a request's rows. bfloat16: about three times the worst seen over the
# trace below (1.56e-2 and 2.5e-3: sharper scores carry rounding further than the tiny configurations' do).
BOUND = {"float32": 1e-4, "heads of 128": 4e-2, "heads of 32": 7.5e-3}
BUCKETS = (1024, 2048, 4096, 8192)


@pytest.fixture(scope="module")
def long_models(tmp_path_factory):
    """name -> (bfloat16 folder, config, plain weights): random weights with the q/k norm weights scaled up."""
    from safetensors.torch import load_file, save_file
    from tie_amd.weights.random_init import write_random_model

    out = {}
    for i, (name, cfg) in enumerate(CONFIGS.items()):
        folder = tmp_path_factory.mktemp(f"long_{i}")
        write_random_model(folder, cfg, seed=41 + i, dtype="bfloat16")
        tensors = load_file(str(folder / "model.safetensors"))
        for key in tensors:
            if key.endswith("q_norm.weight") or key.endswith("k_norm.weight"):
                tensors[key] = (tensors[key].float() * QK_SCALE).to(tensors[key].dtype)
        save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
        out[name] = (str(folder), cfg, load_plain_weights(str(folder)))
    return out


def bucket_of(context):
    bucket = 1024
    while bucket < context:
        bucket *= 2
    return bucket


def crossing_trace(vocab):
    """Requests a (1000 tokens prefilled), c (300), later b (2030) and d (4080), prefilled in portions of up to
    512 between the others' decode steps; the longest live request crosses 1024, 2048 and 4096 keys while all
    decode. Returns (requests' tokens, steps, the most tokens live at a time rounded as the replayer counts)."""
    prefilled = {"a": 1000, "c": 300, "b": 2030, "d": 4080}
    final = {"a": 1000 + 40 + 40 + 30, "c": 300 + 40 + 40 + 30, "b": 2030 + 40 + 30, "d": 4080 + 30}
    tokens = th.make_requests(vocab, [final[r] for r in ("a", "c", "b", "d")], seed=17)
    tokens = dict(zip(("a", "c", "b", "d"), tokens.values()))
    at = {r: 0 for r in tokens}
    steps = []

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    def portion(rid, size):
        n = min(size, prefilled[rid] - at[rid])
        entry = {"id": rid, "tokens": tokens[rid][at[rid]:at[rid] + n], "want": [n - 1] if at[rid] + n == prefilled[rid] else []}
        at[rid] += n
        return entry

    def decoded(rid):
        entry = {"id": rid, "tokens": [tokens[rid][at[rid]]], "want": [0]}
        at[rid] += 1
        return entry

    sizes = [512, 300, 188, 450, 62, 512, 512]
    k = 0
    while at["a"] < prefilled["a"] or at["c"] < prefilled["c"]:          # a and c: portions side by side
        add([portion(r, sizes[k % len(sizes)]) for r in ("a", "c") if at[r] < prefilled[r]])
        k += 1
    for _ in range(40):                                                  # a crosses 1024
        add([decoded("a"), decoded("c")])
    while at["b"] < prefilled["b"]:                                      # b enters, in steps of its own: the decode
        add([portion("b", sizes[k % len(sizes)])])                       # steps around them keep their shapes
        k += 1
    for _ in range(40):                                                  # b crosses 2048
        add([decoded("a"), decoded("b"), decoded("c")])
    while at["d"] < prefilled["d"]:
        add([portion("d", sizes[k % len(sizes)])])
        k += 1
    for i in range(30):                                                  # d crosses 4096
        add([decoded(r) for r in ("a", "b", "c", "d")], end=("a", "b", "c", "d") if i == 29 else ())
    assert all(at[r] == final[r] for r in tokens)
    return tokens, steps, sum(th.round64(n) for n in final.values())


def wanted_positions(steps):
    """request -> the positions whose logits the trace asks for, in order."""
    position, wanted = {}, {}
    for step in steps:
        for e in step["entries"]:
            start = position.get(e["id"], 0)
            wanted.setdefault(e["id"], []).extend(start + w for w in e["want"])
            position[e["id"]] = start + len(e["tokens"])
    return wanted


@pytest.fixture(scope="module")
def expected(long_models):
    out = {}
    for name, (folder, cfg, weights) in long_models.items():
        tokens, steps, pool = crossing_trace(cfg["vocab_size"])
        wanted = wanted_positions(steps)
        want = {rid: plain.forward(weights, cfg, tokens[rid], rows=wanted[rid]).float() for rid in tokens}
        out[name] = (tokens, steps, pool, wanted, want)
    return out


def run_and_compare(replayer, steps, wanted, want, bound, label):
    got = th.collect(replayer, steps)
    worst = 0.0
    for rid, rows in wanted.items():
        mine = torch.stack([got[rid][p] for p in rows])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - want[rid]).abs().amax(dim=1) / want[rid].abs().max()
        bad = err > bound
        assert not bool(bad.any()), (f"{label}: request {rid} first differs at position "
                                     f"{rows[int(torch.argmax(bad.float()))]} (relative error {float(err[bad][0]):.3e}, "
                                     f"allowed {bound:.0e})")
        worst = max(worst, float(err.max()))
    print(f"[observed] {label}: {worst:.3e}")
    return got


@pytest.mark.parametrize("prepares", [True, False])
@pytest.mark.parametrize("use_graphs", [True, False])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_decoding_across_context_buckets_in_bfloat16(long_models, expected, monkeypatch, name, use_graphs, prepares):
    import tie_amd.parts.attention as attention_part
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg, _ = long_models[name]
    tokens, steps, pool, wanted, want = expected[name]
    if not prepares:
        monkeypatch.setattr(attention_part.kernels, "decode_attention_prepares", lambda *a, **k: False)
    calls = {"prepared": 0}
    real = attention_part.kernels.paged_attention_prepared

    def counted(*args, **kwargs):
        calls["prepared"] += 1
        return real(*args, **kwargs)

    monkeypatch.setattr(attention_part.kernels, "paged_attention_prepared", counted)
    replayer = TraceReplayer.from_folder(folder, "bfloat16", pool, block_size=16, use_graphs=use_graphs)
    runner = replayer.runner
    assert runner.use_graphs == use_graphs

    # what every decode-only step did: replayed a recording or not, by the bucket of its longest context
    replays, eager = {b: 0 for b in BUCKETS}, {b: 0 for b in BUCKETS}
    real_step = replayer.run_step
    lengths = {}

    def watched(step):
        for e in step["entries"]:
            lengths[e["id"]] = lengths.get(e["id"], 0) + len(e["tokens"])
        before = runner.graph_replays
        out = real_step(step)
        if all(len(e["tokens"]) == 1 for e in step["entries"]):
            bucket = bucket_of(max(lengths[e["id"]] for e in step["entries"]))
            if runner.graph_replays > before:
                replays[bucket] += 1
            else:
                eager[bucket] += 1
        return out

    replayer.run_step = watched
    run_and_compare(replayer, steps, wanted, want, BOUND[name],
                    f"{name}/bfloat16/graphs {use_graphs}/prepares {prepares}")
    assert replayer.cache.num_free() == replayer.cache.num_blocks
    assert (calls["prepared"] > 0) == prepares
    if use_graphs:
        recorded = {key[2] for key in runner._recorded}
        assert recorded == set(BUCKETS), f"graphs were recorded for the context buckets {sorted(recorded)}"
        # the first step of a shape runs eagerly and is recorded; every later one of that shape replays
        assert all(replays[b] >= 10 for b in BUCKETS), f"replays by bucket: {replays}"
        assert sum(eager.values()) == len(runner._recorded), f"{eager} steps ran eagerly for {len(runner._recorded)} recordings"
    else:
        assert runner.graph_replays == 0 and not runner._recorded


@pytest.mark.parametrize("prepares", [True, False])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_shares_of_one_length_while_sequences_of_300_and_4000_keys_decode_together(long_models, expected, monkeypatch,
                                                                                  name, prepares):
    """The plan for sequences of very different lengths (one length for all shares, a short sequence filling one of
    them) is made for steps of many sequences; here the rule by the step's size is bent to two shares a sequence so
    that four requests meet it: recorded steps and eager ones, the kernel that prepares its queries and the other,
    while the plan changes from step to step with the lengths."""
    import tie_amd.engine.batch as batch_module
    import tie_amd.parts.attention as attention_part
    from tie_amd import kernels
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg, _ = long_models[name]
    tokens, steps, pool, wanted, want = expected[name]
    monkeypatch.setattr(kernels, "decode_splits", lambda *a, **k: 2)
    if not prepares:
        monkeypatch.setattr(attention_part.kernels, "decode_attention_prepares", lambda *a, **k: False)
    plans = []
    real = kernels.decode_share_plan

    def watched(*args, **kwargs):
        plans.append(real(*args, **kwargs))
        return plans[-1]

    monkeypatch.setattr(batch_module.kernels, "decode_share_plan", watched)
    replayer = TraceReplayer.from_folder(folder, "bfloat16", pool, block_size=16, use_graphs=True)
    run_and_compare(replayer, steps, wanted, want, BOUND[name], f"{name}/bfloat16/shares of one length/prepares {prepares}")
    lengths = {length for shares, length in plans if length > 0}
    grids = {shares for shares, length in plans if length > 0}
    assert lengths and len(grids) >= 2 and all(g >= 8 and g & (g - 1) == 0 for g in grids), (sorted(lengths), sorted(grids))
    assert replayer.runner.graph_replays > 50 and {key[3] for key in replayer.runner._recorded} >= {(g,) for g in grids}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_decoding_across_context_buckets_in_float32(long_models, expected, name):
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg, _ = long_models[name]
    tokens, steps, pool, wanted, want = expected[name]
    replayer = TraceReplayer.from_folder(folder, "float32", pool, block_size=16)
    run_and_compare(replayer, steps, wanted, want, BOUND["float32"], f"{name}/float32")
    assert replayer.cache.num_free() == replayer.cache.num_blocks


@pytest.mark.parametrize("name", list(CONFIGS))
def test_a_far_page_matters(long_models, name):
    """The bound of the bfloat16 comparison against a fault among thousands of keys: after a prefill of 4000
    tokens, one page of 16 keys of one layer, 3000 positions back (or the newest whole page), is overwritten with
    another page's, and the next tokens are decoded. Over a few dozen decoded rows at least one row's logits
    must leave the bound - each row's weight sits on its own few dozen keys, and some row's sit on that page."""
    from tie_amd.engine.replay import TraceReplayer

    folder, cfg, weights = long_models[name]
    tokens = th.make_requests(cfg["vocab_size"], [4000 + 48], seed=23)["r0"]
    rows = list(range(3999, len(tokens)))
    want = plain.forward(weights, cfg, tokens, rows=rows).float()
    bound = BOUND[name]

    def worst_error(victim=None, source=None):
        rep = TraceReplayer.from_folder(folder, "bfloat16", th.round64(len(tokens)), block_size=16)
        at = 0
        for size in (1024, 1024, 1024, 927):
            rep.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens[at:at + size], "want": []}], "end": []})
            at += size
        if victim is not None:
            table = rep.requests["a"].tables[0]
            pages = rep.cache.kv[0]
            pages[0, 0, table[victim]] = pages[0, 0, table[source]].clone()       # the first layer's keys
        mine = []
        for p in rows:
            out = rep.run_step({"step": 1, "entries": [{"id": "a", "tokens": [tokens[p]], "want": [0]}], "end": []})
            mine.append(out[0].float().cpu())
        err = (torch.stack(mine) - want).abs().amax(dim=1) / want.abs().max()
        return float(err.max())

    clean = worst_error()
    far = worst_error(victim=1000 // 16, source=2000 // 16)
    near = worst_error(victim=3984 // 16 - 1, source=5)
    print(f"[observed] {name}: clean {clean:.3e}, a far page wrong {far:.3e}, the newest whole page wrong {near:.3e}")
    assert clean < bound
    assert far > 1.5 * bound and near > 1.5 * bound
