"""The parts of a model, each alone and in other arrangements than Qwen3's, on the GPU.

* each built-in part against its plain function, built from a PartSpec as the model builder does;
* a run order that names a layer twice and lets the second call read the first call's cache;
* an attention window, which Qwen3 does not have, through the same part and cache manager;
* a toy mixer with a per-request state of its own, a toy position encoding and a toy architecture,
  all defined HERE and registered from outside: built, loaded with random weights, and stepped
  through the framework's step function without a change to the framework's files.
"""

import dataclasses

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import tolerances
import trace_helpers as th
from conftest import TINY_B, load_plain_weights

pytestmark = pytest.mark.gpu
F64 = torch.float64


def close(got, want, rel, what=""):
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= rel, f"{what}: relative error {err:.3e} > {rel:.0e}"
    if rel >= 1e-3:
        print(f"[observed] {what}: {err:.3e} (allowed {rel:.0e})")


class FakeBatch:
    num_tokens = 0


def make_ctx(T, mode="float32"):
    from tie_amd.parts.base import StepContext, Workspace

    batch = FakeBatch()
    batch.num_tokens = T
    return StepContext(batch, mode, torch.device("cuda:0"), Workspace("cuda:0"), None, None)


def fetcher(tensors, mode="float32"):
    from tie_amd.weights.binder import place_tensor
    from tie_amd.weights.safetensors_io import StoredTensor

    return lambda name, role: place_tensor(StoredTensor.from_tensor(name, tensors[name]), role, mode, "cuda:0")


def test_norm_embedding_feed_forward_and_head_parts_alone():
    from tie_amd.parts import PartSpec, build_part

    g = torch.Generator().manual_seed(1)
    T, D, I, V = 7, 96, 200, 50
    w = {"n": 1 + 0.1 * torch.randn(D, generator=g), "e": torch.randn(V, D, generator=g) * 0.5,
         "g": torch.randn(I, D, generator=g) * 0.1, "u": torch.randn(I, D, generator=g) * 0.1,
         "d": torch.randn(D, I, generator=g) * 0.1, "h": torch.randn(V, D, generator=g) * 0.1}
    fetch = fetcher(w)
    ctx = make_ctx(T)
    x = torch.randn(T, D, generator=g)

    norm = build_part("norm", PartSpec("rms_norm", {"dim": D, "eps": 1e-5, "weight": "n"}))
    assert [(s.name, s.shape, s.role) for s in norm.tensors()] == [("n", (D,), "vector")]
    norm.load_all(fetch, "float32", "cuda:0")
    close(norm.forward(ctx, x.cuda()), plain.rms_norm(x, w["n"], 1e-5), 1e-5, "norm part")

    emb = build_part("embedding", PartSpec("token_embedding", {"vocab": V, "hidden": D, "weight": "e"}))
    emb.load_all(fetch, "float32", "cuda:0")
    ids = [3, 49, 0, 3, 17, 8, 21]
    got = emb.forward(ctx, torch.tensor(ids, dtype=torch.int32, device="cuda"))
    assert torch.equal(got.cpu(), w["e"][ids])

    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden": D, "intermediate": I,
                                                         "names": {"gate": "g", "up": "u", "down": "d"}}))
    assert sorted(s.name for s in ffn.tensors()) == ["d", "g", "u"]
    ffn.load_all(fetch, "float32", "cuda:0")
    residual = x.cuda().clone()
    ffn.forward(ctx, x.cuda(), residual)                      # the part ADDS its result to the residual
    close(residual, x.to(F64) + plain.swiglu(x, w["g"], w["u"], w["d"]), 1e-5, "feed-forward part")

    for tied in (None, "e"):
        head = build_part("head", PartSpec("lm_head", {"vocab": V, "hidden": D, "weight": "h", "tied_to": tied,
                                                       "norm": PartSpec("rms_norm", {"dim": D, "eps": 1e-5, "weight": "n"})}))
        head.load_all(fetch, "float32", "cuda:0")
        rows = torch.tensor([6, 0, 2], dtype=torch.int32, device="cuda")
        want = plain.linear(plain.rms_norm(x[[6, 0, 2]], w["n"], 1e-5), w[tied or "h"])
        close(head.forward(ctx, x.cuda(), rows), want, 1e-5, f"head part tied={tied}")
        names = {s.name: s.optional for s in head.all_tensors()}
        assert names == ({"h": False, "n": False} if tied is None else {"e": False, "h": True, "n": False})


@pytest.mark.parametrize("T", [5, 64, 100, 300])
def test_sums_a_product_leaves_owed_reach_the_stream_through_the_norm_or_settle(T):
    """bfloat16, a long K: the down projection comes as planes of partial sums (decode product up to 64
    rows, tiled product above) that the next norm adds - or ``settle`` does, for parts that know nothing of it."""
    from tie_amd.parts import PartSpec, build_part

    g = torch.Generator().manual_seed(3)
    D, I = 256, 1024
    w = {"n": 1 + 0.1 * torch.randn(D, generator=g), "g": torch.randn(I, D, generator=g) * 0.05,
         "u": torch.randn(I, D, generator=g) * 0.05, "d": torch.randn(D, I, generator=g) * 0.05}
    w = {k: (v.to(torch.bfloat16) if k != "n" else v) for k, v in w.items()}
    fetch = fetcher(w, "bfloat16")
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden": D, "intermediate": I,
                                                         "names": {"gate": "g", "up": "u", "down": "d"}}))
    norm = build_part("norm", PartSpec("rms_norm", {"dim": D, "eps": 1e-5, "weight": "n"}))
    ffn.load_all(fetch, "bfloat16", "cuda:0")
    norm.load_all(fetch, "bfloat16", "cuda:0")
    x = torch.randn(T, D, generator=g)
    h = x.to(torch.bfloat16)
    want = x.to(F64) + plain.swiglu(h.to(F64), w["g"], w["u"], w["d"])

    ctx = make_ctx(T, "bfloat16")
    residual = x.cuda().clone()
    ffn.forward(ctx, h.cuda(), residual)
    # up to 16 rows the whole product is still to be launched (the next norm may ask for it with its own work in
    # the epilogue); above, its planes of partial sums are owed
    assert (ctx._pending if T <= 16 else ctx._owed) is not None, \
        "a product over 1024 of K at this size is expected to leave its sum owed"
    assert torch.equal(residual.cpu(), x)                          # nothing added yet
    normed = norm.forward(ctx, residual)                           # adds what is owed, then normalises
    assert ctx._owed is None and ctx._pending is None
    close(residual, want, 2e-3, "stream after the norm took the owed sums")
    close(normed, plain.rms_norm(want, w["n"].to(F64), 1e-5), 1e-2, "norm of the updated stream")

    ctx = make_ctx(T, "bfloat16")
    residual2 = x.cuda().clone()
    ffn.forward(ctx, h.cuda(), residual2)
    ctx.settle()                                                   # what a block does before a part that does not know
    assert ctx._owed is None and ctx._pending is None and torch.equal(residual2, residual)


@pytest.mark.parametrize("T", [4, 200])
def test_two_products_in_a_row_that_leave_their_sums_owed(T):
    """Two accumulating projections into one stream with no norm between them (a parallel residual, shared
    beside routed experts): the first one's planes must reach the stream before the second reuses their buffer."""
    from tie_amd.parts.linear import Linear

    g = torch.Generator().manual_seed(5)
    D, K = 256, 1024
    w = {"a": (torch.randn(D, K, generator=g) * 0.05).to(torch.bfloat16),
         "b": (torch.randn(D, K, generator=g) * 0.05).to(torch.bfloat16)}
    fetch = fetcher(w, "bfloat16")
    first, second = Linear(["a"], [D], K), Linear(["b"], [D], K)
    first.load(fetch)
    second.load(fetch)
    x1, x2 = torch.randn(T, K, generator=g).to(torch.bfloat16), torch.randn(T, K, generator=g).to(torch.bfloat16)
    stream = torch.randn(T, D, generator=g)
    want = stream.to(F64) + plain.linear(x1.to(F64), w["a"].to(F64)) + plain.linear(x2.to(F64), w["b"].to(F64))
    ctx = make_ctx(T, "bfloat16")
    residual = stream.cuda().clone()
    first(x1.cuda(), residual, accumulate=True, ctx=ctx)
    assert (ctx._pending if T <= 16 else ctx._owed) is not None, \
        "a product over 1024 of K at this size is expected to leave its sum owed"
    second(x2.cuda(), residual, accumulate=True, ctx=ctx)
    ctx.settle()
    close(residual, want, 2e-3, "stream after two owed products")


def test_position_part_holds_the_reference_frequencies():
    from tie_amd.parts import PartSpec, build_part

    for theta, dim in ((1e4, 16), (1e6, 128), (5e5, 80)):
        part = build_part("position", PartSpec("rope_neox", {"head_dim": dim, "theta": theta}))
        part.load_all(None, "float32", "cuda:0")
        inv_freq, rotary_dim, pairing = part.rotary_table()
        assert rotary_dim == dim and pairing == "rotate_half"
        assert np.array_equal(inv_freq.cpu().numpy(), plain.rope_inv_freq(theta, dim))   # bit for bit


# ------------------------------------------------------------------ other arrangements of the attention part
def attention_model(order, window=None, layers=2):
    """A model of ``layers`` attention + SwiGLU layers in Qwen3's tensor names with a free run order and window."""
    from tie_amd.config.qwen3 import Qwen3Config
    from tie_amd.models import LayerCall, Model
    from tie_amd.models.qwen3 import build_qwen3_spec

    cfg = dict(TINY_B, num_hidden_layers=layers)
    spec = build_qwen3_spec(Qwen3Config.from_json(cfg))
    new_layers = []
    for layer in spec.layers:
        mixer = dataclasses.replace(layer.mixer, params={**layer.mixer.params, "window": window})
        new_layers.append(dataclasses.replace(layer, mixer=mixer))
    spec = dataclasses.replace(spec, layers=tuple(new_layers), order=tuple(LayerCall(*o) for o in order))
    return Model(spec), cfg


def plain_with_order(weights, cfg, tokens, order, window=None):
    """Whole-sequence forward with a run order; a call that reads another call's cache uses its keys and values."""
    cfg = plain.normalized_config(cfg)
    T = len(tokens)
    H, KVH, Dh, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    pos = list(range(T))
    x = plain.embed(weights["model.embed_tokens.weight"], tokens)
    kept = {}
    for index, (layer, source) in enumerate(order):
        p = f"model.layers.{layer}."
        h = plain.rms_norm(x, weights[p + "input_layernorm.weight"], eps)
        q = plain.rope_neox(plain.rms_norm(plain.linear(h, weights[p + "self_attn.q_proj.weight"]).view(T, H, Dh),
                                           weights[p + "self_attn.q_norm.weight"], eps), pos, cfg["rope_theta"])
        if source is None:
            k = plain.rope_neox(plain.rms_norm(plain.linear(h, weights[p + "self_attn.k_proj.weight"]).view(T, KVH, Dh),
                                               weights[p + "self_attn.k_norm.weight"], eps), pos, cfg["rope_theta"])
            v = plain.linear(h, weights[p + "self_attn.v_proj.weight"]).view(T, KVH, Dh)
            kept[index] = (k, v)
        else:
            k, v = kept[source]
        a = plain.causal_attention(q, k, v, float(np.float32(1.0) / np.sqrt(np.float32(Dh))), window).reshape(T, H * Dh)
        x = x + plain.linear(a, weights[p + "self_attn.o_proj.weight"])
        h = plain.rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)
        x = x + plain.swiglu(h, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                             weights[p + "mlp.down_proj.weight"])
    x = plain.rms_norm(x, weights["model.norm.weight"], eps)
    return plain.linear(x, weights["lm_head.weight"])


@pytest.mark.parametrize("dtype,tolerance", [("float32", tolerances.FLOAT32), ("bfloat16", tolerances.BFLOAT16["run orders"])])
@pytest.mark.parametrize("order,window", [
    (((0, None), (1, None), (0, None)), None),            # layer 0 runs twice, each call with a cache of its own
    (((0, None), (1, None), (0, 0), (1, 1)), None),       # the later calls read the earlier calls' caches
    (((0, None), (1, None)), 7),                          # a window of 7 keys: pages go back while requests run
    (((0, None), (1, 0)), 20),
])
def test_run_orders_shared_caches_and_windows(tmp_path, order, window, dtype, tolerance):
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.loader import load_model_folder
    from tie_amd.weights.random_init import write_random_model

    model, cfg = attention_model(order, window)
    planes = sum(1 for _, src in order if src is None)
    assert model.cache_plan.groups[0].num_planes == planes and model.cache_plan.groups[0].need.window == window
    folder = write_random_model(tmp_path / "m", cfg, seed=3, dtype="float32" if dtype == "float32" else "bfloat16")
    model.load(load_model_folder(folder).tensors, dtype, "cuda:0")
    weights = load_plain_weights(folder)
    requests = th.make_requests(cfg["vocab_size"], [45, 70, 33], seed=8)
    want = {rid: plain_with_order(weights, cfg, toks, order, window).float() for rid, toks in requests.items()}
    steps, peak = th.mixed(requests, max_live=3, seed=2)
    replayer = TraceReplayer(model, peak if window is None else 96, block_size=4)   # a window needs few pages
    got = th.collect(replayer, steps)
    for rid, ref in want.items():
        mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
        close(mine, ref, tolerance, f"order {order} window {window} request {rid}")
    assert replayer.cache.num_free() == replayer.cache.num_blocks


@pytest.mark.parametrize("dtype,tolerance", [("float32", tolerances.FLOAT32), ("bfloat16", tolerances.BFLOAT16["run orders"])])
def test_projections_with_a_bias_are_a_parameter_of_the_attention_part(dtype, tolerance):
    """An architecture whose q, k, v and o projections have a bias names the vectors in the mixer's parameters:
    no kernel and no file of the package changes. Through the step function (whole, decoded, in portions, mixed)
    against the plain formulas with the bias added; and the bias must matter (without it the check fails)."""
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.models import Model
    from tie_amd.weights.random_init import random_tensors
    from tie_amd.weights.safetensors_io import StoredTensor

    model, cfg = attention_model(((0, None), (1, None)))
    layers = []
    for i, layer in enumerate(model.spec.layers):
        p = f"model.layers.{i}.self_attn."
        bias = {"q": p + "q_proj.bias", "k": p + "k_proj.bias", "v": p + "v_proj.bias", "o": p + "o_proj.bias"}
        layers.append(dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, params={**layer.mixer.params, "bias": bias})))
    model = Model(dataclasses.replace(model.spec, layers=tuple(layers)))
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    tensors = dict(random_tensors(model.expected_tensors(), 9, store, vector_dtype=torch.float32))
    for name in tensors:
        if name.endswith(".bias"):
            tensors[name] = tensors[name] * 20          # init_std 0.02 would leave the bias below the bfloat16 bound
    assert sum(name.endswith(".bias") for name in tensors) == 8
    model.load({n: StoredTensor.from_tensor(n, t) for n, t in tensors.items()}, dtype, "cuda:0")
    weights = {n: t.to(F64) for n, t in tensors.items()}

    def forward(tokens, with_bias=True):
        c = plain.normalized_config(cfg)
        T, H, KVH, Dh, eps = len(tokens), c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
        pos = list(range(T))
        x = plain.embed(weights["model.embed_tokens.weight"], tokens)
        for layer in range(2):
            p = f"model.layers.{layer}."
            b = (lambda n: weights[p + f"self_attn.{n}_proj.bias"]) if with_bias else (lambda n: 0.0)
            h = plain.rms_norm(x, weights[p + "input_layernorm.weight"], eps)
            q = plain.rope_neox(plain.rms_norm((plain.linear(h, weights[p + "self_attn.q_proj.weight"]) + b("q")).view(T, H, Dh),
                                               weights[p + "self_attn.q_norm.weight"], eps), pos, c["rope_theta"])
            k = plain.rope_neox(plain.rms_norm((plain.linear(h, weights[p + "self_attn.k_proj.weight"]) + b("k")).view(T, KVH, Dh),
                                               weights[p + "self_attn.k_norm.weight"], eps), pos, c["rope_theta"])
            v = (plain.linear(h, weights[p + "self_attn.v_proj.weight"]) + b("v")).view(T, KVH, Dh)
            a = plain.causal_attention(q, k, v, float(np.float32(1.0) / np.sqrt(np.float32(Dh))), None).reshape(T, H * Dh)
            x = x + plain.linear(a, weights[p + "self_attn.o_proj.weight"]) + b("o")
            h = plain.rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)
            x = x + plain.swiglu(h, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                                 weights[p + "mlp.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, weights["model.norm.weight"], eps), weights["lm_head.weight"])

    requests = th.make_requests(cfg["vocab_size"], [45, 70, 33], seed=8)
    want = {rid: forward(toks).float() for rid, toks in requests.items()}
    steps, peak = th.mixed(requests, max_live=3, seed=2)
    for label, trace, room in (("whole", th.whole(requests), 192), ("prefill + decode", th.prefill_then_decode(requests), 192),
                               ("mixed", steps, peak)):
        replayer = TraceReplayer(model, room, block_size=4)
        got = th.collect(replayer, trace)
        for rid, ref in want.items():
            mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
            close(mine, ref, tolerance, f"biased projections, {label}, request {rid}")
        assert replayer.cache.num_free() == replayer.cache.num_blocks
    unbiased = forward(requests["r0"], with_bias=False).float()
    assert float((unbiased - want["r0"]).abs().max() / want["r0"].abs().max()) > 10 * tolerance, "the bias does not matter"


def test_a_projection_with_a_bias_alone():
    """``Linear(bias=...)``: the product, then the bias, whether it stores, adds to a stream that planes are still
    owed to, or feeds rows that lack their norm's factor; bfloat16 and float32 rows."""
    from tie_amd import kernels
    from tie_amd.parts.linear import Linear

    g = torch.Generator().manual_seed(6)
    D, K, T = 96, 1024, 5
    w = {"a": (torch.randn(D, K, generator=g) * 0.05).to(torch.bfloat16), "a.bias": torch.randn(D, generator=g),
         "b": (torch.randn(D, K, generator=g) * 0.05).to(torch.bfloat16)}
    fetch = fetcher(w, "bfloat16")
    biased, plain_one = Linear(["a"], [D], K, bias=["a.bias"]), Linear(["b"], [D], K)
    biased.load(fetch)
    plain_one.load(fetch)
    assert [s.name for s in biased.tensors()] == ["a", "a.bias"] and biased.tensors()[1].shape == (D,)
    x = torch.randn(T, K, generator=g).to(torch.bfloat16)
    product = plain.linear(x.to(F64), w["a"].to(F64)) + w["a.bias"].to(F64)
    for out_dtype, bound in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out = torch.full((T, D), float("nan"), dtype=out_dtype, device="cuda")
        biased(x.cuda(), out)
        close(out, product, bound, f"biased product stored as {out_dtype}")
    ctx = make_ctx(T, "bfloat16")
    stream = torch.randn(T, D, generator=g)
    residual = stream.cuda().clone()
    plain_one(x.cuda(), residual, accumulate=True, ctx=ctx)           # left pending or owed
    biased(x.cuda(), residual, accumulate=True, ctx=ctx)
    assert ctx._owed is None and ctx._pending is None and biased.partial_planes(ctx, x.cuda(), "p") is None
    close(residual, stream.to(F64) + plain.linear(x.to(F64), w["b"].to(F64)) + product, 1e-5, "stream after both")
    with pytest.raises(kernels.InvalidArgument):
        Linear(["a", "b"], [D, D], K, bias=["a.bias"])
    with pytest.raises(kernels.InvalidArgument):
        kernels.add_bias(torch.zeros(T, D, device="cuda"), torch.zeros(D + 1, device="cuda"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_a_mixer_alone_and_of_a_feed_forward_alone(tmp_path, dtype):
    """A layer may hold a mixer without a feed-forward or the other way round (an architecture that interleaves
    them otherwise than in pairs; two mixers with caches of their own in what another framework calls one layer).
    Qwen3's layers cut into such halves, twice as many entries in the run order, are the same model: the same
    bits as the whole layers give, through a mixed trace with pages used again."""
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.models import LayerCall, LayerSpec, Model
    from tie_amd.weights.loader import load_model_folder
    from tie_amd.weights.random_init import write_random_model

    whole, cfg = attention_model(((0, None), (1, None), (2, None)), layers=3)
    halves = []
    for layer in whole.spec.layers:
        halves.append(LayerSpec(layer.block, layer.mixer, None, {"pre_mixer": layer.norms["pre_mixer"]}))
        halves.append(LayerSpec(layer.block, None, layer.feed_forward, {"pre_feed_forward": layer.norms["pre_feed_forward"]}))
    cut = Model(dataclasses.replace(whole.spec, layers=tuple(halves), order=tuple(LayerCall(i) for i in range(6))))
    assert [g.num_planes for g in cut.cache_plan.groups] == [3]          # the halves without a mixer need no cache
    with pytest.raises(Exception, match="pre_mixer"):
        Model(dataclasses.replace(whole.spec, layers=(LayerSpec(whole.spec.layers[0].block, whole.spec.layers[0].mixer, None, {}),),
                                  order=(LayerCall(0),)))
    folder = write_random_model(tmp_path / "m", cfg, seed=5, dtype=dtype)
    files = load_model_folder(folder)
    whole.load(files.tensors, dtype, "cuda:0")
    cut.load(files.tensors, dtype, "cuda:0")
    requests = th.make_requests(cfg["vocab_size"], [45, 70, 33, 12], seed=10)
    steps, peak = th.mixed(requests, max_live=3, seed=6)
    got = {}
    for name, model in (("whole", whole), ("cut", cut)):
        replayer = TraceReplayer(model, peak, block_size=16)
        got[name] = th.collect(replayer, steps)
        assert replayer.cache.num_free() == replayer.cache.num_blocks
    for rid in requests:
        for p in got["whole"][rid]:
            assert torch.equal(got["whole"][rid][p], got["cut"][rid][p]), f"request {rid}, position {p}"


# ------------------------------------------------------------------ toy parts, defined and registered here
def register_toy_parts():
    from tie_amd import kernels
    from tie_amd.cache.spec import FixedState
    from tie_amd.parts import FeedForward, Mixer, Position, TensorSpec, register_part

    @register_part("mixer", "toy_decay_undeclared")
    class ToyDecayMixerThatSaysNothing(Mixer):
        """s_t = decay * s_{t-1} + W_in h_t ; out_t = W_out s_t, with s kept per request in a state slot.

        It walks the step's sequences on the host, so a recording of it would hold one step's slots for good -
        and it is written as by someone who never heard of recording: it says nothing about ``capturable``.
        The default must keep it out of HIP graphs."""

        def __init__(self, params):
            super().__init__(params)
            self.hidden, self.width, self.decay = params["hidden"], params["width"], params["decay"]
            self.names = params["names"]

        def cache_need(self):
            return FixedState((self.width,), "float32")

        def tensors(self):
            return [TensorSpec(self.names["in"], (self.width, self.hidden), "matrix", ("normal", 0.2)),
                    TensorSpec(self.names["out"], (self.hidden, self.width), "matrix", ("normal", 0.2))]

        def load(self, fetch, mode, device):
            self.w_in, self.w_out = fetch(self.names["in"], "matrix"), fetch(self.names["out"], "matrix")

        def forward(self, ctx, h, cache, residual):
            u = h.float() @ self.w_in.float().T                               # [T, width]
            row = 0
            for n, slot in zip(ctx.batch.host_new_tokens, ctx.batch.host_state_slots):
                state = cache.state[slot]                                     # carried across portions and steps
                for t in range(row, row + n):                                 # tokens of a sequence in order
                    state.mul_(self.decay).add_(u[t])
                    residual[t] += state @ self.w_out.float().T
                row += n

    assert not any("capturable" in vars(c) for c in ToyDecayMixerThatSaysNothing.__mro__ if c.__module__ == __name__)

    @register_part("mixer", "toy_decay")
    class ToyDecayMixer(ToyDecayMixerThatSaysNothing):
        """The same, by an author who knows that it cannot be recorded and says so."""

        capturable = False

    @register_part("mixer", "toy_decay_on_device")
    class ToyDecayMixerOnDevice(ToyDecayMixer):
        """The same mixer written so that decode-only steps may be recorded: there, one row a sequence, the
        states are gathered and scattered by the step's slot array ON THE DEVICE, and nothing of the step is
        read on the host. (Steps with prompt portions are never recorded and take the loop above.)"""

        capturable = True

        def forward(self, ctx, h, cache, residual):
            if not ctx.batch.all_decode:
                return super().forward(ctx, h, cache, residual)
            slots = cache.state_slots.long()
            state = cache.state.index_select(0, slots) * self.decay + h.float() @ self.w_in.float().T
            cache.state.index_copy_(0, slots, state)
            residual += state @ self.w_out.float().T

    @register_part("feed_forward", "toy_routed")
    class ToyRoutedFeedForward(FeedForward):
        """Router logits in float32, the top k experts per token, softmax over the chosen, ReLU experts.

        ``nonzero`` waits for the GPU, so a model with this part runs every step eagerly."""

        capturable = False

        def __init__(self, params):
            super().__init__(params)
            self.hidden, self.width = params["hidden"], params["width"]
            self.experts, self.top_k, self.names = params["experts"], params["top_k"], params["names"]

        def tensors(self):
            specs = [TensorSpec(self.names["router"], (self.experts, self.hidden), "matrix", ("normal", 0.5))]
            for e in range(self.experts):                      # expert weights: ordinary tensors with an index in the name
                specs.append(TensorSpec(self.names["w1"].format(e=e), (self.width, self.hidden), "matrix", ("normal", 0.2)))
                specs.append(TensorSpec(self.names["w2"].format(e=e), (self.hidden, self.width), "matrix", ("normal", 0.2)))
            return specs

        def load(self, fetch, mode, device):
            self.router = fetch(self.names["router"], "matrix")
            self.w1 = [fetch(self.names["w1"].format(e=e), "matrix") for e in range(self.experts)]
            self.w2 = [fetch(self.names["w2"].format(e=e), "matrix") for e in range(self.experts)]

        def forward(self, ctx, h, residual):
            T = h.shape[0]
            logits = ctx.scratch("toy_routed.logits", (T, self.experts), torch.float32)
            kernels.linear(h, self.router, logits)                                  # the framework's own product
            top, chosen = torch.topk(logits, self.top_k, dim=1)
            gate = torch.softmax(top, dim=1)
            for e in range(self.experts):
                rows, slot = (chosen == e).nonzero(as_tuple=True)
                if rows.numel() == 0:
                    continue
                x = h[rows].contiguous()
                mid = torch.empty(rows.numel(), self.width, dtype=h.dtype, device=h.device)
                kernels.linear(x, self.w1[e], mid)
                mid.clamp_(min=0)
                out = torch.empty(rows.numel(), self.hidden, dtype=torch.float32, device=h.device)
                kernels.linear(mid, self.w2[e], out)
                residual.index_add_(0, rows, out * gate[rows, slot][:, None])

    @register_part("position", "toy_shift")
    class ToyShiftPosition(Position):
        """Not a rotation: adds position * slope to the first dimension of every query and key head."""

        capturable = True         # torch operations on the step's device arrays only

        def __init__(self, params):
            super().__init__(params)
            self.slope = params["slope"]

        def apply(self, ctx, q, k, positions):
            shift = positions.float() * self.slope
            q[:, :, 0] += shift[:, None]
            k[:, :, 0] += shift[:, None]


def unregister_toy_parts():
    from tie_amd.parts import unregister_part

    unregister_part("mixer", "toy_decay")
    unregister_part("mixer", "toy_decay_on_device")
    unregister_part("mixer", "toy_decay_undeclared")
    unregister_part("feed_forward", "toy_routed")
    unregister_part("position", "toy_shift")


def toy_spec(cfg):
    from tie_amd.models import LayerCall, LayerSpec, ModelSpec
    from tie_amd.parts import PartSpec

    D, eps = cfg["hidden_size"], cfg["eps"]
    norm = lambda name: PartSpec("rms_norm", {"dim": D, "eps": eps, "weight": name})
    layers = []
    for l, kind in enumerate(cfg["mixers"]):
        p = f"layers.{l}."
        if kind in ("decay", "decay_on_device", "decay_undeclared"):
            mixer = PartSpec("toy_" + kind, {"hidden": D, "width": cfg["state_width"], "decay": cfg["decay"],
                                           "names": {"in": p + "mix.in", "out": p + "mix.out"}})
        else:
            mixer = PartSpec("paged_attention", {
                "hidden": D, "num_heads": cfg["heads"], "num_kv_heads": cfg["kv_heads"], "head_dim": cfg["head_dim"],
                "scale": cfg["head_dim"] ** -0.5, "window": None, "qk_norm": None,
                "position": PartSpec("toy_shift", {"slope": cfg["slope"]}),
                "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}})
        if cfg["feed_forwards"][l] == "routed":
            ffn = PartSpec("toy_routed", {"hidden": D, "width": cfg["expert_width"], "experts": cfg["experts"],
                                          "top_k": cfg["top_k"],
                                          "names": {"router": p + "router", "w1": p + "experts.{e}.w1",
                                                    "w2": p + "experts.{e}.w2"}})
        else:
            ffn = PartSpec("swiglu", {"hidden": D, "intermediate": cfg["intermediate"],
                                      "names": {"gate": p + "gate", "up": p + "up", "down": p + "down"}})
        layers.append(LayerSpec(PartSpec("pre_norm"), mixer, ffn,
                                {"pre_mixer": norm(p + "n1"), "pre_feed_forward": norm(p + "n2")}))
    return ModelSpec("ToyStateLM", cfg["vocab_size"], D, cfg["max_positions"],
                     PartSpec("token_embedding", {"vocab": cfg["vocab_size"], "hidden": D, "weight": "embed"}),
                     tuple(layers), tuple(LayerCall(l) for l in range(len(layers))),
                     PartSpec("lm_head", {"vocab": cfg["vocab_size"], "hidden": D, "norm": norm("final_norm"),
                                          "weight": "head", "tied_to": "embed"}))


def toy_plain(weights, cfg, tokens):
    T, D = len(tokens), cfg["hidden_size"]
    x = plain.embed(weights["embed"], tokens)
    for l, kind in enumerate(cfg["mixers"]):
        p = f"layers.{l}."
        h = plain.rms_norm(x, weights[p + "n1"], cfg["eps"])
        if kind in ("decay", "decay_on_device", "decay_undeclared"):
            u = plain.linear(h, weights[p + "mix.in"])
            s = torch.zeros(cfg["state_width"], dtype=F64)
            out = []
            for t in range(T):
                s = cfg["decay"] * s + u[t]
                out.append(plain.linear(s[None], weights[p + "mix.out"])[0])
            x = x + torch.stack(out)
        else:
            H, KVH, Dh = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
            q = plain.linear(h, weights[p + "q"]).view(T, H, Dh).clone()
            k = plain.linear(h, weights[p + "k"]).view(T, KVH, Dh).clone()
            v = plain.linear(h, weights[p + "v"]).view(T, KVH, Dh)
            shift = torch.arange(T, dtype=F64) * cfg["slope"]
            q[:, :, 0] += shift[:, None]
            k[:, :, 0] += shift[:, None]
            a = plain.causal_attention(q, k, v, Dh ** -0.5).reshape(T, H * Dh)
            x = x + plain.linear(a, weights[p + "o"])
        h = plain.rms_norm(x, weights[p + "n2"], cfg["eps"])
        if cfg["feed_forwards"][l] == "routed":
            logits = plain.linear(h, weights[p + "router"])
            top, chosen = torch.topk(logits, cfg["top_k"], dim=1)
            gate = torch.softmax(top, dim=1)
            out = torch.zeros_like(x)
            for t in range(T):
                for j in range(cfg["top_k"]):
                    e = int(chosen[t, j])
                    mid = plain.linear(h[t:t + 1], weights[p + f"experts.{e}.w1"]).clamp(min=0)
                    out[t] += gate[t, j] * plain.linear(mid, weights[p + f"experts.{e}.w2"])[0]
            x = x + out
        else:
            x = x + plain.swiglu(h, weights[p + "gate"], weights[p + "up"], weights[p + "down"])
    return plain.linear(plain.rms_norm(x, weights["final_norm"], cfg["eps"]), weights["embed"])


def test_a_toy_architecture_registered_from_outside_runs_through_the_step_function(tmp_path):
    from tie_amd.cache.spec import FixedState, PagedKV
    from tie_amd.config.registry import register_architecture, unregister_architecture
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.random_init import write_random_model

    register_toy_parts()
    register_architecture("ToyStateLM", lambda values: dict(values), toy_spec, model_types=("toy_state",))
    try:
        cfg = {"architectures": ["ToyStateLM"], "vocab_size": 90, "hidden_size": 48, "intermediate": 72,
               "heads": 3, "kv_heads": 1, "head_dim": 16, "state_width": 20, "decay": 0.8, "slope": 0.01,
               "eps": 1e-5, "max_positions": 256, "mixers": ["decay", "attention", "decay"],
               "feed_forwards": ["dense", "routed", "routed"], "experts": 5, "top_k": 2, "expert_width": 24}
        folder = write_random_model(tmp_path / "toy", cfg, seed=4, dtype="float32")   # the parts' TensorSpecs drive it
        replayer = TraceReplayer.from_folder(folder, "float32", 192, block_size=4)    # config.json names the class
        plan = replayer.model.cache_plan
        assert [type(g.need) for g in plan.groups] == [FixedState, PagedKV] and plan.groups[0].num_planes == 2
        weights = load_plain_weights(folder)
        requests = th.make_requests(cfg["vocab_size"], [40, 64, 23, 51], seed=6)
        want = {rid: toy_plain(weights, cfg, toks).float() for rid, toks in requests.items()}
        steps, peak = th.mixed(requests, max_live=3, seed=5)          # portions beside single tokens; slots reused
        got = th.collect(replayer, steps)
        for rid, ref in want.items():
            mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
            close(mine, ref, 1e-4, f"toy model request {rid}")
        assert replayer.cache.num_free_state_slots == replayer.cache.max_state_slots
        # generation through the engine works for it too: the scheduler hands out and takes back state slots
        import tie_amd
        engine = tie_amd.create_engine(replayer.model, kv_blocks=64, block_size=4, max_seqs=2, max_tokens_per_step=16)
        prompt = requests["r2"]
        out = engine.generate(prompt, tie_amd.SamplingParams(max_tokens=5))
        tokens = list(prompt)
        for t in out:
            assert t == int(torch.argmax(toy_plain(weights, cfg, tokens)[-1]))
            tokens.append(t)
    finally:
        unregister_architecture("ToyStateLM")
        unregister_toy_parts()


def changing_live_sets(requests, head, subsets):
    """A trace: every request's first ``head[id]`` tokens in one mixed step, then decode-only steps over the
    live subsets named in turn (so equal step shapes meet different requests and state slots), then the rest."""
    steps = [{"step": 0, "entries": [{"id": r, "tokens": requests[r][:head[r]], "want": list(range(head[r]))}
                                      for r in requests], "end": []}]
    pos = dict(head)
    k = 0
    while any(pos[r] < len(requests[r]) for r in requests):
        chosen = [r for r in subsets[k % len(subsets)] if pos[r] < len(requests[r])]
        k += 1
        if not chosen:
            continue
        entries = [{"id": r, "tokens": [requests[r][pos[r]]], "want": [0]} for r in chosen]
        for r in chosen:
            pos[r] += 1
        steps.append({"step": len(steps), "entries": entries, "end": [r for r in chosen if pos[r] == len(requests[r])]})
    return steps


@pytest.mark.parametrize("kind", ["recorded", "eager", "undeclared"])
def test_the_toy_architecture_in_bfloat16_with_recorded_decode_steps(tmp_path, kind):
    """The serving precision, where decode-only steps are recorded and replayed. A model whose parts all read
    the step on the device is recorded, and replays must follow the step's slots as the live set changes; a
    model with one part that reads the step on the host (or waits for the GPU) must not be recorded at all -
    whether that part says so ("eager") or says nothing ("undeclared": every other part of that model could be
    recorded, so only the default keeps the host-side walk over the state slots out of a graph)."""
    import tie_amd
    from tie_amd.config.registry import register_architecture, unregister_architecture
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.random_init import write_random_model

    register_toy_parts()
    register_architecture("ToyStateLM", lambda values: dict(values), toy_spec, model_types=("toy_state",))
    try:
        cfg = {"architectures": ["ToyStateLM"], "vocab_size": 90, "hidden_size": 48, "intermediate": 72,
               "heads": 3, "kv_heads": 1, "head_dim": 16, "state_width": 20, "decay": 0.8, "slope": 0.01,
               "eps": 1e-5, "max_positions": 256, "experts": 5, "top_k": 2, "expert_width": 24}
        if kind == "recorded":
            cfg.update(mixers=["decay_on_device", "attention", "decay_on_device"], feed_forwards=["dense"] * 3)
        elif kind == "undeclared":
            cfg.update(mixers=["decay_on_device", "attention", "decay_undeclared"], feed_forwards=["dense"] * 3)
        else:
            cfg.update(mixers=["decay", "attention", "decay_on_device"], feed_forwards=["dense", "routed", "dense"])
        folder = write_random_model(tmp_path / "toy", cfg, seed=4, dtype="bfloat16")
        replayer = TraceReplayer.from_folder(folder, "bfloat16", 256, block_size=4)
        assert replayer.runner.use_graphs == (kind == "recorded")
        weights = load_plain_weights(folder)
        requests = th.make_requests(cfg["vocab_size"], [40, 52, 31, 44], seed=6)
        want = {rid: toy_plain(weights, cfg, toks).float() for rid, toks in requests.items()}
        head = {"r0": 20, "r1": 30, "r2": 12, "r3": 25}
        subsets = [("r0", "r1"), ("r2", "r3"), ("r1", "r2"), ("r3", "r0"), ("r0", "r1", "r2"), ("r3", "r2", "r1"),
                   ("r2",), ("r0",), ("r0", "r1", "r2", "r3"), ("r3", "r1", "r0", "r2")]
        got = th.collect(replayer, changing_live_sets(requests, head, subsets))
        for rid, ref in want.items():
            mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
            close(mine, ref, tolerances.BFLOAT16["toy architecture"], f"toy model in bfloat16 ({kind}), request {rid}")
        assert replayer.cache.num_free_state_slots == replayer.cache.max_state_slots
        assert (replayer.runner.graph_replays > 20) == (kind == "recorded")
        # and through the engine, whose scheduler hands the slots out; recording can also be switched off there
        for use_graphs in (None, False):
            engine = tie_amd.create_engine(replayer.model, kv_blocks=64, block_size=4, max_seqs=2,
                                           max_tokens_per_step=16, use_graphs=use_graphs)
            assert engine.runner.use_graphs == (kind == "recorded" and use_graphs is None)
            prompt = requests["r2"]
            out = engine.generate(prompt, tie_amd.SamplingParams(max_tokens=6))
            tokens = list(prompt)
            for t in out:
                row = toy_plain(weights, cfg, tokens)[-1]
                assert float(row.max() - row[t]) <= tolerances.BFLOAT16["toy architecture"] * float(row.abs().max()), \
                    "a token the plain logits do not favour"
                tokens.append(t)
    finally:
        unregister_architecture("ToyStateLM")
        unregister_toy_parts()


# ------------------------------------------------------------------ a norm and an arrangement of other kinds
@pytest.mark.parametrize("dtype,tolerance", [("float32", tolerances.FLOAT32), ("bfloat16", tolerances.BFLOAT16["toy architecture"])])
def test_a_toy_norm_and_a_toy_arrangement_registered_from_outside(dtype, tolerance):
    """A layer norm with a bias (mean and variance: not of the form the products' epilogues can finish) and an
    arrangement with one norm and a parallel residual, ``x += mixer(norm(x)) + feed_forward(norm(x))``, both
    written here with torch operations and without a word about owed sums, pending products, row scales or
    recording: the framework's attention and SwiGLU parts run inside them, the debts are settled before the
    foreign norm reads the stream, and every step stays eager. Against plain formulas, in every way of cutting."""
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.models import LayerCall, LayerSpec, Model, ModelSpec
    from tie_amd.parts import PartSpec, register_part, unregister_part
    from tie_amd.parts.base import Block, Norm, TensorSpec
    from tie_amd.weights.random_init import random_tensors
    from tie_amd.weights.safetensors_io import StoredTensor

    @register_part("norm", "toy_layer_norm")
    class ToyLayerNorm(Norm):
        def __init__(self, params):
            super().__init__(params)
            self.dim, self.eps = int(params["dim"]), float(params["eps"])
            self.names = (params["weight"], params["bias"])

        def tensors(self):
            return [TensorSpec(self.names[0], (self.dim,), "vector", ("one_plus_uniform", 0.1)),
                    TensorSpec(self.names[1], (self.dim,), "vector", ("normal", 0.1))]

        def load(self, fetch, mode, device):
            self.weight, self.bias = fetch(self.names[0], "vector"), fetch(self.names[1], "vector")

        def forward(self, ctx, x, rows=None, out_name="norm.out", out_dtype=None):
            src = x if rows is None else x.index_select(0, rows.long())
            y = torch.nn.functional.layer_norm(src.float(), (self.dim,), self.weight, self.bias, self.eps)
            return y.to(out_dtype or ctx.act_dtype)

    @register_part("block", "toy_parallel")
    class ToyParallelBlock(Block):
        def forward(self, ctx, x, layer, cache):
            h = self.normed(ctx, layer.norms["only"], x, consumer=None)
            layer.mixer.forward(ctx, h, cache, x)
            layer.feed_forward.forward(ctx, h, x)

    try:
        D, H, KVH, Dh, I, V, eps, L = 96, 6, 2, 32, 160, 211, 1e-5, 3
        norm = lambda w, b: PartSpec("toy_layer_norm", {"dim": D, "eps": eps, "weight": w, "bias": b})
        layers = []
        for l in range(L):
            p = f"layers.{l}."
            mixer = PartSpec("paged_attention", {
                "hidden": D, "num_heads": H, "num_kv_heads": KVH, "head_dim": Dh, "scale": Dh ** -0.5, "window": None,
                "qk_norm": None, "position": PartSpec("rope_neox", {"head_dim": Dh, "theta": 10000.0}),
                "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}})
            ffn = PartSpec("swiglu", {"hidden": D, "intermediate": I, "names": {"gate": p + "gate", "up": p + "up", "down": p + "down"}})
            layers.append(LayerSpec(PartSpec("toy_parallel"), mixer, ffn, {"only": norm(p + "ln.w", p + "ln.b")}))
        spec = ModelSpec("ToyParallelLM", V, D, 256, PartSpec("token_embedding", {"vocab": V, "hidden": D, "weight": "embed"}),
                         tuple(layers), tuple(LayerCall(l) for l in range(L)),
                         PartSpec("lm_head", {"vocab": V, "hidden": D, "norm": norm("final.w", "final.b"), "weight": "head",
                                              "tied_to": None}))
        model = Model(spec)
        assert not model.capturable()                     # the toy parts declare nothing: no step is recorded
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        tensors = dict(random_tensors(model.expected_tensors(), 4, store, vector_dtype=torch.float32))
        model.load({n: StoredTensor.from_tensor(n, t) for n, t in tensors.items()}, dtype, "cuda:0")
        w = {n: t.to(F64) for n, t in tensors.items()}

        def layer_norm(x, weight, bias):
            mean = x.mean(-1, keepdim=True)
            var = ((x - mean) ** 2).mean(-1, keepdim=True)
            return (x - mean) / torch.sqrt(var + eps) * weight + bias

        def forward(tokens):
            T = len(tokens)
            pos = list(range(T))
            x = plain.embed(w["embed"], tokens)
            for l in range(L):
                p = f"layers.{l}."
                h = layer_norm(x, w[p + "ln.w"], w[p + "ln.b"])
                q = plain.rope_neox(plain.linear(h, w[p + "q"]).view(T, H, Dh), pos, 10000.0)
                k = plain.rope_neox(plain.linear(h, w[p + "k"]).view(T, KVH, Dh), pos, 10000.0)
                v = plain.linear(h, w[p + "v"]).view(T, KVH, Dh)
                a = plain.causal_attention(q, k, v, Dh ** -0.5).reshape(T, H * Dh)
                x = x + plain.linear(a, w[p + "o"]) + plain.swiglu(h, w[p + "gate"], w[p + "up"], w[p + "down"])
            return plain.linear(layer_norm(x, w["final.w"], w["final.b"]), w["head"])

        requests = th.make_requests(V, [45, 70, 33, 9], seed=12)
        want = {rid: forward(toks).float() for rid, toks in requests.items()}
        steps, peak = th.mixed(requests, max_live=3, seed=4)
        for label, trace, room in (("whole", th.whole(requests), 256), ("prefill + decode", th.prefill_then_decode(requests), 256),
                                   ("portions", th.portions(requests), 256), ("mixed", steps, peak)):
            replayer = TraceReplayer(model, room, block_size=16)
            got = th.collect(replayer, trace)
            for rid, ref in want.items():
                mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
                close(mine, ref, tolerance, f"toy norm and arrangement, {label}, request {rid}")
            assert replayer.cache.num_free() == replayer.cache.num_blocks
            assert replayer.runner.graph_replays == 0
    finally:
        unregister_part("norm", "toy_layer_norm")
        unregister_part("block", "toy_parallel")
