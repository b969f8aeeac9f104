"""Each kernel alone against its plain reference, at sizes other than the engine's.

Head sizes in steps of 16, head counts and groupings that are no powers of two, widths and
vocabularies with tails, scattered and unordered block tables, windows. Where random data would
hide a fault (a far key among hundreds, a window's edge, a page of the cache) the inputs are made
so that it shows.
"""

import math

import numpy as np
import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def close(got, want, rel, what=""):
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= rel, f"{what}: relative error {err:.3e} > {rel:.0e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    from tie_amd import kernels

    table = rnd(37, 100, seed=1, dtype=dtype).cuda()
    ids = i32([3, 0, 36, 3, 17])
    out = torch.empty(5, 100, dtype=torch.float32, device="cuda")
    kernels.embed(table, ids, out)
    assert torch.equal(out.cpu(), table.cpu().float()[ids.cpu().long()])


@pytest.mark.parametrize("n", [16, 100, 1000, 4096, 5120])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rms_norm(n, out_dtype):
    from tie_amd import kernels

    x = rnd(7, n, seed=2, scale=3.0).cuda()
    w = (1 + 0.1 * rnd(n, seed=3)).cuda()
    out = torch.empty(7, n, dtype=out_dtype, device="cuda")
    kernels.rms_norm(x, w, 1e-5, out)
    want = plain.rms_norm(x.cpu(), w.cpu(), 1e-5)
    close(out, want, 1e-5 if out_dtype == torch.float32 else 5e-3, f"rms_norm n={n}")
    rows = i32([6, 0, 3])
    picked = torch.empty(3, n, dtype=out_dtype, device="cuda")
    kernels.rms_norm(x, w, 1e-5, picked, rows)
    assert torch.equal(picked, out[rows.long()])


def test_swiglu():
    from tie_amd import kernels

    gu = rnd(5, 2 * 200, seed=4, scale=2.0).cuda()
    out = torch.empty(5, 200, dtype=torch.float32, device="cuda")
    kernels.swiglu(gu, out)
    g, u = gu.cpu().to(F64)[:, :200], gu.cpu().to(F64)[:, 200:]
    close(out, g / (1 + torch.exp(-g)) * u, 1e-6, "swiglu")
    zero = torch.zeros(1, 8, device="cuda")
    z = torch.empty(1, 4, device="cuda")
    kernels.swiglu(zero, z)
    assert float(z.abs().max()) == 0.0


@pytest.mark.parametrize("T,N,K", [(1, 64, 64), (5, 70, 100), (64, 64, 16), (130, 200, 96), (3, 384, 200)])
@pytest.mark.parametrize("dtypes", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                    (torch.bfloat16, torch.float32)])
def test_gemm_generic(T, N, K, dtypes):
    from tie_amd import kernels

    x = rnd(T, K, seed=5, dtype=dtypes[0]).cuda()
    w = rnd(N, K, seed=6, scale=0.1, dtype=dtypes[1]).cuda()
    out = torch.empty(T, N, dtype=torch.float32, device="cuda")
    kernels.gemm_generic(x, w, out)
    want = plain.linear(x.cpu(), w.cpu())
    close(out, want, 2e-6, f"gemm {T}x{N}x{K}")
    base = rnd(T, N, seed=7).cuda()
    acc = base.clone()
    kernels.gemm_generic(x, w, acc, accumulate=True)
    close(acc, want + base.cpu().to(F64), 2e-6, "gemm accumulate")
    # a row's result does not depend on the other rows of the call
    one = torch.empty(1, N, dtype=torch.float32, device="cuda")
    kernels.gemm_generic(x[T - 1:T].contiguous(), w, one)
    assert torch.equal(one[0], out[T - 1])


@pytest.mark.parametrize("H,KVH,Dh,bs", [(4, 2, 16, 4), (6, 2, 32, 16), (3, 1, 48, 8), (5, 5, 80, 16), (8, 2, 128, 16),
                                         (2, 1, 256, 4), (2, 2, 512, 2)])
def test_qk_norm_rope_kv_write(H, KVH, Dh, bs):
    from tie_amd import kernels

    T, eps, theta = 6, 1e-5, 1e4
    qkv = rnd(T, (H + 2 * KVH) * Dh, seed=8, scale=2.0).cuda()
    qw, kw = (1 + 0.1 * rnd(Dh, seed=9)).cuda(), (1 + 0.1 * rnd(Dh, seed=10)).cuda()
    positions = [0, 1, 5, 77, 300, 4095]
    slots = [9, 2, 31, 4, 17, 0]
    inv_freq = torch.from_numpy(plain.rope_inv_freq(theta, Dh)).cuda()
    NB = 32 // bs + 1
    kc = torch.zeros(NB, KVH, bs, Dh, device="cuda")
    vc = torch.zeros(NB, KVH, Dh, bs, device="cuda")           # values lie transposed inside a page
    q = torch.empty(T, H * Dh, device="cuda")
    kernels.qk_norm_rope_kv_write(qkv, q, qw, kw, eps, inv_freq, i32(positions), i32(slots), kc, vc, H, KVH, Dh, bs)
    x = qkv.cpu()
    q_in = x[:, :H * Dh].view(T, H, Dh)
    k_in = x[:, H * Dh:(H + KVH) * Dh].view(T, KVH, Dh)
    v_in = x[:, (H + KVH) * Dh:].view(T, KVH, Dh)
    q_want = plain.rope_neox(plain.rms_norm(q_in, qw.cpu(), eps), positions, theta)
    k_want = plain.rope_neox(plain.rms_norm(k_in, kw.cpu(), eps), positions, theta)
    close(q.view(T, H, Dh), q_want, 2e-6, "q")
    for t, slot in enumerate(slots):                          # ((page*KVH + h)*bs + offset)*Dh
        close(kc[slot // bs, :, slot % bs], k_want[t], 2e-6, f"k of token {t}")
        assert torch.equal(vc[slot // bs, :, :, slot % bs].cpu(), v_in[t])
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots] = True
    assert float(kc.cpu().view(NB, KVH, bs, Dh).permute(0, 2, 1, 3).reshape(NB * bs, -1)[~written].abs().max()) == 0.0
    # without norm weights and frequencies it is a plain copy; position 0 is the identity of the rotation
    q2 = torch.empty_like(q)
    kernels.qk_norm_rope_kv_write(qkv, q2, None, None, 0.0, None, i32(positions), i32(slots), kc, vc, H, KVH, Dh, bs)
    assert torch.equal(q2, qkv[:, :H * Dh])
    kernels.qk_norm_rope_kv_write(qkv, q2, None, None, 0.0, inv_freq, i32([0] * T), i32(slots), kc, vc, H, KVH, Dh, bs)
    assert torch.equal(q2, qkv[:, :H * Dh])
    # cos and sin from the per-step table: the same bits as computing them per head
    table = torch.empty(T, Dh, device="cuda")
    kernels.rope_angles(i32(positions), inv_freq, table)
    angle = torch.tensor(positions, dtype=torch.float32)[:, None] * inv_freq.cpu()[None, :]
    close(table[:, :Dh // 2], torch.cos(angle.to(F64)), 2e-6, "cos table")
    kc2, vc2, q4 = torch.zeros_like(kc), torch.zeros_like(vc), torch.empty_like(q)
    kernels.qk_norm_rope_kv_write(qkv, q4, qw, kw, eps, inv_freq, i32(positions), i32(slots), kc2, vc2, H, KVH, Dh, bs,
                                  angles=table)
    kc0, vc0, q0 = torch.zeros_like(kc), torch.zeros_like(vc), torch.empty_like(q)
    kernels.qk_norm_rope_kv_write(qkv, q0, qw, kw, eps, inv_freq, i32(positions), i32(slots), kc0, vc0, H, KVH, Dh, bs)
    assert torch.equal(q4, q0) and torch.equal(kc2, kc0) and torch.equal(vc2, vc0)
    # the projection as three planes of partial sums: the same as their sum handed over in one piece
    planes = rnd(3, T, (H + 2 * KVH) * Dh, seed=11).cuda()
    summed = (planes[0] + planes[1]) + planes[2]
    kc1, vc1, kc3, vc3 = (torch.zeros_like(c) for c in (kc, vc, kc, vc))
    q1, q3 = torch.empty_like(q), torch.empty_like(q)
    kernels.qk_norm_rope_kv_write(summed, q1, qw, kw, eps, inv_freq, i32(positions), i32(slots), kc1, vc1, H, KVH, Dh, bs)
    kernels.qk_norm_rope_kv_write(planes[0], q3, qw, kw, eps, inv_freq, i32(positions), i32(slots), kc3, vc3, H, KVH,
                                  Dh, bs, planes=3, plane_stride=planes.stride(0))
    assert torch.equal(q1, q3) and torch.equal(kc1, kc3) and torch.equal(vc1, vc3)

def rotate_pairs(x, positions, inv_freq, rotary_dim, pairing):
    """The first ``rotary_dim`` dimensions of x [T, heads, Dh] rotated as pairs (i, i + rotary_dim/2)
    ("rotate_half") or (2i, 2i + 1) ("interleaved") by position * inv_freq[i]; the rest unchanged."""
    x = x.to(F64)
    out = x.clone()
    half = rotary_dim // 2
    angle = torch.tensor(positions, dtype=torch.float32)[:, None] * inv_freq[None, :]      # float32 angles
    cos, sin = torch.cos(angle.to(F64))[:, None, :], torch.sin(angle.to(F64))[:, None, :]
    if pairing == "rotate_half":
        a, b = x[..., :half], x[..., half:rotary_dim]
        out[..., :half], out[..., half:rotary_dim] = a * cos - b * sin, b * cos + a * sin
    else:
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2], out[..., 1:rotary_dim:2] = a * cos - b * sin, b * cos + a * sin
    return out


@pytest.mark.parametrize("H,KVH,Dh,rotary_dim,bs", [(4, 2, 16, 8, 4), (6, 2, 32, 32, 16), (3, 1, 48, 20, 8),
                                                    (8, 2, 128, 64, 16), (2, 1, 256, 0, 4), (2, 2, 80, 78, 2)])
@pytest.mark.parametrize("pairing", ["rotate_half", "interleaved"])
def test_qk_norm_rope_rotates_part_of_a_head_and_neighbouring_pairs(H, KVH, Dh, rotary_dim, bs, pairing):
    """What the position interface may return beside Qwen3's whole-head halves: a rotation of the first
    rotary_dim dimensions only, and pairs of neighbours; with and without the per-step table of angles."""
    from tie_amd import kernels

    T, eps = 5, 1e-5
    qkv = rnd(T, (H + 2 * KVH) * Dh, seed=18, scale=2.0).cuda()
    qw, kw = (1 + 0.1 * rnd(Dh, seed=19)).cuda(), (1 + 0.1 * rnd(Dh, seed=20)).cuda()
    positions, slots = [0, 3, 77, 300, 4095], [9, 2, 31, 4, 17]
    inv_freq = torch.from_numpy(plain.rope_inv_freq(1e4, max(rotary_dim, 2)))[:rotary_dim // 2].contiguous()
    NB = 32 // bs + 1
    x = qkv.cpu()
    q_in = x[:, :H * Dh].view(T, H, Dh)
    k_in = x[:, H * Dh:(H + KVH) * Dh].view(T, KVH, Dh)
    q_want = rotate_pairs(plain.rms_norm(q_in, qw.cpu(), eps), positions, inv_freq, rotary_dim, pairing)
    k_want = rotate_pairs(plain.rms_norm(k_in, kw.cpu(), eps), positions, inv_freq, rotary_dim, pairing)
    if rotary_dim == Dh and pairing == "rotate_half":
        close(q_want, plain.rope_neox(plain.rms_norm(q_in, qw.cpu(), eps), positions, 1e4), 1e-12, "the test's own rotation")
    table = None
    if rotary_dim:
        table = torch.empty(T, rotary_dim, device="cuda")
        kernels.rope_angles(i32(positions), inv_freq.cuda(), table)
    for angles in (None, table):
        kc = torch.zeros(NB, KVH, bs, Dh, device="cuda")
        vc = torch.zeros(NB, KVH, Dh, bs, device="cuda")
        q = torch.empty(T, H * Dh, device="cuda")
        kernels.qk_norm_rope_kv_write(qkv, q, qw, kw, eps, inv_freq.cuda() if rotary_dim else None, i32(positions),
                                      i32(slots), kc, vc, H, KVH, Dh, bs, angles=angles, rotary_dim=rotary_dim,
                                      pairing=pairing)
        close(q.view(T, H, Dh), q_want, 2e-6, f"q, rotary_dim {rotary_dim}, {pairing}")
        for t, slot in enumerate(slots):
            close(kc[slot // bs, :, slot % bs], k_want[t], 2e-6, f"k of token {t}, rotary_dim {rotary_dim}, {pairing}")


def attention_case(H, KVH, Dh, bs, lens_new, lens_ctx, seed, dtype=torch.float32, window=None, spike=None):
    """Builds a batch of sequences with scattered, unordered block tables; returns kernel inputs and the plain result."""
    rng = np.random.RandomState(seed)
    S = len(lens_ctx)
    MB = max(math.ceil(c / bs) for c in lens_ctx) + 1
    NB = sum(math.ceil(c / bs) for c in lens_ctx) + 3
    pages = list(rng.permutation(NB))
    kc = torch.full((NB, KVH, bs, Dh), float("nan"), dtype=dtype)
    vc = torch.full((NB, KVH, Dh, bs), float("nan"), dtype=dtype)
    tables = np.zeros((S, MB), dtype=np.int32)
    q_rows, want_rows, seq_of_row, query_start = [], [], [], [0]
    for s in range(S):
        ctx, n_new = lens_ctx[s], lens_new[s]
        q = rnd(ctx, H, Dh, seed=seed * 100 + s)
        k = rnd(ctx, KVH, Dh, seed=seed * 100 + s + 50)
        v = rnd(ctx, KVH, Dh, seed=seed * 100 + s + 70)
        if spike is not None:                               # one far key stands out for the last query
            j = spike(ctx)
            k[j] = 0
            k[j, :, 0] = 30.0
            q[ctx - 1] = 0
            q[ctx - 1, :, 0] = 30.0
            v[j] = 5.0
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        table = [int(pages.pop()) for _ in range(math.ceil(ctx / bs))]
        tables[s, :len(table)] = table
        for j in range(ctx):
            kc[table[j // bs], :, j % bs] = k[j]
            vc[table[j // bs], :, :, j % bs] = v[j]
        full = plain.causal_attention(q, k, v, Dh ** -0.5, window)
        q_rows.append(q[ctx - n_new:].reshape(n_new, H * Dh))
        want_rows.append(full[ctx - n_new:].reshape(n_new, H * Dh))
        seq_of_row += [s] * n_new
        query_start.append(query_start[-1] + n_new)
    kc, vc = torch.nan_to_num(kc, nan=1e30), torch.nan_to_num(vc, nan=1e30)   # unused slots hold garbage
    return dict(q=torch.cat(q_rows).cuda().contiguous(), kc=kc.cuda(), vc=vc.cuda(), tables=torch.from_numpy(tables).cuda(),
                query_start=i32(query_start), context_lens=i32(lens_ctx), seq_of_row=i32(seq_of_row),
                want=torch.cat(want_rows)), S


@pytest.mark.parametrize("H,KVH,Dh,bs", [(4, 2, 16, 4), (6, 2, 32, 16), (3, 1, 48, 8), (5, 5, 80, 16), (8, 2, 128, 16),
                                         (2, 1, 256, 4), (1, 1, 512, 2)])
def test_paged_attention_generic_mixed_batch(H, KVH, Dh, bs):
    from tie_amd import kernels

    # a whole prompt, a portion that continues a cached prefix, single decoded tokens, a one-token prompt
    case, S = attention_case(H, KVH, Dh, bs, lens_new=[13, 5, 1, 1, 1], lens_ctx=[13, 29, 40, 300, 1], seed=3)
    out = torch.empty_like(case["q"])
    kernels.paged_attention_generic(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                    case["tables"], case["seq_of_row"], H, Dh ** -0.5)
    close(out, case["want"], 1e-5, f"attention H={H} KVH={KVH} Dh={Dh}")


@pytest.mark.parametrize("where", ["first", "page_edge", "far"])
def test_paged_attention_generic_finds_one_far_key(where):
    from tie_amd import kernels

    spike = {"first": lambda ctx: 0, "page_edge": lambda ctx: 16 * 3 - 1, "far": lambda ctx: ctx - 259}[where]
    case, S = attention_case(4, 2, 32, 16, lens_new=[1, 7], lens_ctx=[700, 523], seed=5, spike=spike)
    out = torch.empty_like(case["q"])
    kernels.paged_attention_generic(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                    case["tables"], case["seq_of_row"], 4, 32 ** -0.5)
    close(out, case["want"], 1e-5, f"spike at {where}")
    assert float(out[0].min()) > 4.9                          # the last query really reads the marked value


@pytest.mark.parametrize("window", [1, 5, 16, 17, 100])
def test_paged_attention_generic_window_edges(window):
    from tie_amd import kernels

    case, S = attention_case(4, 2, 16, 4, lens_new=[9, 1, 20], lens_ctx=[30, 41, 20], seed=7, window=window)
    out = torch.empty_like(case["q"])
    kernels.paged_attention_generic(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                    case["tables"], case["seq_of_row"], 4, 16 ** -0.5, window=window)
    close(out, case["want"], 1e-5, f"window {window}")


def test_paged_attention_generic_bfloat16_cache():
    from tie_amd import kernels

    case, S = attention_case(6, 2, 32, 16, lens_new=[11, 1], lens_ctx=[27, 90], seed=9, dtype=torch.bfloat16)
    out = torch.empty_like(case["q"])
    kernels.paged_attention_generic(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                    case["tables"], case["seq_of_row"], 6, 32 ** -0.5)
    close(out, case["want"], 1e-2, "bfloat16 attention")



@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(16, 8), (70, 96), (384, 200), (100, 4096), (33, 1000)])
def test_skinny_gemm_bf16(M, N, K):
    from tie_amd import kernels

    x = rnd(M, K, seed=21, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=22, scale=0.1, dtype=torch.bfloat16).cuda()
    want = plain.linear(x.cpu(), w.cpu())
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    kernels.skinny_gemm_bf16(x, w, out)
    close(out, want, 1e-5, f"skinny gemm {M}x{N}x{K}")
    base = rnd(M, N, seed=23).cuda()
    acc = base.clone()
    kernels.skinny_gemm_bf16(x, w, acc, accumulate=True)
    close(acc, want + base.cpu().to(F64), 1e-5, "skinny gemm accumulate")
    half = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    kernels.skinny_gemm_bf16(x, w, half)
    close(half, want, 5e-3, "skinny gemm bfloat16 output")
    # a row's result does not depend on how many rows the call holds
    one = torch.empty(1, N, dtype=torch.float32, device="cuda")
    kernels.skinny_gemm_bf16(x[M - 1:M].contiguous(), w, one)
    assert torch.equal(one[0], out[M - 1])
    # cut along K: planes of partial sums that add up to the product, again the same for a row alone
    for splits in (2, 3):
        planes = torch.full((splits, M, N), float("nan"), dtype=torch.float32, device="cuda")
        kernels.skinny_gemm_bf16(x, w, planes, splits=splits)
        close(planes.cpu().to(F64).sum(0), want, 1e-5, f"skinny gemm in {splits} planes")
        alone = torch.empty(splits, 1, N, dtype=torch.float32, device="cuda")
        kernels.skinny_gemm_bf16(x[M - 1:M].contiguous(), w, alone, splits=splits)
        assert torch.equal(alone[:, 0], planes[:, M - 1])


@pytest.mark.parametrize("M", [1, 8, 17, 40, 64])
@pytest.mark.parametrize("N,K,gated", [(10240, 5120, False), (5120, 8192, False), (5120, 25600, False), (1600, 5120, True),
                                       (2048, 6144, False), (4096, 2048, False), (1024, 4032, False)])
def test_skinny_gemm_bf16_at_the_widths_of_other_model_sizes(M, N, K, gated):
    """The projections of the 32B shape (rows of 5120, K up to 25600) and of the 1.7B shape, packed, cut along K
    as the plan says (2, 4 or 8 planes), with every pair of tile count and batch of loads the launcher may pick.
    For the kernel that shares x through LDS they hold ranges of 4, 16, 20 and 40 chunks of k-blocks (fewer than
    its ring is deep, and many rounds of it) and, at K = 4032, a range whose last chunk is half empty."""
    from tie_amd import kernels

    x = rnd(M, K, seed=41, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=42, scale=0.05, dtype=torch.bfloat16).cuda()
    packed = kernels.pack_weight(w)
    if gated:
        g, u = w.cpu().view(N // 16, 2, 8, K)[:, 0].reshape(N // 2, K), w.cpu().view(N // 16, 2, 8, K)[:, 1].reshape(N // 2, K)
        gate, up = plain.linear(x.cpu(), g), plain.linear(x.cpu(), u)
        want = gate / (1 + torch.exp(-gate)) * up
        out = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device="cuda")
        kernels.skinny_gemm_bf16(x, packed, out, gated=True)
        close(out, want, 1e-2, f"gated skinny gemm {M}x{N}x{K}")
        lib = kernels._lib("skinny_gemm_bf16")
        for rt, u in ((0, -1), (3, 1), (6, 1), (8, 1)):      # from memory; through LDS in the three workgroup shapes
            again = torch.full_like(out, float("nan"))
            assert lib.tie_skinny_gemm_bf16_with(x.data_ptr(), packed.data_ptr(), again.data_ptr(), 1, 0, 1, M, N, K, 1, 1,
                                                 rt, u, kernels._stream()) == 0
            assert torch.equal(again, out), f"gated, tiles {rt}, batch {u}: the sums depend on the launch's shape"
        return
    want = plain.linear(x.cpu(), w.cpu())
    splits = kernels.skinny_splits(N, K)
    assert splits in (2, 4, 8)
    planes = torch.full((splits, M, N), float("nan"), dtype=torch.float32, device="cuda")
    kernels.skinny_gemm_bf16(x, packed, planes, splits=splits)
    close(planes.cpu().to(F64).sum(0), want, 1e-5, f"skinny gemm {M}x{N}x{K} in {splits} planes")
    lib = kernels._lib("skinny_gemm_bf16")
    # a row alone (one tile of x, read from memory) and the same row among 64 (x through LDS): the same bits
    alone = torch.empty(splits, 1, N, dtype=torch.float32, device="cuda")
    kernels.skinny_gemm_bf16(x[M - 1:M].contiguous(), packed, alone, splits=splits)
    assert torch.equal(alone[:, 0], planes[:, M - 1])
    # u = -1: x read from memory whatever M and N; u = 1: x through LDS whatever N (for more than 16 rows),
    # in workgroups of rt tiles (3, 6 or 8)
    for rt, u in ((1, 8), (1, 2), (2, 4), (3, 2), (4, 2), (2, 8), (0, -1), (0, 1), (3, 1), (6, 1), (8, 1)):
        again = torch.full_like(planes, float("nan"))
        status = lib.tie_skinny_gemm_bf16_with(x.data_ptr(), packed.data_ptr(), again.data_ptr(), 0, 0, 0, M, N, K, splits, 1,
                                               rt, u, kernels._stream())
        assert status == 0
        assert torch.equal(again, planes), f"tiles {rt}, batch {u}: the sums depend on the launch's shape"


@pytest.mark.parametrize("R,n", [(1, 24), (5, 200), (8, 4096), (64, 1024), (3, 20000)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_add_partials_alone_and_with_rms_norm(R, n, out_dtype):
    from tie_amd import kernels

    x = rnd(R, n, seed=51).cuda()
    planes = rnd(3, R, n, seed=52).cuda()
    w = (1 + 0.1 * rnd(n, seed=53)).cuda()
    total = x.cpu().to(F64) + planes.cpu().to(F64).sum(0)
    added = x.clone()
    kernels.add_partials(added, planes)
    close(added, total, 1e-6, "add_partials")
    both = x.clone()
    out = torch.full((R, n), float("nan"), dtype=out_dtype, device="cuda")
    kernels.add_partials(both, planes, w, 1e-5, out)
    assert torch.equal(both, added)                    # the stream holds the same sum either way
    close(out, plain.rms_norm(total, w.cpu(), 1e-5), 1e-5 if out_dtype == torch.float32 else 5e-3, "add + rms_norm")
    # and the norm of the sum is the norm kernel's own result on the updated stream
    separate = torch.empty_like(out)
    kernels.rms_norm(added, w, 1e-5, separate)
    assert torch.equal(separate, out)



@pytest.mark.parametrize("M,N,K", [(65, 70, 96), (100, 384, 200), (128, 128, 64), (300, 200, 4096), (2048, 256, 512),
                                   (257, 129, 72), (1, 64, 64)])
@pytest.mark.parametrize("tile", [1, 2, 3])
def test_gemm_bf16(M, N, K, tile):
    from tie_amd import kernels

    x = rnd(M, K, seed=31, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=32, scale=0.1, dtype=torch.bfloat16).cuda()
    want = plain.linear(x.cpu(), w.cpu())
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    kernels.gemm_bf16(x, w, out, tile=tile)
    close(out, want, 1e-5, f"gemm {M}x{N}x{K} tile {tile}")
    base = rnd(M, N, seed=33).cuda()
    acc = base.clone()
    kernels.gemm_bf16(x, w, acc, accumulate=True, tile=tile)
    close(acc, want + base.cpu().to(F64), 1e-5, "gemm accumulate")
    half = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    kernels.gemm_bf16(x, w, half, tile=tile)
    close(half, want, 5e-3, "gemm bfloat16 output")
    # a row's result does not depend on the other rows of the call
    few = torch.empty(min(M, 3), N, dtype=torch.float32, device="cuda")
    kernels.gemm_bf16(x[:3].contiguous(), w, few, tile=tile)
    assert torch.equal(few, out[:3])


@pytest.mark.parametrize("M,N,K", [(65, 72, 96), (100, 384, 224), (300, 200, 4096), (2048, 256, 512), (257, 132, 1024),
                                   (513, 516, 352), (1, 64, 128)])
@pytest.mark.parametrize("tile", [4, 5, 6, 7, 8, 9, 10])
def test_gemm_bf16_loaded_straight_into_lds(M, N, K, tile):
    """The tiles whose operand slices bypass registers: ragged M and N, short and long K, every epilogue."""
    from tie_amd import kernels

    x = rnd(M, K, seed=36, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=37, scale=0.1, dtype=torch.bfloat16).cuda()
    want = plain.linear(x.cpu(), w.cpu())
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    kernels.gemm_bf16(x, w, out, tile=tile)
    close(out, want, 1e-5, f"gemm {M}x{N}x{K} tile {tile}")
    base = rnd(M, N, seed=38).cuda()
    acc = base.clone()
    kernels.gemm_bf16(x, w, acc, accumulate=True, tile=tile)
    close(acc, want + base.cpu().to(F64), 1e-5, "gemm accumulate")
    half = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    kernels.gemm_bf16(x, w, half, tile=tile)
    close(half, want, 5e-3, "gemm bfloat16 output")
    few = torch.empty(min(M, 3), N, dtype=torch.float32, device="cuda")
    kernels.gemm_bf16(x[:3].contiguous(), w, few, tile=tile)
    assert torch.equal(few, out[:3])                   # a row's result does not depend on the other rows
    if K // 32 >= 6:
        planes = torch.full((2, M, N), float("nan"), dtype=torch.float32, device="cuda")
        kernels.gemm_bf16(x, w, planes, tile=tile, splits=2)
        close(planes.cpu().to(F64).sum(0), want, 1e-5, "gemm in two planes")
    if N % 16 == 0:
        gate, up = w[: N // 2], w[N // 2:]
        if (N // 2) % 8 == 0:
            gated = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device="cuda")
            kernels.gemm_bf16(x, kernels.interleave_gate_up(gate.contiguous(), up.contiguous()), gated, tile=tile, gated=True)
            g, u = plain.linear(x.cpu(), gate.cpu()), plain.linear(x.cpu(), up.cpu())
            close(gated, g / (1 + torch.exp(-g)) * u, 8e-3, "gated product")


@pytest.mark.parametrize("N,K", [(16, 96), (48, 128), (208, 4096), (1024, 352)])
def test_packed_weight_feeds_both_products_the_same_numbers(N, K):
    """The blocked weight layout changes where bytes lie, not one sum: results equal the row-major ones bit for bit."""
    from tie_amd import kernels

    w = rnd(N, K, seed=51, scale=0.1, dtype=torch.bfloat16).cuda()
    packed = kernels.pack_weight(w)
    assert packed.shape == (N, K) and torch.equal(packed.unpacked(), w)
    # block (t, b): rows 16 t.., k 32 b..; the 8 elements of (row r, chunk c) at (16 c + r) * 8
    blocks = packed.blocks.view(-1)
    t, b, r, c = N // 16 - 1, K // 32 - 1, 5, 2
    at = ((t * (K // 32) + b) * 64 + 16 * c + r) * 8
    assert torch.equal(blocks[at:at + 8], w[16 * t + r, 32 * b + 8 * c:32 * b + 8 * c + 8])
    for M in (1, 8, 40, 64):
        x = rnd(M, K, seed=52 + M, dtype=torch.bfloat16).cuda()
        for splits in (1, 2):
            shape = (M, N) if splits == 1 else (splits, M, N)
            a = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda")
            b_ = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda")
            kernels.skinny_gemm_bf16(x, w, a, splits=splits)
            kernels.skinny_gemm_bf16(x, packed, b_, splits=splits)
            assert torch.equal(a, b_), f"decode product M={M} splits={splits}"
        if N % 16 == 0:
            a = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device="cuda")
            b_ = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device="cuda")
            kernels.skinny_gemm_bf16(x, w, a, gated=True)
            kernels.skinny_gemm_bf16(x, packed, b_, gated=True)
            assert torch.equal(a, b_)
    for M in (40, 64, 65, 128, 300, 513):
        x = rnd(M, K, seed=60 + M, dtype=torch.bfloat16).cuda()
        want = plain.linear(x.cpu(), w.cpu())
        for tile in (4, 5, 6, 7, 8, 9, 10):
            a = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            b_ = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            kernels.gemm_bf16(x, w, a, tile=tile)
            kernels.gemm_bf16(x, packed, b_, tile=tile)
            assert torch.equal(a, b_), f"tiled product M={M} tile={tile}"
            close(b_, want, 1e-5, "tiled product over a packed weight")
        out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        kernels.linear(x, packed, out)                       # left to choose
        close(out, want, 1e-5, "linear over a packed weight")
        s = kernels.gemm_splits(M, N, K, packed=True)
        if s > 1:
            planes = torch.full((s, M, N), float("nan"), dtype=torch.float32, device="cuda")
            kernels.gemm_bf16(x, packed, planes, splits=s)
            close(planes.cpu().to(F64).sum(0), want, 1e-5, f"packed weight in {s} planes")
    with pytest.raises(kernels.InvalidArgument):
        kernels.gemm_bf16(rnd(65, K, seed=1, dtype=torch.bfloat16).cuda(), packed,
                          torch.zeros(65, N, device="cuda"), tile=1)          # only the tiles loaded straight into LDS read the layout
    with pytest.raises(kernels.InvalidArgument):
        kernels.linear(torch.zeros(2, K, device="cuda"), packed, torch.zeros(2, N, device="cuda"))   # float32 input
    assert not kernels.packable(w[:, :64].contiguous()) and not kernels.packable(w.float())


def test_gemm_bf16_straight_into_lds_refuses_what_it_cannot_take():
    from tie_amd import kernels
    from tie_amd.kernels import InvalidArgument

    x = torch.zeros(8, 72, dtype=torch.bfloat16, device="cuda")          # K % 32 != 0
    with pytest.raises(InvalidArgument):
        kernels.gemm_bf16(x, torch.zeros(16, 72, dtype=torch.bfloat16, device="cuda"),
                          torch.zeros(8, 16, device="cuda"), tile=4)
    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")          # two slices only
    with pytest.raises(InvalidArgument):
        kernels.gemm_bf16(x, torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda"),
                          torch.zeros(8, 16, device="cuda"), tile=5)
    # left to choose, the same operands go to a kernel that takes them
    out = torch.full((8, 16), float("nan"), device="cuda")
    kernels.gemm_bf16(x, torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda"), out)
    assert torch.equal(out, torch.zeros_like(out))


@pytest.mark.parametrize("M,N,K,splits", [(65, 70, 1024, 2), (100, 384, 4096, 8), (300, 200, 1536, 3), (128, 128, 520, 2)])
def test_gemm_bf16_in_planes(M, N, K, splits):
    """K cut into ranges: one plane of partial sums a range, which add up to the product."""
    from tie_amd import kernels

    x = rnd(M, K, seed=34, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=35, scale=0.1, dtype=torch.bfloat16).cuda()
    planes = torch.full((splits, M, N), float("nan"), dtype=torch.float32, device="cuda")
    kernels.gemm_bf16(x, w, planes, splits=splits)
    close(planes.cpu().to(F64).sum(0), plain.linear(x.cpu(), w.cpu()), 1e-5, f"gemm {M}x{N}x{K} in {splits} planes")


def run_decode(case, S, H, Dh, nsplit, window=None, depth=0):
    from tie_amd import kernels

    q = case["q"]
    out = torch.full_like(q, float("nan"))
    part_o = torch.empty(S * H * nsplit * Dh, dtype=torch.float32, device="cuda")
    part_ml = torch.empty(S * H * nsplit * 2, dtype=torch.float32, device="cuda")
    kernels.attention_decode_bf16(q, case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                  case["tables"], S, H, Dh ** -0.5, window, nsplit, part_o, part_ml, depth=depth)
    return out


@pytest.mark.parametrize("H,KVH,Dh,bs", [(8, 2, 128, 16), (6, 2, 32, 16), (64, 8, 128, 16), (2, 1, 256, 32), (12, 4, 64, 64),
                                         (16, 1, 128, 16)])
@pytest.mark.parametrize("planes,normed,window", [(1, True, None), (4, True, None), (2, False, None), (4, True, 50)])
def test_attention_decode_that_prepares_its_own_queries(H, KVH, Dh, bs, planes, normed, window):
    """A step of single decoded tokens on the kernel that sums the QKV planes, norms and rotates its queries and
    writes the newest keys and values itself, against the q/k kernel followed by the decode attention: the same
    bits in both cache planes and the same output up to rounding, at lengths where the newest position opens a
    tile or a page."""
    from tie_amd import kernels

    lens = [1, 16, 17, 32, 33, 64, 65, 129, 300, 700, 1000, 2049]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=[1] * len(lens), lens_ctx=lens, seed=43, dtype=torch.bfloat16,
                             window=window)
    width = (H + 2 * KVH) * Dh
    qkv = (rnd(planes, S, width, seed=44) / planes).cuda()
    qw = (1 + 0.1 * rnd(Dh, seed=45)).cuda() if normed else None
    kw = (1 + 0.1 * rnd(Dh, seed=46)).cuda() if normed else None
    eps = 1e-5
    inv_freq = torch.from_numpy(plain.rope_inv_freq(1e4, Dh)).float().cuda()
    positions = i32([c - 1 for c in lens])
    tables = case["tables"]
    slots = i32([int(tables[s, (c - 1) // bs]) * bs + (c - 1) % bs for s, c in enumerate(lens)])
    angles = torch.empty(S, Dh, device="cuda")
    kernels.rope_angles(positions, inv_freq, angles)

    class Batch:
        all_decode, num_seqs, plan_context = True, S, max(lens)
        query_start, context_lens = case["query_start"], case["context_lens"]

    class Step:
        block_tables = tables

    memory = {}

    def scratch(name, shape, dtype):
        return memory.setdefault((name, tuple(shape), dtype), torch.full(tuple(shape), float("nan"), dtype=dtype, device="cuda"))

    # the two kernels, one after the other
    kc1, vc1 = case["kc"].clone(), case["vc"].clone()
    q = torch.empty(S, H * Dh, dtype=torch.bfloat16, device="cuda")
    kernels.qk_norm_rope_kv_write(qkv[0], q, qw, kw, eps, inv_freq, positions, slots, kc1, vc1, H, KVH, Dh, bs,
                                  planes=planes, plane_stride=S * width, angles=angles)
    apart = torch.full_like(q, float("nan"))
    nsplit = kernels.decode_splits(S, KVH, max(lens), bs)
    part_o = torch.empty(S * H * nsplit * Dh, device="cuda")
    part_ml = torch.empty(S * H * nsplit * 2, device="cuda")
    kernels.attention_decode_bf16(q, kc1, vc1, apart, case["query_start"], case["context_lens"], tables, S, H, Dh ** -0.5,
                                  window, nsplit, part_o, part_ml)
    # the one kernel
    kc2, vc2 = case["kc"].clone(), case["vc"].clone()
    assert kernels.decode_attention_prepares(Batch, torch.bfloat16, kc2, H)
    fused = torch.full_like(q, float("nan"))
    kernels.paged_attention_prepared(qkv, qw, kw, eps, angles, True, kc2, vc2, fused, Step, Batch, H, Dh ** -0.5, window,
                                     scratch)
    assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1), "the newest keys or values differ"
    assert not torch.isnan(fused.float()).any()
    # the same queries, keys and values; the newest key is attended to by itself, after the tiles, instead of inside
    # its tile, so the sums round differently
    close(fused, apart, 1e-2, "the kernel that prepares its queries")
    # a cache that holds the token already is left alone
    kc3, vc3 = kc1.clone(), vc1.clone()
    again = torch.full_like(q, float("nan"))
    kernels.paged_attention_prepared(qkv * 3, qw, kw, eps, angles, False, kc3, vc3, again, Step, Batch, H, Dh ** -0.5,
                                     window, scratch)
    assert torch.equal(kc3, kc1) and torch.equal(vc3, vc1)


@pytest.mark.parametrize("H,KVH,Dh,bs", [(6, 2, 32, 16), (5, 5, 80, 16), (8, 2, 128, 16), (2, 1, 256, 32), (4, 4, 112, 64)])
@pytest.mark.parametrize("nsplit,window", [(1, None), (2, None), (5, None), (1, 100), (3, 77)])
def test_attention_decode_bf16_with_tiles_in_flight(H, KVH, Dh, bs, nsplit, window):
    """Pages of 16 positions or more: the kernels that keep two to four tiles of keys in registers against the
    one that looks its pages up per lane and against the plain formula, at lengths around every count of tiles
    that the ring's first, middle and last parts take (1 to 12 tiles a share), with and without a window."""
    lens = [1, 31, 32, 33, 64, 65, 96, 127, 129, 160, 200, 257, 300, 321, 385, 700, 1000]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=[1] * len(lens), lens_ctx=lens, seed=17, dtype=torch.bfloat16,
                             window=window)
    first = run_decode(case, S, H, Dh, nsplit, window=window, depth=1)
    close(first, case["want"], 1e-2, f"decode attention H={H} KVH={KVH} Dh={Dh} bs={bs} splits={nsplit} window={window}")
    for depth in (2, 3, 4):
        again = run_decode(case, S, H, Dh, nsplit, window=window, depth=depth)
        assert torch.equal(again, first), f"{depth} tiles in flight: other bits than one"


@pytest.mark.parametrize("H,KVH,Dh,bs", [(6, 2, 32, 16), (8, 2, 128, 16), (5, 5, 80, 64)])
@pytest.mark.parametrize("nsplit,share_tiles,window", [(8, 4, None), (8, 7, None), (4, 1, None), (3, 100, None),
                                                       (8, 3, 200), (2, 0, None)])
def test_attention_decode_bf16_with_shares_of_one_length(H, KVH, Dh, bs, nsplit, share_tiles, window):
    """Shares of one length for sequences of very different lengths: a short sequence fills one share and leaves
    the others empty, a long one fills several; a length too short to cover a sequence (1 tile in 4 shares against
    32 tiles) falls back to that sequence's own equal shares, one longer than any sequence leaves one share each.
    Against the plain formula, and the same bits whatever the depth of the ring; the kernel that prepares its own
    queries takes the same argument."""
    from tie_amd import kernels

    lens = [1, 33, 64, 129, 300, 1000, 31, 700, 257, 96]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=[1] * len(lens), lens_ctx=lens, seed=19, dtype=torch.bfloat16,
                             window=window)
    length = i32([share_tiles])
    outs = []
    for depth in (2, 3, 4):
        out = torch.full_like(case["q"], float("nan"))
        part_o = torch.full((S * H * nsplit * Dh,), float("nan"), dtype=torch.float32, device="cuda")
        part_ml = torch.full((S * H * nsplit * 2,), float("nan"), dtype=torch.float32, device="cuda")
        kernels.attention_decode_bf16(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                      case["tables"], S, H, Dh ** -0.5, window, nsplit, part_o, part_ml, depth=depth,
                                      share_tiles=length)
        outs.append(out)
    close(outs[0], case["want"], 1e-2, f"decode attention, shares of {share_tiles} tiles in a grid of {nsplit}")
    assert torch.equal(outs[1], outs[0]) and torch.equal(outs[2], outs[0])
    with pytest.raises(Exception, match="more than one share"):
        kernels.attention_decode_bf16(case["q"], case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                      case["tables"], S, H, Dh ** -0.5, window, 1, share_tiles=length)


def test_single_rows_beside_a_portion_with_shares_of_one_length(monkeypatch):
    """A step of a prompt portion and many single decoded rows of very different lengths, through the entry point
    the attention part calls: the single rows go to the decode kernel with shares of one length (the rule by the
    step's size bent to two shares a sequence, so that twelve sequences meet the plan), the portion to the prefill
    kernel; every row against the plain formula."""
    from tie_amd import kernels

    H, KVH, Dh, bs = 8, 2, 128, 16
    lens_ctx = [300, 1000, 40, 1000, 90, 33, 64, 700, 17, 130, 257, 50, 31]
    lens_new = [70] + [1] * 12
    case, S = attention_case(H, KVH, Dh, bs, lens_new=lens_new, lens_ctx=lens_ctx, seed=23, dtype=torch.bfloat16)
    monkeypatch.setattr(kernels, "decode_splits", lambda *a, **k: 2)
    monkeypatch.setattr(kernels, "SINGLE_ROWS_RIDE_ALONG", 0)
    plans = []
    real = kernels.decode_share_plan

    def watched(*args, **kwargs):
        plans.append(real(*args, **kwargs))
        return plans[-1]

    monkeypatch.setattr(kernels, "decode_share_plan", watched)

    class Batch:
        all_decode, num_seqs, plan_context, memo = False, S, 1024, {}
        host_new_tokens, host_context_lens = lens_new, lens_ctx
        query_start, context_lens, seq_of_row = case["query_start"], case["context_lens"], case["seq_of_row"]

    class Step:
        block_tables = case["tables"]

    memory = {}

    def scratch(name, shape, dtype):
        return memory.setdefault((name, tuple(shape), dtype), torch.full(tuple(shape), float("nan"), dtype=dtype, device="cuda"))

    out = torch.full_like(case["q"], float("nan"))
    for _ in range(2):                                       # the second call takes the step's plan from its memo
        kernels.paged_attention(case["q"], case["kc"], case["vc"], out, Step, Batch, H, Dh ** -0.5, None, scratch)
    assert len(plans) == 1 and plans[0][0] >= 8 and plans[0][1] >= 4, plans
    close(out, case["want"], 1e-2, "a portion beside single rows in shares of one length")


@pytest.mark.parametrize("H,KVH,Dh,bs", [(4, 2, 16, 4), (6, 2, 32, 16), (3, 1, 48, 8), (5, 5, 80, 16), (8, 2, 128, 16),
                                         (16, 1, 64, 4), (2, 1, 256, 32)])
@pytest.mark.parametrize("nsplit", [1, 3, 8])
def test_attention_decode_bf16(H, KVH, Dh, bs, nsplit):
    lens = [1, 31, 32, 33, 300, 700, 64]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=[1] * len(lens), lens_ctx=lens, seed=13, dtype=torch.bfloat16)
    out = run_decode(case, S, H, Dh, nsplit)
    close(out, case["want"], 1e-2, f"decode attention H={H} KVH={KVH} Dh={Dh} bs={bs} splits={nsplit}")


@pytest.mark.parametrize("nsplit", [1, 16, 64])
def test_attention_decode_bf16_groups_of_eight_query_heads(nsplit):
    """64 query heads over 8 KV heads of 128 (the 32B shape's geometry), contexts around 4096."""
    H, KVH, Dh = 64, 8, 128
    case, S = long_decode_case(H, KVH, Dh, 16, [4096, 4001, 33], seed=35, spike_back=30)
    out = run_decode(case, S, H, Dh, nsplit)
    close(out, case["want"], 1e-2, f"decode attention, groups of 8, {nsplit} shares")


@pytest.mark.parametrize("where", ["first", "page_edge", "tile_edge", "far", "last"])
@pytest.mark.parametrize("nsplit", [1, 5])
def test_attention_decode_bf16_finds_one_far_key(where, nsplit):
    spike = {"first": lambda ctx: 0, "page_edge": lambda ctx: 16 * 3 - 1, "tile_edge": lambda ctx: 32 * 7,
             "far": lambda ctx: ctx - 259, "last": lambda ctx: ctx - 2}[where]
    case, S = attention_case(8, 2, 64, 16, lens_new=[1, 1], lens_ctx=[700, 523], seed=15, dtype=torch.bfloat16,
                             spike=spike)
    out = run_decode(case, S, 8, 64, nsplit)
    close(out, case["want"], 1e-2, f"spike at {where}")
    assert float(out.float().min()) > 4.9


@pytest.mark.parametrize("window", [1, 5, 32, 33, 100])
def test_attention_decode_bf16_window_edges(window):
    lens = [30, 41, 20, 200]
    case, S = attention_case(4, 2, 32, 4, lens_new=[1] * 4, lens_ctx=lens, seed=17, dtype=torch.bfloat16, window=window)
    for nsplit in (1, 4):
        out = run_decode(case, S, 4, 32, nsplit, window=window)
        close(out, case["want"], 1e-2, f"decode window {window} splits {nsplit}")


def long_decode_case(H, KVH, Dh, bs, lens_ctx, seed, spike_back):
    """Decode rows over long contexts (vectorised filling, the plain result for the last row only).

    Key ``ctx - spike_back`` of every sequence is made to stand out for the last query, with a value of 5
    in every dimension: a share of keys that is dropped, read twice or merged with a wrong weight shows."""
    rng = np.random.RandomState(seed)
    S = len(lens_ctx)
    MB = max(math.ceil(c / bs) for c in lens_ctx) + 1
    NB = sum(math.ceil(c / bs) for c in lens_ctx) + 3
    pages = torch.from_numpy(rng.permutation(NB).astype(np.int64))
    kc = torch.full((NB, KVH, bs, Dh), 1e30, dtype=torch.bfloat16)          # unused slots hold garbage
    vc = torch.full((NB, KVH, Dh, bs), 1e30, dtype=torch.bfloat16)
    tables = np.zeros((S, MB), dtype=np.int32)
    q_rows, want_rows, used = [], [], 0
    for s, ctx in enumerate(lens_ctx):
        q = rnd(1, H, Dh, seed=seed * 100 + s)
        k = rnd(ctx, KVH, Dh, seed=seed * 100 + s + 50)
        v = rnd(ctx, KVH, Dh, seed=seed * 100 + s + 70)
        j = ctx - spike_back
        k[j] = 0
        k[j, :, 0] = 30.0
        q[0] = 0
        q[0, :, 0] = 30.0
        v[j] = 5.0
        q, k, v = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
        n_pages = math.ceil(ctx / bs)
        table = pages[used:used + n_pages]
        used += n_pages
        tables[s, :n_pages] = table.numpy()
        pos = torch.arange(ctx)
        kc[table[pos // bs], :, pos % bs] = k
        vc[table[pos // bs], :, :, pos % bs] = v
        q_rows.append(q.reshape(1, H * Dh))
        want_rows.append(plain.causal_attention_tail(q, k, v, Dh ** -0.5).reshape(1, H * Dh))
    return dict(q=torch.cat(q_rows).cuda().contiguous(), kc=kc.cuda(), vc=vc.cuda(), tables=torch.from_numpy(tables).cuda(),
                query_start=i32(list(range(S + 1))), context_lens=i32(lens_ctx), want=torch.cat(want_rows)), S


@pytest.mark.parametrize("nsplit", [32, 64, 129, 256])
def test_attention_decode_bf16_many_key_shares(nsplit):
    """The numbers of shares that serving contexts get (32 at 4096 keys, up to 256): every merge width."""
    H, KVH, Dh = 8, 2, 128
    case, S = long_decode_case(H, KVH, Dh, 16, [8200, 16001, 12288], seed=31, spike_back=7000)
    out = run_decode(case, S, H, Dh, nsplit)
    close(out, case["want"], 1e-2, f"decode attention over long contexts, {nsplit} shares")
    assert float(out.float().min()) > 4.9


@pytest.mark.parametrize("H,KVH", [(4, 1), (8, 2), (16, 4)])
def test_attention_decode_bf16_one_sequence_past_32k(H, KVH):
    """One sequence alone at 40 000 keys with few KV heads: the plan asks for as many shares as it may."""
    from tie_amd import kernels

    Dh, ctx = 64, 40000
    nsplit = kernels.decode_splits(1, KVH, 65536, 8)
    assert nsplit == kernels.MAX_KEY_SPLITS or KVH > 8
    case, S = long_decode_case(H, KVH, Dh, 16, [ctx], seed=33, spike_back=39000)
    out = run_decode(case, S, H, Dh, nsplit)
    close(out, case["want"], 1e-2, f"decode attention, one sequence of {ctx} keys, {nsplit} shares")
    assert float(out.float().min()) > 4.9



def run_prefill(case, H, KVH, lens_new, window=None, nsplit=1, staging=0):
    from tie_amd import kernels

    q = case["q"]
    out = torch.full_like(q, float("nan"))
    Dh = q.shape[1] // H
    items = torch.tensor(kernels.prefill_items(lens_new, H // KVH), dtype=torch.int32).cuda()
    extra = {}
    if nsplit > 1:          # the keys of every item in shares, merged by a second kernel
        rows = q.shape[0]
        extra = dict(nsplit=nsplit, merge_rows=i32(list(range(rows))),
                     part_o=torch.full((rows * H * nsplit * Dh,), float("nan"), dtype=torch.float32, device="cuda"),
                     part_ml=torch.full((rows * H * nsplit * 2,), float("nan"), dtype=torch.float32, device="cuda"))
    kernels.attention_prefill_bf16(q, case["kc"], case["vc"], out, case["query_start"], case["context_lens"],
                                   case["tables"], items, H, Dh ** -0.5, window, staging=staging, **extra)
    return out


def test_attention_kernels_over_cache_planes_beyond_4_gb():
    """Pages that lie more than 4 GB into a cache plane of 4.5 GB (byte offsets that no 32-bit number holds): the
    prefill kernel that loads straight into LDS, the decode kernel with its tiles in flight, and the same kernel
    making its own queries and writing the newest key and value there."""
    from tie_amd import kernels

    H, KVH, Dh, bs = 8, 8, 128, 16
    NB = (9 << 29) // (KVH * bs * Dh * 2)                   # 4.5 GB a plane
    kc = torch.zeros(NB, KVH, bs, Dh, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros(NB, KVH, Dh, bs, dtype=torch.bfloat16, device="cuda")
    lens = [70, 300]
    rng = np.random.RandomState(5)
    far = list(NB - 1 - rng.permutation(64))                # the last pages of the plane
    assert min(far) * KVH * bs * Dh * 2 > 1 << 32
    tables = np.zeros((len(lens), 32), dtype=np.int32)
    qs, ks, vs = [], [], []
    for s, ctx in enumerate(lens):
        q, k, v = (rnd(ctx, n, Dh, seed=60 + 3 * s + i).to(torch.bfloat16) for i, n in enumerate((H, KVH, KVH)))
        for j in range(math.ceil(ctx / bs)):
            page = int(far.pop())
            tables[s, j] = page
            rows = slice(j * bs, min(ctx, (j + 1) * bs))
            kc[page, :, :rows.stop - rows.start] = k[rows].transpose(0, 1).cuda()
            vc[page, :, :, :rows.stop - rows.start] = v[rows].permute(1, 2, 0).cuda()
        qs.append(q), ks.append(k), vs.append(v)
    tables = torch.from_numpy(tables).cuda()
    scale = Dh ** -0.5
    whole = [plain.causal_attention(q.float(), k.float(), v.float(), scale) for q, k, v in zip(qs, ks, vs)]
    # the prompts whole
    q_all = torch.cat([q.reshape(len(q), H * Dh) for q in qs]).cuda()
    out = torch.full_like(q_all, float("nan"))
    items = torch.tensor(kernels.prefill_items(lens, H // KVH), dtype=torch.int32).cuda()
    kernels.attention_prefill_bf16(q_all, kc, vc, out, i32([0, lens[0], sum(lens)]), i32(lens), tables, items, H, scale,
                                   staging=2)
    close(out, torch.cat([w.reshape(len(w), H * Dh) for w in whole]), 1e-2, "prefill attention beyond 4 GB")
    # the last rows as decoded tokens
    q_last = torch.stack([q[-1].reshape(H * Dh) for q in qs]).cuda()
    want_last = torch.stack([w[-1].reshape(H * Dh) for w in whole])
    for nsplit in (1, 2):
        got = torch.full_like(q_last, float("nan"))
        kernels.attention_decode_bf16(q_last, kc, vc, got, i32([0, 1, 2]), i32(lens), tables, 2, H, scale, None, nsplit,
                                      torch.empty(2 * H * nsplit * Dh, device="cuda"),
                                      torch.empty(2 * H * nsplit * 2, device="cuda"), depth=3)
        close(got, want_last, 1e-2, f"decode attention beyond 4 GB, {nsplit} shares")
    # the same rows from a projection's output: no norm, angles of position 0 (cos 1, sin 0) leave q and k as they are
    width = (H + 2 * KVH) * Dh
    qkv = torch.stack([torch.cat([q[-1].reshape(-1), k[-1].reshape(-1), v[-1].reshape(-1)]).float() for q, k, v in zip(qs, ks, vs)])
    angles = torch.cat([torch.ones(2, Dh // 2), torch.zeros(2, Dh // 2)], dim=1).cuda()
    for s, ctx in enumerate(lens):                          # the kernel has to write these itself
        kc[tables[s, (ctx - 1) // bs], :, (ctx - 1) % bs] = 7.0
        vc[tables[s, (ctx - 1) // bs], :, :, (ctx - 1) % bs] = 7.0

    class Batch:
        all_decode, num_seqs, plan_context = True, 2, 4096
        query_start, context_lens = i32([0, 1, 2]), i32(lens)

    class Step:
        block_tables = tables

    got = torch.full_like(q_last, float("nan"))
    kernels.paged_attention_prepared(qkv.view(1, 2, width).cuda().contiguous(), None, None, 0.0, angles, True, kc, vc, got,
                                     Step, Batch, H, scale, None, lambda name, shape, dtype: torch.empty(shape, dtype=dtype, device="cuda"))
    close(got, want_last, 1e-2, "decode attention that prepares its queries, beyond 4 GB")
    for s, ctx in enumerate(lens):
        page, off = int(tables[s, (ctx - 1) // bs]), (ctx - 1) % bs
        assert torch.equal(kc[page, :, off].cpu(), ks[s][-1]) and torch.equal(vc[page, :, :, off].cpu(), vs[s][-1])


@pytest.mark.parametrize("H,KVH,Dh,bs", [(8, 2, 128, 16), (6, 2, 32, 16), (12, 2, 64, 32), (2, 1, 256, 16), (3, 3, 128, 64),
                                         (16, 2, 64, 16)])
@pytest.mark.parametrize("nsplit,window", [(1, None), (3, None), (1, 100), (2, 45)])
def test_attention_prefill_bf16_tiles_copied_or_loaded_straight(H, KVH, Dh, bs, nsplit, window):
    """Both ways of staging the key tiles (through registers; straight into LDS, a page's block of 16 keys per
    wave) against the plain formula: whole prompts, portions over cached prefixes that start and end inside
    tiles and pages, one-row portions, with a window and with the keys cut into shares."""
    from tie_amd import kernels

    assert kernels.prefill_loads_straight(Dh, bs)
    lens_new, lens_ctx = [13, 5, 1, 70, 2, 200, 64, 33], [13, 29, 300, 150, 33, 777, 64, 1000]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=lens_new, lens_ctx=lens_ctx, seed=29, dtype=torch.bfloat16,
                             window=window)
    for staging in (1, 2):
        out = run_prefill(case, H, KVH, lens_new, window=window, nsplit=nsplit, staging=staging)
        close(out, case["want"], 1e-2, f"prefill attention staging {staging} H={H} KVH={KVH} Dh={Dh} bs={bs} "
                                      f"splits={nsplit} window={window}")


@pytest.mark.parametrize("H,KVH,Dh,bs", [(4, 2, 16, 4), (6, 2, 32, 16), (3, 1, 48, 8), (5, 5, 80, 16), (8, 2, 128, 16),
                                         (16, 1, 64, 4), (12, 2, 64, 16), (2, 1, 256, 32)])
def test_attention_prefill_bf16_mixed_batch(H, KVH, Dh, bs):
    # a whole prompt, a portion that continues a cached prefix, single decoded tokens, a one-token prompt, 70 rows
    lens_new, lens_ctx = [13, 5, 1, 1, 1, 70, 2], [13, 29, 40, 300, 1, 150, 33]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=lens_new, lens_ctx=lens_ctx, seed=23, dtype=torch.bfloat16)
    out = run_prefill(case, H, KVH, lens_new)
    close(out, case["want"], 1e-2, f"prefill attention H={H} KVH={KVH} Dh={Dh} bs={bs}")


@pytest.mark.parametrize("H,KVH,Dh,bs", [(8, 2, 128, 16), (2, 2, 64, 8), (6, 3, 32, 4)])
@pytest.mark.parametrize("nsplit", [1, 3, 8])
def test_attention_prefill_bf16_long_portions(H, KVH, Dh, bs, nsplit):
    # several key tiles per workgroup, row tiles that end inside a tile, a long cached prefix; with nsplit > 1
    # every item's keys are cut into shares (short items leave some of them empty) and merged
    lens_new, lens_ctx = [300, 130, 64, 33], [300, 1000, 64, 129]
    case, S = attention_case(H, KVH, Dh, bs, lens_new=lens_new, lens_ctx=lens_ctx, seed=24, dtype=torch.bfloat16)
    out = run_prefill(case, H, KVH, lens_new, nsplit=nsplit)
    close(out, case["want"], 1e-2, f"prefill attention, long portions, H={H} KVH={KVH} Dh={Dh} bs={bs} splits={nsplit}")


def test_prefill_items_cover_the_rows_the_kernel_takes_per_item():
    """The item list is built on the host, the rows an item covers are the kernel's: the two must agree, or
    items overlap (and with key shares two workgroups then write one row's partial results)."""
    from tie_amd import kernels

    lib = kernels._lib("attention_prefill_bf16", 64)
    for group in (1, 2, 3, 4, 5, 8, 16):
        rows = int(lib.tie_attention_prefill_rows_per_item(group))
        items = kernels.prefill_items([rows * 2 + 5], group)
        assert [first for _, first in items] == [0, rows, 2 * rows], f"group of {group}"


@pytest.mark.parametrize("where", ["first", "page_edge", "tile_edge", "tile_edge_64", "far", "last"])
def test_attention_prefill_bf16_finds_one_far_key(where):
    spike = {"first": lambda ctx: 0, "page_edge": lambda ctx: 16 * 3 - 1, "tile_edge": lambda ctx: 32 * 7,
             "tile_edge_64": lambda ctx: 64 * 5 - 1, "far": lambda ctx: ctx - 259, "last": lambda ctx: ctx - 2}[where]
    lens_new = [40, 7]
    case, S = attention_case(8, 2, 64, 16, lens_new=lens_new, lens_ctx=[700, 523], seed=25, dtype=torch.bfloat16, spike=spike)
    out = run_prefill(case, 8, 2, lens_new)
    close(out, case["want"], 1e-2, f"spike at {where}")
    assert float(out[39].float().min()) > 4.9 and float(out[46].float().min()) > 4.9


@pytest.mark.parametrize("window", [1, 5, 32, 33, 100])
def test_attention_prefill_bf16_window_edges(window):
    lens_new, lens_ctx = [9, 1, 20, 50], [30, 41, 20, 200]
    case, S = attention_case(4, 2, 32, 4, lens_new=lens_new, lens_ctx=lens_ctx, seed=27, dtype=torch.bfloat16, window=window)
    for nsplit in (1, 4):
        out = run_prefill(case, 4, 2, lens_new, window=window, nsplit=nsplit)
        close(out, case["want"], 1e-2, f"prefill window {window} splits {nsplit}")


def test_argmax_and_sample_kernels():
    from tie_amd import kernels

    logits = rnd(4, 1537, seed=11, scale=2.0)
    logits[1, 900] = logits[1, 30] = 50.0                      # a tie: the lowest id
    logits[2, 5] = float("nan")
    logits = logits.cuda()
    out = torch.empty(4, dtype=torch.int32, device="cuda")
    kernels.argmax_rows(logits, out)
    assert out.tolist() == [int(torch.argmax(logits[0])), 30, -1, int(torch.argmax(logits[3]))]
    top = torch.empty(4, device="cuda")
    kernels.argmax_rows(logits, out, top)                     # the maximum itself comes along on request
    assert out.tolist()[1] == 30 and float(top[1]) == 50.0 and float(top[0]) == float(logits[0].max())
    # frequencies of log {0.7, 0.2, 0.1} at temperature 1 (the reference's sampler test), many rows at once
    R = 4000
    rows = torch.log(torch.tensor([0.7, 0.2, 0.1])).repeat(R, 1).cuda()
    g = torch.Generator().manual_seed(1)
    uniform = torch.rand(R, generator=g, dtype=torch.float64).cuda()
    drawn = torch.empty(R, dtype=torch.int32, device="cuda")
    kernels.sample_rows(rows, torch.ones(R, device="cuda"), uniform, drawn)
    freq = torch.bincount(drawn.cpu().long(), minlength=3).double() / R
    assert freq[0] == pytest.approx(0.7, abs=0.03) and freq[1] == pytest.approx(0.2, abs=0.03)
    # the draw inverts the cumulative sum in index order
    want = torch.searchsorted(torch.cumsum(torch.tensor([0.7, 0.2, 0.1], dtype=torch.float64), 0) / 1.0, uniform.cpu() * 1.0,
                              right=True).clamp(max=2)
    assert (drawn.cpu().long() == want).float().mean() > 0.999


@pytest.mark.parametrize("vocab", [7, 1537, 50257, 151936])
def test_temperature_sampling_kernel_draws_what_the_host_rule_draws(vocab):
    """The walk in index order, against ``sample`` with the same uniform numbers: vocabularies that are no
    multiple of the kernel's pieces of 256 (and rows that start off 16 bytes), -inf logits, temperatures; the
    odd rows; only the rows listed, with the maxima given."""
    import numpy as np
    from tie_amd import kernels
    from tie_amd.sampling import RandomStream, SamplingParams, sample

    g = torch.Generator().manual_seed(vocab)
    temperatures = [1.0, 0.5, 3.0, 0.05, 1.0, 0.8]
    R = len(temperatures)
    logits = torch.randn(R, vocab, generator=g) * 3
    logits[4, torch.randperm(vocab, generator=g)[:vocab // 2]] = float("-inf")
    logits[5, -1] = logits[5].max() + 3                       # most of the weight on the row's last logit
    dev = logits.cuda()
    inv_t = torch.tensor([float(np.float32(1.0) / np.float32(t)) for t in temperatures], device="cuda")
    streams, host_streams = [RandomStream(i) for i in range(R)], [RandomStream(i) for i in range(R)]
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    host = logits.numpy()
    for d in range(40):
        uniform = torch.tensor([s.unit() for s in streams], dtype=torch.float64).cuda()
        kernels.sample_rows(dev, inv_t, uniform, out)
        want = [sample(host[i], SamplingParams(temperature=temperatures[i]), host_streams[i]) for i in range(R)]
        assert out.tolist() == want, f"draw {d}"
    listed = torch.tensor([4, 1], dtype=torch.int32, device="cuda")
    again = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    kernels.sample_rows(dev, inv_t, uniform, again, listed, dev.max(dim=1).values.contiguous())
    assert again.tolist() == [-7, want[1], -7, -7, want[4], -7]
    odd = torch.randn(3, vocab, generator=g)
    odd[0, vocab // 2] = float("nan")
    odd[1] = float("-inf")
    odd[2, 5] = odd[2, 2] = float("inf")
    three = torch.empty(3, dtype=torch.int32, device="cuda")
    kernels.sample_rows(odd.cuda(), inv_t[:3].contiguous(), uniform[:3].contiguous(), three)
    assert three.tolist() == [-1, -2, 2]


@pytest.mark.parametrize("vocab", [300, 5000, 151936])
def test_temperature_sampling_never_picks_a_token_of_weight_zero(vocab):
    """Uniform numbers at the very end of [0, 1): the walk ends at the last token that weighs anything, also where
    rounding lets the kernel's sums disagree by an ulp; never at a -inf logit behind it, wherever the row's last
    finite logit lies (in the last piece of 256, in an earlier one, in the first)."""
    import numpy as np
    from tie_amd import kernels

    g = torch.Generator().manual_seed(vocab)
    ends = sorted({1, 2, 255, 256, 257, vocab // 3, vocab - 257, vocab - 1, vocab} & set(range(1, vocab + 1)))
    logits = torch.randn(len(ends), vocab, generator=g) * 2
    for r, end in enumerate(ends):
        logits[r, end:] = float("-inf")
        logits[r, end - 1] = logits[r, :end].max()        # weighs at least 1 / vocab of the total at any temperature
    dev = logits.cuda()
    R = len(ends)
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    for inv_t in (1.0, 0.37, 2.9):
        for u in (np.nextafter(1.0, 0.0), 1.0 - 2.0 ** -52, 1.0 - 2.0 ** -50, 1.0 - 1e-13):
            kernels.sample_rows(dev, torch.full((R,), inv_t, device="cuda"),
                                torch.full((R,), u, dtype=torch.float64, device="cuda"), out)
            for r, end in enumerate(ends):
                assert int(out[r]) == end - 1, f"row ending at {end}, uniform 1 - {1.0 - u:.3g}, 1/T {inv_t}"


@pytest.mark.parametrize("vocab", [1000, 151936])
def test_sampling_kernel_with_top_k_and_top_p_draws_what_the_host_rule_draws(vocab):
    """The kernel that selects instead of sorting, against ``sample`` (sort, sums in double precision), draw by
    draw with the same uniform numbers: every combination of top-k and top-p, logits with many exact ties (steps
    of 0.25, so that the k-th value and the top-p boundary fall among equals and the ids decide), -inf logits,
    a tiny temperature, all logits equal. Rows not listed keep what the output held."""
    import numpy as np
    from tie_amd import kernels
    from tie_amd.sampling import RandomStream, SamplingParams, sample

    g = torch.Generator().manual_seed(vocab)
    smooth = torch.randn(vocab, generator=g) * 3
    stepped = (torch.randn(vocab, generator=g) * 2 / 0.25).round() * 0.25
    holes = smooth.clone()
    holes[torch.randperm(vocab, generator=g)[:vocab // 3]] = float("-inf")
    flat = torch.full((vocab,), 1.5)
    cases = []
    for name, row in (("smooth", smooth), ("stepped", stepped), ("holes", holes), ("flat", flat)):
        for temperature in (1.0, 0.6, 2.5, 1e-3):
            for top_k in (0, 1, 7, 50, vocab - 1, vocab + 5):
                for top_p in (1.0, 0.95, 0.5, 0.02):
                    if top_k in (0, vocab + 5) and top_p == 1.0:
                        continue
                    cases.append((name, row, temperature, top_k, top_p))
    cases, draws = (cases[::7], 4) if vocab > 10000 else (cases, 6)     # the host rule sorts every large row: fewer of them
    R = len(cases)
    logits = torch.stack([c[1] for c in cases]).cuda()
    inv_t = torch.tensor([float(np.float32(1.0) / np.float32(c[2])) for c in cases], device="cuda")
    top_k = torch.tensor([c[3] for c in cases], dtype=torch.int32, device="cuda")
    top_p = torch.tensor([c[4] for c in cases], dtype=torch.float32, device="cuda")
    streams = [RandomStream(i) for i in range(R)]
    host_streams = [RandomStream(i) for i in range(R)]
    host_rows = {name: row.numpy() for name, row, *_ in cases}
    out = torch.empty(R, dtype=torch.int32, device="cuda")
    for d in range(draws):
        uniform = torch.tensor([s.unit() for s in streams], dtype=torch.float64).cuda()
        out.fill_(-7)
        kernels.sample_rows_filtered(logits, inv_t, uniform, top_k, top_p, out)
        got = out.tolist()
        for i, (name, _, temperature, k, p) in enumerate(cases):
            want = sample(host_rows[name], SamplingParams(temperature=temperature, top_k=k, top_p=p), host_streams[i])
            assert got[i] == want, f"{name} T={temperature} top_k={k} top_p={p} draw {d}: {got[i]} != {want}"
    # only the rows listed
    listed = torch.tensor([3, 0, R - 1], dtype=torch.int32, device="cuda")
    again = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    kernels.sample_rows_filtered(logits, inv_t, uniform, top_k, top_p, again, listed)
    again = again.tolist()
    assert [again[i] for i in (3, 0, R - 1)] == [got[i] for i in (3, 0, R - 1)]
    # the maxima given by the caller (the sampler has them from the argmax kernel)
    given = torch.empty(R, dtype=torch.int32, device="cuda")
    kernels.sample_rows_filtered(logits, inv_t, uniform, top_k, top_p, given, row_max=logits.max(dim=1).values.contiguous())
    assert given.tolist() == got
    assert all(t == -7 for i, t in enumerate(again) if i not in (3, 0, R - 1))
    # a NaN and a row of -inf are reported, a +inf logit wins
    odd = torch.randn(3, vocab, generator=g)
    odd[0, 11] = float("nan")
    odd[1] = float("-inf")
    odd[2, 40] = odd[2, 90] = float("inf")
    three = torch.empty(3, dtype=torch.int32, device="cuda")
    kernels.sample_rows_filtered(odd.cuda(), inv_t[:3].contiguous(), uniform[:3].contiguous(), top_k[:3].contiguous(),
                                 top_p[:3].contiguous(), three)
    assert three.tolist() == [-1, -2, 40]


def test_kernels_refuse_what_they_cannot_take():
    from tie_amd import kernels
    from tie_amd.errors import InvalidArgument, KernelUnavailable

    with pytest.raises(KernelUnavailable, match="no CPU fallback"):
        kernels.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-6, torch.zeros(2, 8))
    with pytest.raises(InvalidArgument):
        kernels.rms_norm(torch.zeros(2, 8).cuda(), torch.ones(4).cuda(), 1e-6, torch.zeros(2, 8).cuda())
    with pytest.raises(InvalidArgument):
        kernels.gemm_generic(torch.zeros(2, 8).cuda(), torch.zeros(4, 6).cuda(), torch.zeros(2, 4).cuda())
    with pytest.raises(InvalidArgument, match="head_dim"):
        kernels.qk_norm_rope_kv_write(torch.zeros(1, 3 * 1024).cuda(), torch.zeros(1, 1024).cuda(), None, None, 0.0, None,
                                      i32([0]), i32([0]), torch.zeros(1, 1, 4, 1024).cuda(),
                                      torch.zeros(1, 1, 1024, 4).cuda(), 1, 1, 1024, 4)
    with pytest.raises(InvalidArgument):
        kernels.embed(torch.zeros(4, 8, dtype=torch.float16).cuda(), i32([0]), torch.zeros(1, 8).cuda())


@pytest.mark.parametrize("M", [1, 8, 40, 65, 300])
@pytest.mark.parametrize("I,K", [(8, 64), (200, 96), (1000, 512)])
def test_gated_product_is_silu_gate_times_up(M, I, K):
    from tie_amd import kernels

    x = rnd(M, K, seed=41, dtype=torch.bfloat16).cuda()
    gate = rnd(I, K, seed=42, scale=0.2, dtype=torch.bfloat16).cuda()
    up = rnd(I, K, seed=43, scale=0.2, dtype=torch.bfloat16).cuda()
    w = kernels.interleave_gate_up(gate, up)
    assert torch.equal(w[:8], gate[:8]) and torch.equal(w[8:16], up[:8])
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device="cuda")
    kernels.linear_swiglu(x, w, out)
    g, u = plain.linear(x.cpu(), gate.cpu()), plain.linear(x.cpu(), up.cpu())
    close(out, g / (1 + torch.exp(-g)) * u, 6e-3, f"gated product M={M} I={I}")
    if M <= 64:
        big = torch.empty_like(out)
        kernels.gemm_bf16(x, w, big, gated=True)                    # both kernels hold the same epilogue
        close(big, out.float(), 8e-3, "gated product, tiled kernel")


def test_random_weights_are_the_same_bits_on_the_gpu_and_on_the_host():
    """``random_tensor(..., device="cuda")`` against the host's draw, bit for bit: normal values (the central
    rational function and the near tails with their root and logarithm series; the far tail beyond 6.7 standard
    deviations comes up about once in 10^11 draws and is not met by sampling), norm weights, sizes that are no
    multiple of the kernel's block, float32 and the two 16-bit roundings, and a whole model folder."""
    from conftest import TINY_B
    from tie_amd.models.builder import expected_tensors_for_config
    from tie_amd.weights import random_init as ri
    from tie_amd.weights.binder import TensorSpec

    for shape, init, role in (((1537, 1031), ("normal", 0.02), "matrix"), ((3, 5, 7), ("normal", 1.0), "matrix"),
                              ((4097,), ("one_plus_uniform", 0.1), "vector"), ((1,), ("normal", 0.5), "matrix")):
        for dtype in (torch.float32, torch.bfloat16, torch.float16):
            spec = TensorSpec("model.layers.3.x.weight", shape, role, init)
            host = ri.random_tensor(spec, 17, dtype, "cpu")
            dev = ri.random_tensor(spec, 17, dtype, "cuda")
            assert dev.is_cuda and dev.dtype == dtype and tuple(dev.shape) == shape
            same = torch.equal(dev.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                               host.view(torch.int16 if dtype != torch.float32 else torch.int32))
            assert same, f"{shape} {init} {dtype}: {int((dev.cpu() != host).sum())} elements differ"
    tails = ri.random_tensor(TensorSpec("t", (1 << 22,), "matrix", ("normal", 1.0)), 1, torch.float32, "cuda")
    assert float(tails.abs().max()) > 4.5                      # the tail branch ran (and matched above at 1.6 M values)
    specs = [s for s in expected_tensors_for_config(TINY_B) if not s.optional]
    on_host = dict(ri.random_tensors(specs, 5, torch.bfloat16, "cpu", vector_dtype=torch.float32))
    on_gpu = dict(ri.random_tensors(specs, 5, torch.bfloat16, "cuda", vector_dtype=torch.float32))
    assert list(on_host) == list(on_gpu)
    for name, t in on_host.items():
        assert torch.equal(on_gpu[name].cpu().float(), t.float()), name


@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (3, 4096, 4096), (8, 96, 12288), (16, 1024, 160), (16, 8192, 128),
                                   (7, 5200, 96)])
@pytest.mark.parametrize("packed", [True, False])
def test_decode_product_with_the_norms_work_in_its_epilogue(M, N, K, packed):
    """The product that ends a sub-layer adds to the stream in place and leaves bf16(stream * weight) and the sums
    of the stream's squares per 16-column tile; the products that read those rows multiply their sums by
    1 / sqrt(sum of squares / n + eps) - stored whole, in planes over K, or under the gated activation. Against
    the formulas in float64, and the stream's new value bit for bit against the same product without the
    epilogue's extra work. Chained, the two give what RMSNorm between two products gives (src/model/qwen3.cpp:
    230-235: o_proj, add, rms_norm, gate/up)."""
    from tie_amd import kernels

    x = rnd(M, K, seed=41, dtype=torch.bfloat16).cuda()
    w = rnd(N, K, seed=42, scale=0.05, dtype=torch.bfloat16).cuda()
    weight = kernels.pack_weight(w) if packed and kernels.packable(w) else w
    if packed and weight is w:
        pytest.skip("this shape cannot be packed")
    stream = rnd(M, N, seed=43).cuda()
    norm_w = (1 + 0.1 * rnd(N, seed=44)).cuda()
    plainly = stream.clone()
    kernels.skinny_gemm_bf16(x, weight, plainly, accumulate=True)
    want = stream.cpu().to(F64) + plain.linear(x.cpu(), w.cpu())
    # waves a workgroup and k-blocks a batch of loads: four waves (the sums of the product without the epilogue's
    # work, bit for bit), and the wider workgroups that packed weights get where the output is narrow; last, the rule
    for waves, loads in ([(4, 0), (8, 8), (8, 4), (16, 4), (16, 2), (0, 0)] if packed else [(4, 0), (0, 0)]):
        got = stream.clone()
        rows = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        squares = torch.full((M, N // 16), float("nan"), device="cuda")
        kernels.skinny_gemm_bf16(x, weight, got, accumulate=True, next_norm=(norm_w, rows, squares), waves=waves, loads=loads)
        if waves == 4:
            assert torch.equal(got, plainly), "the stream differs from the product without the norm's work"
        close(got, want, 1e-5, f"stream, {waves} waves")
        assert torch.equal(rows, (got * norm_w).to(torch.bfloat16)), f"rows for the next norm, {waves} waves"
        close(squares, (got.cpu().to(F64) ** 2).view(M, N // 16, 16).sum(-1), 1e-6, f"sums of squares, {waves} waves")
    with pytest.raises(kernels.InvalidArgument):
        kernels.skinny_gemm_bf16(x, weight, got.clone(), accumulate=True, next_norm=(norm_w, rows, squares), waves=5)

    # the consumers: x2 = rows (no 1 / rms yet) against a second weight
    eps = 1e-5
    inv = 1.0 / torch.sqrt((got.cpu().to(F64) ** 2).mean(-1, keepdim=True) + eps)
    scale = kernels.RowScale(squares, N, eps)
    N2 = 192
    w2 = rnd(N2, N, seed=45, scale=0.05, dtype=torch.bfloat16).cuda()
    weight2 = kernels.pack_weight(w2) if packed and kernels.packable(w2) else w2
    unscaled = plain.linear(rows.cpu(), w2.cpu())
    out = torch.empty(M, N2, device="cuda")
    kernels.skinny_gemm_bf16(rows, weight2, out, row_scale=scale)
    close(out, unscaled * inv, 1e-5, "scaled product")
    if N % 256 == 0:                                   # planes over K need k-blocks enough for every range
        planes = torch.empty(4, M, N2, device="cuda")
        kernels.skinny_gemm_bf16(rows, weight2, planes, splits=4, row_scale=scale)
        close(planes.sum(0), unscaled * inv, 1e-5, "scaled product in four planes")
    gate, up = w2[:N2 // 2], w2[N2 // 2:]
    both = kernels.interleave_gate_up(gate.contiguous(), up.contiguous())
    both = kernels.pack_weight(both) if packed and kernels.packable(both) else both
    act = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device="cuda")
    kernels.linear_swiglu(rows, both, act, row_scale=scale)
    g, u = unscaled[:, :N2 // 2] * inv, unscaled[:, N2 // 2:] * inv
    close(act, g / (1 + torch.exp(-g)) * u, 1e-2, "gated product of scaled sums")
    # and against the norm itself: (stream * inv * norm_w) @ w2^T, the reference's order of operations
    normed = plain.rms_norm(got.cpu().to(F64), norm_w.cpu().to(F64), eps)
    close(out, plain.linear(normed, w2.cpu()), 1e-2, "the two epilogues against RMSNorm between the products")
    # rows that go where no epilogue applies the factor get it in place
    copy = rows.clone()
    kernels.scale_rows(copy, scale)
    close(copy, rows.cpu().to(F64) * inv, 1e-2, "rows scaled in place")
    with pytest.raises(kernels.InvalidArgument):
        kernels.skinny_gemm_bf16(rnd(17, K, dtype=torch.bfloat16).cuda(), weight, torch.empty(17, N, device="cuda"),
                                 row_scale=scale)


@pytest.mark.parametrize("Dh,bs,planes", [(128, 16, 1), (64, 8, 2), (256, 32, 1), (32, 16, 4), (128, 4, 1)])
@pytest.mark.parametrize("cache_dtype", [torch.bfloat16, torch.float16])
def test_values_of_a_portion_reach_the_cache_in_pieces_of_eight_tokens(Dh, bs, planes, cache_dtype):
    """From 32 rows on the values are stored by a kernel that takes eight consecutive rows of a dimension at once
    where their slots are eight consecutive, aligned positions of one page, and one by one elsewhere: runs that
    start inside a page, a sequence that ends in the middle of a group, scattered single slots. The same bits as
    the rows written a few at a time (the kernel that writes a token a workgroup), and the plain transposition."""
    from tie_amd import kernels

    H, KVH, eps = 4, 2, 1e-6
    NB = 40
    rng = np.random.RandomState(5)
    # rows of the step: a run aligned to a page, a run that starts at position 3 of a page, scattered slots, and a
    # run that ends 5 rows into a group
    pages = rng.permutation(NB)
    runs = []
    runs += [pages[0] * bs + i for i in range(min(bs, 24))] + [pages[1] * bs + i for i in range(bs)]
    runs += [pages[2] * bs + 3 + i for i in range(bs - 3)] + [pages[3] * bs + i for i in range(bs)]
    runs += [int(pages[4 + i] * bs + rng.randint(bs)) for i in range(9)]
    runs += [pages[20] * bs + i for i in range(min(bs, 13))]
    while len(runs) < 40:
        runs.append(int(pages[21 + len(runs) % 10] * bs + len(runs) % bs))
    assert len(set(runs)) == len(runs)
    T = len(runs)
    width = (H + 2 * KVH) * Dh
    qkv = rnd(planes, T, width, seed=61).cuda()
    summed = qkv[0].clone()
    for p in range(1, planes):
        summed = summed + qkv[p]
    qw, kw = (1 + 0.1 * rnd(Dh, seed=62)).cuda(), (1 + 0.1 * rnd(Dh, seed=63)).cuda()
    inv_freq = torch.from_numpy(plain.rope_inv_freq(1e4, Dh)).cuda()
    positions, slots = i32(list(range(T))), i32(runs)
    q_dtype = torch.bfloat16 if cache_dtype == torch.bfloat16 else torch.float32
    x = qkv if q_dtype == torch.float32 else qkv        # float32 sums either way

    def run(rows):
        kc = torch.zeros(NB, KVH, bs, Dh, device="cuda", dtype=cache_dtype)
        vc = torch.zeros(NB, KVH, Dh, bs, device="cuda", dtype=cache_dtype)
        q = torch.empty(T, H * Dh, device="cuda", dtype=q_dtype)
        for first in range(0, T, rows):
            n = min(rows, T - first)
            kernels.qk_norm_rope_kv_write(x[0, first:first + n], q[first:first + n], qw, kw, eps, inv_freq,
                                          positions[first:first + n], slots[first:first + n], kc, vc, H, KVH, Dh, bs,
                                          planes=planes, plane_stride=T * width)
        return q, kc, vc

    q_all, k_all, v_all = run(T)            # one call: 40 rows or more, the values by the kernel of their own
    q_few, k_few, v_few = run(7)            # a few rows a call: the kernel that writes a token a workgroup
    assert torch.equal(q_all, q_few) and torch.equal(k_all, k_few)
    assert torch.equal(v_all, v_few), "the values differ between the two ways of writing them"
    want = summed[:, (H + KVH) * Dh:].view(T, KVH, Dh).cpu()
    for t, slot in enumerate(runs):
        assert torch.equal(v_all[slot // bs, :, :, slot % bs].cpu(), want[t].to(cache_dtype)), f"row {t}, slot {slot}"
    assert int((v_all != 0).sum()) <= T * KVH * Dh          # nothing written beside the rows' slots
