"""How far the products' own choice of kernel, tile and ranges of K lies from the best forced choice.

For the four projections of a layer shape (QKV, O, gate/up, down) at a list of row counts, every candidate
the launchers can be forced to - the decode product reading x from memory (1 to 4 weight tiles a
workgroup, 2 to 8 k-blocks a batch of loads) or sharing it through LDS (3, 6 or 8 tiles a workgroup), the tiled
product (64-row tiles from 17 to 64 rows, tiles of 64 and 128 rows up to 128, of 128 and 256 rows above), each in 1 to 8
ranges of K - is timed together with what its
consumer has to do for it (planes: the kernel that adds them to the stream and norms; one plane: accumulate in
place, then the norm kernel), in a recorded chain over several copies of the weight so that no cache holds it.
The product's own choice is timed the same way. Prints a line a point and a summary:

    python3 -m tie_amd.bench.product_sweep --shape 3b --rows 1,8,16,24,32,48,64

Shapes are (hidden, q width, kv width, intermediate); ``--sizes`` names another. Needs a GPU. The reference has no
counterpart (its CPU backend has one product, src/backend/cpu/cpu_backend.cpp:33-95).
"""
from __future__ import annotations

import argparse
import json
import sys

SHAPES = {"0.6b": (1024, 2048, 1024, 3072), "1.7b": (2048, 2048, 1024, 6144), "4b": (2560, 4096, 1024, 9728),
          "3b": (3072, 3072, 1024, 8192), "8b": (4096, 4096, 1024, 12288), "14b": (5120, 5120, 1024, 17408),
          "32b": (5120, 8192, 1024, 25600), "70b": (8192, 8192, 1024, 28672)}


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--shape", choices=sorted(SHAPES), default="3b")
    parser.add_argument("--sizes", default=None, help="hidden,q width,kv width,intermediate instead of --shape")
    parser.add_argument("--rows", default="1,4,8,16,24,32,48,64")
    parser.add_argument("--json", default=None, help="also append one JSON object a point (all candidates) to this file")
    args = parser.parse_args(argv)

    import torch

    from .. import kernels

    if not torch.cuda.is_available():
        print("product_sweep needs a GPU", file=sys.stderr)
        return 1
    dev = "cuda"
    torch.manual_seed(0)
    D, Q, KV, I = tuple(int(v) for v in args.sizes.split(",")) if args.sizes else SHAPES[args.shape]
    name_of_shape = args.sizes or args.shape
    rows = [int(m) for m in args.rows.split(",")]
    lib = kernels._lib("skinny_gemm_bf16")

    def timed(fn, copies):
        for i in range(copies):
            fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(copies):
                fn(i)
        for _ in range(2):
            graph.replay()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(6):
            graph.replay()
        end.record()
        end.synchronize()
        return start.elapsed_time(end) / 6 / copies * 1e3

    regrets = []
    for proj, N, K, gated in (("qkv", Q + 2 * KV, D, False), ("o", D, Q, False), ("gate/up", 2 * I, D, True),
                              ("down", D, I, False)):
        copies = max(3, min(12, int(600e6 / (N * K * 2))))
        weights = [kernels.pack_weight((torch.randn(N, K, device=dev) * 0.02).bfloat16()) for _ in range(copies)]
        norm_weight = torch.ones(N, device=dev)
        for M in rows:
            x = torch.randn(M, K, device=dev).bfloat16()
            stream = torch.randn(M, N, device=dev)
            normed = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            act = torch.empty(M, N // 2, device=dev, dtype=torch.bfloat16)
            planes = {s: torch.empty(s, M, N, device=dev) for s in (2, 4, 8)}

            def consume(s):
                if s > 1:
                    kernels.add_partials(stream, planes[s], norm_weight, 1e-6, normed)
                else:
                    kernels.rms_norm(stream, norm_weight, 1e-6, normed)

            if gated:
                def own(i):
                    kernels.linear_swiglu(x, weights[i], act)
            else:
                decode = kernels.decode_product_rows(M, weights[0])
                if decode:
                    own_splits = kernels.skinny_splits(N, K) if M <= 16 else kernels.few_rows_plan(M, N, K)[2]
                else:
                    own_splits = kernels.gemm_splits(M, N, K, True)

                def own(i):
                    if own_splits > 1:
                        (kernels.skinny_gemm_bf16 if decode else kernels.gemm_bf16)(x, weights[i], planes[own_splits],
                                                                                    splits=own_splits)
                    else:
                        kernels.linear(x, weights[i], stream, True)
                    consume(own_splits)
            t_own = timed(own, copies)
            results = []
            for s in ((1,) if gated else (1, 2, 4, 8)):
                if s > 1 and K // s < 256:
                    continue
                variants = [(rt, -u) for rt in (1, 2, 3, 4) for u in (2, 4, 8)] if M <= 64 else []
                if 16 < M <= 64:
                    variants += [(3, 1), (6, 1), (8, 1)]
                for rt, u in variants:
                    out = act if gated else (planes[s] if s > 1 else stream)

                    def forced(i, rt=rt, u=u, s=s, out=out):
                        status = lib.tie_skinny_gemm_bf16_with(
                            x.data_ptr(), weights[i].data_ptr(), out.data_ptr(), 1 if gated else 0,
                            0 if (gated or s > 1) else 1, int(gated), M, N, K, s, 1, rt, u, kernels._stream())
                        if status != 0:
                            raise RuntimeError(status)
                        if not gated:
                            consume(s)
                    label = (f"x through LDS, {rt} tiles a workgroup, {s} ranges" if u == 1 else
                             f"x from memory, {rt} tiles a workgroup, batches of {-u}, {s} ranges")
                    try:
                        results.append((timed(forced, copies), label))
                    except RuntimeError:
                        pass
                if M > 16:
                    tiles_tried = ((8, "64 x 256"), (9, "64 x 128")) if M <= 64 else \
                        ((6, "128 x 256"), (7, "128 x 128"), (8, "64 x 256"), (9, "64 x 128")) if M <= 128 else \
                        ((4, "256 x 256"), (10, "256 x 192"), (5, "256 x 128"), (6, "128 x 256"), (7, "128 x 128"))
                    for tile, shape in tiles_tried:
                        def tiled(i, tile=tile, s=s):
                            if gated:
                                kernels.gemm_bf16(x, weights[i], act, gated=True, tile=tile)
                            elif s > 1:
                                kernels.gemm_bf16(x, weights[i], planes[s], tile=tile, splits=s)
                            else:
                                kernels.gemm_bf16(x, weights[i], stream, accumulate=True, tile=tile)
                            if not gated:
                                consume(s)
                        try:
                            results.append((timed(tiled, copies), f"tiles of {shape}, {s} ranges"))
                        except Exception:
                            pass
            results.sort()
            best_t, best_label = results[0]
            regrets.append(t_own / best_t)
            print(f"{name_of_shape} {proj} [{N} x {K}] {M} rows: own choice {t_own:.1f} us, best {best_t:.1f} us ({best_label}); "
                  f"own / best = {t_own / best_t:.3f}", flush=True)
            if args.json:
                with open(args.json, "a") as fh:
                    fh.write(json.dumps({"shape": name_of_shape, "proj": proj, "N": N, "K": K, "M": M, "gated": gated,
                                         "own": t_own, "all": [(round(t, 2), n) for t, n in results]}) + "\n")
        del weights
        torch.cuda.empty_cache()
    over = sum(1 for r in regrets if r > 1.05)
    print(f"{name_of_shape}: own / best over {len(regrets)} points: mean {sum(regrets) / len(regrets):.3f}, worst {max(regrets):.3f}, "
          f"above 1.05 on {over}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
