"""Times single kernels against their rooflines on one MI355X.

    python -m prelude_amd.bench_kernels [stream] [gemm] [tall] [dispatch] [normed] [cuts] [decode] [prefill] [elementwise] [sampling] [--shape 4b|8b|32b]

Each line gives the kernel's time (device events around repeated launches,
operands rotated over copies larger than the caches where the kernel streams
memory), the rate it reached and that rate as a fraction of the published peak
(HBM 8 TB/s, dense bfloat16 MFMA 2.5 PFLOP/s).  The shapes are those of the
Qwen3 sizes the benchmark configurations name.
"""
from __future__ import annotations

import argparse
import math

import torch

from .ops import kernels as K

HBM_PEAK = 8.0e12
MFMA_PEAK = 2.5e15
SHAPES = {   # hidden, intermediate, heads, kv heads, head_dim, vocabulary
    "0.6b": (1024, 3072, 16, 8, 128, 151936),
    "1.7b": (2048, 6144, 16, 8, 128, 151936),
    "4b": (2560, 9728, 32, 8, 128, 151936),
    "8b": (4096, 12288, 32, 8, 128, 151936),
    "14b": (5120, 17408, 40, 8, 128, 151936),
    "32b": (5120, 25600, 64, 8, 128, 151936),
}


def timeit(fn, variants: int, iters: int = 50) -> float:
    """Microseconds per call of fn(i), i cycling over the operand copies."""
    for i in range(5):
        fn(i % variants)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(iters):
        fn(i % variants)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters * 1e3


def line(name: str, us: float, nbytes: float = 0.0, flops: float = 0.0) -> None:
    parts = [f"{name:46s} {us:9.1f} us"]
    if nbytes:
        rate = nbytes / us * 1e6
        parts.append(f"{rate / 1e9:8.0f} GB/s  {rate / HBM_PEAK:5.2f} of HBM peak")
    if flops:
        rate = flops / us * 1e6
        parts.append(f"{rate / 1e12:8.1f} TFLOP/s  {rate / MFMA_PEAK:5.2f} of MFMA peak")
    print("  ".join(parts), flush=True)


def bench_stream(dev, shape) -> None:
    """The rate a kernel that does nothing but read reaches over 8 GB: what the published 8 TB/s comes to here."""
    from ._native import check, kernels
    nbytes = 8 << 30
    buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    buf.zero_()
    for blocks in (1024, 2048, 4096, 8192, 16384):
        out = torch.zeros(blocks, dtype=torch.int32, device=dev)
        us = timeit(lambda i: check(kernels().pa_stream_read(K._stream(), buf.data_ptr(), nbytes, out.data_ptr(), blocks)), 1, iters=10)
        line(f"read 8 GB, {blocks} workgroups of 256 threads", us, nbytes=nbytes)


def bench_gemm(dev, shape) -> None:
    h, inter, nh, nkv, hd, vocab = shape
    weights = {"qkv": ((nh + 2 * nkv) * hd, h), "o": (h, nh * hd), "gate_up (SiLU*up)": (2 * inter, h),
               "down": (h, inter), "head (f32 out)": (vocab, h)}
    for name, (n, k) in weights.items():
        copies = max(2, int(600e6 // (n * k * 2)))
        rows = [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        tiles = [K.pack_tiles(w) for w in rows]
        silu = name.startswith("gate_up")
        f32 = torch.float32 if name.startswith("head") else None
        for m in (1, 8, 16):
            x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
            us = timeit(lambda i: K.gemm_skinny(x, tiles[i], out_dtype=f32, silu_mul_epilogue=silu), copies)
            line(f"gemm {name} [{n}x{k}] M={m} tiled", us, nbytes=n * k * 2)
        # what the engine's dispatcher sends 32 to 128 rows to (the product with X staged in LDS where it measured
        # faster: cut into slices of K for o and down, whose reader adds them; SiLU*up in its epilogue), and the
        # library beside it
        weights_of = [K.LinearWeight(r, t) for r, t in zip(rows, tiles)]
        for m in (32, 64, 128):
            x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
            if silu:
                us = timeit(lambda i: K.linear_silu_mul(x, weights_of[i]), copies, iters=20)
            else:
                us = timeit(lambda i: K.linear(x, weights_of[i], out_dtype=f32, slices_ok=name in ("o", "down")), copies, iters=20)
            line(f"gemm {name} [{n}x{k}] M={m} as dispatched", us, nbytes=n * k * 2)
            if silu:
                us = timeit(lambda i: K.silu_mul(K.gemm_library(x, rows[i])), copies, iters=20)
            elif f32 is not None:
                us = timeit(lambda i: K.to_f32(K.gemm_library(x, rows[i])), copies, iters=20)
            else:
                us = timeit(lambda i: K.gemm_library(x, rows[i]), copies, iters=20)
            line(f"gemm {name} [{n}x{k}] M={m} library" + (" + SiLU*up" if silu else " + widening" if f32 is not None else ""),
                 us, nbytes=n * k * 2)
        x = torch.randn(2048, k, device=dev, dtype=torch.bfloat16)
        us = timeit(lambda i: K.gemm_library(x, rows[i]), copies, iters=20)
        line(f"gemm {name} [{n}x{k}] M=2048 library", us, flops=2.0 * 2048 * n * k)
        del rows, tiles, weights_of


def bench_tall(dev, shape) -> None:
    """Products of 129 to 1,024 rows: the kernel tiled both ways (``gemm_tall``: in four slices of K for o and down,
    which the norm after them adds; with the activation in its epilogue for gate_up) beside the library (with
    its separate activation kernel for gate_up), weights rotated over 600 MB so that they come from memory.  Which
    of the two a step takes is ``ops.kernels.linear``'s choice, made from whole prompt steps, not from these."""
    h, inter, nh, nkv, hd, vocab = shape
    weights = {"qkv": ((nh + 2 * nkv) * hd, h), "o": (h, nh * hd), "gate_up (act*up)": (2 * inter, h), "down": (h, inter)}
    for name, (n, k) in weights.items():
        copies = max(2, int(600e6 // (n * k * 2)))
        rows = [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        tiles = [K.pack_tiles(w) for w in rows]
        gated = name.startswith("gate_up")
        slices = K._tall_slices(k) if name in ("o", "down") else 1
        for m in (129, 192, 256, 384, 512, 1024):
            x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
            flops = 2.0 * m * n * k
            us = timeit(lambda i: K.gemm_tall(x, tiles[i], silu_mul_epilogue=gated, slices=slices), copies, iters=20)
            line(f"gemm {name} [{n}x{k}] M={m} tall" + (f" in {slices} slices" if slices > 1 else ""), us, flops=flops)
            if gated:
                us = timeit(lambda i: K.silu_mul(K.gemm_library(x, rows[i])), copies, iters=20)
            else:
                us = timeit(lambda i: K.gemm_library(x, rows[i]), copies, iters=20)
            line(f"gemm {name} [{n}x{k}] M={m} library" + (" + act*up" if gated else ""), us, flops=flops)
        del rows, tiles


def graph_time(fns, iters: int = 10) -> float:
    """Microseconds per call of the chain ``fns`` (one call per operand copy), replayed from a captured graph: what a
    kernel costs inside a step, where no launch waits for the host."""
    for f in fns:
        f()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for f in fns:
            f()
    g.replay()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        g.replay()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters / len(fns) * 1e3


def bench_dispatch(dev, shape) -> None:
    """Every product of the shape at 1 to 512 rows as ``ops.kernels.linear`` / ``linear_gated`` dispatch it against
    every kernel forced, each with its reader behind it (the residual add + norm for o and down, which takes a
    product's slices as they are), inside a graph, weights rotated so that they come from memory.  A line ends in
    ``<<<`` where the dispatcher's choice is more than a twentieth behind the best kernel."""
    h, inter, nh, nkv, hd, _ = shape
    prods = {"qkv": ((nh + 2 * nkv) * hd, h, "tensor"), "o": (h, nh * hd, "norm"), "gate_up": (2 * inter, h, "gated"),
             "down": (h, inter, "norm")}
    for pname, (n, k, kind) in prods.items():
        copies = max(3, min(12, int(700e6 // (n * k * 2))))
        rows = [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        lws = [K.LinearWeight(r, K.pack_tiles(r)) for r in rows]
        gain = torch.ones(n, device=dev)
        for m in (1, 4, 8, 12, 16, 20, 24, 32, 48, 64, 96, 128, 160, 192, 256, 384, 512):
            x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
            res = torch.randn(m, n, device=dev, dtype=torch.bfloat16)
            norm = lambda y: K.rmsnorm(y, gain, 1e-6, residual=res)
            cands = {}
            if kind == "tensor":
                cands["dispatched"] = lambda w: K.linear(x, w)
                if m <= 64:
                    cands["skinny"] = lambda w: K.gemm_skinny(x, w.tiles)
                if m <= 128:
                    cands["mid"] = lambda w: K.gemm_mid(x, w.tiles)
                    s = K.gemm_mid_slices(n, k)
                    if s > 1:
                        cands["mid sliced + sum"] = lambda w: K.gemm_mid(x, w.tiles, slices=s).materialize()
                cands["library"] = lambda w: K.gemm_library(x, w.rows)
                if m > 16:
                    cands["tall"] = lambda w: K.gemm_tall(x, w.tiles)
            elif kind == "norm":
                cands["dispatched"] = lambda w: norm(K.linear(x, w, slices_ok=True))
                if m <= 64:
                    cands["skinny"] = lambda w: norm(K.gemm_skinny(x, w.tiles))
                if m <= 128:
                    s = K.gemm_mid_slices(n, k)
                    if s > 1:
                        cands["mid sliced"] = lambda w: norm(K.gemm_mid(x, w.tiles, slices=s))
                    cands["mid"] = lambda w: norm(K.gemm_mid(x, w.tiles))
                cands["library"] = lambda w: norm(K.gemm_library(x, w.rows))
                if m > 16:
                    s4 = K._tall_slices(k)
                    if s4 > 1:
                        cands["tall sliced"] = lambda w: norm(K.gemm_tall(x, w.tiles, slices=s4))
                    cands["tall"] = lambda w: norm(K.gemm_tall(x, w.tiles))
            else:
                cands["dispatched"] = lambda w: K.linear_gated(x, w, "silu")
                if m <= 64:
                    cands["skinny"] = lambda w: K.gemm_skinny(x, w.tiles, silu_mul_epilogue=True)
                if m <= 128:
                    cands["mid"] = lambda w: K.gemm_mid(x, w.tiles, silu_mul_epilogue=True)
                cands["library"] = lambda w: K.silu_mul(K.gemm_library(x, w.rows))
                if m > 16:
                    cands["tall"] = lambda w: K.gemm_tall(x, w.tiles, silu_mul_epilogue=True)
            t = {c: graph_time([(lambda w=w, f=f: f(w)) for w in lws]) for c, f in cands.items()}
            d = t.pop("dispatched")
            best = min(t, key=t.get)
            print(f"{pname:8s} [{n:6d} x {k:6d}] M={m:4d}: dispatched {d:7.1f} us  best {best:16s} {t[best]:7.1f}   " +
                  "  ".join(f"{c} {v:.1f}" for c, v in t.items()) + ("  <<<" if d > 1.05 * t[best] + 0.3 else ""), flush=True)
        del rows, lws


def bench_normed(dev, shape) -> None:
    """The residual add + RMSNorm and the gated product behind it at 1 to 16 rows: the two kernels apart (the product
    as ``linear_gated`` dispatches it) against the one kernel that does both, inside a graph, weights from memory."""
    h, inter = shape[0], shape[1]
    n, k = 2 * inter, h
    copies = max(3, min(12, int(700e6 // (n * k * 2))))
    rows = [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
    lws = [K.LinearWeight(r, K.pack_tiles(r)) for r in rows]
    gain = torch.ones(k, device=dev)
    for m in (1, 2, 4, 6, 8, 12, 16):
        x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
        res = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
        apart = graph_time([(lambda w=w: K.linear_gated(K.rmsnorm(x, gain, 1e-6, residual=res), w, "silu")) for w in lws])
        if not K.gated_after_norm_supported(x, res, lws[0]):
            print(f"norm + gate_up [{n:6d} x {k:6d}] M={m:4d}: apart {apart:7.1f} us  (the one kernel does not take this)", flush=True)
            continue
        fused = graph_time([(lambda w=w: K.linear_gated_after_norm(x, res, gain, 1e-6, w, "silu")) for w in lws])
        print(f"norm + gate_up [{n:6d} x {k:6d}] M={m:4d}: apart {apart:7.1f} us  in one kernel {fused:7.1f} us", flush=True)


def bench_cuts(dev, shape, page: int = 16) -> None:
    """The prefill attention as its launcher cuts the work against every cut forced (tiles paired, unpaired, or
    unpaired with the tiles slowest over the grid; 1 or 2 heads a wavefront, 1 or 2 head groups a workgroup), over
    prompts of 256 to 8,192 tokens, several prompts a step and portions behind long contexts; every cut gives the
    same bits."""
    _, _, nh, nkv, hd, _ = shape
    sizes = [(1, t, t) for t in (256, 512, 1024, 1536, 2048, 3072, 4096, 6144, 8192)]
    sizes += [(n, 512, 512) for n in (2, 3, 4, 6, 8, 16)] + [(3, 1024, 1024), (2, 2048, 2048), (3, 2048, 2048), (1, 512, 4096), (1, 2048, 8192)]
    for nseq, t, ctx in sizes:
        pages = nseq * ctx // page
        kc = torch.randn(pages, nkv, page, hd, device=dev, dtype=torch.bfloat16)
        vc = torch.randn(pages, nkv, hd, page, device=dev, dtype=torch.bfloat16)
        table = torch.randperm(pages, device=dev).to(torch.int32).view(nseq, ctx // page)
        q = torch.randn(nseq * t, nh, hd, device=dev, dtype=torch.bfloat16)
        seqs = torch.arange(nseq, device=dev, dtype=torch.int32)
        cu = torch.arange(0, (nseq + 1) * t, t, device=dev, dtype=torch.int32)
        lens = torch.full((nseq,), ctx, device=dev, dtype=torch.int32)
        out = torch.empty_like(q)
        scale = 1 / math.sqrt(hd)
        run = lambda cut: timeit(lambda i: K.attention_prefill(q, kc, vc, table, seqs, cu, lens, out, t, 0, scale,
                                                               min_prefix=ctx - t, cut=cut), 1, iters=15)
        for _ in range(3):
            run(None)
        res = {}
        for heads, groups in ((1, 1), (1, 2), (2, 1), (2, 2)):
            for paired in (0, 1, 2):
                try:
                    res[f"{heads} heads x {groups}{('', ' paired', ' tiles slowest')[paired]}"] = run((paired, heads, groups, 1))
                except Exception:   # a cut this shape does not have
                    pass
        us = min(run(None), run(None))
        best = min(res, key=res.get)
        flops = 2.0 * nseq * nh * hd * t * (2 * ctx - t)
        print(f"prefill attention {nseq:2d} x {t:5d} tokens, context {ctx:5d}: launcher {us:7.1f} us ({flops / us / 1e6 / MFMA_PEAK * 1e12:.2f} of peak)  "
              f"best cut {best} {res[best]:7.1f}  ratio {us / res[best]:.3f}", flush=True)


def bench_decode(dev, shape, page: int = 16) -> None:
    _, _, nh, nkv, hd, _ = shape
    for batch, ctx in ((1, 4096), (8, 512), (8, 4096), (8, 32768), (64, 4096)):
        pages = batch * ctx // page
        per_copy = pages * nkv * page * hd * 2 * 2
        copies = max(2, min(8, int(1.2e9 // per_copy)))
        kcs = [torch.randn(pages, nkv, page, hd, device=dev, dtype=torch.bfloat16) for _ in range(copies)]
        vcs = [torch.randn(pages, nkv, hd, page, device=dev, dtype=torch.bfloat16) for _ in range(copies)]
        table = torch.randperm(pages, device=dev).to(torch.int32).view(batch, ctx // page)
        q = torch.randn(batch, nh, hd, device=dev, dtype=torch.bfloat16)
        seqs = torch.arange(batch, device=dev, dtype=torch.int32)
        cu = torch.arange(batch + 1, device=dev, dtype=torch.int32)
        lens = torch.full((batch,), ctx, device=dev, dtype=torch.int32)
        out = torch.empty_like(q)
        scale = 1 / math.sqrt(hd)
        us = timeit(lambda i: K.attention_decode(q, kcs[i], vcs[i], table, seqs, cu, lens, out, ctx, 0, scale), copies)
        line(f"decode attention + merge, batch {batch}, context {ctx}", us, nbytes=per_copy)
        del kcs, vcs


def bench_prefill(dev, shape, page: int = 16) -> None:
    _, _, nh, nkv, hd, _ = shape
    for nseq, t, ctx in ((1, 512, 512), (4, 512, 512), (16, 512, 512), (1, 2048, 2048), (1, 2048, 8192), (1, 8192, 8192)):
        pages = nseq * ctx // page
        kc = torch.randn(pages, nkv, page, hd, device=dev, dtype=torch.bfloat16)
        vc = torch.randn(pages, nkv, hd, page, device=dev, dtype=torch.bfloat16)
        table = torch.randperm(pages, device=dev).to(torch.int32).view(nseq, ctx // page)
        q = torch.randn(nseq * t, nh, hd, device=dev, dtype=torch.bfloat16)
        seqs = torch.arange(nseq, device=dev, dtype=torch.int32)
        cu = torch.arange(0, (nseq + 1) * t, t, device=dev, dtype=torch.int32)
        lens = torch.full((nseq,), ctx, device=dev, dtype=torch.int32)
        out = torch.empty_like(q)
        scale = 1 / math.sqrt(hd)
        us = timeit(lambda i: K.attention_prefill(q, kc, vc, table, seqs, cu, lens, out, t, 0, scale, min_prefix=ctx - t), 1, iters=20)
        line(f"prefill attention, {nseq} x {t} tokens, context {ctx}", us, flops=2.0 * nseq * nh * hd * t * (2 * ctx - t))


def bench_elementwise(dev, shape, page: int = 16) -> None:
    h, inter, nh, nkv, hd, _ = shape
    for t in (8, 2048):
        x = torch.randn(t, h, device=dev, dtype=torch.bfloat16)
        r = torch.randn(t, h, device=dev, dtype=torch.bfloat16)
        w = torch.ones(h, device=dev)
        line(f"residual add + RMSNorm, {t} tokens", timeit(lambda i: K.rmsnorm(x, w, 1e-6, residual=r), 1), nbytes=t * h * 2 * 4)
        gu = torch.randn(t, 2 * inter, device=dev, dtype=torch.bfloat16)
        line(f"SiLU*up, {t} tokens", timeit(lambda i: K.silu_mul(gu), 1), nbytes=t * inter * 2 * 3)
        qkv = torch.randn(t, (nh + 2 * nkv) * hd, device=dev, dtype=torch.bfloat16)
        nw = torch.ones(hd, device=dev)
        cos = torch.randn(4096, hd // 2, device=dev)
        pos = torch.arange(t, device=dev, dtype=torch.int32)
        kc = torch.zeros(max(t // page, 1), nkv, page, hd, device=dev, dtype=torch.bfloat16)
        vc = torch.zeros(max(t // page, 1), nkv, hd, page, device=dev, dtype=torch.bfloat16)
        line(f"QK-norm + RoPE + cache write, {t} tokens",
             timeit(lambda i: K.qknorm_rope_kv(qkv, nw, nw, cos, cos, pos, pos, kc, vc, nh, nkv, hd, hd, 1e-6), 1),
             nbytes=t * (nh * 2 + nkv * 4) * hd * 2)


def bench_sampling(dev, shape) -> None:
    vocab = shape[5]
    for rows in (1, 8, 64):
        logits = torch.randn(rows, vocab, device=dev) * 3
        u = torch.rand(rows, device=dev)
        full = lambda v, dt=torch.float32: torch.full((rows,), v, dtype=dt, device=dev)
        line(f"argmax, {rows} rows of {vocab}", timeit(lambda i: K.argmax(logits), 1), nbytes=rows * vocab * 4)
        for name, k, p in (("temperature", 0, 1.0), ("top-p 0.9", 0, 0.9), ("top-k 50", 50, 1.0), ("top-k 50, top-p 0.9", 50, 0.9)):
            args = (logits, full(0.7), full(k, torch.int32), full(p), u)
            us = timeit(lambda i: K.sample(*args, any_top_k=k > 0, any_top_p=p < 1.0), 1)
            line(f"draw, {rows} rows, {name}", us)


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("what", nargs="*", help="stream, gemm, tall, decode, prefill, elementwise, sampling (default: all these); dispatch, normed, cuts (sweeps, on request)")
    ap.add_argument("--shape", default="4b", choices=sorted(SHAPES))
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_kernels needs a GPU")
        return 1
    dev = torch.device("cuda:0")
    shape = SHAPES[args.shape]
    todo = args.what or ["stream", "gemm", "tall", "decode", "prefill", "elementwise", "sampling"]
    print(f"Qwen3-{args.shape.upper()} shapes: hidden {shape[0]}, intermediate {shape[1]}, {shape[2]} heads, "
          f"{shape[3]} KV heads, head_dim {shape[4]}, vocabulary {shape[5]}")
    for name in todo:
        {"stream": bench_stream, "gemm": bench_gemm, "tall": bench_tall, "dispatch": bench_dispatch, "normed": bench_normed, "cuts": bench_cuts, "decode": bench_decode, "prefill": bench_prefill, "elementwise": bench_elementwise,
         "sampling": bench_sampling}[name](dev, shape)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
