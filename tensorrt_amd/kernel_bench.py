"""Per-kernel timings on the benchmark configurations other than the headline one.

    python -m tensorrt_amd.kernel_bench [--steps N]

Prints one line per kernel: average launch time (events around back-to-back launches on the launch
stream), achieved algorithmic bandwidth or arithmetic rate, and its fraction of the MI355X peak
(HBM 8 TB/s, dense FP16 MFMA 2.5 PFLOP/s, dense INT8 MFMA 5 POP/s).  Inputs are synthetic and
seeded, resident in HBM; torch is only the allocator.  bench.py remains the one-line contract; this
is the table behind the per-kernel figures quoted in the design notes.
"""
from __future__ import annotations

import argparse
import ctypes as C
import time

import numpy as np

PEAK_HBM = 8.0e12
PEAK_F16 = 2.5e15
PEAK_I8 = 5.0e15


def f32_bits(x) -> int:
    return int(np.float32(x).view(np.uint32))


def half2_bits(x) -> int:
    h = int(np.float16(x).view(np.uint16))
    return h | (h << 16)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--seed", type=int, default=1)
    args = ap.parse_args()

    import torch
    from tensorrt_amd import capi, workloads
    api = capi.api()
    stream = torch.cuda.current_stream().cuda_stream
    r = np.random.default_rng(args.seed)

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def timeit(fn):
        for _ in range(10):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / args.steps

    # the GPU raises its clocks over the first tens of milliseconds of load
    warm = torch.randn((4096, 4096), dtype=torch.float16, device="cuda")
    t_end = time.perf_counter() + 0.3
    while time.perf_counter() < t_end:
        torch.mm(warm, warm)
        torch.cuda.synchronize()
    del warm

    rows = []

    def report(name, t, nbytes=None, ops=None, peak_ops=None):
        if nbytes is not None:
            rows.append((name, t * 1e6, f"{nbytes / t / 1e9:8.1f} GB/s", nbytes / t / PEAK_HBM, "hbm"))
        else:
            rows.append((name, t * 1e6, f"{ops / t / 1e12:8.1f} Top/s", ops / t / peak_ops, "mfma"))

    # ---- SkipLayerNorm fp32, [8,128,768] (+bias) ------------------------------------------------
    n_rows, ld = 8 * 128, 768
    x, s = (dev(r.standard_normal((n_rows, ld)).astype(np.float32)) for _ in range(2))
    g = dev(r.uniform(0.5, 1.5, ld).astype(np.float32))
    b = dev((0.1 * r.standard_normal(ld)).astype(np.float32))
    bias = dev((0.02 * r.standard_normal(ld)).astype(np.float32))
    o = torch.empty_like(x)
    t = timeit(lambda: api.check(api.skip_layer_norm_fp32(stream, ld, n_rows * ld, x.data_ptr(), s.data_ptr(),
                                                          b.data_ptr(), g.data_ptr(), o.data_ptr(), bias.data_ptr())))
    report("SkipLN fp32 1024x768", t, nbytes=n_rows * ld * 3 * 4 + 3 * ld * 4)

    # ---- BERT-base EmbLN + SkipLN fp16, B=32 S=128 E=768 ----------------------------------------
    S, B, ld, vocab = 128, 32, 768, 30522
    word = dev((0.02 * r.standard_normal((vocab, ld))).astype(np.float16))
    pos = dev((0.02 * r.standard_normal((512, ld))).astype(np.float16))
    tok = dev((0.02 * r.standard_normal((2, ld))).astype(np.float16))
    g32 = dev(r.uniform(0.5, 1.5, ld).astype(np.float32))
    b32 = dev((0.1 * r.standard_normal(ld)).astype(np.float32))
    ids = dev(r.integers(0, vocab, (S, B)).astype(np.int32))
    segs = dev(r.integers(0, 2, (S, B)).astype(np.int32))
    emb = torch.empty((S * B, ld), dtype=torch.float16, device="cuda")
    t = timeit(lambda: api.check(api.emb_layer_norm_fp16(stream, ld, B, S, ids.data_ptr(), segs.data_ptr(),
                                                         b32.data_ptr(), g32.data_ptr(), word.data_ptr(),
                                                         pos.data_ptr(), tok.data_ptr(), vocab, 2, emb.data_ptr())))
    # gathered word rows + output + ids; the position/type rows are shared and stay in cache
    report("EmbLN fp16 B32 S128 E768", t, nbytes=S * B * (2 * ld * 2 + 8) + S * ld * 2 + 2 * ld * 2)
    lens = r.integers(64, 129, B)
    mask = dev((np.arange(S)[:, None] < lens[None, :]).astype(np.int32))
    pm = torch.zeros((B, 512), dtype=torch.int32, device="cuda")
    t = timeit(lambda: api.check(api.convert_mask(S, B, 2, 2, 1, mask.data_ptr(), pm.data_ptr(), stream)))
    report("packed mask B32 S128", t, nbytes=S * B * 4 + B * 512 * 4)
    n_rows = S * B
    xs = dev(r.standard_normal((n_rows, ld)).astype(np.float16))
    gh, bh = g32.half(), b32.half()
    biash = dev((0.02 * r.standard_normal(ld)).astype(np.float16))
    oh = torch.empty_like(emb)
    t = timeit(lambda: api.check(api.skip_layer_norm_fp16(stream, ld, n_rows * ld, emb.data_ptr(), xs.data_ptr(),
                                                          bh.data_ptr(), gh.data_ptr(), oh.data_ptr(),
                                                          biash.data_ptr())))
    report("SkipLN fp16 4096x768", t, nbytes=n_rows * ld * 3 * 2 + 3 * ld * 2)

    # ---- the same kernels at a size where the launch itself no longer matters -------------------
    n_big = 65536
    xb = torch.randn((n_big, ld), dtype=torch.float16, device="cuda")
    sb = torch.randn((n_big, ld), dtype=torch.float16, device="cuda")
    ob = torch.empty_like(xb)
    t = timeit(lambda: api.check(api.skip_layer_norm_fp16(stream, ld, n_big * ld, xb.data_ptr(), sb.data_ptr(),
                                                          bh.data_ptr(), gh.data_ptr(), ob.data_ptr(),
                                                          biash.data_ptr())))
    report("SkipLN fp16 65536x768", t, nbytes=n_big * ld * 3 * 2 + 3 * ld * 2)
    Sb, Bb = 384, 256
    idsb = dev(r.integers(0, vocab, (Sb, Bb)).astype(np.int32))
    segsb = dev(r.integers(0, 2, (Sb, Bb)).astype(np.int32))
    embb = torch.empty((Sb * Bb, ld), dtype=torch.float16, device="cuda")
    t = timeit(lambda: api.check(api.emb_layer_norm_fp16(stream, ld, Bb, Sb, idsb.data_ptr(), segsb.data_ptr(),
                                                         b32.data_ptr(), g32.data_ptr(), word.data_ptr(),
                                                         pos.data_ptr(), tok.data_ptr(), vocab, 2, embb.data_ptr())))
    report("EmbLN fp16 B256 S384 E768", t, nbytes=Sb * Bb * (2 * ld * 2 + 8) + Sb * ld * 2 + 2 * ld * 2)
    del xb, sb, ob, embb

    # ---- fused attention FP16, BERT-base, B=32, var-seqlen ---------------------------------------
    for S in (128, 384):
        B, N, d = 32, 12, 64
        lens = r.integers(S // 2, S + 1, B)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        T = int(cu[-1])
        qkv = dev((r.standard_normal((T, 3 * N * d)) / 8).astype(np.float16))
        out = torch.empty((T, N * d), dtype=torch.float16, device="cuda")
        dcu = dev(cu)
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = qkv.data_ptr(), out.data_ptr(), dcu.data_ptr()
        p.qkv_stride_in_bytes, p.o_stride_in_bytes = 3 * N * d * 2, N * d * 2
        p.b, p.h, p.s, p.d = B, N, S, d
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        t = timeit(lambda: api.check(api.fused_mha_run(stream, 1, C.byref(p))))
        ops = 4.0 * d * N * float(np.sum(lens.astype(np.float64) ** 2))
        report(f"fused MHA fp16 B32 S{S} N12", t, ops=ops, peak_ops=PEAK_F16)

    # ---- BERT-large INT8 layer pieces in the linear layouts ------------------------------------
    wl = workloads.int8_layer(64, 384, N=16, seed=args.seed)
    T, E, N = wl.T, wl.E, wl.N
    qkv_lin = np.ascontiguousarray(wl.qkv_tc.reshape(T, 3, N, 64).transpose(0, 2, 1, 3)).reshape(T, 3 * E)
    dq = dev(qkv_lin)
    ctx = torch.empty((T, E), dtype=torch.int8, device="cuda")
    dcu = dev(wl.cu)
    p = capi.FmhaParams()
    p.qkv_ptr, p.o_ptr, p.cu_seqlens = dq.data_ptr(), ctx.data_ptr(), dcu.data_ptr()
    p.qkv_stride_in_bytes, p.o_stride_in_bytes = 3 * E, E
    p.b, p.h, p.s, p.d = wl.B, N, wl.S, 64
    p.scale_bmm1 = f32_bits(wl.s_qkv * wl.s_qkv * np.float32(0.125))
    p.scale_softmax, p.scale_bmm2 = f32_bits(127.0), f32_bits(wl.dq_probs * wl.s_qkv / np.float32(0.01))
    t = timeit(lambda: api.check(api.fused_mha_run(stream, 2, C.byref(p))))
    report("fused MHA int8 (linear) B64 S384 N16", t, ops=wl.mha_ops(), peak_ops=PEAK_I8)
    skip = dev(wl.skip_tc)
    gam, bet = dev(wl.gamma), dev(wl.beta)
    outq = torch.empty((T, E), dtype=torch.int8, device="cuda")
    t = timeit(lambda: api.check(api.skip_layer_norm_dqq(stream, E, T * E, ctx.data_ptr(), skip.data_ptr(),
                                                         bet.data_ptr(), gam.data_ptr(), outq.data_ptr(), 0,
                                                         0.01, float(wl.s_skip), 20.0)))
    report(f"SkipLN int8 linear {T}x1024", t, nbytes=T * E * 3 + 2 * E * 2)

    # ---- SkipLayerNorm with nothing in the last-level cache: operands rotate through more than 256 MB -----
    Tq = 33289
    n_sets = 12  # 12 x 3 x 34 MB = 1.2 GB
    sets = [tuple(torch.randint(-127, 128, (32, Tq, 32), dtype=torch.int8, device="cuda") for _ in range(3))
            for _ in range(n_sets)]
    gh1, bh1 = dev(r.uniform(0.5, 1.5, 1024).astype(np.float16)), dev((0.1 * r.standard_normal(1024)).astype(np.float16))
    turn = [0]

    def skipln_rotating():
        xi, si, oi = sets[turn[0] % n_sets]
        turn[0] += 1
        api.check(api.skipln_interleaved_large_hface(stream, 1024, Tq, xi.data_ptr(), si.data_ptr(), bh1.data_ptr(),
                                                     gh1.data_ptr(), oi.data_ptr(), 0.02, 0.02, 30.0))

    t = timeit(skipln_rotating)
    report(f"SkipLN int8 kCHW32 {Tq}x1024, rotating 1.2 GB", t, nbytes=Tq * 1024 * 3 + 2 * 1024 * 2)
    xi, si, oi = sets[0]
    t = timeit(lambda: api.check(api.skipln_interleaved_large_hface(
        stream, 1024, Tq, xi.data_ptr(), si.data_ptr(), bh1.data_ptr(), gh1.data_ptr(), oi.data_ptr(), 0.02, 0.02, 30.0)))
    report(f"SkipLN int8 kCHW32 {Tq}x1024, same buffers", t, nbytes=Tq * 1024 * 3 + 2 * 1024 * 2)
    del sets, xi, si, oi
    n_sets = 6  # 6 x 3 x 100 MB
    sets = [tuple(torch.randn((n_big, ld), dtype=torch.float16, device="cuda") for _ in range(3)) for _ in range(n_sets)]
    turn[0] = 0

    def skipln16_rotating():
        xi, si, oi = sets[turn[0] % n_sets]
        turn[0] += 1
        api.check(api.skip_layer_norm_fp16(stream, ld, n_big * ld, xi.data_ptr(), si.data_ptr(), bh.data_ptr(),
                                           gh.data_ptr(), oi.data_ptr(), biash.data_ptr()))

    t = timeit(skipln16_rotating)
    report(f"SkipLN fp16 {n_big}x768, rotating 1.8 GB", t, nbytes=n_big * ld * 3 * 2 + 3 * ld * 2)
    del sets

    # ---- the linear layers and reformats of the BERT-large INT8 encoder, B=128, 33289 tokens -------------

    def qnormal(shape):
        v = torch.randn(shape, device="cuda")
        return torch.clamp(torch.round(v * (127.0 / float(v.abs().max()))), -127, 127).to(torch.int8)

    for name, K, Nn, epi in (("QKV projection", 1024, 3072, capi.LINEAR_AFFINE),
                             ("attention output projection", 1024, 1024, capi.LINEAR_AFFINE),
                             ("feed-forward 1 + GELU", 1024, 4096, capi.LINEAR_GELU),
                             ("feed-forward 2", 4096, 1024, capi.LINEAR_AFFINE)):
        a8, w8 = qnormal((K // 32, Tq, 32)), qnormal((K // 32, Nn, 32))
        al = torch.full((Nn,), 2e-4, device="cuda")
        be = torch.zeros(Nn, device="cuda")
        o8 = torch.empty((Nn // 32, Tq, 32), dtype=torch.int8, device="cuda")
        lp = capi.Int8LinearParams()
        lp.a, lp.w, lp.alpha, lp.beta, lp.out = a8.data_ptr(), w8.data_ptr(), al.data_ptr(), be.data_ptr(), o8.data_ptr()
        lp.T, lp.K, lp.N = Tq, K, Nn
        lp.a_interleaved = lp.w_interleaved = lp.out_interleaved = 1
        lp.epilogue, lp.out_scale = epi, 30.0
        t = timeit(lambda: api.check(api.int8_linear(stream, C.byref(lp))))
        report(f"INT8 linear {name} {Tq}x{K}x{Nn}", t, ops=2.0 * Tq * K * Nn, peak_ops=PEAK_I8)
        del a8, w8, o8
    # ---- FP16 linear layers of a BERT-base FP16 encoder, B=128 x S=128 tokens ---------------------------
    Th = 16384
    for name, K, Nn, epi in (("feed-forward 1 + GELU", 768, 3072, capi.LINEAR_GELU),
                             ("feed-forward 2", 3072, 768, capi.LINEAR_AFFINE)):
        ah = torch.randn((Th, K), dtype=torch.float16, device="cuda")
        wh = torch.randn((Nn, K), dtype=torch.float16, device="cuda") * (K ** -0.5)
        al = torch.ones(Nn, device="cuda")
        be = torch.zeros(Nn, device="cuda")
        oh = torch.empty((Th, Nn), dtype=torch.float16, device="cuda")
        hp = capi.Fp16LinearParams()
        hp.a, hp.w, hp.alpha, hp.beta, hp.out = ah.data_ptr(), wh.data_ptr(), al.data_ptr(), be.data_ptr(), oh.data_ptr()
        hp.T, hp.K, hp.N, hp.epilogue = Th, K, Nn, epi
        t = timeit(lambda: api.check(api.fp16_linear(stream, C.byref(hp))))
        report(f"FP16 linear {name} {Th}x{K}x{Nn}", t, ops=2.0 * Th * K * Nn, peak_ops=PEAK_F16)
        del ah, wh, oh
    xh = torch.randn((Tq, 1024), dtype=torch.float16, device="cuda")
    x8 = torch.empty((32, Tq, 32), dtype=torch.int8, device="cuda")
    t = timeit(lambda: api.check(api.quantize_fp16_to_interleaved(stream, Tq, 1024, xh.data_ptr(), 0.03, x8.data_ptr())))
    report(f"quantise fp16 -> kCHW32 int8 {Tq}x1024", t, nbytes=Tq * 1024 * 3)
    t = timeit(lambda: api.check(api.dequantize_interleaved_to_fp16(stream, Tq, 1024, x8.data_ptr(), 0.03, xh.data_ptr())))
    report(f"dequantise kCHW32 int8 -> fp16 {Tq}x1024", t, nbytes=Tq * 1024 * 3)

    print(f"{'kernel':52s} {'us':>9s} {'achieved':>16s} {'of peak':>8s}  bound")
    for name, us, ach, frac, bound in rows:
        print(f"{name:52s} {us:9.2f} {ach:>16s} {frac:8.3f}  {bound}")


if __name__ == "__main__":
    main()
