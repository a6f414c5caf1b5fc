"""Per-kernel timings on the benchmark configurations other than the headline pass, and the on-box instruction rates.

bench.py imports `config_rows` and `microbench` and puts their results into its JSON line (keys `configs` and
`microbench`); `python -m tensorrt_amd.kernel_bench [--steps N]` prints the same rows as a table.

Every row: average launch time (events around back-to-back launches on the launch stream), the algorithmic bytes
or operations of one launch, the achieved rate and its fraction of the MI355X peak (HBM 8 TB/s, dense FP16 MFMA
2.5 PFLOP/s, dense INT8 MFMA 5 POP/s), and what torch's CPU kernels need for the same subgraph on this host's cores
(the stand-in for onnxruntime, which is not installed).  Inputs are synthetic and seeded, resident in HBM; torch is
only the allocator.
"""
from __future__ import annotations

import argparse
import ctypes as C
import os
import time

import numpy as np

PEAK_HBM = 8.0e12
PEAK_F16 = 2.5e15
PEAK_I8 = 5.0e15
PEAK_F32_MFMA = 157.3e12


def f32_bits(x) -> int:
    return int(np.float32(x).view(np.uint32))


def half2_bits(x) -> int:
    h = int(np.float16(x).view(np.uint16))
    return h | (h << 16)


def _microbench_lib():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtrtamd_microbench.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `python -m tensorrt_amd.build`")
    lib = C.CDLL(path)
    lib.trtamd_microbench_mfma_i8.restype = C.c_float
    lib.trtamd_microbench_mfma_i8.argtypes = [C.c_int] * 4 + [C.c_void_p] * 2
    lib.trtamd_microbench_valu.restype = C.c_float
    lib.trtamd_microbench_valu.argtypes = [C.c_int] * 3 + [C.c_void_p] * 3
    lib.trtamd_microbench_mfma_valu.restype = C.c_float
    lib.trtamd_microbench_mfma_valu.argtypes = [C.c_int] * 5 + [C.c_void_p] * 2
    lib.trtamd_microbench_mfma_valu_split.restype = C.c_float
    lib.trtamd_microbench_mfma_valu_split.argtypes = [C.c_int] * 5 + [C.c_void_p] * 2
    lib.trtamd_microbench_empty.restype = C.c_float
    lib.trtamd_microbench_empty.argtypes = [C.c_int] * 2 + [C.c_void_p]
    return lib


def microbench(torch, cus: int = 256) -> dict:
    """Instruction rates of this GPU (csrc/bench/microbench.hip): INT8 MFMA with four independent accumulators per
    wavefront and four wavefronts per SIMD, on zero and on random operands; the vector-ALU instructions of the softmax;
    whether the matrix pipe runs beside the vector ALU; the cost of an empty launch."""
    lib = _microbench_lib()
    out = torch.zeros(cus * 8 * 256, dtype=torch.int32, device="cuda")
    zero = torch.zeros(512, dtype=torch.int32, device="cuda")
    rnd = torch.randint(-2 ** 31, 2 ** 31 - 1, (512,), dtype=torch.int32, device="cuda")
    clocks = torch.zeros(2 * cus * 8, dtype=torch.int64, device="cuda")
    wps, chains, iters = 4, 4, 8192
    blocks = cus * wps
    res = {"waves_per_simd": wps, "independent_accumulators": chains}
    # integer operations per instruction and wavefront: 16x16x64 -> 2*16*16*64, 32x32x32 -> 2*32*32*32
    for shape, name, ops in ((0, "v_mfma_i32_16x16x64_i8", 2 * 16 * 16 * 64), (1, "v_mfma_i32_32x32x32_i8", 2 * 32 * 32 * 32)):
        for data, dn in ((zero, "zero_operands"), (rnd, "random_operands")):
            ms = lib.trtamd_microbench_mfma_i8(shape, chains, blocks, iters, data.data_ptr(), out.data_ptr())
            res[f"{name}.{dn}.TOP/s"] = round(blocks * 4 * iters * chains * ops / (ms * 1e-3) / 1e12, 1)
    # a dependent chain: one wavefront per SIMD with a single accumulator (each MFMA waits for the one before it)
    ms = lib.trtamd_microbench_mfma_i8(0, 1, cus, iters, zero.data_ptr(), out.data_ptr())
    res["v_mfma_i32_16x16x64_i8.one_wave_per_simd_one_accumulator.TOP/s"] = round(
        cus * 4 * iters * 2 * 16 * 16 * 64 / (ms * 1e-3) / 1e12, 1)
    names = ["v_fma_f32", "v_exp_f32", "v_add_f32", "v_perm_b32", "v_max3_i32", "v_cvt_pk_u8_f32",
             "fma+exp+add+fma (softmax inner sequence)", "v_max3_f32", "v_max_f32", "v_mul_f32", "v_lshl_or_b32",
             "v_cvt_f32_i32", "v_cvt_f32_ubyte0", "v_dot4_i32_i8", "v_rcp_f32", "v_med3_f32", "v_add_u32"]
    valu = {}
    mhz = []
    for op, name in enumerate(names):
        ms = lib.trtamd_microbench_valu(op, blocks, iters, rnd.data_ptr(), out.data_ptr(), clocks.data_ptr())
        c = clocks[: 2 * blocks].view(blocks, 2).double().cpu().numpy()
        mhz.append(float((c[:, 0] / np.maximum(c[:, 1], 1)).mean() * 100))
        valu[name] = ms * 1e-3 / (iters * 8 * wps)          # seconds per wavefront instruction (group) and SIMD
    clock = float(np.median(mhz)) * 1e6
    res["shader_clock_MHz_under_vector_load"] = round(clock / 1e6)
    res["cycles_per_wave_instruction"] = {k: round(v * clock, 2) for k, v in valu.items()}
    res["ns_per_wave_instruction"] = {k: round(v * 1e9, 3) for k, v in valu.items()}
    alone = {}
    for op in (0, 1):
        ms = lib.trtamd_microbench_valu(op, cus, iters, rnd.data_ptr(), out.data_ptr(), clocks.data_ptr())
        alone[names[op]] = round(ms * 1e-3 / (iters * 8) * clock, 2)
    res["cycles_per_wave_instruction_one_wave_per_simd"] = alone
    # one instruction stream: ns per step of one MFMA followed by n independent vector instructions, and of the same
    # n vector instructions without the MFMA (the control); four wavefronts per SIMD and one
    co = {}
    for w in (wps, 1):
        for kind, kname in ((0, "v_fma_f32"), (1, "v_exp_f32"), (2, "fma,exp,add,fma")):
            row = {}
            for nv in (0, 4, 8, 12, 16, 24, 32):
                t = []
                for with_mfma in (1, 0):
                    ms = lib.trtamd_microbench_mfma_valu(nv, kind, with_mfma, cus * w, iters // 2, rnd.data_ptr(),
                                                         out.data_ptr())
                    t.append(round(ms * 1e-3 / (iters // 2 * 4 * w) * 1e9, 2))
                row[str(nv)] = t
            co[f"{kname},waves_per_simd={w}"] = row
    res["ns_per_step_[mfma_16x16x64_then_n_vector_instructions,n_vector_instructions_alone]_one_stream"] = co
    # across wavefronts: per SIMD as many wavefronts that only issue MFMAs (4 per iteration) as wavefronts that only
    # issue v_fma_f32 (nv per iteration, 16 independent chains); workgroups of eight wavefronts, wgs_per_cu of them
    # on a CU; ns per iteration and SIMD for the MFMA wavefronts alone, the vector wavefronts alone, and both
    split = {}
    for wgs in (1, 2):
        for nv in (32, 64):
            for pad in (0, 1, 2, 3, 4):
                t = []
                for roles in (1, 2, 3):
                    ms = lib.trtamd_microbench_mfma_valu_split(cus * wgs, iters, nv, pad, roles, rnd.data_ptr(),
                                                               out.data_ptr())
                    t.append(round(ms * 1e-3 / iters * 1e9, 1))
                split[f"wgs_per_cu={wgs},nv={nv},s_nop7_behind_each_mfma={pad}"] = t
    res["ns_per_iteration_[mfma_wavefronts_only,vector_wavefronts_only,both]_on_one_simd"] = split
    res["empty_launch_us"] = {f"{b}x{t}": round(lib.trtamd_microbench_empty(b, t, out.data_ptr()) * 1e3, 2)
                              for b, t in ((256, 256), (1041, 512), (2048, 256))}
    return res


def _cpu_time(fn, budget_s=0.4):
    """Seconds per call of a torch-CPU subgraph (one warm-up call, then as many as fit the budget)."""
    fn()
    t0 = time.perf_counter()
    n = 0
    while True:
        fn()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 50:
            return el / n


def config_rows(api, torch, steps: int = 100, seed: int = 1, cpu: bool = True, launch_floor_us: float | None = None) -> list:
    """The kernels of configs[0..3] (and of the unfused attention path) at their stated sizes.  launch_floor_us: what
    an empty kernel costs back to back on this box (microbench()["empty_launch_us"]); bandwidth-bound rows then also
    carry the rate over the time above that floor, which is what the kernel itself decides at these small sizes."""
    from tensorrt_amd import capi, workloads
    stream = torch.cuda.current_stream().cuda_stream
    r = np.random.default_rng(seed)
    cores = min(len(os.sched_getaffinity(0)), 16)
    if cpu:
        torch.set_num_threads(cores)
    F = torch.nn.functional

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def timeit(fn):
        # the GPU raises its clocks over the first tens of milliseconds of load: 0.15 s of untimed launches first
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < 0.15:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / steps

    rows = []

    def report(config, kernel, dtype, shape, t, nbytes=None, ops=None, peak_ops=None, cpu_s=None, note=None):
        row = {"config": config, "kernel": kernel, "dtype": dtype, "shape": shape, "gpu_us": round(t * 1e6, 2)}
        if nbytes is not None:
            row.update({"algorithmic_bytes": int(nbytes), "achieved": round(nbytes / t / 1e9, 1), "unit": "GB/s",
                        "roofline": "HBM 8 TB/s", "frac": round(nbytes / t / PEAK_HBM, 4)})
            if launch_floor_us is not None and t * 1e6 > launch_floor_us + 0.2:
                above = t - launch_floor_us * 1e-6
                row.update({"empty_launch_us": launch_floor_us, "frac_above_empty_launch": round(nbytes / above / PEAK_HBM, 4)})
        else:
            row.update({"algorithmic_ops": float(ops), "achieved": round(ops / t / 1e12, 2), "unit": "TOP/s",
                        "roofline": f"MFMA {peak_ops / 1e12:.1f} TOP/s", "frac": round(ops / t / peak_ops, 4)})
        if cpu_s is not None:
            row["cpu_ms"] = round(cpu_s * 1e3, 3)
            row["cpu"] = f"torch-CPU fallback (onnxruntime unavailable), {cores} cores"
        if note:
            row["note"] = note
        rows.append(row)

    # ---- C1: SkipLayerNorm fp32, [8,128,768] + bias -------------------------------------------------
    n_rows, ld = 8 * 128, 768
    hx, hs = (r.standard_normal((n_rows, ld)).astype(np.float32) for _ in range(2))
    hg = r.uniform(0.5, 1.5, ld).astype(np.float32)
    hb = (0.1 * r.standard_normal(ld)).astype(np.float32)
    hbias = (0.02 * r.standard_normal(ld)).astype(np.float32)
    x, s, g, b, bias = dev(hx), dev(hs), dev(hg), dev(hb), dev(hbias)
    o = torch.empty_like(x)
    t = timeit(lambda: api.check(api.skip_layer_norm_fp32(stream, ld, n_rows * ld, x.data_ptr(), s.data_ptr(),
                                                          b.data_ptr(), g.data_ptr(), o.data_ptr(), bias.data_ptr())))
    cpu_s = None
    if cpu:
        cx, cs, cg, cb, cbias = (torch.from_numpy(a) for a in (hx, hs, hg, hb, hbias))
        cpu_s = _cpu_time(lambda: F.layer_norm(cx + cs + cbias, (ld,), cg, cb, 1e-12))
    report("C1", "SkipLN v5 (skipln_rows_kernel)", "fp32", "1024x768", t, nbytes=n_rows * ld * 3 * 4 + 3 * ld * 4,
           cpu_s=cpu_s)

    # ---- C2: BERT-base EmbLN + SkipLN fp16, B=32 S=128 E=768 ---------------------------------------
    S, B, ld, vocab = 128, 32, 768, 30522
    hword = (0.02 * r.standard_normal((vocab, ld))).astype(np.float16)
    hpos = (0.02 * r.standard_normal((512, ld))).astype(np.float16)
    htok = (0.02 * r.standard_normal((2, ld))).astype(np.float16)
    word, pos, tok = dev(hword), dev(hpos), dev(htok)
    g32 = dev(r.uniform(0.5, 1.5, ld).astype(np.float32))
    b32 = dev((0.1 * r.standard_normal(ld)).astype(np.float32))
    hids = r.integers(0, vocab, (S, B)).astype(np.int32)
    hsegs = r.integers(0, 2, (S, B)).astype(np.int32)
    ids, segs = dev(hids), dev(hsegs)
    emb = torch.empty((S * B, ld), dtype=torch.float16, device="cuda")
    t = timeit(lambda: api.check(api.emb_layer_norm_fp16(stream, ld, B, S, ids.data_ptr(), segs.data_ptr(),
                                                         b32.data_ptr(), g32.data_ptr(), word.data_ptr(),
                                                         pos.data_ptr(), tok.data_ptr(), vocab, 2, emb.data_ptr())))
    cpu_s = None
    if cpu:
        cw, cp, ct = (torch.from_numpy(a.astype(np.float32)) for a in (hword, hpos, htok))
        ci, cseg = torch.from_numpy(hids.astype(np.int64)), torch.from_numpy(hsegs.astype(np.int64))
        cg32, cb32 = g32.cpu(), b32.cpu()
        cpu_s = _cpu_time(lambda: F.layer_norm(cw[ci] + ct[cseg] + cp[:S, None, :], (ld,), cg32, cb32, 1e-12))
    # gathered word rows + output + ids; the position/type rows are shared and stay in cache
    report("C2", "EmbLN v6 (embln_kernel)", "fp16", "4096x768, vocab 30522", t,
           nbytes=S * B * (2 * ld * 2 + 8) + S * ld * 2 + 2 * ld * 2, cpu_s=cpu_s)
    n_rows = S * B
    hxs = r.standard_normal((n_rows, ld)).astype(np.float16)
    xs = dev(hxs)
    gh, bh = g32.half(), b32.half()
    biash = dev((0.02 * r.standard_normal(ld)).astype(np.float16))
    oh = torch.empty_like(emb)
    t = timeit(lambda: api.check(api.skip_layer_norm_fp16(stream, ld, n_rows * ld, emb.data_ptr(), xs.data_ptr(),
                                                          bh.data_ptr(), gh.data_ptr(), oh.data_ptr(),
                                                          biash.data_ptr())))
    cpu_s = None
    if cpu:
        ce, cxs = emb.float().cpu(), torch.from_numpy(hxs.astype(np.float32))
        cgh, cbh, cbi = gh.float().cpu(), bh.float().cpu(), biash.float().cpu()
        cpu_s = _cpu_time(lambda: F.layer_norm(ce + cxs + cbi, (ld,), cgh, cbh, 1e-12))
    report("C2", "SkipLN v5 (skipln_rows_kernel)", "fp16", "4096x768", t, nbytes=n_rows * ld * 3 * 2 + 3 * ld * 2,
           cpu_s=cpu_s)
    # the same kernel where the launch itself no longer matters, operands rotating through more than the 256 MB cache
    n_big, n_sets = 65536, 6
    sets = [tuple(torch.randn((n_big, ld), dtype=torch.float16, device="cuda") for _ in range(3)) for _ in range(n_sets)]
    turn = [0]

    def skipln16_rotating():
        xi, si, oi = sets[turn[0] % n_sets]
        turn[0] += 1
        api.check(api.skip_layer_norm_fp16(stream, ld, n_big * ld, xi.data_ptr(), si.data_ptr(), bh.data_ptr(),
                                           gh.data_ptr(), oi.data_ptr(), biash.data_ptr()))

    t = timeit(skipln16_rotating)
    report("C2 x16 rows", "SkipLN v5 (skipln_rows_kernel)", "fp16", "65536x768, rotating 1.8 GB", t,
           nbytes=n_big * ld * 3 * 2 + 3 * ld * 2, note="nothing in the last-level cache")
    del sets

    # ---- C3: fused attention FP16, BERT-base, B=32, var-seqlen (v5) ---------------------------------
    for S in (128, 384):
        B, N, d = 32, 12, 64
        lens = r.integers(S // 2, S + 1, B)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        T = int(cu[-1])
        hq = (r.standard_normal((T, 3 * N * d)) / 8).astype(np.float16)
        qkv = dev(hq)
        out = torch.empty((T, N * d), dtype=torch.float16, device="cuda")
        dcu = dev(cu)
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = qkv.data_ptr(), out.data_ptr(), dcu.data_ptr()
        p.qkv_stride_in_bytes, p.o_stride_in_bytes = 3 * N * d * 2, N * d * 2
        p.b, p.h, p.s, p.d = B, N, S, d
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        t = timeit(lambda: api.check(api.fused_mha_run(stream, 1, C.byref(p))))
        ops = 4.0 * d * N * float(np.sum(lens.astype(np.float64) ** 2))
        cpu_s = None
        if cpu:
            cq = torch.from_numpy(hq.astype(np.float32)).reshape(T, N, 3, d)

            def attn_cpu():
                for bb in range(B):
                    lo, hi = int(cu[bb]), int(cu[bb + 1])
                    q, k, v = (cq[lo:hi, :, i].transpose(0, 1) for i in range(3))
                    torch.softmax(q @ k.transpose(1, 2) * 0.125, -1) @ v
            cpu_s = _cpu_time(attn_cpu)
        report("C3", "QKV-to-context v5 (fmha_f16_prefix_kernel)", "fp16", f"B=32 N=12 S={S}, {T} tokens", t, ops=ops,
               peak_ops=PEAK_F16, cpu_s=cpu_s)

    # ---- C3, the fixed [S,B,N,3,d] layout with the packed key mask (v4 plugin with a mask input) ----------
    for S in (128, 384):
        B, N, d = 32, 12, 64
        lens = r.integers(S // 2, S + 1, B)
        hq = (r.standard_normal((S, B, 3 * N * d)) / 8).astype(np.float16)
        qkv = dev(hq)
        out = torch.empty((S, B, N * d), dtype=torch.float16, device="cuda")
        mask = dev((np.arange(S)[:, None] < lens[None, :]).astype(np.int32))
        words = 6144 if S == 384 else 512
        packed = torch.zeros((B, words), dtype=torch.int32, device="cuda")
        wm, wn = (2, 2) if S <= 128 else (1, 8)
        api.check(api.convert_mask(S, B, wm, wn, 1, mask.data_ptr(), packed.data_ptr(), stream))
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.packed_mask_ptr = qkv.data_ptr(), out.data_ptr(), packed.data_ptr()
        p.qkv_stride_in_bytes, p.o_stride_in_bytes = 3 * B * N * d * 2, B * N * d * 2
        p.packed_mask_stride_in_bytes = words * 4
        p.b, p.h, p.s, p.d = B, N, S, d
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        t = timeit(lambda: api.check(api.fused_mha_run(stream, 1, C.byref(p))))
        report("C3", "QKV-to-context v4, packed mask (fmha_f16_kernel)", "fp16", f"S={S} B=32 N=12, fixed layout", t,
               ops=4.0 * d * N * float(np.sum(lens.astype(np.float64) ** 2)), peak_ops=PEAK_F16,
               note="every query row of the S x B tensor is computed; ops count valid lengths only")

    # ---- unfused attention (FP32, other head sizes, S > 512) ------------------------------------------
    # head sizes up to 128: one launch, a query's scores in registers up to S = 512 and two passes over the keys beyond
    # (larger head sizes: two MFMA GEMMs around a softmax with the S x S scores in the workspace)
    for dt, tname, type_id, peak in ((np.float16, "fp16", 1, PEAK_F16), (np.float32, "fp32", 0, PEAK_F32_MFMA)):
        for S, B, N, d in ((128, 32, 12, 64), (384, 32, 12, 64), (1024, 4, 12, 64)):
            hq = (r.standard_normal((S, B, 3 * N * d)) / 8).astype(dt)
            qkv = dev(hq)
            out = torch.empty((S, B, N * d), dtype=qkv.dtype, device="cuda")
            ws = torch.empty((api.unfused_mha_workspace_size(type_id, S, B, N),), dtype=torch.uint8, device="cuda")
            t = timeit(lambda: api.check(api.unfused_mha(stream, type_id, S, B, N, d, qkv.data_ptr(), 0,
                                                         out.data_ptr(), ws.data_ptr())))
            one = S <= 512
            report("C3 shape, unfused path",
                   "QKV-to-context v4 (attention_in_registers_kernel)" if one
                   else "QKV-to-context v4 (attention_two_pass_kernel)", tname,
                   f"S={S} B={B} N={N} d={d}, all keys", t, ops=4.0 * d * N * B * S * S, peak_ops=peak,
                   note="one launch, scores in registers" if one else "one launch, two passes over the keys")

    # ---- C4: BERT-large INT8 layer, B=64, lengths U[192,384] -----------------------------------------
    wl = workloads.int8_layer(64, 384, N=16, seed=seed)
    T, E, N = wl.T, wl.E, wl.N
    dq = dev(workloads.interleave32(wl.qkv_tc))
    ctx = torch.empty((T * E,), dtype=torch.int8, device="cuda")
    dcu = dev(wl.cu)
    p = capi.FmhaParams()
    p.qkv_ptr, p.o_ptr, p.cu_seqlens = dq.data_ptr(), ctx.data_ptr(), dcu.data_ptr()
    p.qkv_stride_in_bytes = p.o_stride_in_bytes = T
    p.b, p.h, p.s, p.d = wl.B, N, wl.S, 64
    p.interleaved = 1
    p.scale_bmm1 = f32_bits(wl.s_qkv * wl.s_qkv * np.float32(0.125))
    p.scale_softmax, p.scale_bmm2 = f32_bits(127.0), f32_bits(wl.dq_probs * wl.s_qkv / np.float32(0.01))
    t = timeit(lambda: api.check(api.fused_mha_run(stream, 2, C.byref(p))))
    cpu_s = None
    if cpu:
        nseq = 8
        cq = torch.from_numpy(wl.qkv_tc[: int(wl.cu[nseq])].astype(np.float32) * float(wl.s_qkv))

        def attn8_cpu():
            for bb in range(nseq):
                lo, hi = int(wl.cu[bb]), int(wl.cu[bb + 1])
                q, k, v = (cq[lo:hi, i * E:(i + 1) * E].reshape(hi - lo, N, 64).transpose(0, 1) for i in range(3))
                torch.softmax(q @ k.transpose(1, 2) * 0.125, -1) @ v
        cpu_s = _cpu_time(attn8_cpu) * wl.B / nseq
    report("C4", "QKV-to-context v6 (fmha_i8_prefix_kernel)", "int8", f"B=64 N=16 S=384, {T} tokens, kCHW32", t,
           ops=wl.mha_ops(), peak_ops=PEAK_I8, cpu_s=cpu_s,
           note="CPU: the de-quantised FP32 subgraph on 8 sequences, scaled to 64" if cpu else None)
    # the same attention in the linear layout of the v5 plugin ([T, 3E], channel order [N][3][d])
    dql = dev(np.ascontiguousarray(wl.qkv_tc.reshape(T, 3, N, 64).transpose(0, 2, 1, 3)).reshape(T, 3 * E))
    ctxl = torch.empty((T, E), dtype=torch.int8, device="cuda")
    pl = capi.FmhaParams()
    pl.qkv_ptr, pl.o_ptr, pl.cu_seqlens = dql.data_ptr(), ctxl.data_ptr(), dcu.data_ptr()
    pl.qkv_stride_in_bytes, pl.o_stride_in_bytes = 3 * E, E
    pl.b, pl.h, pl.s, pl.d = wl.B, N, wl.S, 64
    pl.scale_bmm1, pl.scale_softmax, pl.scale_bmm2 = p.scale_bmm1, p.scale_softmax, p.scale_bmm2
    t = timeit(lambda: api.check(api.fused_mha_run(stream, 2, C.byref(pl))))
    report("C4", "QKV-to-context v5 (fmha_i8_prefix_kernel, linear layout)", "int8",
           f"B=64 N=16 S=384, {T} tokens, [T,3E]", t, ops=wl.mha_ops(), peak_ops=PEAK_I8)
    skip = dev(workloads.interleave32(wl.skip_tc))
    gam, bet = dev(wl.gamma), dev(wl.beta)
    outq = torch.empty((T * E,), dtype=torch.int8, device="cuda")
    t = timeit(lambda: api.check(api.skipln_interleaved_large_hface(stream, E, T, ctx.data_ptr(), skip.data_ptr(),
                                                                   bet.data_ptr(), gam.data_ptr(), outq.data_ptr(),
                                                                   0.01, float(wl.s_skip), 20.0)))
    cpu_s = None
    if cpu:
        ca, cs2 = (torch.randn(T, E) for _ in range(2))
        cg, cb = torch.from_numpy(wl.gamma.astype(np.float32)), torch.from_numpy(wl.beta.astype(np.float32))
        cpu_s = _cpu_time(lambda: F.layer_norm(ca + cs2, (E,), cg, cb, 1e-12))
    report("C4", "SkipLN v7 (skipln_interleaved_kernel)", "int8", f"{T}x1024 kCHW32, same buffers", t,
           nbytes=T * E * 3 + 2 * E * 2, cpu_s=cpu_s, note="operands resident in the 256 MB last-level cache")
    n_sets = 12
    sets = [tuple(torch.randint(-127, 128, (32, T, 32), dtype=torch.int8, device="cuda") for _ in range(3))
            for _ in range(n_sets)]
    turn[0] = 0

    def skipln_rotating():
        xi, si, oi = sets[turn[0] % n_sets]
        turn[0] += 1
        api.check(api.skipln_interleaved_large_hface(stream, E, T, xi.data_ptr(), si.data_ptr(), bet.data_ptr(),
                                                     gam.data_ptr(), oi.data_ptr(), 0.02, 0.02, 30.0))

    t = timeit(skipln_rotating)
    report("C4", "SkipLN v7 (skipln_interleaved_kernel)", "int8", f"{T}x1024 kCHW32, rotating 0.7 GB", t,
           nbytes=T * E * 3 + 2 * E * 2, note="nothing in the last-level cache")
    del sets
    # ---- C5 SkipLN size, cold ---------------------------------------------------------------------
    Tq = 33289
    sets = [tuple(torch.randint(-127, 128, (32, Tq, 32), dtype=torch.int8, device="cuda") for _ in range(3))
            for _ in range(n_sets)]
    turn[0] = 0

    def skipln_rotating5():
        xi, si, oi = sets[turn[0] % n_sets]
        turn[0] += 1
        api.check(api.skipln_interleaved_large_hface(stream, E, Tq, xi.data_ptr(), si.data_ptr(), bet.data_ptr(),
                                                     gam.data_ptr(), oi.data_ptr(), 0.02, 0.02, 30.0))

    t = timeit(skipln_rotating5)
    report("C5", "SkipLN v7 (skipln_interleaved_kernel)", "int8", f"{Tq}x1024 kCHW32, rotating 1.2 GB", t,
           nbytes=Tq * E * 3 + 2 * E * 2, note="nothing in the last-level cache")
    del sets
    return rows


def extra_rows(api, torch, steps: int = 100) -> list:
    """Linear layers and reformats of the encoders (the table behind the design notes; not part of bench.py's line)."""
    from tensorrt_amd import capi
    stream = torch.cuda.current_stream().cuda_stream
    rows = []

    def timeit(fn):
        # the GPU raises its clocks over the first tens of milliseconds of load: 0.15 s of untimed launches first
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < 0.15:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / steps

    def qnormal(shape):
        v = torch.randn(shape, device="cuda")
        return torch.clamp(torch.round(v * (127.0 / float(v.abs().max()))), -127, 127).to(torch.int8)

    Tq = 33289
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
        ops = 2.0 * Tq * K * Nn
        rows.append({"kernel": f"INT8 linear {name} {Tq}x{K}x{Nn}", "gpu_us": round(t * 1e6, 2),
                     "achieved": round(ops / t / 1e12, 1), "unit": "TOP/s", "frac": round(ops / t / PEAK_I8, 4)})
        del a8, w8, o8
        # the vendor library on the same product (hipBLASLt behind torch._int_mm: row-major operands, INT32 output
        # and no epilogue, so four times the output bytes and none of the requantisation); a comparison, not a leg
        # of any workload
        if epi == capi.LINEAR_AFFINE and hasattr(torch, "_int_mm"):
            Tp = (Tq + 7) // 8 * 8   # _int_mm wants a multiple of 8 rows
            A, Wt = qnormal((Tp, K)), qnormal((Nn, K)).t()
            try:
                t = timeit(lambda: torch._int_mm(A, Wt))
                ops = 2.0 * Tp * K * Nn
                rows.append({"kernel": f"  vendor library, torch._int_mm {Tp}x{K}x{Nn}, INT32 output", "gpu_us": round(t * 1e6, 2),
                             "achieved": round(ops / t / 1e12, 1), "unit": "TOP/s", "frac": round(ops / t / PEAK_I8, 4)})
            except RuntimeError:
                pass   # not every build of torch has the INT8 product
            del A, Wt
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
        ops = 2.0 * Th * K * Nn
        rows.append({"kernel": f"FP16 linear {name} {Th}x{K}x{Nn}", "gpu_us": round(t * 1e6, 2),
                     "achieved": round(ops / t / 1e12, 1), "unit": "TOP/s", "frac": round(ops / t / PEAK_F16, 4)})
        if epi == capi.LINEAR_AFFINE:
            bh = torch.zeros(Nn, dtype=torch.float16, device="cuda")
            t = timeit(lambda: torch.nn.functional.linear(ah, wh, bh))
            rows.append({"kernel": f"  vendor library, torch linear {Th}x{K}x{Nn}, FP16 + bias", "gpu_us": round(t * 1e6, 2),
                         "achieved": round(ops / t / 1e12, 1), "unit": "TOP/s", "frac": round(ops / t / PEAK_F16, 4)})
        del ah, wh, oh
    xh = torch.randn((Tq, 1024), dtype=torch.float16, device="cuda")
    x8 = torch.empty((32, Tq, 32), dtype=torch.int8, device="cuda")
    for name, fn in (("quantise fp16 -> kCHW32 int8", lambda: api.check(api.quantize_fp16_to_interleaved(
                          stream, Tq, 1024, xh.data_ptr(), 0.03, x8.data_ptr()))),
                     ("dequantise kCHW32 int8 -> fp16", lambda: api.check(api.dequantize_interleaved_to_fp16(
                          stream, Tq, 1024, x8.data_ptr(), 0.03, xh.data_ptr())))):
        t = timeit(fn)
        nb = Tq * 1024 * 3
        rows.append({"kernel": f"{name} {Tq}x1024", "gpu_us": round(t * 1e6, 2), "achieved": round(nb / t / 1e9, 1),
                     "unit": "GB/s", "frac": round(nb / t / PEAK_HBM, 4)})
    return rows


def attention_rows(api, torch, steps: int = 200) -> list:
    """The cu_seqlens attention kernels alone, on device-generated operands: INT8 (interleaved layout) at the encoder's
    and the layer workload's shapes and with full-length sequences, FP16 at the BERT-base shapes.  Used to time a plugin
    library against its MFMA-less diagnostic build (`--ablation`), whose results are wrong on purpose."""
    from tensorrt_amd import capi
    stream = torch.cuda.current_stream().cuda_stream
    rows = []

    def timeit(fn):
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < 0.25:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e-3 / steps)
        return best

    def run(name, lens, N, S, int8):
        lens = np.asarray(lens)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        T, E = int(cu[-1]), N * 64
        gen = torch.Generator(device="cuda")
        gen.manual_seed(1)
        x = torch.randn((T, 3 * E), device="cuda", generator=gen)
        p = capi.FmhaParams()
        dcu = torch.from_numpy(cu).cuda()
        if int8:
            qkv = torch.clamp(torch.round(x * (127 / 4.5)), -127, 127).to(torch.int8)
            out = torch.zeros(T * E, dtype=torch.int8, device="cuda")
            sq = 4.5 / 127
            p.qkv_stride_in_bytes = p.o_stride_in_bytes = T
            p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = f32_bits(sq * sq * 0.125), f32_bits(127.0), f32_bits(sq / 127 / 0.01)
            p.interleaved = 1
        else:
            qkv = (x / 8).half()
            out = torch.zeros((T, E), dtype=torch.float16, device="cuda")
            p.qkv_stride_in_bytes, p.o_stride_in_bytes = 2 * 3 * E, 2 * E
            p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = qkv.data_ptr(), out.data_ptr(), dcu.data_ptr()
        p.b, p.h, p.s, p.d = len(lens), N, S, 64
        t = timeit(lambda: api.check(api.fused_mha_run(stream, 2 if int8 else 1, C.byref(p))))
        ops = 4.0 * 64 * N * float(np.sum(lens.astype(np.float64) ** 2))
        rows.append({"kernel": name, "gpu_us": round(t * 1e6, 2), "achieved": round(ops / t / 1e12, 1), "unit": "TOP/s",
                     "frac": round(ops / t / (PEAK_I8 if int8 else PEAK_F16), 4)})

    r = np.random.default_rng(1)
    run("INT8 v6, 128 sequences U[128,384], 16 heads (encoder)", r.integers(128, 385, 128), 16, 384, True)
    run("INT8 v6, 64 sequences U[192,384], 16 heads (layer)", np.random.default_rng(1).integers(192, 385, 64), 16, 384, True)
    run("INT8 v6, 128 sequences of 384, 16 heads", np.full(128, 384), 16, 384, True)
    run("FP16 v5, 32 sequences U[192,384], 12 heads", np.random.default_rng(1).integers(192, 385, 32), 12, 384, False)
    run("FP16 v5, 32 sequences U[64,128], 12 heads", np.random.default_rng(1).integers(64, 129, 32), 12, 128, False)
    run("FP16 v5, 64 sequences of 384, 12 heads", np.full(64, 384), 12, 384, False)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--ablation", action="store_true",
                    help="time the cu_seqlens attention kernels of lib/libtrtamd_ablation.so (the MFMAs left out; "
                         "`python -m tensorrt_amd.build --ablation`) and, in a second process, of the plugin library")
    ap.add_argument("--attention-only", action="store_true", help="only the attention rows of --ablation, this library")
    args = ap.parse_args()

    if args.ablation:
        # two libraries that export the same symbols do not go into one process: a child per library
        import subprocess
        import sys
        import tensorrt_amd
        for lib in (os.path.join(os.path.dirname(tensorrt_amd.library_path()), "libtrtamd_ablation.so"),
                    tensorrt_amd.library_path()):
            print(f"== {os.path.basename(lib)}", flush=True)
            env = dict(os.environ, TRTAMD_KERNEL_BENCH_LIBRARY=lib)
            subprocess.run([sys.executable, "-m", "tensorrt_amd.kernel_bench", "--attention-only", "--steps",
                            str(args.steps)], env=env, check=True)
        return

    import torch
    if os.environ.get("TRTAMD_KERNEL_BENCH_LIBRARY"):
        import tensorrt_amd
        tensorrt_amd._LIB = os.environ["TRTAMD_KERNEL_BENCH_LIBRARY"]   # the diagnostic build, this process only
    from tensorrt_amd import capi
    api = capi.api()
    # the GPU raises its clocks over the first tens of milliseconds of load
    warm = torch.randn((4096, 4096), dtype=torch.float16, device="cuda")
    t_end = time.perf_counter() + 0.3
    while time.perf_counter() < t_end:
        torch.mm(warm, warm)
        torch.cuda.synchronize()
    del warm
    if args.attention_only:
        for row in attention_rows(api, torch, args.steps):
            print(f"{row['kernel']:60s} {row['gpu_us']:9.2f} us {row['achieved']:9.1f} {row['unit']:>5s} {row['frac']:8.4f}",
                  flush=True)
        return
    print(f"{'config':22s} {'kernel':62s} {'shape':44s} {'us':>9s} {'achieved':>14s} {'of peak':>8s} {'CPU ms':>9s}")
    mb = microbench(torch)
    for row in config_rows(api, torch, args.steps, args.seed, cpu=not args.no_cpu,
                           launch_floor_us=mb["empty_launch_us"]["256x256"]):
        print(f"{row['config']:22s} {row['kernel']:62s} {row['shape']:44s} {row['gpu_us']:9.2f} "
              f"{row['achieved']:9.1f} {row['unit']:>5s} {row['frac']:8.3f} {row.get('cpu_ms', float('nan')):9.2f}")
    for row in extra_rows(api, torch, args.steps):
        print(f"{'':22s} {row['kernel']:107s} {row['gpu_us']:9.2f} {row['achieved']:9.1f} {row['unit']:>5s} {row['frac']:8.3f}")
    for k, v in mb.items():
        print(f"{k}: {v}")


if __name__ == "__main__":
    main()
