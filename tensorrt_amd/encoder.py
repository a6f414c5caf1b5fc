"""INT8 BERT encoder assembled from the plugin library, the way a TensorRT network for it is laid out.

The reference's own builder for this network (demo/BERT) is gone from the tree (CHANGELOG.md:23-24);
what is left is what each plugin expects of its neighbours (plugin/bertQKVToContextPlugin/README.md:20-35,
plugin/skipLayerNormPlugin/README.md, plugin/embLayerNormPlugin/README.md).  This module plays the
engine's part for one network: it creates the plugins through the registry by name and version,
re-creates them from their serialised fields as engine deserialisation does, owns the activation
buffers, folds quantisation scales into the linear layers and enqueues everything in order on one
stream:

    EmbLayerNorm (var-seqlen, FP16)            CustomEmbLayerNormPluginDynamic v4
    Quantize + reformat to kCHW32                (TensorRT inserts it; explicit call here)
    per layer:
        QKV projection      INT8 GEMM            (TensorRT core; trtamd_int8_linear here)
        attention           CustomQKVToContextPluginDynamic v6 (INT8 interleaved, var-seqlen)
        output projection   INT8 GEMM
        residual + LN       CustomSkipLayerNormPluginDynamic v7 (INT8 interleaved)
        feed-forward 1      INT8 GEMM + GELU
        feed-forward 2      INT8 GEMM
        residual + LN       CustomSkipLayerNormPluginDynamic v7
    Dequantize + reformat to linear FP16

torch is the allocator (and computes amax during calibration); every operation on the timed path is
a call into libtrtamd_bert_plugins.so.
"""
from __future__ import annotations

import ctypes as C
import dataclasses

import numpy as np

from . import capi
from .plugin import (DataType, PluginField, PluginFieldType, TensorDesc, TensorFormat, TensorRTPhase,
                     get_plugin_registry, last_log)

EMBLN = "CustomEmbLayerNormPluginDynamic"
SKIPLN = "CustomSkipLayerNormPluginDynamic"
QKV = "CustomQKVToContextPluginDynamic"
HEAD = 64


@dataclasses.dataclass
class EncoderConfig:
    hidden: int = 1024
    heads: int = 16
    ffn: int = 4096
    layers: int = 24
    vocab: int = 30522
    max_pos: int = 512
    type_vocab: int = 2
    max_seqlen: int = 384
    seed: int = 1

    def __post_init__(self):
        if self.hidden != self.heads * HEAD:
            raise ValueError("the INT8 interleaved attention plugin serves heads of 64 channels")


def _i32(name, v):
    return PluginField(name, np.array([v], np.int32), PluginFieldType.INT32)


def _f32(name, v):
    return PluginField(name, np.array([v], np.float32), PluginFieldType.FLOAT32)


def _through_runtime(creator, plugin, what):
    """Engine deserialisation: a runtime-phase plugin rebuilt from the serialised fields."""
    if plugin is None:
        raise RuntimeError(f"{what}: createPlugin failed: {last_log()}")
    rt = creator.create_plugin(what, plugin.get_fields_to_serialize(), TensorRTPhase.RUNTIME)
    if rt is None:
        raise RuntimeError(f"{what}: runtime createPlugin failed: {last_log()}")
    return rt


def quantize_rows(w: np.ndarray):
    """Per-output-channel symmetric INT8: q[n] = clip(rne(w[n] * 127 / amax_n)), scale[n] = amax_n / 127."""
    amax = np.maximum(np.abs(w).max(axis=1), 1e-8).astype(np.float32)
    scale = (amax / np.float32(127)).astype(np.float32)
    q = np.clip(np.rint(w / scale[:, None]), -127, 127).astype(np.int8)
    return q, scale


class Linear:
    """One INT8 fully-connected layer: weights [N][K] quantised per row, kept on the GPU in the interleaved
    layout [K/32][N][32]; alpha/beta hold the folded scales once the activation scales are known."""

    def __init__(self, api, torch, w: np.ndarray, bias: np.ndarray, stream: int):
        self.api, self.torch = api, torch
        self.N, self.K = w.shape
        self.w_q, self.s_w = quantize_rows(w.astype(np.float32))
        self.bias = bias.astype(np.float32)
        lin = torch.from_numpy(self.w_q).cuda()
        self.w_dev = torch.empty((self.K // 32, self.N, 32), dtype=torch.int8, device="cuda")
        api.check(api.int8_linear_to_interleaved(stream, self.N, self.K, lin.data_ptr(), self.w_dev.data_ptr()))
        torch.cuda.synchronize()
        self.alpha = self.beta = None
        self.alpha_h = self.beta_h = None
        self.epilogue = capi.LINEAR_AFFINE
        self.out_scale = 1.0

    def fold(self, s_in: float, s_out: float, gelu: bool = False):
        """out8 = sat8(rne(y / s_out)) with y = s_in * s_w[n] * acc + bias[n] (then GELU)."""
        s_in, s_out = np.float32(s_in), np.float32(s_out)
        if gelu:
            a = (s_in * self.s_w).astype(np.float32)
            b = self.bias.copy()
            self.epilogue, self.out_scale = capi.LINEAR_GELU, float(np.float32(1) / s_out)
        else:
            a = (s_in * self.s_w / s_out).astype(np.float32)
            b = (self.bias / s_out).astype(np.float32)
            self.epilogue, self.out_scale = capi.LINEAR_AFFINE, 1.0
        self.alpha_h, self.beta_h = a, b
        self.alpha = self.torch.from_numpy(a).cuda()
        self.beta = self.torch.from_numpy(b).cuda()

    def params(self, a_ptr: int, out_ptr: int, T: int, epilogue=None) -> capi.Int8LinearParams:
        p = capi.Int8LinearParams()
        p.a, p.w, p.alpha, p.beta, p.out = a_ptr, self.w_dev.data_ptr(), self.alpha.data_ptr(), self.beta.data_ptr(), out_ptr
        p.T, p.K, p.N = T, self.K, self.N
        p.a_interleaved, p.w_interleaved = 1, 1
        p.epilogue = self.epilogue if epilogue is None else epilogue
        p.out_interleaved = 0 if p.epilogue in (capi.LINEAR_RAW_INT32, capi.LINEAR_AFFINE_FP16) else 1
        p.out_scale = self.out_scale
        return p


def split_runs(cu, parts: int) -> list:
    """Cuts a packed batch (cu_seqlens `cu`, [B + 1]) into at most `parts` runs of whole sequences with about the same
    number of tokens each: the i-th cut is the sequence boundary nearest to i / parts of the tokens that still leaves
    every later run a sequence.  Returns [(first sequence, one past the last)]; runs without tokens are left out."""
    cu = np.asarray(cu, np.int64)
    B = len(cu) - 1
    parts = max(1, min(int(parts), B))
    cuts = [0]
    for i in range(1, parts):
        lo, hi = cuts[-1] + 1, B - (parts - i)
        cuts.append(lo + int(np.argmin(np.abs(cu[lo:hi + 1] - cu[-1] * i / parts))))
    cuts.append(B)
    return [(cuts[i], cuts[i + 1]) for i in range(len(cuts) - 1) if cu[cuts[i + 1]] > cu[cuts[i]]]


class Int8BertEncoder:
    """Random-initialised BERT encoder (weights ~N(0, 0.02), LayerNorm gamma ~U(0.5, 1.5), beta ~N(0, 0.1))
    running as INT8 in the 32-interleaved layout."""

    def __init__(self, cfg: EncoderConfig):
        import torch
        self.torch, self.cfg = torch, cfg
        self.api = capi.api()
        self.stream = torch.cuda.current_stream().cuda_stream
        reg = get_plugin_registry()
        r = np.random.default_rng(cfg.seed)
        E, F = cfg.hidden, cfg.ffn
        f32t = PluginFieldType.FLOAT32

        emb = dict(beta=(0.1 * r.standard_normal(E)).astype(np.float32),
                   gamma=r.uniform(0.5, 1.5, E).astype(np.float32),
                   word=(0.02 * r.standard_normal((cfg.vocab, E))).astype(np.float32),
                   tok=(0.02 * r.standard_normal((cfg.type_vocab, E))).astype(np.float32),
                   pos=(0.02 * r.standard_normal((cfg.max_pos, E))).astype(np.float32))
        self.emb_weights = emb
        c = reg.get_creator(EMBLN, "4")
        self.emb_plugin = _through_runtime(c, c.create_plugin("embeddings", [
            PluginField("bert_embeddings_layernorm_beta", emb["beta"], f32t),
            PluginField("bert_embeddings_layernorm_gamma", emb["gamma"], f32t),
            PluginField("bert_embeddings_word_embeddings", emb["word"], f32t),
            PluginField("bert_embeddings_token_type_embeddings", emb["tok"], f32t),
            PluginField("bert_embeddings_position_embeddings", emb["pos"], f32t),
            _i32("output_fp16", 1)]), "embeddings")

        cq = reg.get_creator(QKV, "6")
        cs = reg.get_creator(SKIPLN, "7")
        self.layers = []
        for li in range(cfg.layers):
            L = {}
            for name, n, k in (("qkv", 3 * E, E), ("proj", E, E), ("ffn1", F, E), ("ffn2", E, F)):
                w = (0.02 * r.standard_normal((n, k))).astype(np.float32)
                b = (0.02 * r.standard_normal(n)).astype(np.float32)
                L[name] = Linear(self.api, torch, w, b, self.stream)
            L["attention"] = _through_runtime(cq, cq.create_plugin(f"l{li}_attention", [
                _i32("hidden_size", E), _i32("num_heads", cfg.heads), _f32("dq_probs", 1.0 / 127.0)]), f"l{li}_attention")
            for ln in ("ln1", "ln2"):
                gamma = r.uniform(0.5, 1.5, E).astype(np.float16)
                beta = (0.1 * r.standard_normal(E)).astype(np.float16)
                L[ln + "_gamma"], L[ln + "_beta"] = gamma, beta
                L[ln] = _through_runtime(cs, cs.create_plugin(f"l{li}_{ln}", [
                    PluginField("beta", beta, PluginFieldType.FLOAT16),
                    PluginField("gamma", gamma, PluginFieldType.FLOAT16)]), f"l{li}_{ln}")
            L["scales"] = {}
            self.layers.append(L)
        self.s_emb = None
        self.T = self.B = 0
        self.buf = {}
        self.calibrated = False

    # ---- buffers -------------------------------------------------------------------------------------
    def _bind(self, ids: np.ndarray, segs: np.ndarray, cu: np.ndarray):
        torch, cfg = self.torch, self.cfg
        T, B = int(cu[-1]), len(cu) - 1
        if len(ids) != T or len(segs) != T:
            raise ValueError("ids and segment ids must hold one entry per packed token")
        E, F = cfg.hidden, cfg.ffn
        if T != self.T or B != self.B:
            i8 = lambda c: torch.empty((c // 32, T, 32), dtype=torch.int8, device="cuda")
            self.buf = dict(emb=torch.empty((T, E), dtype=torch.float16, device="cuda"),
                            emb2=torch.empty((1,), dtype=torch.int32, device="cuda"),
                            x=i8(E), qkv=i8(3 * E), ctx=i8(E), ao=i8(E), h=i8(E), m=i8(F), f=i8(E),
                            out=torch.empty((T, E), dtype=torch.float16, device="cuda"),
                            dummy=torch.zeros((cfg.max_seqlen,), dtype=torch.int32, device="cuda"))
            self.T, self.B = T, B
        self.buf["ids"] = torch.from_numpy(np.ascontiguousarray(ids, np.int32)).cuda()
        self.buf["segs"] = torch.from_numpy(np.ascontiguousarray(segs, np.int32)).cuda()
        self.buf["cu"] = torch.from_numpy(np.ascontiguousarray(cu, np.int32)).cuda()
        self._concurrent = None   # its sub-batches point into the tensors replaced above

    # ---- single operations -----------------------------------------------------------------------------
    def _check(self, st, what):
        if st != 0:
            raise RuntimeError(f"{what} failed with status {st}: {last_log() or self.api.last_error_str()}")

    def _embed(self):
        b, cfg = self.buf, self.cfg
        T, B, E = self.T, self.B, cfg.hidden
        ins = [TensorDesc([T], DataType.INT32), TensorDesc([T], DataType.INT32), TensorDesc([B + 1], DataType.INT32),
               TensorDesc([cfg.max_seqlen], DataType.INT32)]
        outs = [TensorDesc([T, E, 1, 1], DataType.HALF), TensorDesc([], DataType.INT32)]
        p = self.emb_plugin
        self._check(p.on_shape_change(ins, outs), "embeddings onShapeChange")
        self._check(p.enqueue(ins, outs, [b["ids"].data_ptr(), b["segs"].data_ptr(), b["cu"].data_ptr(),
                                          b["dummy"].data_ptr()], [b["emb"].data_ptr(), b["emb2"].data_ptr()], 0,
                              self.stream), "embeddings enqueue")

    def _linear(self, lin: Linear, src, dst, epilogue=None):
        p = lin.params(src.data_ptr(), dst.data_ptr(), self.T, epilogue)
        self.api.check(self.api.int8_linear(self.stream, C.byref(p)))

    def _attention(self, L, s_qkv, s_ctx):
        b, cfg = self.buf, self.cfg
        T, B, E = self.T, self.B, cfg.hidden
        fmt = TensorFormat.CHW32
        ins = [TensorDesc([1, 3 * E, T, 1], DataType.INT8, fmt, s_qkv), TensorDesc([B + 1], DataType.INT32),
               TensorDesc([cfg.max_seqlen], DataType.INT32)]
        outs = [TensorDesc([1, E, T, 1], DataType.INT8, fmt, s_ctx)]
        p = L["attention"]
        self._check(p.on_shape_change(ins, outs), "attention onShapeChange")
        self._check(p.enqueue(ins, outs, [b["qkv"].data_ptr(), b["cu"].data_ptr(), b["dummy"].data_ptr()],
                              [b["ctx"].data_ptr()], 0, self.stream), "attention enqueue")

    def _skipln(self, plugin, src, s_src, skip, s_skip, dst, s_dst):
        T, E = self.T, self.cfg.hidden
        fmt = TensorFormat.CHW32
        shape = [1, E, T, 1]
        ins = [TensorDesc(shape, DataType.INT8, fmt, s_src), TensorDesc(shape, DataType.INT8, fmt, s_skip)]
        outs = [TensorDesc(shape, DataType.INT8, fmt, s_dst)]
        self._check(plugin.on_shape_change(ins, outs), "skipLayerNorm onShapeChange")
        self._check(plugin.enqueue(ins, outs, [src.data_ptr(), skip.data_ptr()], [dst.data_ptr()], 0, self.stream),
                    "skipLayerNorm enqueue")

    # ---- calibration ------------------------------------------------------------------------------------
    def _amax_linear(self, lin: Linear, src, s_in, scratch, gelu=False) -> float:
        """amax of the layer's real-valued output on the current batch (FP16 epilogue into scratch)."""
        torch = self.torch
        lin.fold(s_in, 1.0)
        view = scratch[: self.T * lin.N].view(self.T, lin.N)
        self._linear(lin, src, view, capi.LINEAR_AFFINE_FP16)
        y = view.float()
        if gelu:
            y = torch.nn.functional.gelu(y)
        return float(y.abs().max())

    def _amax_int8(self, t) -> int:
        return int(t.to(self.torch.int16).abs().max())

    def calibrate(self, ids, segs, cu, margin: float = 1.05):
        """Sets every activation scale to amax/127 measured on this batch, layer by layer (what a
        calibrator does at build time) and folds the scales into the linear layers."""
        torch, cfg = self.torch, self.cfg
        self._bind(ids, segs, cu)
        b = self.buf
        T, E, F = self.T, cfg.hidden, cfg.ffn
        scratch = torch.empty((T * max(3 * E, F),), dtype=torch.float16, device="cuda")
        to_scale = lambda amax: float(np.float32(max(amax, 1e-6) * margin / 127.0))

        self._embed()
        self.s_emb = to_scale(float(b["emb"].float().abs().max()))
        self.api.check(self.api.quantize_fp16_to_interleaved(self.stream, T, E, b["emb"].data_ptr(), self.s_emb,
                                                             b["x"].data_ptr()))
        s_x = self.s_emb
        for L in self.layers:
            sc = L["scales"]
            sc["x"] = s_x
            sc["qkv"] = to_scale(self._amax_linear(L["qkv"], b["x"], s_x, scratch))
            L["qkv"].fold(s_x, sc["qkv"])
            self._linear(L["qkv"], b["x"], b["qkv"])
            # attention output is a convex combination of V rows: start from the QKV scale, then tighten
            self._attention(L, sc["qkv"], sc["qkv"])
            sc["ctx"] = float(np.float32(sc["qkv"] * max(self._amax_int8(b["ctx"]), 1) * margin / 127.0))
            self._attention(L, sc["qkv"], sc["ctx"])
            sc["ao"] = to_scale(self._amax_linear(L["proj"], b["ctx"], sc["ctx"], scratch))
            L["proj"].fold(sc["ctx"], sc["ao"])
            self._linear(L["proj"], b["ctx"], b["ao"])
            sc["h"] = self._calibrate_skipln(L, "ln1", b["ao"], sc["ao"], b["x"], s_x, b["h"], margin)
            sc["m"] = to_scale(self._amax_linear(L["ffn1"], b["h"], sc["h"], scratch, gelu=True))
            L["ffn1"].fold(sc["h"], sc["m"], gelu=True)
            self._linear(L["ffn1"], b["h"], b["m"])
            sc["f"] = to_scale(self._amax_linear(L["ffn2"], b["m"], sc["m"], scratch))
            L["ffn2"].fold(sc["m"], sc["f"])
            self._linear(L["ffn2"], b["m"], b["f"])
            sc["out"] = self._calibrate_skipln(L, "ln2", b["f"], sc["f"], b["h"], sc["h"], b["x"], margin)
            s_x = sc["out"]
        torch.cuda.synchronize()
        self.calibrated = True

    def _calibrate_skipln(self, L, ln, src, s_src, skip, s_skip, dst, margin) -> float:
        # a normalised row has |z| <= sqrt(E); start wide, measure, tighten
        gamma, beta = L[ln + "_gamma"].astype(np.float32), L[ln + "_beta"].astype(np.float32)
        wide = float(np.float32((8.0 * np.abs(gamma).max() + np.abs(beta).max()) / 127.0))
        self._skipln(L[ln], src, s_src, skip, s_skip, dst, wide)
        s = float(np.float32(wide * max(self._amax_int8(dst), 1) * margin / 127.0))
        self._skipln(L[ln], src, s_src, skip, s_skip, dst, s)
        return s

    # ---- inference ------------------------------------------------------------------------------------
    def enqueue(self, ids=None, segs=None, cu=None, capture: dict | None = None):
        """One forward pass over the packed batch; returns the FP16 [T, hidden] output tensor (device).
        With ids=None the inputs of the previous call are reused (steady-state timing).  `capture`, if
        given, receives a host copy of every intermediate tensor, keyed "l<i>.<name>"."""
        if not self.calibrated:
            raise RuntimeError("calibrate() first: the activation scales are not set")
        if ids is not None:
            self._bind(ids, segs, cu)
        b, api = self.buf, self.api
        T, E = self.T, self.cfg.hidden

        def keep(key, t):
            if capture is not None:
                capture[key] = t.detach().cpu().numpy().copy()

        self._embed()
        keep("emb", b["emb"])
        api.check(api.quantize_fp16_to_interleaved(self.stream, T, E, b["emb"].data_ptr(), self.s_emb, b["x"].data_ptr()))
        for i, L in enumerate(self.layers):
            sc = L["scales"]
            keep(f"l{i}.x", b["x"])
            self._linear(L["qkv"], b["x"], b["qkv"])
            keep(f"l{i}.qkv", b["qkv"])
            self._attention(L, sc["qkv"], sc["ctx"])
            keep(f"l{i}.ctx", b["ctx"])
            self._linear(L["proj"], b["ctx"], b["ao"])
            keep(f"l{i}.ao", b["ao"])
            self._skipln(L["ln1"], b["ao"], sc["ao"], b["x"], sc["x"], b["h"], sc["h"])
            keep(f"l{i}.h", b["h"])
            self._linear(L["ffn1"], b["h"], b["m"])
            keep(f"l{i}.m", b["m"])
            self._linear(L["ffn2"], b["m"], b["f"])
            keep(f"l{i}.f", b["f"])
            self._skipln(L["ln2"], b["f"], sc["f"], b["h"], sc["h"], b["x"], sc["out"])
        keep("x_out", b["x"])
        api.check(api.dequantize_interleaved_to_fp16(self.stream, T, E, b["x"].data_ptr(), self.layers[-1]["scales"]["out"]
                                                     if self.layers else self.s_emb, b["out"].data_ptr()))
        keep("out", b["out"])
        return b["out"]

    # ---- the native runner ------------------------------------------------------------------------------
    def build_native(self):
        """Hands the built network (quantised weights, folded scales, calibrated activation scales) to the C++
        runner of include/trtamd_encoder_runtime.h, which then owns its own plugin objects and device weights."""
        if not self.calibrated:
            raise RuntimeError("calibrate() first: the activation scales are not set")
        api, cfg = self.api, self.cfg
        c = capi.EncoderConfig(hidden=cfg.hidden, heads=cfg.heads, ffn=cfg.ffn, layers=cfg.layers, vocab=cfg.vocab,
                               max_pos=cfg.max_pos, type_vocab=cfg.type_vocab, max_seqlen=cfg.max_seqlen)
        h = api.encoder_create(C.byref(c))
        if not h:
            raise RuntimeError(f"trtamd_encoder_create: {api.last_error_str()}")
        host = lambda a, dt: np.ascontiguousarray(a, dtype=dt)
        ptr = lambda a: a.ctypes.data
        w = self.emb_weights
        keep = [host(w[k], np.float32) for k in ("beta", "gamma", "word", "tok", "pos")]
        e = capi.EncoderEmbedding(*[ptr(a) for a in keep], self.s_emb)
        api.check(api.encoder_set_embedding(h, C.byref(e)))
        for i, L in enumerate(self.layers):
            sc = L["scales"]
            d = capi.EncoderLayer()
            hold = []
            for name in ("qkv", "proj", "ffn1", "ffn2"):
                lin = L[name]
                arrs = [host(lin.w_q, np.int8), host(lin.alpha_h, np.float32), host(lin.beta_h, np.float32)]
                hold += arrs
                setattr(d, name, capi.EncoderLinear(*[ptr(a) for a in arrs]))
            d.ffn1_out_scale = L["ffn1"].out_scale
            for field, key in (("ln1_gamma", "ln1_gamma"), ("ln1_beta", "ln1_beta"), ("ln2_gamma", "ln2_gamma"),
                               ("ln2_beta", "ln2_beta")):
                a = host(L[key], np.float16)
                hold.append(a)
                setattr(d, field, ptr(a))
            d.s_x, d.s_qkv, d.s_ctx, d.s_ao = sc["x"], sc["qkv"], sc["ctx"], sc["ao"]
            d.s_h, d.s_f, d.s_out = sc["h"], sc["f"], sc["out"]
            api.check(api.encoder_set_layer(h, i, C.byref(d)))
            del hold
        self._native = h
        self._native_ws = None
        return h

    def enqueue_native(self, ids=None, segs=None, cu=None, stream=None):
        """One forward pass through the C++ runner (same network, same scales); returns the FP16 output tensor.
        `stream` (a raw stream handle) overrides the stream the encoder was built on, e.g. a stream under graph
        capture: the call only launches kernels, so it can be recorded and replayed."""
        if getattr(self, "_native", None) is None:
            self.build_native()
        if ids is not None:
            self._bind(ids, segs, cu)
        api, b = self.api, self.buf
        self.prepare_native()
        api.check(api.encoder_enqueue(self._native, b["ids"].data_ptr(), b["segs"].data_ptr(), b["cu"].data_ptr(), self.B,
                                      self.T, self._native_ws.data_ptr(), b["out_native"].data_ptr(),
                                      self.stream if stream is None else stream))
        return b["out_native"]

    def prepare_concurrent(self, parts: int = 2):
        """The caller's side of enqueue_native_concurrent: the bound batch cut into `parts` runs of whole sequences with
        about the same number of tokens, each with its own cu_seqlens and workspace; execution contexts reserved."""
        torch, api, b = self.torch, self.api, self.buf
        if getattr(self, "_native", None) is None:
            self.build_native()
        self.prepare_native()
        cu = b["cu"].cpu().numpy().astype(np.int64)
        runs = split_runs(cu, parts)
        api.check(api.encoder_reserve_contexts(self._native, max(len(runs), 1)))
        batches = (capi.EncoderBatch * max(len(runs), 1))()
        keep = []
        E = self.cfg.hidden
        for i, (lo, hi) in enumerate(runs):
            t0, t1 = int(cu[lo]), int(cu[hi])
            sub_cu = torch.from_numpy((cu[lo:hi + 1] - cu[lo]).astype(np.int32)).cuda()
            ws = torch.empty((api.encoder_workspace_size(self._native, t1 - t0),), dtype=torch.uint8, device="cuda")
            keep += [sub_cu, ws]
            q = batches[i]
            q.ids = b["ids"].data_ptr() + 4 * t0
            q.segment_ids = b["segs"].data_ptr() + 4 * t0
            q.cu_seqlens = sub_cu.data_ptr()
            q.batch, q.tokens = hi - lo, t1 - t0
            q.workspace = ws.data_ptr()
            q.out = b["out_native"].data_ptr() + 2 * E * t0
        self._concurrent = (batches, len(runs), keep, parts)
        return len(runs)

    def enqueue_native_concurrent(self, parts: int = 2, stream=None):
        """One forward pass of the bound batch as `parts` sub-batches that the C++ runner executes at the same time
        (trtamd_encoder_enqueue_concurrent).  Sequences do not interact, so the output tensor holds the same bits as
        enqueue_native's; the sub-batches fill the compute units that each other's kernel tails leave idle."""
        if getattr(self, "_concurrent", None) is None or self._concurrent[3] != parts:
            self.prepare_concurrent(parts)
        batches, n = self._concurrent[:2]
        self.api.check(self.api.encoder_enqueue_concurrent(self._native, batches, n,
                                                           self.stream if stream is None else stream))
        return self.buf["out_native"]

    def prepare_native(self):
        """The caller's side of an enqueue that must not allocate: workspace and output tensor for the bound batch."""
        torch, b = self.torch, self.buf
        need = self.api.encoder_workspace_size(self._native, self.T)
        if self._native_ws is None or self._native_ws.numel() < need:
            self._native_ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
        if "out_native" not in b or b["out_native"].shape[0] != self.T:
            b["out_native"] = torch.empty((self.T, self.cfg.hidden), dtype=torch.float16, device="cuda")

    def destroy_native(self):
        h = getattr(self, "_native", None)
        if h:
            self.api.encoder_destroy(h)
            self._native = None
            self._concurrent = None

    def __del__(self):
        h = getattr(self, "_native", None)
        if h:
            self.api.encoder_destroy(h)
            self._native = None

    # ---- accounting ------------------------------------------------------------------------------------
    def gemm_ops(self) -> float:
        """Integer operations of the linear layers of one pass (2 per multiply-accumulate)."""
        E, F = self.cfg.hidden, self.cfg.ffn
        return 2.0 * self.T * (3 * E * E + E * E + 2 * E * F) * self.cfg.layers
