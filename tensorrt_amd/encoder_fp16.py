"""FP16 BERT encoder assembled from the plugin library: the FP16 counterpart of encoder.Int8BertEncoder.

    EmbLayerNorm (var-seqlen, FP16)       CustomEmbLayerNormPluginDynamic v4
    per layer:
        QKV projection    FP16 GEMM + bias    (TensorRT core / CustomFCPluginDynamic; trtamd_fp16_linear here)
        attention         CustomQKVToContextPluginDynamic v5, type_id 1, var_seqlen 1 (fused FP16 MHA on cu_seqlens)
        output projection FP16 GEMM           (its bias travels in the SkipLayerNorm that follows)
        residual + LN     CustomSkipLayerNormPluginDynamic v6, type_id 1, with bias
        feed-forward 1    FP16 GEMM + bias + GELU
        feed-forward 2    FP16 GEMM
        residual + LN     CustomSkipLayerNormPluginDynamic v6, with bias

All tensors are linear: activations [T, C] over the packed tokens, weights [N][K] (QKV rows ordered
[head][q|k|v][64], plugin/bertQKVToContextPlugin/README.md:27-30).  torch is the allocator; every operation is a call
into libtrtamd_bert_plugins.so.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .encoder import EMBLN, HEAD, QKV, SKIPLN, EncoderConfig, _i32, _through_runtime
from .plugin import DataType, PluginField, PluginFieldType, TensorDesc, get_plugin_registry, last_log


class Fp16Linear:
    """out = f(a @ w.T * alpha + beta) through trtamd_fp16_linear; alpha is 1, beta the bias (or 0)."""

    def __init__(self, torch, w: np.ndarray, bias: np.ndarray | None, gelu: bool = False):
        self.N, self.K = w.shape
        self.w_h = w.astype(np.float16)
        self.bias_h = (np.zeros(self.N, np.float32) if bias is None else bias.astype(np.float32))
        self.alpha_h = np.ones(self.N, np.float32)
        self.gelu = gelu
        self.w = torch.from_numpy(self.w_h).cuda()
        self.alpha = torch.from_numpy(self.alpha_h).cuda()
        self.beta = torch.from_numpy(self.bias_h).cuda()

    def params(self, a_ptr: int, out_ptr: int, T: int) -> capi.Fp16LinearParams:
        p = capi.Fp16LinearParams()
        p.a, p.w, p.alpha, p.beta, p.out = a_ptr, self.w.data_ptr(), self.alpha.data_ptr(), self.beta.data_ptr(), out_ptr
        p.T, p.K, p.N = T, self.K, self.N
        p.epilogue = capi.LINEAR_GELU if self.gelu else capi.LINEAR_AFFINE
        return p


class Fp16BertEncoder:
    """Random-initialised BERT encoder (weights ~N(0, 0.02), LayerNorm gamma ~U(0.5, 1.5), beta ~N(0, 0.1)) in FP16."""

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

        cq = reg.get_creator(QKV, "5")
        cs = reg.get_creator(SKIPLN, "6")
        self.layers = []
        for li in range(cfg.layers):
            L = {}
            w = lambda n, k: (0.02 * r.standard_normal((n, k))).astype(np.float32)
            b = lambda n: (0.02 * r.standard_normal(n)).astype(np.float32)
            L["qkv"] = Fp16Linear(torch, w(3 * E, E), b(3 * E))
            L["proj"] = Fp16Linear(torch, w(E, E), None)
            L["ffn1"] = Fp16Linear(torch, w(F, E), b(F), gelu=True)
            L["ffn2"] = Fp16Linear(torch, w(E, F), None)
            attention = cq.create_plugin(f"l{li}_attention", [
                _i32("type_id", int(DataType.HALF)), _i32("hidden_size", E), _i32("num_heads", cfg.heads),
                _i32("has_mask", 1), _i32("var_seqlen", 1)])
            if attention is None:
                raise RuntimeError(f"l{li}_attention: createPlugin failed: {last_log()}")
            # the builder configures a plugin before it serialises it (this version stores the configured S and B)
            nominal = cfg.max_seqlen
            ins = [TensorDesc([nominal, 3 * E, 1, 1], DataType.HALF), TensorDesc([1], DataType.INT32),
                   TensorDesc([2], DataType.INT32), TensorDesc([cfg.max_seqlen], DataType.INT32)]
            if attention.configure_plugin(ins, [TensorDesc([nominal, E, 1, 1], DataType.HALF)]) != 0:
                raise RuntimeError(f"l{li}_attention: configurePlugin failed: {last_log()}")
            L["attention"] = _through_runtime(cq, attention, f"l{li}_attention")
            for ln in ("ln1", "ln2"):
                gamma = r.uniform(0.5, 1.5, E).astype(np.float32)
                beta = (0.1 * r.standard_normal(E)).astype(np.float32)
                bias = b(E)   # the bias of the linear layer in front of this LayerNorm
                L[ln + "_gamma"], L[ln + "_beta"], L[ln + "_bias"] = gamma, beta, bias
                L[ln] = _through_runtime(cs, cs.create_plugin(f"l{li}_{ln}", [
                    _i32("type_id", int(DataType.HALF)), PluginField("beta", beta, f32t),
                    PluginField("gamma", gamma, f32t), PluginField("bias", bias, f32t)]), f"l{li}_{ln}")
            self.layers.append(L)
        self.T = self.B = 0
        self.buf = {}

    def _bind(self, ids: np.ndarray, segs: np.ndarray, cu: np.ndarray):
        torch, cfg = self.torch, self.cfg
        T, B = int(cu[-1]), len(cu) - 1
        if len(ids) != T or len(segs) != T:
            raise ValueError("ids and segment ids must hold one entry per packed token")
        E, F = cfg.hidden, cfg.ffn
        if T != self.T or B != self.B:
            h = lambda c: torch.empty((T, c), dtype=torch.float16, device="cuda")
            self.buf = dict(x=h(E), qkv=h(3 * E), ctx=h(E), ao=h(E), h=h(E), m=h(F), f=h(E),
                            emb2=torch.empty((1,), dtype=torch.int32, device="cuda"),
                            mask=torch.zeros((1,), dtype=torch.int32, device="cuda"),
                            dummy=torch.zeros((cfg.max_seqlen,), dtype=torch.int32, device="cuda"))
            self.T, self.B = T, B
        self.buf["ids"] = torch.from_numpy(np.ascontiguousarray(ids, np.int32)).cuda()
        self.buf["segs"] = torch.from_numpy(np.ascontiguousarray(segs, np.int32)).cuda()
        self.buf["cu"] = torch.from_numpy(np.ascontiguousarray(cu, np.int32)).cuda()

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
                                          b["dummy"].data_ptr()], [b["x"].data_ptr(), b["emb2"].data_ptr()], 0,
                              self.stream), "embeddings enqueue")

    def _linear(self, lin: Fp16Linear, src, dst):
        p = lin.params(src.data_ptr(), dst.data_ptr(), self.T)
        self.api.check(self.api.fp16_linear(self.stream, C.byref(p)))

    def _attention(self, L):
        b, cfg = self.buf, self.cfg
        T, B, E = self.T, self.B, cfg.hidden
        ins = [TensorDesc([T, 3 * E, 1, 1], DataType.HALF), TensorDesc([1], DataType.INT32),
               TensorDesc([B + 1], DataType.INT32), TensorDesc([cfg.max_seqlen], DataType.INT32)]
        outs = [TensorDesc([T, E, 1, 1], DataType.HALF)]
        p = L["attention"]
        self._check(p.on_shape_change(ins, outs), "attention onShapeChange")
        self._check(p.enqueue(ins, outs, [b["qkv"].data_ptr(), b["mask"].data_ptr(), b["cu"].data_ptr(),
                                          b["dummy"].data_ptr()], [b["ctx"].data_ptr()], 0, self.stream),
                    "attention enqueue")

    def _skipln(self, plugin, src, skip, dst):
        T, E = self.T, self.cfg.hidden
        d = TensorDesc([T, 1, E, 1, 1], DataType.HALF)
        self._check(plugin.on_shape_change([d, d], [d]), "skipLayerNorm onShapeChange")
        self._check(plugin.enqueue([d, d], [d], [src.data_ptr(), skip.data_ptr()], [dst.data_ptr()], 0, self.stream),
                    "skipLayerNorm enqueue")

    def enqueue(self, ids=None, segs=None, cu=None, capture: dict | None = None):
        """One forward pass over the packed batch; returns the FP16 [T, hidden] output tensor (device).
        With ids=None the inputs of the previous call are reused.  `capture`, if given, receives host copies of
        every intermediate tensor under the names emb, l<i>.qkv, l<i>.ctx, l<i>.ao, l<i>.h, l<i>.m, l<i>.f, l<i>.out."""
        if ids is not None:
            self._bind(ids, segs, cu)
        b = self.buf

        def keep(key, t):
            if capture is not None:
                capture[key] = t.detach().cpu().numpy().copy()

        self._embed()
        keep("emb", b["x"])
        for i, L in enumerate(self.layers):
            self._linear(L["qkv"], b["x"], b["qkv"])
            keep(f"l{i}.qkv", b["qkv"])
            self._attention(L)
            keep(f"l{i}.ctx", b["ctx"])
            self._linear(L["proj"], b["ctx"], b["ao"])
            keep(f"l{i}.ao", b["ao"])
            self._skipln(L["ln1"], b["ao"], b["x"], b["h"])
            keep(f"l{i}.h", b["h"])
            self._linear(L["ffn1"], b["h"], b["m"])
            keep(f"l{i}.m", b["m"])
            self._linear(L["ffn2"], b["m"], b["f"])
            keep(f"l{i}.f", b["f"])
            self._skipln(L["ln2"], b["f"], b["h"], b["x"])
            keep(f"l{i}.out", b["x"])
        return b["x"]

    def flops(self) -> float:
        """Floating-point operations of one pass over the current batch: linear layers and attention (2 per MAC)."""
        cfg = self.cfg
        E, F = cfg.hidden, cfg.ffn
        cu = self.buf["cu"].cpu().numpy().astype(np.float64)
        lens = np.diff(cu)
        linear = 2.0 * self.T * (3 * E * E + E * E + 2 * E * F)
        attention = 4.0 * HEAD * cfg.heads * float(np.sum(lens * lens))
        return (linear + attention) * cfg.layers
