"""The FP16 encoder chain (embedding -> [QKV GEMM, fused FP16 attention v5, projection, SkipLayerNorm v6 with bias,
FFN + GELU, FFN, SkipLayerNorm v6] x L) on the GPU, every operation checked against the CPU oracle applied to that
operation's own GPU inputs (|a - b| <= 2e-3 + 1e-2 |b|)."""
import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, rng
from tensorrt_amd.encoder import EncoderConfig
from tensorrt_amd.encoder_fp16 import Fp16BertEncoder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def setup():
    cfg = EncoderConfig(hidden=768, heads=12, ffn=3072, layers=2, vocab=1000, max_pos=512, max_seqlen=384, seed=11)
    enc = Fp16BertEncoder(cfg)
    r = rng(12)
    lens = np.array([50, 128, 7, 101, 1, 384])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    ids = r.integers(0, cfg.vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    cap = {}
    out = enc.enqueue(ids, segs, cu, capture=cap)
    import torch
    torch.cuda.synchronize()
    return cfg, enc, ids, segs, cu, cap, out.cpu().numpy()


def test_embedding(setup):
    cfg, enc, ids, segs, cu, cap, _ = setup
    w = enc.emb_weights
    tabs = {k: w[k].astype(np.float16) for k in ("word", "pos", "tok")}
    ref, _, _ = oracle.embln(1, ids, segs, cu, w["beta"], w["gamma"], tabs["word"], tabs["pos"], tabs["tok"],
                             cfg.max_seqlen, len(cu) - 1)
    assert_fp_close(cap["emb"], ref, what="embedding")


@pytest.mark.parametrize("layer", [0, 1])
def test_layer_operations(setup, layer):
    cfg, enc, ids, segs, cu, cap, _ = setup
    E, N = cfg.hidden, cfg.heads
    L = enc.layers[layer]
    g = lambda k: cap[f"l{layer}.{k}"]
    x = cap["emb"] if layer == 0 else cap[f"l{layer - 1}.out"]

    def linear(name, src):
        lin = L[name]
        return oracle.fp16_linear(src, lin.w_h, lin.alpha_h, lin.bias_h, gelu=lin.gelu)

    def skipln(ln, src, skip):
        h = lambda a: a.astype(np.float16)
        return oracle.skipln(src, skip, h(L[ln + "_beta"]), h(L[ln + "_gamma"]), h(L[ln + "_bias"]))

    assert_fp_close(g("qkv"), linear("qkv", x), what="QKV projection")
    assert_fp_close(g("ctx"), oracle.mha_fused_f16_packed(g("qkv"), cu, N, 64), what="attention")
    assert_fp_close(g("ao"), linear("proj", g("ctx")), what="output projection")
    assert_fp_close(g("h"), skipln("ln1", g("ao"), x), what="SkipLayerNorm 1")
    assert_fp_close(g("m"), linear("ffn1", g("h")), what="feed-forward 1 + GELU")
    assert_fp_close(g("f"), linear("ffn2", g("m")), what="feed-forward 2")
    assert_fp_close(g("out"), skipln("ln2", g("f"), g("h")), what="SkipLayerNorm 2")


def test_output_is_finite_and_repeatable(setup):
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    assert np.isfinite(out.astype(np.float32)).all() and float(np.abs(out.astype(np.float32)).max()) > 1.0
    again = enc.enqueue()
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy().view(np.uint16), out.view(np.uint16))
