"""The INT8 encoder chain (embedding -> quantise -> [QKV GEMM, attention, projection, SkipLN, FFN, SkipLN] x L
-> dequantise) on the GPU, every operation checked against the CPU oracle applied to that operation's own
GPU inputs.  Teacher forcing keeps each comparison at the single-operation bar (INT8 within 1 LSB, FP16 within
tolerance) while still proving the wiring: layouts, channel orders, plugin versions and the scale folded into
every step."""
import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, assert_int8_close, int8_attention_parity, rng
from tensorrt_amd import capi
from tensorrt_amd.encoder import EncoderConfig, Int8BertEncoder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def setup():
    cfg = EncoderConfig(hidden=768, heads=12, ffn=3072, layers=2, vocab=1000, max_pos=512, max_seqlen=384, seed=7)
    enc = Int8BertEncoder(cfg)
    r = rng(9)
    lens = np.array([50, 128, 7, 101, 1, 384])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    ids = r.integers(0, cfg.vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    enc.calibrate(ids, segs, cu)
    cap = {}
    out = enc.enqueue(ids, segs, cu, capture=cap)
    import torch
    torch.cuda.synchronize()
    return cfg, enc, ids, segs, cu, cap, out.cpu().numpy()


def il(x, T, C):
    return oracle.deinterleave(np.ascontiguousarray(x).ravel(), T, C)


def test_scales_are_calibrated(setup):
    cfg, enc, *_ = setup
    for L in enc.layers:
        for k in ("x", "qkv", "ctx", "ao", "h", "m", "f", "out"):
            assert 0 < L["scales"][k] < 10, (k, L["scales"][k])


def test_activations_use_the_int8_range(setup):
    cfg, enc, ids, segs, cu, cap, _ = setup
    for k, v in cap.items():
        if v.dtype == np.int8:
            amax = int(np.abs(v.astype(np.int16)).max())
            assert 100 <= amax <= 128, f"{k}: amax {amax} (calibration should place amax near 127/1.05)"


def test_embedding_and_quantiser(setup):
    cfg, enc, ids, segs, cu, cap, _ = setup
    w = enc.emb_weights
    tabs = {k: w[k].astype(np.float16) for k in ("word", "pos", "tok")}
    ref, _, _ = oracle.embln(1, ids, segs, cu, w["beta"], w["gamma"], tabs["word"], tabs["pos"], tabs["tok"],
                             cfg.max_seqlen, len(cu) - 1)
    assert_fp_close(cap["emb"], ref, what="embedding")
    want = oracle.quantize_f16_interleave(cap["emb"], enc.s_emb)
    assert np.array_equal(cap["l0.x"], want)


@pytest.mark.parametrize("layer", [0, 1])
def test_layer_operations(setup, layer):
    check_layer(setup, layer)


@pytest.fixture(scope="module")
def setup_large():
    """The benchmark's network (BERT-large: hidden 1024, 16 heads, feed-forward 4096, 24 layers) on a few short
    sequences, so that the oracle can follow every operation of every layer in seconds."""
    cfg = EncoderConfig(hidden=1024, heads=16, ffn=4096, layers=24, vocab=1000, max_pos=512, max_seqlen=384, seed=11)
    enc = Int8BertEncoder(cfg)
    r = rng(12)
    lens = np.array([33, 384, 1, 140])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    ids = r.integers(0, cfg.vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    enc.calibrate(ids, segs, cu)
    cap = {}
    out = enc.enqueue(ids, segs, cu, capture=cap)
    import torch
    torch.cuda.synchronize()
    return cfg, enc, ids, segs, cu, cap, out.cpu().numpy()


def test_every_layer_of_the_24_layer_network(setup_large):
    """Depth: the same per-operation checks on all 24 layers of the benchmark's network, each operation against the
    oracle applied to the tensor the GPU chain fed it, down to the dequantised output."""
    cfg, enc, ids, segs, cu, cap, out = setup_large
    for layer in range(cfg.layers):
        check_layer(setup_large, layer)
    want = oracle.dequantize_deinterleave_f16(cap["x_out"], enc.layers[-1]["scales"]["out"])
    assert np.array_equal(out, want)
    # the chain has not collapsed on the way down: the last layer still uses the INT8 range
    assert int(np.abs(cap["x_out"].astype(np.int32)).max()) >= 100


def check_layer(setup, layer):
    cfg, enc, ids, segs, cu, cap, _ = setup
    T, E, F, N = int(cu[-1]), cfg.hidden, cfg.ffn, cfg.heads
    L, sc = enc.layers[layer], enc.layers[layer]["scales"]
    g = lambda k: cap[f"l{layer}.{k}"]

    def linear(name, src, gelu=False):
        lin = L[name]
        return oracle.int8_linear(src, lin.w_q, lin.alpha_h, lin.beta_h,
                                  oracle.LINEAR_GELU if gelu else oracle.LINEAR_AFFINE, out_scale=lin.out_scale,
                                  a_interleaved=True, out_interleaved=True)

    assert_int8_close(g("qkv"), linear("qkv", g("x")), what="QKV projection", max_frac_off=1e-3)

    # attention: the interleaved tensor's channel order is [3][N][64]; the oracle takes [T][N][3][64]
    qkv_lin = il(g("qkv"), T, 3 * E).reshape(T, 3, N, 64).transpose(0, 2, 1, 3).reshape(T, 3 * E)
    s_q, s_ctx, dqp = np.float32(sc["qkv"]), np.float32(sc["ctx"]), np.float32(np.float32(1.0) / np.float32(127.0))
    s1 = np.float32(np.float32(s_q * s_q) * (np.float32(1) / np.sqrt(np.float32(64))))
    s2 = np.float32(np.float32(dqp * s_q) / s_ctx)
    # the kernel run again on the captured tensor must reproduce the captured context bytes, with bit-exact first
    # accumulators, probabilities within one step (<= 1e-5 of them off), an exact second product and bit-exact
    # rows wherever the probabilities agree
    int8_attention_parity(qkv_lin, cu, N, s1, np.float32(1) / dqp, s2, interleaved=True, S=cfg.max_seqlen,
                          expect=il(g("ctx"), T, E))

    assert_int8_close(g("ao"), linear("proj", g("ctx")), what="output projection", max_frac_off=1e-3)

    def skipln(ln, src, s_src, skip, s_skip, s_out):
        st, ref, _ = oracle.skipln_interleaved(0, src.ravel(), skip.ravel(), L[ln + "_beta"], L[ln + "_gamma"], E, T,
                                               np.float32(s_src), np.float32(s_skip), np.float32(1) / np.float32(s_out))
        assert st == 0
        return ref

    assert_int8_close(g("h").ravel(), skipln("ln1", g("ao"), sc["ao"], g("x"), sc["x"], sc["h"]), what="SkipLN 1")
    assert_int8_close(g("m"), linear("ffn1", g("h"), gelu=True), what="FFN 1 + GELU", max_frac_off=2e-3)
    assert_int8_close(g("f"), linear("ffn2", g("m")), what="FFN 2", max_frac_off=1e-3)
    nxt = cap[f"l{layer + 1}.x"] if layer + 1 < cfg.layers else cap["x_out"]
    assert_int8_close(nxt.ravel(), skipln("ln2", g("f"), sc["f"], g("h"), sc["h"], sc["out"]), what="SkipLN 2")


def test_output_dequantiser_and_repeatability(setup):
    cfg, enc, ids, segs, cu, cap, out = setup
    want = oracle.dequantize_deinterleave_f16(cap["x_out"], enc.layers[-1]["scales"]["out"])
    assert np.array_equal(out, want)
    assert np.isfinite(out.astype(np.float32)).all() and float(np.abs(out.astype(np.float32)).max()) > 1.0
    # a second pass over the same inputs (the steady-state call the benchmark times) gives the same bytes
    import torch
    again = enc.enqueue()
    torch.cuda.synchronize()
    assert np.array_equal(again.cpu().numpy(), out)


def test_native_runner_matches_the_python_chain(setup):
    """The C++ runner builds its own plugin objects and device weights from the same built network; its output
    is the same bytes, on the calibration batch and on a batch of another shape."""
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    got = enc.enqueue_native(ids, segs, cu)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), out)
    r = rng(17)
    lens = np.array([3, 200, 64])
    cu2 = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ids2 = r.integers(0, cfg.vocab, int(cu2[-1])).astype(np.int32)
    segs2 = r.integers(0, 2, int(cu2[-1])).astype(np.int32)
    want = enc.enqueue(ids2, segs2, cu2).cpu().numpy()
    got = enc.enqueue_native(ids2, segs2, cu2)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    enc.enqueue(ids, segs, cu)   # leave the fixture's buffers as the other tests expect them


def test_native_runner_replays_from_a_captured_graph(setup):
    """enqueue launches kernels only (no allocation, copy, memset or synchronisation), so a caller can record it
    into a graph.  Every replay is checked, with eager work on the same buffers between the replays."""
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    first = enc.enqueue_native(ids, segs, cu)
    torch.cuda.synchronize()
    assert np.array_equal(first.cpu().numpy(), out)
    r = rng(23)
    ids2 = r.integers(0, cfg.vocab, ids.size).astype(np.int32)
    want2 = enc.enqueue_native(ids2, segs, cu).cpu().numpy()
    enc.enqueue_native(ids, segs, cu)
    torch.cuda.synchronize()
    assert not np.array_equal(want2, out)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        result = enc.enqueue_native(stream=torch.cuda.current_stream().cuda_stream)
    d_ids = enc.buf["ids"]
    for k, (tokens, want) in enumerate([(ids, out), (ids2, want2), (ids, out), (ids2, want2)]):
        d_ids.copy_(torch.from_numpy(tokens))          # eager: new inputs in place
        result.fill_(float("nan"))                     # eager: the previous result is gone
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(result.cpu().numpy(), want), f"replay {k}"
    enc.enqueue(ids, segs, cu)   # leave the fixture's buffers as the other tests expect them


def test_first_enqueue_of_a_fresh_runner_can_be_captured(setup):
    """The very first enqueue of a newly built runner launches kernels only: every device allocation and copy of
    its plugins happened in set_embedding / set_layer.  It is recorded into a graph without any eager pass before
    it, and every replay gives the eager bytes."""
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    enc.destroy_native()
    enc.build_native()                      # new plugin objects, new device weights; nothing enqueued yet
    enc._bind(ids, segs, cu)
    enc.prepare_native()                    # the caller's buffers
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        result = enc.enqueue_native(stream=torch.cuda.current_stream().cuda_stream)
    for k in range(3):
        result.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(result.cpu().numpy(), out), f"replay {k}"
    enc.enqueue(ids, segs, cu)


@pytest.mark.parametrize("parts", [2, 3])
def test_concurrent_sub_batches_give_the_single_pass_bytes(setup, parts):
    """The batch cut into runs of whole sequences that the runner executes at the same time (one execution context,
    i.e. one set of plugin clones, per run; side streams forked from and joined to the caller's stream) must give the
    bytes of the single enqueue, eagerly and on every replay of a captured graph with eager work in between."""
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    enc.enqueue_native(ids, segs, cu)
    torch.cuda.synchronize()
    n = enc.prepare_concurrent(parts)
    assert n == parts
    result = enc.buf["out_native"]
    for _ in range(2):
        result.fill_(float("nan"))
        got = enc.enqueue_native_concurrent(parts)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), out)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            enc.enqueue_native_concurrent(parts, stream=stream.cuda_stream)
    r = rng(29)
    ids2 = r.integers(0, cfg.vocab, ids.size).astype(np.int32)
    d_ids = enc.buf["ids"]
    d_ids.copy_(torch.from_numpy(ids2))
    want2 = enc.enqueue_native().cpu().numpy()
    assert not np.array_equal(want2, out)
    for k, (tokens, want) in enumerate([(ids, out), (ids2, want2), (ids, out)]):
        d_ids.copy_(torch.from_numpy(tokens))
        result.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(result.cpu().numpy(), want), f"replay {k}"
    enc.enqueue(ids, segs, cu)   # leave the fixture's buffers as the other tests expect them


def test_concurrent_enqueue_refuses_more_parts_than_contexts(setup):
    from tensorrt_amd import capi
    cfg, enc, ids, segs, cu, cap, out = setup
    enc.enqueue_native(ids, segs, cu)
    enc.prepare_concurrent(2)
    three = (capi.EncoderBatch * 9)()
    st = enc.api.encoder_enqueue_concurrent(enc._native, three, 9, enc.stream)
    assert st != 0 and "contexts" in enc.api.last_error_str()
    assert enc.api.encoder_reserve_contexts(enc._native, 9) != 0
    enc.enqueue(ids, segs, cu)


def test_concurrent_enqueue_with_degenerate_batches(setup):
    """One sequence cannot be cut (one part), and a run of empty sequences has no rows (it is left out): both still
    give the single enqueue's bytes."""
    import torch
    cfg, enc, ids, segs, cu, cap, out = setup
    r = rng(31)
    for lens in ([77], [0, 0, 150, 40], [90, 60, 0, 0]):
        cu2 = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        ids2 = r.integers(0, cfg.vocab, int(cu2[-1])).astype(np.int32)
        segs2 = r.integers(0, 2, int(cu2[-1])).astype(np.int32)
        want = enc.enqueue_native(ids2, segs2, cu2).cpu().numpy().copy()
        n = enc.prepare_concurrent(2)
        assert n == (1 if len(lens) == 1 else 2)
        enc.buf["out_native"].fill_(float("nan"))
        got = enc.enqueue_native_concurrent(2)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want), lens
    enc.enqueue(ids, segs, cu)
