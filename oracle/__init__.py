"""CPU oracle for the BERT plugin hot path (numpy front end over ``bert_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the CPU-baseline leg
of the benchmark.  The shipped package never imports it.

Every wrapper takes and returns numpy arrays; binary16 tensors are ``np.float16``.  The C source
carries the reference citations; this module only marshals arguments.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile bert_oracle.c with gcc (a few seconds)."""
    src = os.path.join(_HERE, "bert_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_convert_mask.restype = C.c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return None if a is None else np.ascontiguousarray(a, dtype=dt)


class MhaGeom(C.Structure):
    _fields_ = [("B", C.c_int32), ("N", C.c_int32), ("d", C.c_int32), ("tokStrideIn", C.c_int64),
                ("tokStrideOut", C.c_int64), ("headStrideIn", C.c_int64), ("headStrideOut", C.c_int64)]


class MhaSeq(C.Structure):
    _fields_ = [("inBase", C.c_int64), ("outBase", C.c_int64), ("nq", C.c_int32), ("nk", C.c_int32)]


# ------------------------------------------------------------------------------------------------
# conversions
# ------------------------------------------------------------------------------------------------

def f32_to_f16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.float16)
    lib().orc_f32_to_f16(_p(x), _p(out), C.c_int64(x.size))
    return out


def float4_to_char4(v):
    v = _c(v, np.float32)
    out = np.empty(v.shape, np.int8)
    lib().orc_float4_to_char4(_p(v), _p(out), C.c_int64(v.size))
    return out


def quantize(v, q_scale):
    v = _c(v, np.float32)
    out = np.empty(v.shape, np.int8)
    lib().orc_quantize(_p(v), C.c_float(q_scale), _p(out), C.c_int64(v.size))
    return out


def interleave(x_tc):
    """[T, C] int8 -> [C/32][T][32] bytes."""
    x_tc = _c(x_tc, np.int8)
    t, c = x_tc.shape
    out = np.empty(t * c, np.int8)
    lib().orc_interleave(_p(x_tc), _p(out), C.c_int64(t), C.c_int(c))
    return out


def deinterleave(x_il, t, c):
    x_il = _c(x_il, np.int8)
    out = np.empty((t, c), np.int8)
    lib().orc_deinterleave(_p(x_il), _p(out), C.c_int64(t), C.c_int(c))
    return out


# ------------------------------------------------------------------------------------------------
# SkipLayerNorm
# ------------------------------------------------------------------------------------------------

def skipln(x, skip, beta, gamma, bias=None):
    """computeSkipLayerNorm<T,hasBias>; T from x.dtype (float32 / float16); x is [rows, ld]."""
    rows, ld = x.shape
    if x.dtype == np.float32:
        args = [_c(a, np.float32) for a in (x, skip, beta, gamma)]
        b = _c(bias, np.float32)
        out = np.empty((rows, ld), np.float32)
        lib().orc_skipln_f32(C.c_int(ld), C.c_int64(rows), _p(args[0]), _p(args[1]), _p(args[2]), _p(args[3]),
                             _p(b), _p(out))
        return out
    assert x.dtype == np.float16
    args = [_c(a, np.float16) for a in (x, skip, beta, gamma)]
    b = _c(bias, np.float16)
    out = np.empty((rows, ld), np.float16)
    lib().orc_skipln_f16(C.c_int(ld), C.c_int64(rows), _p(args[0]), _p(args[1]), _p(args[2]), _p(args[3]), _p(b),
                         _p(out))
    return out


def skipln_dqq(x, skip, beta, gamma, bias, dq_in, dq_skip, q_scale):
    """computeSkipLayerNormDQQ<hasBias>: int8 [rows, ld] in, int8 out.  Returns (status, out)."""
    rows, ld = x.shape
    x, skip = _c(x, np.int8), _c(skip, np.int8)
    beta, gamma, bias = _c(beta, np.float16), _c(gamma, np.float16), _c(bias, np.float16)
    out = np.zeros((rows, ld), np.int8)
    st = lib().orc_skipln_dqq(C.c_int(ld), C.c_int64(rows), _p(x), _p(skip), _p(beta), _p(gamma), _p(bias), _p(out),
                              C.c_float(dq_in), C.c_float(dq_skip), C.c_float(q_scale))
    return st, out


def skipln_interleaved(variant, x_il, skip_il, beta, gamma, ld, total, dq_in, dq_skip, q_scale, q_skip_scale=0.0,
                       force=-1):
    """launch_{small,large}_{hface,mtron}.  variant 0 HFace, 1 MTron.  Flat [ld/32][total][32] int8 arrays.
    Returns (status, out, preln-or-None)."""
    x_il, skip_il = _c(x_il, np.int8), _c(skip_il, np.int8)
    beta, gamma = _c(beta, np.float16), _c(gamma, np.float16)
    out = np.zeros(ld * total, np.int8)
    pre = np.zeros(ld * total, np.int8) if variant == 1 else None
    st = lib().orc_skipln_interleaved(C.c_int(variant), C.c_int(force), C.c_int(ld), C.c_int64(total), _p(x_il),
                                      _p(skip_il), _p(beta), _p(gamma), _p(out), _p(pre), C.c_float(dq_in),
                                      C.c_float(dq_skip), C.c_float(q_scale), C.c_float(q_skip_scale))
    return st, out, pre


# ------------------------------------------------------------------------------------------------
# EmbLayerNorm, maskIdx, packed mask
# ------------------------------------------------------------------------------------------------

def embln(mode, ids, segs, cu, beta, gamma, word, pos, tok, S, B, out_rows=None):
    """mode 0 fixed ([S,B] ids), 1 HFace, 2 MTron (packed ids + cu_seqlens).
    Tables' dtype selects T.  Returns (out, skip-or-None, valid[rows] uint8)."""
    is_half = int(word.dtype == np.float16)
    ld = word.shape[1]
    ids, segs = _c(ids, np.int32).ravel(), _c(segs, np.int32).ravel()
    cu = _c(cu, np.int32)
    rows = ids.size if out_rows is None else out_rows
    w32, p32, t32 = (_c(a.astype(np.float32), np.float32) for a in (word, pos, tok))
    beta, gamma = _c(beta, np.float32), _c(gamma, np.float32)
    out = np.zeros((rows, ld), np.float32)
    skip = np.zeros((rows, ld), np.float32) if mode == 2 else None
    valid = np.zeros(rows, np.uint8)
    lib().orc_embln(C.c_int(mode), C.c_int(is_half), C.c_int(ld), C.c_int(B), C.c_int(S), _p(ids), _p(segs), _p(cu),
                    _p(beta), _p(gamma), _p(w32), _p(p32), _p(t32), C.c_int32(word.shape[0]),
                    C.c_int32(tok.shape[0]), _p(out), _p(skip), _p(valid))
    dt = word.dtype
    return out.astype(dt), (None if skip is None else skip.astype(dt)), valid


def mask_idx(mask_sb):
    mask_sb = _c(mask_sb, np.int32)
    s, b = mask_sb.shape
    out = np.empty(b, np.int32)
    lib().orc_mask_idx(C.c_int(s), C.c_int(b), _p(mask_sb), _p(out))
    return out


def packed_mask_geometry(S, warps_m, warps_n, warps_k=1):
    xm = (S + 16 * warps_m - 1) // (16 * warps_m)
    xn = (S + 16 * warps_n - 1) // (16 * warps_n)
    return xm, xn, warps_m * warps_n * warps_k * 32


def convert_mask(mask_sb, warps_m, warps_n, warps_k=1):
    """convertMask / fillSBSMaskKernel.  Returns (packed [B, xmmas_m*threads] uint32, overreads)."""
    mask_sb = _c(mask_sb, np.int32)
    s, b = mask_sb.shape
    xm, _, thr = packed_mask_geometry(s, warps_m, warps_n, warps_k)
    out = np.zeros((b, xm * thr), np.uint32)
    over = lib().orc_convert_mask(C.c_uint32(s), C.c_uint32(b), C.c_uint32(warps_m), C.c_uint32(warps_n),
                                  C.c_uint32(warps_k), _p(mask_sb), _p(out))
    return out, int(over)


# ------------------------------------------------------------------------------------------------
# softmax and attention
# ------------------------------------------------------------------------------------------------

def scaled_softmax(x, rsqrt_head_size, mask_idx_=None):
    """x: [B, N, S, S] (float32 or float16)."""
    is_half = int(x.dtype == np.float16)
    b, n, s, _ = x.shape
    xin = _c(x.astype(np.float32), np.float32)
    out = np.empty_like(xin)
    mi = _c(mask_idx_, np.int32)
    lib().orc_scaled_softmax(C.c_int(is_half), C.c_int(s), C.c_int(b), C.c_int(n), C.c_float(rsqrt_head_size), _p(mi),
                             _p(xin), _p(out))
    return out.astype(x.dtype)


def _geom_fixed(S, B, N, d, lens_k, all_queries=True):
    g = MhaGeom(B, N, d, 3 * B * N * d, B * N * d, 3 * d, d)
    seqs = (MhaSeq * B)()
    for b in range(B):
        seqs[b] = MhaSeq(b * 3 * N * d, b * N * d, S if all_queries else int(lens_k[b]), int(lens_k[b]))
    return g, seqs


def _geom_packed(cu, N, d):
    B = len(cu) - 1
    g = MhaGeom(B, N, d, 3 * N * d, N * d, 3 * d, d)
    seqs = (MhaSeq * B)()
    for b in range(B):
        ln = int(cu[b + 1] - cu[b])
        seqs[b] = MhaSeq(int(cu[b]) * 3 * N * d, int(cu[b]) * N * d, ln, ln)
    return g, seqs


def mha_unfused_fixed(qkv, S, B, N, d, mask_idx_=None):
    """UnfusedMHARunner on [S,B,N,3,d]; returns [S,B,N,d] in qkv.dtype."""
    is_half = int(qkv.dtype == np.float16)
    lens = np.full(B, S, np.int32) if mask_idx_ is None else np.minimum(np.asarray(mask_idx_), S)
    g, seqs = _geom_fixed(S, B, N, d, lens)
    x = _c(qkv.astype(np.float32).ravel(), np.float32)
    out = np.zeros(S * B * N * d, np.float32)
    lib().orc_mha_unfused(C.c_int(is_half), C.byref(g), seqs, _p(x), _p(out))
    return out.reshape(S, B, N * d).astype(qkv.dtype)


def mha_fused_f16_fixed(qkv, S, B, N, d, lens_k):
    g, seqs = _geom_fixed(S, B, N, d, lens_k)
    x = _c(qkv.astype(np.float32).ravel(), np.float32)
    out = np.zeros(S * B * N * d, np.float32)
    lib().orc_mha_fused_f16(C.byref(g), seqs, _p(x), _p(out))
    return out.reshape(S, B, N * d).astype(np.float16)


def mha_fused_f16_packed(qkv, cu, N, d):
    """qkv [T, 3*N*d] float16 ([T,N,3,d]); returns [T, N*d] float16."""
    g, seqs = _geom_packed(cu, N, d)
    T = qkv.shape[0]
    x = _c(qkv.astype(np.float32).ravel(), np.float32)
    out = np.zeros(T * N * d, np.float32)
    lib().orc_mha_fused_f16(C.byref(g), seqs, _p(x), _p(out))
    return out.reshape(T, N * d).astype(np.float16)


def _run_i8(g, seqs, qkv, out_elems, B, N, scales, want_ints, maxq, maxk):
    x = _c(qkv.ravel(), np.int8)
    out = np.zeros(out_elems, np.int8)
    a1 = p8 = a2 = None
    if want_ints:
        a1 = np.zeros((B, N, maxq, maxk), np.int32)
        p8 = np.zeros((B, N, maxq, maxk), np.int8)
        a2 = np.zeros(out_elems, np.int32)
    lib().orc_mha_fused_i8(C.byref(g), seqs, _p(x), _p(out), C.c_float(scales[0]), C.c_float(scales[1]),
                           C.c_float(scales[2]), C.c_int32(maxq), C.c_int32(maxk), _p(a1), _p(p8), _p(a2))
    return out, a1, p8, a2


def mha_fused_i8_packed(qkv, cu, N, d, scale_bmm1, scale_softmax, scale_bmm2, want_ints=False):
    """qkv [T, 3*N*d] int8 ([T,N,3,d]).  Returns out [T, N*d] int8 (+ acc1, p8, acc2 if want_ints)."""
    g, seqs = _geom_packed(cu, N, d)
    T = qkv.shape[0]
    B = len(cu) - 1
    maxl = int(np.max(np.diff(cu))) if B else 0
    out, a1, p8, a2 = _run_i8(g, seqs, qkv, T * N * d, B, N, (scale_bmm1, scale_softmax, scale_bmm2), want_ints, maxl,
                              maxl)
    out = out.reshape(T, N * d)
    if want_ints:
        return out, a1, p8, a2.reshape(T, N * d)
    return out


def mha_fused_i8_fixed(qkv, S, B, N, d, lens_k, scale_bmm1, scale_softmax, scale_bmm2, want_ints=False):
    """qkv [S,B,N,3,d] int8 with a prefix key mask of lens_k[b]; all S query rows are computed."""
    g, seqs = _geom_fixed(S, B, N, d, lens_k)
    out, a1, p8, a2 = _run_i8(g, seqs, qkv, S * B * N * d, B, N, (scale_bmm1, scale_softmax, scale_bmm2), want_ints, S,
                              S)
    out = out.reshape(S, B, N * d)
    if want_ints:
        return out, a1, p8, a2.reshape(S, B, N * d)
    return out


def zero_padding_2d(src_bytes, spitch, dpitch, height):
    src = _c(src_bytes, np.uint8)
    dst = np.empty(height * dpitch, np.uint8)
    lib().orc_zero_padding_2d(_p(src), _p(dst), C.c_int64(height), C.c_int(spitch), C.c_int(dpitch), C.c_int(1))
    return dst


# ------------------------------------------------------------------------------------------------
# INT8 linear layer between the plugins
# ------------------------------------------------------------------------------------------------

LINEAR_AFFINE, LINEAR_GELU, LINEAR_RAW_INT32, LINEAR_AFFINE_FP16 = 0, 1, 2, 3


def int8_linear(a, w, alpha=None, beta=None, epilogue=LINEAR_AFFINE, out_scale=1.0, a_interleaved=False,
                out_interleaved=False):
    """a: int8 [T,K] (or [K/32,T,32] if a_interleaved); w: int8 [N,K]; alpha, beta: float32 [N].

    Returns int8 [T,N] (or [N/32,T,32] if out_interleaved), int32 [T,N] for LINEAR_RAW_INT32,
    float16 [T,N] for LINEAR_AFFINE_FP16.
    """
    a = _c(a, np.int8)
    w = _c(w, np.int8)
    N, K = w.shape
    T = a.shape[1] if a_interleaved else a.shape[0]
    alpha = _c(alpha, np.float32)
    beta = _c(beta, np.float32)
    if epilogue == LINEAR_RAW_INT32:
        out = np.zeros((T, N), np.int32)
    elif epilogue == LINEAR_AFFINE_FP16:
        out = np.zeros((T, N), np.float16)
    else:
        out = np.zeros((N // 32, T, 32) if out_interleaved else (T, N), np.int8)
    rc = lib().orc_int8_linear(C.c_int64(T), C.c_int(K), C.c_int(N), _p(a), C.c_int(int(a_interleaved)), _p(w),
                               _p(alpha), _p(beta), C.c_int(epilogue), C.c_float(out_scale),
                               C.c_int(int(out_interleaved)), _p(out))
    if rc != 0:
        raise ValueError("orc_int8_linear rejected its arguments")
    return out


def quantize_f16_interleave(x, scale):
    """x: float16 [T,C]; returns int8 [C/32,T,32] = clamp(rne(x / scale), -128, 127)."""
    x = _c(x, np.float16)
    T, Cc = x.shape
    out = np.zeros((Cc // 32, T, 32), np.int8)
    lib().orc_quantize_f16_interleave(_p(x), C.c_float(scale), _p(out), C.c_int64(T), C.c_int(Cc))
    return out


def dequantize_deinterleave_f16(q, scale):
    """q: int8 [C/32,T,32]; returns float16 [T,C] = binary16(q * scale)."""
    q = _c(q, np.int8)
    nslab, T, _ = q.shape
    out = np.zeros((T, nslab * 32), np.float16)
    lib().orc_dequantize_deinterleave_f16(_p(q), C.c_float(scale), _p(out), C.c_int64(T), C.c_int(nslab * 32))
    return out


def fp16_linear(a, w, alpha, beta, gelu=False):
    """a: float16 [T,K]; w: float16 [N,K]; alpha, beta: float32 [N].  Returns float16 [T,N]."""
    a, w = _c(a, np.float16), _c(w, np.float16)
    T, K = a.shape
    N = w.shape[0]
    out = np.zeros((T, N), np.float16)
    rc = lib().orc_fp16_linear(C.c_int64(T), C.c_int(K), C.c_int(N), _p(a), _p(w), _p(_c(alpha, np.float32)),
                               _p(_c(beta, np.float32)), C.c_int(int(gelu)), _p(out))
    if rc != 0:
        raise ValueError("orc_fp16_linear rejected its arguments")
    return out
