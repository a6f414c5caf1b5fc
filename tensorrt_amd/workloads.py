"""Seeded synthetic inputs of the benchmark configurations (shapes and distributions of the
BERT-large INT8 layer: 16 heads x 64, hidden 1024, variable sequence lengths).

Pure numpy; used by bench.py, the smoke check and tests.  Nothing here touches the GPU.
"""
from __future__ import annotations

import dataclasses

import numpy as np

HEAD = 64


def interleave32(x_tc: np.ndarray) -> np.ndarray:
    """[T, C] int8 -> bytes of TensorFormat::kCHW32 for a [1,C,T,1] tensor, i.e. [C/32][T][32]."""
    t, c = x_tc.shape
    return np.ascontiguousarray(x_tc.reshape(t, c // 32, 32).transpose(1, 0, 2)).reshape(-1)


def deinterleave32(x_il: np.ndarray, t: int, c: int) -> np.ndarray:
    return np.ascontiguousarray(x_il.reshape(c // 32, t, 32).transpose(1, 0, 2)).reshape(t, c)


def quantize_amax(x: np.ndarray):
    """q = clip(rne(x * 127/amax), -127, 127), scale = amax/127 (per tensor)."""
    amax = float(np.abs(x).max())
    scale = np.float32(amax / 127.0)
    q = np.clip(np.rint(x * (127.0 / amax)), -127, 127).astype(np.int8)
    return q, scale


@dataclasses.dataclass
class Int8Layer:
    """One BERT-large INT8 layer's plugin inputs (packed tokens, 32-interleaved layouts)."""
    B: int
    S: int
    N: int
    lens: np.ndarray          # [B]
    cu: np.ndarray            # [B+1] int32
    qkv_tc: np.ndarray        # [T, 3*N*64] int8, channel order [3][N][64] (the v6 plugin's)
    s_qkv: np.float32
    skip_tc: np.ndarray       # [T, N*64] int8 residual stream
    s_skip: np.float32
    gamma: np.ndarray         # [E] float16
    beta: np.ndarray          # [E] float16
    dq_probs: np.float32

    @property
    def T(self) -> int:
        return int(self.cu[-1])

    @property
    def E(self) -> int:
        return self.N * HEAD

    def mha_ops(self) -> float:
        """Algorithmic integer operations of the two attention GEMMs: sum_b 4 * L_b^2 * d * N."""
        return float(4.0 * HEAD * self.N * np.sum(self.lens.astype(np.float64) ** 2))

    def mha_bytes(self) -> float:
        return float(self.T) * 4 * self.E

    def skipln_bytes(self, n_out: int = 1) -> float:
        """rows * E * (2 + n_out) bytes of INT8 tensors + gamma/beta."""
        return float(self.T) * self.E * (2 + n_out) + 2 * 2 * self.E


def int8_layer(B: int, S: int, N: int = 16, min_len: int | None = None, seed: int = 1) -> Int8Layer:
    r = np.random.default_rng(seed)
    lo = S // 2 if min_len is None else min_len
    lens = r.integers(lo, S + 1, B)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    E = N * HEAD
    qkv, s_qkv = quantize_amax(r.standard_normal((T, 3 * E), dtype=np.float32))
    skip, s_skip = quantize_amax(r.standard_normal((T, E), dtype=np.float32))
    gamma = r.uniform(0.5, 1.5, E).astype(np.float16)
    beta = (r.standard_normal(E) * 0.1).astype(np.float16)
    return Int8Layer(B, S, N, lens, cu, qkv, s_qkv, skip, s_skip, gamma, beta, np.float32(1.0 / 127.0))
