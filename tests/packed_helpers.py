"""Builds weights in burn's packed block-32 layout (pack.rs:940-985) the way the reference's quantizer does
for its tests (symmetric per-block scale = max|w| / qmax, codes rounded to nearest), and an independent f64
evaluation of x . dequantize(w) to judge the packed GEMV against, as nn/packed_gemv.rs:1593-1624 does."""
import numpy as np


def quantize_block32(w: np.ndarray, bits: int):
    """w [K, N] f32 -> (codes int8 [K, N], scales f32 [K, N/32]); blocks run along N."""
    k, n = w.shape
    qmax = (1 << (bits - 1)) - 1
    blocks = w.reshape(k, n // 32, 32)
    scales = (np.abs(blocks).max(axis=2) / qmax).astype(np.float32)
    safe = np.where(scales > 0, scales, 1).astype(np.float32)
    codes = np.clip(np.rint(blocks / safe[:, :, None]), -qmax - 1, qmax).astype(np.int8).reshape(k, n)
    return codes, scales


def pack_words(codes: np.ndarray, bits: int) -> np.ndarray:
    """Element j of a word at bits j*bits, two's complement, words running along N."""
    k, n = codes.shape
    per = 32 // bits
    fields = (codes.astype(np.int64) & ((1 << bits) - 1)).reshape(k, n // per, per)
    shifts = (np.arange(per, dtype=np.int64) * bits)[None, None, :]
    return (fields << shifts).sum(axis=2).astype(np.uint32)


def reference_f64(codes, scales, x):
    w = codes.astype(np.float64) * np.repeat(scales.astype(np.float64), 32, axis=1)
    return x.astype(np.float64) @ w
