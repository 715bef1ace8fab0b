"""Seeded synthetic inputs for the sparse MoE block: weights, GGUF-packed banks, activations.

The generator is the reference's test generator, SplitMix64 with a 24-bit uniform
(models/qwen4exp/experts.rs:1162-1189), and the synthetic Q4_K / Q8_0 / Q5_1 / Q5_K blocks
follow its ``synth_blocks`` draw order and scale ranges (experts.rs:1209-1237), so a bank
built here from a seed is byte-identical to the one the reference's tests build from the
same seed.  SplitMix64's state after n draws is ``seed + n*GAMMA``, so every stream is
generated in one vectorised numpy pass.

Normals are Box-Muller over two 53-bit uniforms of the same stream, the construction in
nn/refarith.rs:108-125.
"""
from __future__ import annotations

import numpy as np

GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)

# ggml type ids (gguf.rs:298-324)
F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 2, 3, 6, 7, 8, 12, 13, 14, 30

BLOCK_SIZE = {F32: 1, F16: 1, BF16: 1, Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256}
BLOCK_BYTES = {F32: 4, F16: 2, BF16: 2, Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210}

# f16 header fields of a synthetic block: (byte offset, low, high).  Q8_0, Q5_1, Q4_K and Q5_K are
# the reference's ranges (experts.rs:1209-1237); the others are this package's own, chosen to give
# weights of the same magnitude.
SCALE_FIELDS = {
    Q8_0: [(0, 0.002, 0.02)],
    Q5_1: [(0, 0.005, 0.05), (2, -0.4, 0.0)],
    Q4_K: [(0, 0.0005, 0.003), (2, 0.0005, 0.003)],
    Q5_K: [(0, 0.0003, 0.002), (2, 0.0003, 0.002)],
    Q4_0: [(0, 0.005, 0.05)],
    Q4_1: [(0, 0.005, 0.05), (2, -0.4, 0.0)],
    Q5_0: [(0, 0.003, 0.03)],
    Q6_K: [(208, 0.00002, 0.0002)],
}


def row_bytes(dtype: int, in_dim: int) -> int:
    bs = BLOCK_SIZE[dtype]
    if in_dim % bs:
        raise ValueError(f"row width {in_dim} is not whole blocks of {bs}")
    return in_dim // bs * BLOCK_BYTES[dtype]


class SplitMix64:
    """Counter-based SplitMix64: draw i (0-based) mixes ``seed + (i+1)*GAMMA``."""

    def __init__(self, seed: int):
        self.state = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next_u64(self, n: int) -> np.ndarray:
        with np.errstate(over="ignore"):
            idx = np.arange(1, n + 1, dtype=np.uint64)
            z = self.state + idx * GAMMA
            self.state = self.state + np.uint64(n) * GAMMA
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            return z ^ (z >> np.uint64(31))

    @staticmethod
    def _to_uniform(u64: np.ndarray, lo: float, hi: float) -> np.ndarray:
        # 24 random bits / 2^24, then (hi-lo)*u and lo+span as two f32 roundings.
        u = (u64 >> np.uint64(40)).astype(np.float32) / np.float32(16777216.0)
        span = (np.float32(hi) - np.float32(lo)) * u
        return (np.float32(lo) + span).astype(np.float32)

    @staticmethod
    def _to_byte(u64: np.ndarray) -> np.ndarray:
        return (u64 >> np.uint64(56)).astype(np.uint8)

    def uniform(self, lo: float, hi: float, n: int) -> np.ndarray:
        return self._to_uniform(self.next_u64(n), lo, hi)

    def bytes(self, n: int) -> np.ndarray:
        return self._to_byte(self.next_u64(n))

    def uniform_vec(self, n: int) -> np.ndarray:
        """experts.rs:1186-1188: n values uniform in [-1, 1)."""
        return self.uniform(-1.0, 1.0, n)

    def normal(self, n: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
        """Box-Muller over pairs of 53-bit uniforms (nn/refarith.rs:110-120), narrowed to f32."""
        u = self.next_u64(2 * n)
        u = ((u >> np.uint64(11)).astype(np.float64) + 0.5) / float(1 << 53)
        g = np.sqrt(-2.0 * np.log(u[0::2])) * np.cos(2.0 * np.pi * u[1::2])
        return (mean + std * g).astype(np.float32)


def f16_bits(v: np.ndarray) -> np.ndarray:
    """f32 -> IEEE half, round to nearest even, as little-endian u16."""
    return np.asarray(v, dtype=np.float32).astype(np.float16).view(np.uint16)


def synth_blocks(dtype: int, blocks: int, rng: SplitMix64) -> np.ndarray:
    """``blocks`` sane blocks of ``dtype``: finite, modest f16 scales and random quant bits
    (experts.rs:1209-1237).  Draws are consumed block by block in the reference's order:
    the scale uniform(s) first, then one draw per payload byte."""
    if dtype not in SCALE_FIELDS:
        raise ValueError(f"no synthetic blocks for ggml type {dtype}")
    fields = SCALE_FIELDS[dtype]
    bb = BLOCK_BYTES[dtype]
    heads = len(fields)
    head_bytes = {o + i for o, _, _ in fields for i in (0, 1)}
    body = np.array([i for i in range(bb) if i not in head_bytes])
    per = heads + len(body)
    out = np.empty((blocks, bb), dtype=np.uint8)
    # Generate in slabs so a multi-hundred-MB bank never holds 8x its size in u64 draws.
    slab = max(1, (1 << 22) // per)
    for b0 in range(0, blocks, slab):
        nb = min(slab, blocks - b0)
        draws = rng.next_u64(nb * per).reshape(nb, per)
        for h, (off, lo, hi) in enumerate(fields):
            bits = f16_bits(SplitMix64._to_uniform(draws[:, h], lo, hi))
            out[b0:b0 + nb, off] = (bits & 0xFF).astype(np.uint8)
            out[b0:b0 + nb, off + 1] = (bits >> 8).astype(np.uint8)
        out[b0:b0 + nb, body] = SplitMix64._to_byte(draws[:, heads:])
    return out.reshape(-1)


def synth_bank(dtype: int, ne, rng: SplitMix64) -> np.ndarray:
    """A whole bank ``ne = [in_dim, out_dim, n_experts]`` (experts.rs:1239-1242): bytes are
    expert-major, then row-major, each row whole blocks."""
    in_dim, out_dim, n_experts = ne
    if dtype in (F32, F16, BF16):
        raise ValueError("use dense_bank for float types")
    blocks = in_dim // BLOCK_SIZE[dtype] * out_dim * n_experts
    return synth_blocks(dtype, blocks, rng)


def dense_bank(dtype: int, ne, rng: SplitMix64, std: float = 0.02) -> np.ndarray:
    """A float bank ``[n_experts, out_dim, in_dim]`` ~ N(0, std) stored as F32 / F16 / BF16
    bytes in GGUF order."""
    in_dim, out_dim, n_experts = ne
    w = rng.normal(in_dim * out_dim * n_experts, 0.0, std)
    return encode_float(w, dtype)


def encode_float(w: np.ndarray, dtype: int) -> np.ndarray:
    w = np.asarray(w, dtype=np.float32).reshape(-1)
    if dtype == F32:
        return w.view(np.uint8).copy()
    if dtype == F16:
        return w.astype(np.float16).view(np.uint8).copy()
    if dtype == BF16:
        b = w.view(np.uint32)
        # round to nearest even on the dropped 16 bits
        r = ((b >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
        return ((b + r) >> np.uint32(16)).astype(np.uint16).view(np.uint8).copy()
    raise ValueError(f"not a float type: {dtype}")


def random_bank_fast(dtype: int, ne, seed: int) -> np.ndarray:
    """Benchmark-sized banks: same block structure and scale ranges as ``synth_blocks`` but
    drawn from numpy's PCG64 (hundreds of MB per second).  Not byte-compatible with the
    reference's test generator; used where only the shape and statistics matter."""
    in_dim, out_dim, n_experts = ne
    g = np.random.Generator(np.random.PCG64(seed))
    blocks = in_dim // BLOCK_SIZE[dtype] * out_dim * n_experts
    bb = BLOCK_BYTES[dtype]
    out = g.integers(0, 256, size=(blocks, bb), dtype=np.uint8)
    if dtype not in SCALE_FIELDS:
        raise ValueError(f"no fast bank for ggml type {dtype}")
    for off, lo, hi in SCALE_FIELDS[dtype]:
        bits = f16_bits(g.uniform(lo, hi, size=blocks).astype(np.float32))
        out[:, off] = (bits & 0xFF).astype(np.uint8)
        out[:, off + 1] = (bits >> 8).astype(np.uint8)
    return out.reshape(-1)


# --- burn's packed block-32 layout (pack.rs:940-985), for the packed-GEMV op -------------------

def quantize_block32(w: np.ndarray, bits: int):
    """w [K, N] f32 -> (codes int8 [K, N], scales f32 [K, N/32]): symmetric per-block scale max|w| / qmax, codes
    rounded to nearest; blocks run along N."""
    k, n = w.shape
    qmax = (1 << (bits - 1)) - 1
    blocks = w.reshape(k, n // 32, 32)
    scales = (np.abs(blocks).max(axis=2) / qmax).astype(np.float32)
    safe = np.where(scales > 0, scales, 1).astype(np.float32)
    codes = np.clip(np.rint(blocks / safe[:, :, None]), -qmax - 1, qmax).astype(np.int8).reshape(k, n)
    return codes, scales


def pack_words(codes: np.ndarray, bits: int) -> np.ndarray:
    """int8 codes [K, N] -> u32 words [K, N*bits/32]: element j of a word at bits j*bits, two's complement,
    words running along N."""
    k, n = codes.shape
    per = 32 // bits
    fields = (codes.astype(np.int64) & ((1 << bits) - 1)).reshape(k, n // per, per)
    shifts = (np.arange(per, dtype=np.int64) * bits)[None, None, :]
    return (fields << shifts).sum(axis=2).astype(np.uint32)
