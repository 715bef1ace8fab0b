"""Pins the oracle's GGUF codec (oracle/moe_oracle.c) against
  * the reference's own known-answer blocks (gguf.rs:2379-2447, 2654-2662),
  * numpy's IEEE half conversion over all 65 536 bit patterns,
  * an independent vectorised numpy dequantizer written from the block layouts.
"""
import numpy as np
import pytest

from mummu_amd import synth
from oracle import binding as orc


def f16b(v):
    return np.array([v], dtype=np.float16).view(np.uint8)


def test_float_widths_dequantize_exactly():
    # gguf.rs:2379-2393
    assert orc.dequantize(orc.F32, np.array([1.5], dtype=np.float32)).tolist() == [1.5]
    assert orc.dequantize(orc.F16, f16b(-0.25)).tolist() == [-0.25]
    bf16 = np.array([np.array([2.0], dtype=np.float32).view(np.uint32)[0] >> 16], dtype=np.uint16)
    assert orc.dequantize(orc.BF16, bf16).tolist() == [2.0]


def test_q8_0_block_matches_hand_computation():
    # gguf.rs:2395-2405
    block = np.concatenate([f16b(0.5), (np.arange(32, dtype=np.int8) - 16).view(np.uint8)])
    out = orc.dequantize(orc.Q8_0, block)
    assert out.size == 32
    assert out[0] == 0.5 * -16.0 and out[16] == 0.0 and out[31] == 0.5 * 15.0


def test_q4_k_superblock_matches_hand_computation():
    # gguf.rs:2407-2429
    block = np.zeros(144, dtype=np.uint8)
    block[0:2] = f16b(1.0)
    block[2:4] = f16b(0.5)
    block[4], block[5], block[8], block[12] = 2, 3, 1, 0x21
    block[16] = 0x51
    block[16 + 64] = 0x04
    out = orc.dequantize(orc.Q4_K, block)
    assert out.size == 256
    assert out[0] == 1.5 and out[32] == 15.0 and out[128] == 3.0 and out[1] == -0.5


def test_q6_k_superblock_matches_hand_computation():
    # gguf.rs:2431-2447
    block = np.zeros(210, dtype=np.uint8)
    block[0] = 0x0F
    block[128] = 0b11
    block[192] = 2
    block[194] = 1
    block[208:210] = f16b(1.0)
    out = orc.dequantize(orc.Q6_K, block)
    assert out[0] == 62.0 and out[32] == -32.0 and out[64] == 0.0


def test_partial_blocks_and_unknown_types_are_refused():
    # gguf.rs:2654-2662
    with pytest.raises(orc.OracleError):
        orc.dequantize(orc.Q8_0, np.zeros(33, dtype=np.uint8))
    with pytest.raises(orc.OracleError):
        orc.dequantize(orc.Q8_0, np.zeros(0, dtype=np.uint8))
    with pytest.raises(orc.OracleError):
        orc.dequantize(15, np.zeros(292, dtype=np.uint8))  # Q8_K is an activation format


def test_f16_to_f32_is_exact_for_every_bit_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.dequantize(orc.F16, bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


# --- an independent numpy statement of the two hot formats, from the layouts -----------

def np_dequant_q8_0(raw):
    b = raw.reshape(-1, 34)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)
    return (d * b[:, 2:].view(np.int8).astype(np.float32)).reshape(-1)


def np_dequant_q4_k(raw):
    b = raw.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)
    s = b[:, 4:16].astype(np.uint8)
    sc = np.empty((b.shape[0], 8), dtype=np.uint8)
    mn = np.empty((b.shape[0], 8), dtype=np.uint8)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0x0F) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    qs = b[:, 16:].reshape(-1, 4, 32)
    q = np.concatenate([qs & 0x0F, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)
    ds = (d * sc.astype(np.float32))[:, :, None]
    mins = (dmin * mn.astype(np.float32))[:, :, None]
    return ((ds * q).astype(np.float32) - mins).astype(np.float32).reshape(-1)


def _f16col(b, off):
    return b[:, off:off + 2].copy().view(np.float16).astype(np.float32)


def _k4_scales(s):
    """The 6-bit (scale, min) pairs of a Q4_K / Q5_K super-block from its 12 packed bytes."""
    sc = np.empty((s.shape[0], 8), dtype=np.float32)
    mn = np.empty((s.shape[0], 8), dtype=np.float32)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0x0F) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    return sc, mn


def np_dequant_q5_k(raw):
    # 176 B: d, dmin, 12 B scales, 32 B fifth bits (bit 2c / 2c+1 of byte l: chunk c, low / high nibble), 128 B nibbles
    b = raw.reshape(-1, 176)
    d, dmin = _f16col(b, 0), _f16col(b, 2)
    sc, mn = _k4_scales(b[:, 4:16])
    qh = b[:, 16:48]
    qs = b[:, 48:].reshape(-1, 4, 32)
    q = np.empty((b.shape[0], 8, 32), dtype=np.float32)
    for c in range(4):
        q[:, 2 * c] = (qs[:, c] & 0x0F) + 16 * ((qh >> (2 * c)) & 1)
        q[:, 2 * c + 1] = (qs[:, c] >> 4) + 16 * ((qh >> (2 * c + 1)) & 1)
    ds = (d * sc)[:, :, None]
    mins = (dmin * mn)[:, :, None]
    return ((ds * q).astype(np.float32) - mins).astype(np.float32).reshape(-1)


def np_dequant_q6_k(raw):
    # 210 B: 128 B low nibbles, 64 B two-bit tops, 16 signed scales (one per 16 elements), d
    b = raw.reshape(-1, 210)
    ql = b[:, 0:128].reshape(-1, 2, 64)
    qh = b[:, 128:192].reshape(-1, 2, 32)
    sc = b[:, 192:208].view(np.int8).astype(np.float32).reshape(-1, 2, 8)
    d = _f16col(b, 208)
    out = np.empty((b.shape[0], 2, 4, 32), dtype=np.float32)
    for g in range(4):  # elements 32g .. 32g+31 of a 128-element half
        lo = ql[:, :, (g & 1) * 32:(g & 1) * 32 + 32]
        lo = (lo >> 4) if g >= 2 else (lo & 0x0F)
        q = (lo | (((qh >> (2 * g)) & 3) << 4)).astype(np.int16) - 32
        s = np.repeat(sc[:, :, 2 * g:2 * g + 2], 16, axis=2)  # scale index l / 16 + 2g
        out[:, :, g] = ((d[:, :, None] * s).astype(np.float32) * q.astype(np.float32)).astype(np.float32)
    return out.reshape(-1)


def _legacy_codes(b, qs_off, qh_off=None):
    """Elements 0..15 are the low nibbles, 16..31 the high ones; bit j of qh tops element j."""
    qs = b[:, qs_off:qs_off + 16]
    q = np.concatenate([qs & 0x0F, qs >> 4], axis=1).astype(np.uint32)
    if qh_off is not None:
        qh = b[:, qh_off:qh_off + 4].copy().view(np.uint32)
        q |= ((qh >> np.arange(32, dtype=np.uint32)[None, :]) & 1) << 4
    return q.astype(np.float32)


def np_dequant_legacy(dtype, raw):
    b = raw.reshape(-1, synth.BLOCK_BYTES[dtype])
    d = _f16col(b, 0)
    if dtype == synth.Q4_0:
        return (d * (_legacy_codes(b, 2) - 8.0)).astype(np.float32).reshape(-1)
    if dtype == synth.Q5_0:
        return (d * (_legacy_codes(b, 6, 2) - 16.0)).astype(np.float32).reshape(-1)
    m = _f16col(b, 2)
    q = _legacy_codes(b, 4) if dtype == synth.Q4_1 else _legacy_codes(b, 8, 4)
    return ((d * q).astype(np.float32) + m).astype(np.float32).reshape(-1)


NP_DECODERS = {
    synth.Q5_K: np_dequant_q5_k, synth.Q6_K: np_dequant_q6_k,
    synth.Q4_0: lambda r: np_dequant_legacy(synth.Q4_0, r), synth.Q4_1: lambda r: np_dequant_legacy(synth.Q4_1, r),
    synth.Q5_0: lambda r: np_dequant_legacy(synth.Q5_0, r), synth.Q5_1: lambda r: np_dequant_legacy(synth.Q5_1, r),
}


@pytest.mark.parametrize("dtype", sorted(NP_DECODERS), ids=lambda t: f"type{t}")
def test_the_other_block_types_match_an_independent_numpy_dequantizer_bit_for_bit(dtype):
    # sane synthetic blocks, then raw random bytes (any f16 pattern as a scale: finite outputs compared as bits)
    raw = synth.synth_blocks(dtype, 200, synth.SplitMix64(11 + dtype))
    assert np.array_equal(orc.dequantize(dtype, raw).view(np.uint32), NP_DECODERS[dtype](raw).view(np.uint32))
    g = np.random.Generator(np.random.PCG64(dtype))
    raw = g.integers(0, 256, size=synth.BLOCK_BYTES[dtype] * 64, dtype=np.uint8)
    with np.errstate(all="ignore"):
        a, b = orc.dequantize(dtype, raw), NP_DECODERS[dtype](raw)
    fin = np.isfinite(b)
    assert np.array_equal(a[fin].view(np.uint32), b[fin].view(np.uint32))
    assert np.array_equal(np.isnan(a), np.isnan(b))


def test_the_reference_known_answers_hold_for_the_numpy_decoders_too():
    # gguf.rs:2549-2592, 2638-2652, 2431-2447: the same hand-computed blocks, so the second opinion is itself pinned
    import json
    import os
    golden = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")))
    seen = set()
    for case in golden["codec"]:
        if case["type"] in NP_DECODERS:
            out = NP_DECODERS[case["type"]](np.array(case["bytes"], dtype=np.uint8))
            for i, v in case["expect"].items():
                assert out[int(i)] == np.float32(v), (case["cite"], i)
            seen.add(case["type"])
    assert seen == set(NP_DECODERS)


@pytest.mark.parametrize("seed", [1, 0x5EED])
def test_q4_k_and_q8_0_match_an_independent_numpy_dequantizer_bit_for_bit(seed):
    rng = synth.SplitMix64(seed)
    raw = synth.synth_blocks(synth.Q4_K, 300, rng)
    assert np.array_equal(orc.dequantize(orc.Q4_K, raw).view(np.uint32), np_dequant_q4_k(raw).view(np.uint32))
    raw = synth.synth_blocks(synth.Q8_0, 500, rng)
    assert np.array_equal(orc.dequantize(orc.Q8_0, raw).view(np.uint32), np_dequant_q8_0(raw).view(np.uint32))


def test_fully_random_bytes_still_agree_with_numpy():
    # scales are arbitrary f16 patterns here (inf/NaN included): compare bit patterns of finite outputs
    g = np.random.Generator(np.random.PCG64(7))
    raw = g.integers(0, 256, size=144 * 64, dtype=np.uint8)
    a, b = orc.dequantize(orc.Q4_K, raw), np_dequant_q4_k(raw)
    fin = np.isfinite(b)
    assert np.array_equal(a[fin].view(np.uint32), b[fin].view(np.uint32))
    assert np.array_equal(np.isnan(a), np.isnan(b))


def test_block_geometry():
    # gguf.rs:331-382
    for t, bs, bb in [(orc.F32, 1, 4), (orc.F16, 1, 2), (orc.BF16, 1, 2), (orc.Q8_0, 32, 34), (orc.Q4_K, 256, 144),
                      (orc.Q5_K, 256, 176), (orc.Q6_K, 256, 210), (orc.Q5_1, 32, 24), (orc.Q4_0, 32, 18)]:
        assert orc.block_size(t) == bs and orc.block_bytes(t) == bb
    # OLMoE row and expert sizes
    assert orc.row_bytes(orc.Q4_K, 2048) == 1152 and orc.row_bytes(orc.Q4_K, 1024) == 576
    assert 2 * 1024 * 1152 + 2048 * 576 == 3_538_944
    assert 2 * 1024 * orc.row_bytes(orc.Q8_0, 2048) + 2048 * orc.row_bytes(orc.Q8_0, 1024) == 6_684_672


def test_synth_blocks_follow_the_reference_generator():
    # SplitMix64 known values: seed 0 -> 0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4 (the
    # published reference outputs of the algorithm experts.rs:1165-1171 spells out)
    r = synth.SplitMix64(0)
    v = r.next_u64(2)
    assert int(v[0]) == 0xE220A8397B1DCDAF and int(v[1]) == 0x6E789E6AA1B965F4
    # scale ranges of synth_blocks (experts.rs:1213-1226)
    raw = synth.synth_blocks(synth.Q4_K, 64, synth.SplitMix64(3)).reshape(-1, 144)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)
    assert d.min() >= 0.0005 - 1e-6 and d.max() <= 0.003 + 1e-6
    raw = synth.synth_blocks(synth.Q8_0, 64, synth.SplitMix64(3)).reshape(-1, 34)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)
    assert d.min() >= 0.002 - 1e-5 and d.max() <= 0.02 + 1e-5
    # a stream split in two equals one stream (state arithmetic)
    a = synth.SplitMix64(9)
    b = synth.SplitMix64(9)
    assert np.array_equal(np.concatenate([a.next_u64(5), a.next_u64(7)]), b.next_u64(12))
