"""Every GGUF block type of the reference's dequantizer (gguf.rs:1535-1797) on the device:
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K and Q6_K next to Q8_0 and Q4_K - bit-exact dequantization against
the oracle, and expert banks of those types (mixed the way shipped files mix them,
experts.rs:1838-1879: gate/up Q4_K or Q5_K, down Q5_1 or Q8_0; Q6_K downs as llama.cpp's
Q4_K_M recipe writes them) through the decode kernels: routing bit-exact, outputs within 2e-3
of the f64 product of the dequantized weights, measured as the reference measures it
(experts.rs:1264-1271)."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu

QUANT = [M.Q4_0, M.Q4_1, M.Q5_0, M.Q5_1, M.Q8_0, M.Q4_K, M.Q5_K, M.Q6_K]
NAME = {M.Q4_0: "Q4_0", M.Q4_1: "Q4_1", M.Q5_0: "Q5_0", M.Q5_1: "Q5_1", M.Q8_0: "Q8_0", M.Q4_K: "Q4_K", M.Q5_K: "Q5_K",
        M.Q6_K: "Q6_K"}


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


@pytest.mark.parametrize("t", QUANT, ids=[NAME[t] for t in QUANT])
def test_dequantize_is_bit_exact_for_every_block_type(t):
    # synthetic blocks with sane scales, then blocks of raw random bytes whose f16 fields are
    # whatever the bytes say (subnormals, huge values, infinities; where both sides are NaN the
    # payload is not compared)
    blocks = synth.synth_blocks(t, 300, synth.SplitMix64(40 + t))
    raw = np.random.Generator(np.random.PCG64(t)).integers(0, 256, size=64 * synth.BLOCK_BYTES[t], dtype=np.uint8)
    for data in (blocks, raw):
        got = M.dequantize(t, data)
        want = orc.dequantize(t, data)
        assert got.shape == want.shape
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), np.flatnonzero(~same)[:8]
    with pytest.raises(M.MoeError):
        M.dequantize(t, blocks[:-1])  # not whole blocks (gguf.rs:1411-1416)


# (gate/up type, down type, hidden, inter, experts, k)
CASES = [
    (M.Q5_K, M.Q5_1, 512, 256, 8, 2),
    (M.Q4_K, M.Q6_K, 512, 256, 8, 2),
    (M.Q6_K, M.Q8_0, 512, 256, 8, 4),
    (M.Q4_0, M.Q4_0, 512, 256, 8, 2),
    (M.Q4_1, M.Q5_0, 512, 96, 8, 2),      # 96-wide rows: 3 units, not a power of two
    (M.Q5_0, M.Q4_1, 256, 64, 4, 2),
    (M.Q5_1, M.Q4_K, 512, 256, 8, 8),     # k = E
    (M.Q8_0, M.Q5_K, 512, 256, 16, 2),
    (M.Q5_K, M.Q5_1, 2560, 640, 16, 8),   # the shipped qwen4exp geometry (experts.rs:1849): 80 and 20 units per row
    (M.Q4_K, M.Q8_0, 2560, 640, 16, 8),
    (M.Q4_K, M.Q6_K, 2048, 1024, 64, 8),  # OLMoE shape, Q4_K_M-style down bank
    (M.Q8_0, M.Q4_0, 4352, 64, 4, 2),     # 136 units per gate/up row: three units per lane
    (M.Q4_0, M.Q8_0, 256, 2560, 4, 2),    # 80 units per down row: two units per lane
]


@pytest.mark.parametrize("gt,dt,H,I,E,k", CASES, ids=[f"{NAME[c[0]]}-{NAME[c[1]]}-{c[2]}x{c[3]}" for c in CASES])
def test_mixed_type_banks_match_the_oracle(gt, dt, H, I, E, k):
    seed = 7 * gt + dt + H
    gate = synth.random_bank_fast(gt, [H, I, E], seed)
    up = synth.random_bank_fast(gt, [H, I, E], seed + 1)
    down = synth.random_bank_fast(dt, [I, H, E], seed + 2)
    router = normal((E, H), seed + 3, 0.05).astype(np.float16)
    n = 21
    x = normal((n, H), seed + 4)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, gt, up, gt, down, dt)
        outs = {c: m.forward(x[:c], k, True) for c in (1, 5, n)}
        batched_from = m.batched_from(0)
        ids, w = m.last_routing(n, k)
        hits_before = m.take_hits()
        e0 = int(ids[0, 0])
        one = m.expert_run(0, e0, x[:3])
        gate_e = m.dequantize_expert(0, "gate", e0)
        down_e = m.dequantize_expert(0, "down", e0)
    assert hits_before.sum() == (1 + 5 + n) * k
    banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F16, x, k, True)
    assert np.array_equal(ids, oids.astype(np.int32))
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    for c, got in outs.items():
        err = orc.rel_err(got, want[:c], mag[:c])
        assert err.max() <= 2e-3, f"{c} tokens: max relative error {err.max():.3e}"
    # below the batched path (the 21-token call takes it where the shape allows the grouped GEMM) a
    # token's result does not depend on how many tokens share the call
    assert np.array_equal(outs[1].view(np.uint32), outs[5][:1].view(np.uint32))
    if n < batched_from:
        assert np.array_equal(outs[5].view(np.uint32), outs[n][:5].view(np.uint32))
    # one expert alone (ExpertExec::run) is a top-1 routing to it with weight 1: same closeness
    want1, mag1 = orc.moe_ref_f64(banks, np.full((3, 1), e0, np.uint32), np.ones((3, 1), np.float32), x[:3])
    assert orc.rel_err(one, want1, mag1).max() <= 2e-3
    assert orc.rel_err(orc.expert_ffn(banks, e0, x[:3]), want1, mag1).max() <= 2e-3  # and so is the oracle's own f32 path
    # the resident bytes decode to the oracle's weights, bit for bit
    rb_g, rb_d = orc.row_bytes(gt, H), orc.row_bytes(dt, I)
    og = orc.dequantize(gt, gate[e0 * I * rb_g:(e0 + 1) * I * rb_g]).reshape(I, H)
    od = orc.dequantize(dt, down[e0 * H * rb_d:(e0 + 1) * H * rb_d]).reshape(H, I)
    assert np.array_equal(gate_e.view(np.uint32), og.view(np.uint32))
    assert np.array_equal(down_e.view(np.uint32), od.view(np.uint32))


# many tokens: dispatch + grouped GEMM on the int8 matrix cores, every block type on either side
PREFILL = [
    (M.Q5_K, M.Q6_K, 512, 256, 8, 2, 300),
    (M.Q6_K, M.Q5_K, 512, 256, 8, 2, 300),
    (M.Q4_0, M.Q4_1, 512, 256, 8, 2, 130),
    (M.Q4_1, M.Q4_0, 512, 256, 8, 2, 77),
    (M.Q5_0, M.Q5_1, 512, 256, 8, 4, 200),
    (M.Q5_1, M.Q5_0, 512, 256, 8, 2, 515),
    (M.Q4_K, M.Q6_K, 1024, 512, 16, 4, 1027),
    (M.Q5_K, M.Q5_1, 2560, 640, 32, 10, 96),   # qwen4exp geometry, top-10
    (M.Q4_K, M.Q5_1, 512, 96, 8, 2, 300),      # 96-wide rows are not whole 64-element K steps: per-assignment kernels
]


@pytest.mark.parametrize("gt,dt,H,I,E,k,n", PREFILL, ids=[f"{NAME[c[0]]}-{NAME[c[1]]}-{c[2]}x{c[3]}-{c[6]}" for c in PREFILL])
def test_many_tokens_match_the_oracle_for_every_block_type(gt, dt, H, I, E, k, n):
    gate = synth.random_bank_fast(gt, [H, I, E], 1 + gt)
    up = synth.random_bank_fast(gt, [H, I, E], 2 + gt)
    down = synth.random_bank_fast(dt, [I, H, E], 3 + dt)
    router = normal((E, H), 4, 0.05).astype(np.float16)
    x = normal((n, H), 5)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, gt, up, gt, down, dt)
        got = m.forward(x, k, False)
        hits = m.take_hits()
        ids, w = m.last_routing(n, k)
        again = m.forward(x, k, False)
    banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F16, x, k, False)
    assert np.array_equal(ids, oids.astype(np.int32))
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    assert hits.tolist() == np.bincount(oids.reshape(-1), minlength=E).tolist()
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    err = orc.rel_err(got, want, mag)
    assert err.max() <= 2e-3, f"max relative error {err.max():.3e}"
