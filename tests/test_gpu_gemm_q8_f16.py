"""Q8_0 banks on the batched path: the grouped GEMM of the f16 banks with every weight d * code held exactly as
two halfs, against the f64 product of the dequantized weights, beside the int8 form it replaces
(MUMMU_GEMM_Q8_F16=0).  Tolerance as the reference measures it (experts.rs:1264-1271): 2e-3.  x and the
activations between the two products are halfs in this form, as for F16 and BF16 banks; a bank whose largest
|d| * 127 leaves the half range keeps the int8 form."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def banks_of(H, I, E, seed):
    return (synth.random_bank_fast(M.Q8_0, [H, I, E], seed), synth.random_bank_fast(M.Q8_0, [H, I, E], seed + 1),
            synth.random_bank_fast(M.Q8_0, [I, H, E], seed + 2))


def run(monkeypatch, half_form, H, I, E, k, x, banks, seed=1):
    monkeypatch.setenv("MUMMU_GEMM_Q8_F16", "1" if half_form else "0")
    gate, up, down = banks
    router = normal((E, H), seed + 3, 0.05).astype(np.float16)
    n = x.shape[0]
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, M.Q8_0, up, M.Q8_0, down, M.Q8_0)
        got = m.forward(x, k, True)
        again = m.forward(x, k, True)
        ids, w = m.last_routing(n, k)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), "the batched path is not deterministic"
    ob = orc.LayerBanks(H, I, E, gate, up, down, orc.Q8_0)
    _, oids, ow, _ = orc.moe_forward(ob, router, orc.F16, x, k, True)
    assert np.array_equal(ids, oids.astype(np.int32))
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    want, mag = orc.moe_ref_f64(ob, oids, ow, x)
    return got, orc.rel_err(got, want, mag)


# (H, I, E, k, tokens): about 75 rows per expert (128-row tiles), 19 (32-row tiles), 50 (96-row tiles), 16 on 64 experts
# with a ragged router wave, 48 on a row of two K steps, 513 (several 64-row tiles per expert)
SHAPES = [
    (1024, 512, 8, 2, 300),
    (1024, 512, 16, 4, 77),
    (512, 256, 8, 2, 200),
    (2048, 1024, 64, 8, 131),
    (128, 128, 4, 2, 97),
    (1024, 512, 4, 2, 1027),
]


@pytest.mark.parametrize("H,I,E,k,n", SHAPES)
def test_half_form_matches_the_f64_reference(monkeypatch, H, I, E, k, n):
    x = normal((n, H), 5 + n)
    banks = banks_of(H, I, E, 10 + n)
    got, err = run(monkeypatch, True, H, I, E, k, x, banks, seed=10 + n)
    assert err.max() <= 2e-3, f"max relative error {err.max():.3e}"
    got8, err8 = run(monkeypatch, False, H, I, E, k, x, banks, seed=10 + n)
    assert err8.max() <= 2e-3, f"int8 form: max relative error {err8.max():.3e}"
    assert not np.array_equal(got, got8), "the switch did not change the arithmetic: is the half form running?"


def test_a_bank_with_a_scale_outside_the_half_range_keeps_the_int8_form(monkeypatch):
    # one block of the up bank with d = 1000: d * 128 is no finite half, so the layer is not eligible and both
    # settings of the switch run the same kernels
    H, I, E, k, n = 512, 256, 8, 2, 200
    x = normal((n, H), 91)
    gate, up, down = banks_of(H, I, E, 92)
    up = up.copy()
    bits = int(np.array([1000.0], dtype=np.float16).view(np.uint16)[0])
    blk = 34 * 1234
    up[blk], up[blk + 1] = bits & 0xFF, bits >> 8
    # (no accuracy bar here: the hidden unit behind that block is a thousand times its neighbours, the case the
    # 16-bit block-scaled activations of the int8 form are known to lose small elements in)
    got, _ = run(monkeypatch, True, H, I, E, k, x, (gate, up, down), seed=93)
    got8, _ = run(monkeypatch, False, H, I, E, k, x, (gate, up, down), seed=93)
    assert np.all(np.isfinite(got))
    assert np.array_equal(got.view(np.uint32), got8.view(np.uint32))


def test_a_scale_of_512_with_a_code_of_minus_128_keeps_the_int8_form(monkeypatch):
    # d = 512 and a code of -128 (the reference's encoder never writes one, a file may hold it): d * code = -65536 is
    # no finite half, so |d| must stay BELOW 512 for the half form and this layer keeps the integer one
    H, I, E, k, n = 512, 256, 8, 2, 200
    x = normal((n, H), 94)
    gate, up, down = banks_of(H, I, E, 95)
    up = up.copy()
    bits = int(np.array([512.0], dtype=np.float16).view(np.uint16)[0])
    blk = 34 * 77
    up[blk], up[blk + 1] = bits & 0xFF, bits >> 8
    up[blk + 2] = 0x80  # code -128
    got, _ = run(monkeypatch, True, H, I, E, k, x, (gate, up, down), seed=96)
    got8, _ = run(monkeypatch, False, H, I, E, k, x, (gate, up, down), seed=96)
    assert np.all(np.isfinite(got))
    assert np.array_equal(got.view(np.uint32), got8.view(np.uint32))


def test_weights_small_enough_that_the_low_halfs_are_subnormal(monkeypatch):
    # d around 4e-4 (weights up to 0.07, the size a trained model's are): d * code is a normal half, its low half
    # (below 2^-14) a subnormal one, which the vector and the matrix units both keep
    H, I, E, k, n = 512, 256, 8, 2, 150
    x = normal((n, H), 71)
    g = np.random.Generator(np.random.PCG64(72))
    banks = []
    for i, (a, b) in enumerate(((H, I), (H, I), (I, H))):
        bank = synth.random_bank_fast(M.Q8_0, [a, b, E], 73 + i).reshape(-1, 34).copy()
        d = g.uniform(2e-4, 6e-4, size=bank.shape[0]).astype(np.float16).view(np.uint16)
        bank[:, 0], bank[:, 1] = (d & 0xFF).astype(np.uint8), (d >> 8).astype(np.uint8)
        banks.append(bank.reshape(-1))
    got, err = run(monkeypatch, True, H, I, E, k, x, tuple(banks), seed=76)
    assert err.max() <= 2e-3, f"max relative error {err.max():.3e}"
