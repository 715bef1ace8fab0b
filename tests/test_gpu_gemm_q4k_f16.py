"""Q4_K banks on the batched path: the grouped GEMM on the f16 matrix units (exact sc*q halfs against
activations held as pairs of halfs) against the f64 product of the dequantized weights, beside the int8
form it replaces (MUMMU_GEMM_Q4K_F16=0).  Tolerance as the reference measures it (experts.rs:1264-1271):
2e-3 is the reference's bar; the f16-unit form carries 22 bits per activation and is held to 3e-5 here."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu

ORC = {M.Q4_K: orc.Q4_K, M.Q6_K: orc.Q6_K, M.Q8_0: orc.Q8_0}


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def run(monkeypatch, f16_units, H, I, E, k, x, down_type=M.Q4_K, seed=1):
    monkeypatch.setenv("MUMMU_GEMM_Q4K_F16", "1" if f16_units else "0")
    gate = synth.random_bank_fast(M.Q4_K, [H, I, E], seed)
    up = synth.random_bank_fast(M.Q4_K, [H, I, E], seed + 1)
    down = synth.random_bank_fast(down_type, [I, H, E], seed + 2)
    router = normal((E, H), seed + 3, 0.05).astype(np.float16)
    n = x.shape[0]
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, M.Q4_K, up, M.Q4_K, down, down_type)
        got = m.forward(x, k, True)
        again = m.forward(x, k, True)
        ids, w = m.last_routing(n, k)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), "the batched path is not deterministic"
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.Q4_K, orc.Q4_K, ORC[down_type])
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F16, x, k, True)
    assert np.array_equal(ids, oids.astype(np.int32))
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    return got, orc.rel_err(got, want, mag)


# (H, I, E, k, tokens): 64-row tiles with ragged second tiles, 32-row tiles, one tile per expert, a token
# count that leaves a partial router wave, the smallest K-quant row (one super-block per down row)
SHAPES = [
    (1024, 512, 8, 2, 300),
    (1024, 512, 16, 4, 77),
    (512, 256, 8, 2, 200),
    (2048, 1024, 64, 8, 131),
    (256, 256, 4, 2, 97),
]


@pytest.mark.parametrize("H,I,E,k,n", SHAPES)
def test_f16_units_match_the_f64_reference_at_f32_accuracy(monkeypatch, H, I, E, k, n):
    x = normal((n, H), 5 + n)
    got, err = run(monkeypatch, True, H, I, E, k, x, seed=10 + n)
    assert err.max() <= 3e-5, f"max relative error {err.max():.3e}"
    got8, err8 = run(monkeypatch, False, H, I, E, k, x, seed=10 + n)
    assert err8.max() <= 2e-3, f"int8 form: max relative error {err8.max():.3e}"
    assert not np.array_equal(got, got8), "the switch did not change the arithmetic: is the f16-unit form running?"


@pytest.mark.parametrize("tile_rows", [16, 32, 64])
@pytest.mark.parametrize("H,I,E,k,n", [(1024, 512, 8, 2, 300), (2048, 1024, 64, 8, 40), (256, 256, 4, 2, 97)])
def test_every_tile_form_on_the_same_batch(monkeypatch, tile_rows, H, I, E, k, n):
    # MUMMU_GEMM_TILE_ROWS forces the 16-, 32- or 64-row form, whatever the cost model would pick: full tiles, ragged
    # last tiles and experts with a row or two (or none) under each of them
    monkeypatch.setenv("MUMMU_GEMM_TILE_ROWS", str(tile_rows))
    x = normal((n, H), 70 + n)
    _, err = run(monkeypatch, True, H, I, E, k, x, seed=60 + n)
    assert err.max() <= 3e-5, f"{tile_rows}-row tiles: max relative error {err.max():.3e}"


@pytest.mark.parametrize("down_type", [M.Q6_K, M.Q8_0])
def test_q4k_gate_up_feeding_a_down_bank_of_another_type(monkeypatch, down_type):
    # the gate/up launch takes the f16 units and writes the 16-bit byte planes the int8 down product reads
    H, I, E, k, n = 1024, 512, 8, 2, 260
    x = normal((n, H), 21)
    _, err = run(monkeypatch, True, H, I, E, k, x, down_type=down_type, seed=40)
    assert err.max() <= 2e-3, f"max relative error {err.max():.3e}"


def test_rows_with_one_element_standing_out_keep_their_small_elements(monkeypatch):
    # one element of every row 2000 times the others: the 16-bit block-scaled form rounds the elements that share
    # its 64-element block to 1/65024 of it; a pair of halfs keeps 22 bits of every element down to 2^-24 of the
    # row's largest, and one power-of-two scale per row changes nothing in that
    H, I, E, k, n = 1024, 512, 8, 2, 300
    x = normal((n, H), 33)
    x[:, 7] = 2000.0 * np.sign(x[:, 7])
    x[::3, 900] = -2500.0
    _, err = run(monkeypatch, True, H, I, E, k, x, seed=50)
    assert err.max() <= 3e-5, f"max relative error {err.max():.3e}"


def test_rows_of_zeros_and_tiny_and_huge_rows(monkeypatch):
    H, I, E, k, n = 512, 256, 8, 2, 150
    x = normal((n, H), 44)
    x[3] = 0.0
    x[10] *= np.float32(1e-30)
    x[20] *= np.float32(1e20)
    got, err = run(monkeypatch, True, H, I, E, k, x, seed=60)
    assert np.all(np.isfinite(got[[3, 10]]))
    assert np.all(got[3] == 0.0)
    keep = np.ones(n, dtype=bool)
    keep[20] = False   # (|x|^2-sized products of a 1e20 row overflow f32 in the reference arithmetic as well)
    assert err[keep].max() <= 3e-5, f"max relative error {err[keep].max():.3e}"
