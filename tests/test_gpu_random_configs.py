"""Seeded random configurations through the C ABI: block type (all eleven), hidden and intermediate
widths, expert count, top-k, router flavour and dtype, normalisation and token count are drawn
together, so that combinations nobody wrote down by hand cross the path switches too (decode
kernels with the routing inside, the per-assignment kernels, dispatch + grouped GEMM with one or
two K steps per stage, float banks fused or not, BF16 banks on the f16 units).  Every case is held
to the same bar as the hand-written ones: routing bit-exact against the oracle, outputs within 1e-5
(float banks on the decode kernels) or 2e-3 of the f64 product of the dequantized weights, measured
as the reference measures it (experts.rs:1264-1271)."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu

QUANT = [M.Q4_0, M.Q4_1, M.Q5_0, M.Q5_1, M.Q8_0, M.Q4_K, M.Q5_K, M.Q6_K]
FLOAT = [M.F32, M.F16, M.BF16]
KQ = (M.Q4_K, M.Q5_K, M.Q6_K)


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def bank(t, ne, seed):
    if t in FLOAT:
        return synth.encode_float(normal((ne[2], ne[1], ne[0]), seed, 0.05), t)
    return synth.random_bank_fast(t, ne, seed)


def draw(seed):
    g = np.random.Generator(np.random.PCG64(1000 + seed))
    kind = g.integers(0, 4)
    if kind == 0:      # both sides the same quantized type
        gt = dt = QUANT[g.integers(0, len(QUANT))]
    elif kind == 1:    # mixed quantized types
        gt, dt = QUANT[g.integers(0, len(QUANT))], QUANT[g.integers(0, len(QUANT))]
    elif kind == 2:    # float banks
        gt = dt = FLOAT[g.integers(0, len(FLOAT))]
    else:              # anything with anything
        pool = QUANT + FLOAT
        gt, dt = pool[g.integers(0, len(pool))], pool[g.integers(0, len(pool))]
    # widths: whole blocks of the type that reads them; sometimes multiples of 64 / 128 (grouped GEMM, one or two K
    # steps per stage), sometimes not
    unit_h = 256 if gt in KQ else 32
    unit_i = 256 if dt in KQ else 32
    H = int(unit_h * g.integers(1, 1 + 1280 // unit_h))
    I = int(unit_i * g.integers(1, 1 + 768 // unit_i))
    E = int(g.choice([2, 3, 8, 17, 64, 65, 130]))
    k = int(g.integers(1, min(E, 16) + 1))
    n = int(g.choice([1, 2, 3, 5, 8, 9, 13, 20, 33, 64, 130]))
    flavour = int(g.integers(0, 2))
    norm = bool(flavour) or bool(g.integers(0, 2))
    rt = [M.F32, M.F16, M.BF16][g.integers(0, 3)]
    return gt, dt, H, I, E, k, n, flavour, norm, rt


@pytest.mark.parametrize("seed", range(96))
def test_a_random_configuration_matches_the_oracle(seed):
    gt, dt, H, I, E, k, n, flavour, norm, rt = draw(seed)
    gate, up, down = bank(gt, [H, I, E], 3 * seed), bank(gt, [H, I, E], 3 * seed + 1), bank(dt, [I, H, E], 3 * seed + 2)
    router32 = normal((E, H), 7000 + seed, 0.05)
    router = synth.encode_float(router32, rt)
    x = normal((n, H), 9000 + seed)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n, router_flavour=flavour) as m:
        m.load_layer(0, router, rt, gate, gt, up, gt, down, dt)
        got = m.forward(x, k, norm)
        ids, w = m.last_routing(n, k)
        hits = m.take_hits()
        again = m.forward(x, k, norm)
        batched_from = m.batched_from(0)
    banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
    ort = {M.F32: orc.F32, M.F16: orc.F16, M.BF16: orc.BF16}[rt]
    _, oids, ow, _ = orc.moe_forward(banks, router, ort, x, k, norm, flavour)
    what = f"seed {seed}: types {gt}/{dt}, H {H}, I {I}, E {E}, k {k}, n {n}, flavour {flavour}, norm {norm}, router {rt}"
    assert np.array_equal(ids, oids.astype(np.int32)), what
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), what
    assert hits.tolist() == np.bincount(oids.reshape(-1), minlength=E).tolist(), what
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), what
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    # float banks on the decode kernels multiply exact f32 values of the weights (F32, BF16 and F16 alike) by the f32
    # activations; from batched_from on the 16-bit types take the f16 matrix units, where x is rounded to halfs
    exact_float = gt in (M.F32, M.BF16, M.F16) and dt in (M.F32, M.BF16, M.F16) and n < batched_from
    tol = 1e-5 if exact_float else 2e-3
    # (outputs 100 times smaller than the batch's typical magnitude - a token whose hidden row is all but zero - are
    # held to the tolerance against that floor, not against their own magnitude)
    err = orc.rel_err(got, want, np.maximum(mag, 1e-2 * np.median(mag))).max()
    assert err <= tol, f"{what}: max relative error {err:.3e} > {tol}"
