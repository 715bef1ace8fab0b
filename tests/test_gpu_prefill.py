"""Batched (prefill) path at small shapes where the f64 reference covers every token: streaming
router, three-launch dispatch over several chunks, grouped GEMMs with every tile size, ragged
token counts, hit counters taken from the dispatch scan.  Routing must be bit-exact against the
oracle, outputs within 2e-3 (f16 / quantized banks) of the f64 product of the dequantized
weights, measured as the reference measures it (experts.rs:1264-1271)."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def banks_for(kind, H, I, E, seed):
    if kind in ("F16", "BF16", "F32"):
        t, ot = {"F16": (M.F16, orc.F16), "BF16": (M.BF16, orc.BF16), "F32": (M.F32, orc.F32)}[kind]
        mk = lambda i, o, s: synth.encode_float(normal(E * o * i, s, 0.05), t)
        return mk(H, I, seed), mk(H, I, seed + 1), mk(I, H, seed + 2), t, ot
    t, ot = {"Q8_0": (M.Q8_0, orc.Q8_0), "Q4_K": (M.Q4_K, orc.Q4_K)}[kind]
    mk = lambda i, o, s: synth.random_bank_fast(t, [i, o, E], s)
    return mk(H, I, seed), mk(H, I, seed + 1), mk(I, H, seed + 2), t, ot


# (bank kind, H, I, E, k, tokens): token counts chosen to hit 32/64/96/128-row tiles, partial
# last tiles, a ragged last router wave and more than one 1024-assignment dispatch chunk
CASES = [
    ("F16", 512, 256, 8, 2, 77),      # ~19 rows per expert -> 32-row tiles
    ("F16", 512, 256, 8, 2, 200),     # 50 per expert -> 96-row tiles
    ("F16", 512, 256, 8, 4, 130),     # 65 per expert -> 96/128-row tiles
    ("F16", 1024, 512, 16, 4, 1027),  # 257 per expert -> several 64-row tiles, 5 dispatch chunks, odd token count
    ("F16", 256, 256, 128, 8, 1500),  # 12 dispatch chunks over 128 experts: every chunk's workgroup scans the counts itself
    ("BF16", 512, 256, 8, 2, 130),    # bf16 weights become halfs on the way into LDS
    ("BF16", 1024, 512, 16, 4, 515),
    ("F32", 512, 256, 8, 2, 77),      # f32 matrix cores, everything f32: held to 1e-5
    ("F32", 1024, 512, 16, 4, 515),
    ("Q8_0", 512, 256, 8, 2, 77),
    ("Q8_0", 1024, 512, 16, 4, 515),
    ("Q4_K", 512, 256, 8, 2, 200),
    ("Q4_K", 1024, 512, 16, 4, 1027),
]


@pytest.mark.parametrize("kind,H,I,E,k,n", CASES)
def test_prefill_matches_the_oracle(kind, H, I, E, k, n):
    gate, up, down, mt, ot = banks_for(kind, H, I, E, 100 + n)
    router = normal((E, H), 7 + n, 0.05).astype(np.float16)
    x = normal((n, H), 11 + n)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, mt, up, mt, down, mt)
        m.take_hits()
        got = m.forward(x, k, True)
        hits = m.take_hits()
        ids, w = m.last_routing(n, k)
        again = m.forward(x, k, True)
        one = m.forward(x[:1], k, True)  # the same token alone takes the decode kernels
    banks = orc.LayerBanks(H, I, E, gate, up, down, ot)
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F16, x, k, True)
    assert np.array_equal(ids, oids.astype(np.int32))
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    assert hits.tolist() == np.bincount(oids.reshape(-1), minlength=E).tolist()
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), "the batched path is not deterministic"
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    tol = 1e-5 if kind == "F32" else 2e-3
    err = orc.rel_err(got, want, mag)
    assert err.max() <= tol, f"max relative error {err.max():.3e}"
    assert orc.rel_err(one, want[:1], mag[:1]).max() <= tol


def test_prefill_with_experts_nobody_picks_and_two_everybody_picks():
    # router rows rigged: expert 0 takes all the probability for every token, every other
    # probability underflows to 0, and the tie at 0 goes to the lowest id (expert 1): two experts
    # serve all rows, six serve none
    H, I, E, k, n = 512, 256, 8, 2, 300
    gate, up, down, mt, ot = banks_for("F16", H, I, E, 5)
    router = normal((E, H), 9, 0.02)
    x = np.abs(normal((n, H), 10)) + 0.1
    router[0] = 1.0
    router[1] = -1.0
    router = router.astype(np.float16)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, mt, up, mt, down, mt)
        got = m.forward(x, k, False)
        hits = m.take_hits()
    banks = orc.LayerBanks(H, I, E, gate, up, down, ot)
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F16, x, k, False)
    assert hits.tolist() == [n, n, 0, 0, 0, 0, 0, 0]
    assert np.all(oids[:, 0] == 0) and np.all(oids[:, 1] == 1)
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    assert orc.rel_err(got, want, mag).max() <= 2e-3
