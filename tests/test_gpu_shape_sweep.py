"""A sweep over awkward shapes through every kernel family: hidden and intermediate widths that
are not powers of two (lane groups with idle lanes, rows of two to four units per lane), expert
counts that are not multiples of 64, top-k from 1 to 16, token counts on both sides of every path
switch (1, 2..8 inline routing, 9.. per-assignment kernels, dispatch + grouped GEMM from 7 tokens
for F16 banks and 19 for block-quantized ones where the shape allows it), mixed
bank types, both router flavours.  Routing must be bit-exact, outputs within the path's tolerance
of the f64 product of the dequantized weights."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def bank(t, ne, seed):
    if t in (M.F32, M.F16, M.BF16):
        w = normal((ne[2], ne[1], ne[0]), seed, 0.05)
        return synth.encode_float(w, t)
    return synth.random_bank_fast(t, ne, seed)


# (gate/up type, down type, H, I, E, k, flavour)
SHAPES = [
    (M.Q8_0, M.Q8_0, 96, 32, 3, 1, 0),          # 3 units per row, odd expert count, top-1
    (M.Q8_0, M.Q4_0, 160, 96, 5, 5, 1),         # k = E
    (M.Q4_0, M.Q8_0, 320, 160, 60, 6, 0),       # 10 and 5 units per row
    (M.Q4_K, M.Q4_K, 768, 256, 100, 8, 1),      # 3 super-blocks per row, 100 experts (two per lane)
    (M.Q4_K, M.Q8_0, 2304, 1408, 12, 2, 0),     # 72 units: two per lane with idle lanes; 44 units in the down rows
    (M.Q5_K, M.Q6_K, 1280, 512, 160, 10, 1),    # 160 experts (eight-per-lane router), top-10
    (M.Q6_K, M.Q5_K, 512, 768, 16, 16, 1),      # top-16: widest fused down+combine
    (M.Q8_0, M.Q8_0, 5120, 64, 4, 2, 0),        # 160 units: three per lane
    (M.Q8_0, M.Q8_0, 64, 4096, 4, 2, 0),        # 128 units in the down rows: two per lane there
    (M.F16, M.F16, 192, 64, 6, 3, 0),           # float banks, widths not multiples of 128
    (M.BF16, M.F32, 100, 36, 7, 2, 1),          # scalar (non-vector) float loads
    (M.F32, M.Q8_0, 128, 64, 9, 4, 0),          # float gate/up feeding a quantized down bank
    (M.Q4_1, M.F16, 256, 48, 8, 3, 1),          # quantized gate/up feeding a float down bank
]
TOKENS = [1, 2, 6, 7, 8, 9, 18, 19, 31, 33, 70]


@pytest.mark.parametrize("gt,dt,H,I,E,k,flavour", SHAPES, ids=[f"{s[0]}-{s[1]}-{s[2]}x{s[3]}-E{s[4]}k{s[5]}f{s[6]}" for s in SHAPES])
def test_awkward_shapes_match_the_oracle_on_every_path(gt, dt, H, I, E, k, flavour):
    seed = H + 7 * I + 13 * E + k
    gate, up, down = bank(gt, [H, I, E], seed), bank(gt, [H, I, E], seed + 1), bank(dt, [I, H, E], seed + 2)
    router = normal((E, H), seed + 3, 0.05)
    nmax = max(TOKENS)
    x = normal((nmax, H), seed + 4)
    norm = bool(flavour) or (seed % 2 == 0)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=nmax, router_flavour=flavour) as m:
        m.load_layer(0, router, M.F32, gate, gt, up, gt, down, dt)
        m.take_hits()
        outs, routes = {}, {}
        for n in TOKENS:
            outs[n] = m.forward(x[:n], k, norm)
            routes[n] = m.last_routing(n, k)
        hits = m.take_hits()
        batched_from = m.batched_from(0)
    banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
    _, oids, ow, _ = orc.moe_forward(banks, router, orc.F32, x, k, norm, flavour)
    want, mag = orc.moe_ref_f64(banks, oids, ow, x)
    all_float = gt in (M.F32, M.BF16) and dt in (M.F32, M.BF16)
    tol = 1e-5 if all_float else 2e-3
    served = np.zeros(E, np.int64)
    for n in TOKENS:
        ids, w = routes[n]
        assert np.array_equal(ids, oids[:n].astype(np.int32)), n
        assert np.array_equal(w.view(np.uint32), ow[:n].view(np.uint32)), n
        err = orc.rel_err(outs[n], want[:n], mag[:n]).max()
        # (the batched path rounds the activations of BF16 banks to f16, as it does for F16 banks)
        tol_n = 2e-3 if n >= batched_from and M.BF16 in (gt, dt) else tol
        assert err <= tol_n, f"{n} tokens: max relative error {err:.3e}"
        served += np.bincount(oids[:n].reshape(-1), minlength=E)
    assert hits.tolist() == served.tolist()
    # below the batched path a token's result does not depend on its company
    for n in (2, 6, 7, 8, 9, 18, 19, 31):
        if n < batched_from:
            assert np.array_equal(outs[1].view(np.uint32), outs[n][:1].view(np.uint32)), n
