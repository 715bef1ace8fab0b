"""The XCD-aware workgroup order of the multi-token decode launches (mummu_moe_set_tile_order: tokens that share an
expert read its rows through one XCD's L2) against the plain order, through the C ABI: the same routing and the same
output bits for every bank type, with row-tile counts that are and are not multiples of eight, beyond eight tokens
(the launches that read the routing from memory), in the layer stack, on graph replays, and when the caller's logits
(mummu_moe_routed) pile every token on the same experts."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def make(H, I, E, k, gt, dt, seed, layers=1, flavour=0, max_tokens=32):
    g = np.random.Generator(np.random.PCG64(seed))
    m = M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=layers, max_tokens=max_tokens, rms_norm_eps=1e-5, router_flavour=flavour)
    kept = []
    for l in range(layers):
        gate = synth.random_bank_fast(gt, [H, I, E], seed + 10 * l + 1)
        up = synth.random_bank_fast(gt, [H, I, E], seed + 10 * l + 2)
        down = synth.random_bank_fast(dt, [I, H, E], seed + 10 * l + 3)
        router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.05)).astype(np.float16)
        gamma = (1.0 + 0.1 * g.standard_normal(H)).astype(np.float32)
        m.load_layer(l, router, M.F16, gate, gt, up, gt, down, dt, rms_gamma=gamma)
        kept.append((router, gate, up, down, gamma))
    return m, g, kept


SHAPES = [
    # H, I, E, k, gate/up type, down type, flavour
    (2048, 1024, 64, 8, M.Q4_K, M.Q4_K, 0),    # the headline shape: 64 gate/up tiles, 256 down tiles
    (2048, 768, 128, 8, M.Q4_K, M.Q6_K, 1),    # 48 gate/up tiles
    (2560, 640, 512, 10, M.Q4_K, M.Q5_1, 1),   # top-10 of 512, 40 gate/up tiles, rows wider than a wave
    (1024, 160, 32, 4, M.Q8_0, M.Q8_0, 0),     # 3 gate/up tiles (64 rows each): most of the eight XCD columns hold nothing
    (512, 256, 16, 6, M.Q5_K, M.Q5_K, 0),
    (256, 128, 8, 8, M.Q6_K, M.Q4_0, 0),       # top-8 of 8: every token on every expert; one gate/up tile
    (768, 4096, 24, 3, M.Q5_0, M.Q4_1, 0),     # hidden rows of 4096: two units per lane in the down product
]


@pytest.mark.parametrize("H,I,E,k,gt,dt,flavour", SHAPES, ids=[f"H{s[0]}-I{s[1]}-E{s[2]}-k{s[3]}-{s[4]}-{s[5]}" for s in SHAPES])
def test_tile_order_gives_the_bits_of_the_plain_order(H, I, E, k, gt, dt, flavour, monkeypatch):
    monkeypatch.setenv("MUMMU_GEMM_MIN_TOKENS", "1000000")  # the decode kernels at every size
    m, g, kept = make(H, I, E, k, gt, dt, 8100 + E + I, flavour=flavour)
    with m:
        for n in (2, 3, 5, 8, 9, 17, 25):
            x = g.standard_normal((n, H), dtype=np.float32)
            if n >= 5:
                x[1] = x[0]            # two tokens with the same routing: every expert of theirs serves both
                x[n - 1] = 0.5 * x[0]  # (a scaled row keeps the routing's order but not its weights)
            m.set_tile_order(True)
            got = m.forward(x, k, flavour == 1)
            r1 = m.last_routing(n, k)
            m.set_tile_order(False)
            want = m.forward(x, k, flavour == 1)
            r0 = m.last_routing(n, k)
            assert np.array_equal(r1[0], r0[0]) and np.array_equal(bits(r1[1]), bits(r0[1])), f"{n} tokens: routing"
            assert np.array_equal(bits(got), bits(want)), f"{n} tokens"
            # a token alone gives the same bits as in the batch
            for t in (0, n - 1):
                alone = m.forward(x[t:t + 1], k, flavour == 1)
                assert np.array_equal(bits(alone[0]), bits(got[t])), f"token {t} of {n}"
        # and against the oracle: its routing, the f64 product within the quantized banks' tolerance
        router, gate, up, down, _ = kept[0]
        banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
        _, ids, w, _ = orc.moe_forward(banks, router, orc.F16, x, k, flavour == 1, flavour)
        assert np.array_equal(r1[0], ids.astype(np.int32)) and np.array_equal(bits(r1[1]), bits(w))
        ref, mag = orc.moe_ref_f64(banks, ids, w, x)
        assert float(orc.rel_err(got, ref, mag).max()) <= 2e-3


def test_tile_order_in_the_layer_stack():
    H, I, E, k, L = 2048, 256, 64, 8, 3
    m, g, _ = make(H, I, E, k, M.Q8_0, M.Q8_0, 8300, layers=L)
    with m:
        for n in (4, 8, 12):
            x = (3.0 * g.standard_normal((n, H), dtype=np.float32)).astype(np.float32)
            m.set_tile_order(True)
            got, ids1 = m.stack_forward(x, k, False, return_ids=True)
            m.set_tile_order(False)
            want, ids0 = m.stack_forward(x, k, False, return_ids=True)
            assert np.array_equal(ids1, ids0)
            assert np.array_equal(bits(got), bits(want)), f"{n} tokens"


def test_tile_order_on_graph_replays():
    H, I, E, k = 2048, 1024, 64, 8
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, 8400)
    with m:
        shapes = (8, 4, 2, 6)
        xs = [g.standard_normal((n, H), dtype=np.float32) for n in shapes]
        want = [m.forward(x, k, False) for x in xs]
        m.set_tile_order(True)
        xd = [M.DeviceBuffer.from_array(x) for x in xs]
        od = [M.DeviceBuffer(x.nbytes) for x in xs]
        m.graph_begin()
        for n, x, o in zip(shapes, xd, od):
            m.forward_device(0, x, n, k, False, o)
        graph = m.graph_end()
        for rep in range(3):
            for o, x in zip(od, xs):
                o.upload(np.full(x.shape, np.nan, np.float32))
            graph.launch()
            m.check()
            for n, o, w in zip(shapes, od, want):
                assert np.array_equal(bits(o.download(np.float32, (n, H))), bits(w)), (rep, n)
            xs = [g.standard_normal((n, H), dtype=np.float32) for n in shapes]
            for d, x in zip(xd, xs):
                d.upload(x)
            m.set_tile_order(False)
            want = [m.forward(x, k, False) for x in xs]
            m.set_tile_order(True)
        graph.close()


def test_tile_order_when_every_token_takes_the_same_experts(monkeypatch):
    # the caller's logits (mummu_moe_routed) send all 32 tokens to the same eight experts, then spread them so that
    # every expert serves exactly four
    monkeypatch.setenv("MUMMU_GEMM_MIN_TOKENS", "1000000")
    H, I, E, k = 1024, 512, 64, 8
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, 8500)
    with m:
        n = 32
        x = g.standard_normal((n, H), dtype=np.float32)
        piled = np.tile(g.standard_normal((1, E), dtype=np.float32), (n, 1)) + 1e-3 * g.standard_normal((n, E), dtype=np.float32)
        spread = np.full((n, E), -5.0, np.float32)
        for t in range(n):
            spread[t, [(8 * (t % 8) + j) % E for j in range(8)]] = 1.0 + 0.1 * g.standard_normal(8).astype(np.float32)
        for logits in (piled, spread):
            m.set_tile_order(True)
            got = m.routed_moe(0, logits, x, n, k)
            m.set_tile_order(False)
            want = m.routed_moe(0, logits, x, n, k)
            assert np.array_equal(bits(got), bits(want))
