"""The two-launch decode form (router logits, routing and gate/up in one kernel whose workgroups exchange the
logits through their XCD's L2) against the three-launch form it replaces, through the C ABI: the same routing and
the same output bits, with and without the fused RmsNorm, on graph replays, and when every workgroup is made to
give up waiting and compute the logits itself (spin bound 0) - the failure path is forced from the host, no kernel
waits for anything that does not come."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def make(H, I, E, k, gt, dt, rt, seed, layers=1, flavour=0):
    g = np.random.Generator(np.random.PCG64(seed))
    m = M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=layers, max_tokens=8, rms_norm_eps=1e-5, router_flavour=flavour)
    kept = []
    for l in range(layers):
        gate = synth.random_bank_fast(gt, [H, I, E], seed + 10 * l + 1)
        up = synth.random_bank_fast(gt, [H, I, E], seed + 10 * l + 2)
        down = synth.random_bank_fast(dt, [I, H, E], seed + 10 * l + 3)
        r32 = g.standard_normal((E, H), dtype=np.float32) * np.float32(0.05)
        router = r32 if rt == M.F32 else (r32.astype(np.float16) if rt == M.F16 else synth.encode_float(r32, M.BF16).view(np.uint16).reshape(E, H))
        gamma = (1.0 + 0.1 * g.standard_normal(H)).astype(np.float32)
        m.load_layer(l, router, rt, gate, gt, up, gt, down, dt, rms_gamma=gamma)
        kept.append((router, gate, up, down, gamma))
    return m, g, kept


SHAPES = [
    # H, I, E, k, gate/up type, down type, router type, flavour
    (2048, 1024, 64, 8, M.Q4_K, M.Q4_K, M.F16, 0),   # the headline shape: one router row per workgroup
    (2048, 768, 128, 8, M.Q4_K, M.Q4_K, M.F16, 1),   # three rows per workgroup, two experts per routing lane
    (1024, 256, 16, 4, M.Q8_0, M.Q6_K, M.F32, 0),    # more workgroups than router rows, two rows of a wave per iteration
    (512, 512, 256, 8, M.Q5_K, M.Q8_0, M.BF16, 0),   # 32 rows per workgroup: eight rounds of its four waves
    (256, 1024, 8, 2, M.Q4_0, M.Q5_1, M.F16, 1),     # a row narrower than a wave's 512-element chunk
]


@pytest.mark.parametrize("H,I,E,k,gt,dt,rt,flavour", SHAPES, ids=[f"H{s[0]}-E{s[2]}-k{s[3]}" for s in SHAPES])
def test_two_launches_give_the_bits_of_three(H, I, E, k, gt, dt, rt, flavour):
    m, g, kept = make(H, I, E, k, gt, dt, rt, 4000 + E, flavour=flavour)
    with m:
        usable, _ = m.router_exchange_state()
        assert usable, "this device deals workgroups to its XCDs round-robin: the two-launch form must be on"
        for n in (1, 3, 8):
            x = g.standard_normal((n, H), dtype=np.float32)
            m.set_router_exchange(2)
            two = m.forward(x, k, flavour == 1)
            r2 = m.last_routing(n, k)
            assert m.router_exchange_state()[1] == 0, "no workgroup should have had to give up waiting"
            m.set_router_exchange(2, 0)  # nobody waits: every workgroup computes all logits itself
            alone = m.forward(x, k, flavour == 1)
            assert m.router_exchange_state()[1] > 0
            m.set_router_exchange(False)
            three = m.forward(x, k, flavour == 1)
            r3 = m.last_routing(n, k)
            assert np.array_equal(r2[0], r3[0]) and np.array_equal(bits(r2[1]), bits(r3[1])), f"{n} tokens: routing"
            assert np.array_equal(bits(two), bits(three)), f"{n} tokens"
            assert np.array_equal(bits(alone), bits(three)), f"{n} tokens, no exchange"
        # and the routing is the oracle's
        router, gate, up, down, _ = kept[0]
        banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
        rtype = {M.F32: orc.F32, M.F16: orc.F16, M.BF16: orc.BF16}[rt]
        _, ids, w, _ = orc.moe_forward(banks, router, rtype, x, k, flavour == 1, flavour)
        assert np.array_equal(r2[0], ids.astype(np.int32)) and np.array_equal(bits(r2[1]), bits(w))


def test_stack_with_the_norm_inside_the_fused_launch():
    H, I, E, k, L = 2048, 256, 64, 8, 3
    m, g, _ = make(H, I, E, k, M.Q8_0, M.Q8_0, M.F16, 5000, layers=L)
    with m:
        for n in (1, 5):
            x = (3.0 * g.standard_normal((n, H), dtype=np.float32)).astype(np.float32)
            m.set_router_exchange(2)
            two, ids2 = m.stack_forward(x, k, False, return_ids=True)
            m.set_router_exchange(False)
            three, ids3 = m.stack_forward(x, k, False, return_ids=True)
            assert np.array_equal(ids2, ids3)
            assert np.array_equal(bits(two), bits(three)), f"{n} tokens"
        assert m.router_exchange_state()[1] == 0


def test_graph_replays_of_the_two_launch_form():
    # every replay moves the exchange's epoch on: records of the replay before must never be taken for fresh ones
    H, I, E, k = 2048, 1024, 64, 8
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, M.F16, 6000)
    with m:
        xs = [g.standard_normal((1, H), dtype=np.float32) for _ in range(4)]
        m.set_router_exchange(False)
        want = [m.forward(x, k, False) for x in xs]
        m.set_router_exchange(True)
        xd = [M.DeviceBuffer.from_array(x) for x in xs]
        od = [M.DeviceBuffer(H * 4) for _ in xs]
        m.graph_begin()
        for x, o in zip(xd, od):
            m.forward_device(0, x, 1, k, False, o)
        graph = m.graph_end()
        for rep in range(5):
            for o in od:
                o.upload(np.zeros((1, H), np.float32))
            graph.launch()
            m.check()
            for o, w in zip(od, want):
                assert np.array_equal(bits(o.download(np.float32, (1, H))), bits(w)), rep
            # new inputs through the same buffers: stale logits of the previous replay would show here
            xs = [g.standard_normal((1, H), dtype=np.float32) for _ in range(4)]
            m.set_router_exchange(False)
            want = [m.forward(x, k, False) for x in xs]
            m.set_router_exchange(True)
            for d, x in zip(xd, xs):
                d.upload(x)
        graph.close()
        assert m.router_exchange_state()[1] == 0
