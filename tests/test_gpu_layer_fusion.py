"""The one-launch decode form (router logits, routing, gate/up and the down product of every routed expert in one
kernel, the experts' hidden rows passed between the workgroups of an XCD through its L2) against the two- and
three-launch forms it replaces, through the C ABI: the same routing and the same output bits, with and without the
fused RmsNorm, with a shared expert beside it, on graph replays, and when every workgroup is made to give up waiting
and compute everything it needs itself (spin bound 0) - the failure path is forced from the host, no kernel waits
for anything that does not come."""
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
    (2048, 1024, 64, 8, M.Q4_K, M.Q4_K, M.F16, 0),   # the headline shape: 64 workgroups per slot, 32 down rows each
    (2048, 768, 128, 8, M.Q4_K, M.Q4_K, M.F16, 1),   # 48 workgroups per slot: 43 down rows each needed, 64 given
    (2048, 1024, 64, 8, M.Q8_0, M.Q8_0, M.F16, 0),   # the 16-layer stack's banks
    (2048, 1024, 64, 8, M.Q4_K, M.Q6_K, M.F16, 0),   # a Q4_K_M-style file: part of ffn_down in Q6_K
    (1024, 256, 16, 8, M.Q8_0, M.Q6_K, M.F32, 0),    # two gate/up rows of a wave per iteration: two hidden blocks per workgroup
    (512, 512, 32, 8, M.Q4_K, M.Q8_0, M.BF16, 0),    # four blocks per workgroup, 16 workgroups per slot
    (256, 1024, 8, 8, M.Q8_0, M.Q4_K, M.F16, 1),     # top-8 of 8: every expert; a row narrower than a wave's chunk
]


@pytest.mark.parametrize("H,I,E,k,gt,dt,rt,flavour", SHAPES, ids=[f"H{s[0]}-I{s[1]}-E{s[2]}-{s[4]}-{s[5]}" for s in SHAPES])
def test_one_launch_gives_the_bits_of_two_and_three(H, I, E, k, gt, dt, rt, flavour):
    m, g, kept = make(H, I, E, k, gt, dt, rt, 7000 + E + I, flavour=flavour)
    with m:
        assert m.router_exchange_state()[0], "this device deals workgroups to its XCDs round-robin: the fused forms must be on"
        for n in (1, 3, 8):
            x = g.standard_normal((n, H), dtype=np.float32)
            m.set_router_exchange(2)
            m.set_layer_fusion(2)
            m.kernel_timing(True)
            one = m.forward(x, k, flavour == 1)
            r1 = m.last_routing(n, k)
            launched = {name for name, (_, cnt) in m.kernel_times().items() if cnt}
            m.kernel_timing(False)
            assert launched == {"decode_layer", "combine"}, launched
            assert m.router_exchange_state()[1] == 0, "no workgroup should have had to give up waiting"
            m.set_router_exchange(2, 0)  # nobody waits: every workgroup computes all logits and all hidden blocks itself
            alone = m.forward(x, k, flavour == 1)
            assert m.router_exchange_state()[1] > 0
            m.set_router_exchange(2)
            m.set_layer_fusion(False)
            two = m.forward(x, k, flavour == 1)
            m.set_router_exchange(False)
            three = m.forward(x, k, flavour == 1)
            r3 = m.last_routing(n, k)
            assert np.array_equal(r1[0], r3[0]) and np.array_equal(bits(r1[1]), bits(r3[1])), f"{n} tokens: routing"
            assert np.array_equal(bits(one), bits(three)), f"{n} tokens"
            assert np.array_equal(bits(two), bits(three)), f"{n} tokens, two launches"
            assert np.array_equal(bits(alone), bits(three)), f"{n} tokens, no exchange"
        # and the routing is the oracle's, the output within the quantized banks' tolerance of the f64 product
        router, gate, up, down, _ = kept[0]
        banks = orc.LayerBanks(H, I, E, gate, up, down, gt, gt, dt)
        rtype = {M.F32: orc.F32, M.F16: orc.F16, M.BF16: orc.BF16}[rt]
        _, ids, w, _ = orc.moe_forward(banks, router, rtype, x, k, flavour == 1, flavour)
        assert np.array_equal(r1[0], ids.astype(np.int32)) and np.array_equal(bits(r1[1]), bits(w))
        want, mag = orc.moe_ref_f64(banks, ids, w, x)
        assert float(orc.rel_err(one, want, mag).max()) <= 2e-3


def test_stack_with_the_norm_inside_the_one_launch_form():
    H, I, E, k, L = 2048, 256, 64, 8, 3
    m, g, _ = make(H, I, E, k, M.Q8_0, M.Q8_0, M.F16, 7500, layers=L)
    with m:
        for n in (1, 5):
            x = (3.0 * g.standard_normal((n, H), dtype=np.float32)).astype(np.float32)
            m.set_router_exchange(2)
            m.set_layer_fusion(2)
            one, ids1 = m.stack_forward(x, k, False, return_ids=True)
            m.set_router_exchange(False)
            three, ids3 = m.stack_forward(x, k, False, return_ids=True)
            assert np.array_equal(ids1, ids3)
            assert np.array_equal(bits(one), bits(three)), f"{n} tokens"
        assert m.router_exchange_state()[1] == 0


def test_graph_replays_of_the_one_launch_form():
    # every step moves the exchange's epoch on and every captured launch has a salt of its own: blocks of the step or
    # the replay before must never be taken for fresh ones
    H, I, E, k = 2048, 1024, 64, 8
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, M.F16, 7600)
    with m:
        xs = [g.standard_normal((1, H), dtype=np.float32) for _ in range(4)]
        m.set_router_exchange(False)
        want = [m.forward(x, k, False) for x in xs]
        m.set_router_exchange(True)
        m.set_layer_fusion(2)
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
            # new inputs through the same buffers: stale blocks of the previous replay would show here
            xs = [g.standard_normal((1, H), dtype=np.float32) for _ in range(4)]
            m.set_router_exchange(False)
            want = [m.forward(x, k, False) for x in xs]
            m.set_router_exchange(True)
            for d, x in zip(xd, xs):
                d.upload(x)
        graph.close()
        assert m.router_exchange_state()[1] == 0


def test_shared_expert_beside_the_one_launch_form():
    H, I, E, k, IS = 1024, 512, 32, 8, 512
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, M.F16, 7700)
    with m:
        sh = [synth.random_bank_fast(M.Q4_K, ne, 7700 + 50 + j) for j, ne in enumerate(([H, IS, 1], [H, IS, 1], [IS, H, 1]))]
        gate_vec = (g.standard_normal(H, dtype=np.float32) * np.float32(0.05)).astype(np.float32)
        m.load_shared_expert(0, IS, sh[0], M.Q4_K, sh[1], M.Q4_K, sh[2], M.Q4_K, gate_vec)
        for n in (1, 4):
            x = g.standard_normal((n, H), dtype=np.float32)
            m.set_router_exchange(2)
            m.set_layer_fusion(2)
            one = m.forward(x, k, False)
            m.set_router_exchange(False)
            three = m.forward(x, k, False)
            assert np.array_equal(bits(one), bits(three)), f"{n} tokens"


def test_deferred_sums_give_the_same_bits_eagerly_and_in_graph_replays():
    # the sum over a step's eight rows done by the NEXT step's launch: a chain of eager calls ended by flush / check,
    # and a captured graph (whose last node is the last step's sum), each against the three-launch form
    H, I, E, k = 2048, 1024, 64, 8
    m, g, _ = make(H, I, E, k, M.Q4_K, M.Q4_K, M.F16, 7800, layers=2)
    with m:
        for n in (1, 3):
            xs = [g.standard_normal((n, H), dtype=np.float32) for _ in range(5)]
            m.set_router_exchange(False)
            want = [m.forward(x, k, False, layer=i % 2) for i, x in enumerate(xs)]
            m.set_router_exchange(2)
            m.set_deferred_combine(True)
            xd = [M.DeviceBuffer.from_array(x) for x in xs]
            od = [M.DeviceBuffer(n * H * 4) for _ in xs]
            for o in od:
                o.upload(np.full((n, H), 7.0, np.float32))
            m.kernel_timing(True)
            for i, (x, o) in enumerate(zip(xd, od)):
                m.forward_device(i % 2, x, n, k, False, o)
            m.check()  # enqueues the last step's sum
            counts = {name: cnt for name, (_, cnt) in m.kernel_times().items() if cnt}
            m.kernel_timing(False)
            assert counts == {"decode_layer": 5, "combine": 1}, counts
            for i, (o, w) in enumerate(zip(od, want)):
                assert np.array_equal(bits(o.download(np.float32, (n, H))), bits(w)), (n, i)
            # the routing of the last call is the one last_routing reports
            m.set_router_exchange(False)
            m.forward(xs[-1], k, False, layer=0)
            r3 = m.last_routing(n, k)
            m.set_router_exchange(2)
            m.forward_device(0, xd[-1], n, k, False, od[-1])
            r1 = m.last_routing(n, k)
            assert np.array_equal(r1[0], r3[0]) and np.array_equal(bits(r1[1]), bits(r3[1]))
            # a graph of the same steps, replayed with new inputs
            m.graph_begin()
            for i, (x, o) in enumerate(zip(xd, od)):
                m.forward_device(i % 2, x, n, k, False, o)
            graph = m.graph_end()
            for rep in range(4):
                for o in od:
                    o.upload(np.zeros((n, H), np.float32))
                graph.launch()
                m.check()
                for i, (o, w) in enumerate(zip(od, want)):
                    assert np.array_equal(bits(o.download(np.float32, (n, H))), bits(w)), (n, rep, i)
                xs = [g.standard_normal((n, H), dtype=np.float32) for _ in range(5)]
                m.set_router_exchange(False)
                want = [m.forward(x, k, False, layer=i % 2) for i, x in enumerate(xs)]
                m.set_router_exchange(2)
                for d, x in zip(xd, xs):
                    d.upload(x)
            graph.close()
            m.set_deferred_combine(False)
        assert m.router_exchange_state()[1] == 0


def test_a_deferred_step_that_reads_the_pending_output_waits_for_it():
    # x of a step = out of the step before: the pending sum must be enqueued ahead of the launch, not inside it
    H, I, E, k = 1024, 512, 32, 8
    m, g, _ = make(H, I, E, k, M.Q8_0, M.Q8_0, M.F16, 7900)
    with m:
        x = g.standard_normal((1, H), dtype=np.float32)
        m.set_router_exchange(False)
        y1 = m.forward(x, k, False)
        y2 = m.forward(y1, k, False)
        m.set_router_exchange(True)
        m.set_deferred_combine(True)
        a, b, c = M.DeviceBuffer.from_array(x), M.DeviceBuffer(H * 4), M.DeviceBuffer(H * 4)
        m.forward_device(0, a, 1, k, False, b)
        m.forward_device(0, b, 1, k, False, c)
        m.check()
        assert np.array_equal(bits(b.download(np.float32, (1, H))), bits(y1))
        assert np.array_equal(bits(c.download(np.float32, (1, H))), bits(y2))
