"""The entry point that allocates nothing (mummu_moe_forward_device_noalloc) against the entry point it is a variant
of (mummu_moe_forward_device), through the C ABI: same result bits on two calls in a row, the second with fewer
tokens, and its limits refused with a message."""
import numpy as np
import pytest

from mummu_amd import _lib
from mummu_amd import moe as M
from mummu_amd import synth

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("H,I,E,k,gt,dt", [(2048, 1024, 64, 8, M.Q4_K, M.Q4_K), (512, 256, 16, 4, M.Q8_0, M.Q6_K)],
                         ids=["olmoe-q4k", "small-q8_0-q6k"])
def test_noalloc_forward_gives_the_bits_of_forward_device_on_two_calls_in_a_row(H, I, E, k, gt, dt):
    gate = synth.random_bank_fast(gt, [H, I, E], 901)
    up = synth.random_bank_fast(gt, [H, I, E], 902)
    down = synth.random_bank_fast(dt, [I, H, E], 903)
    g = np.random.Generator(np.random.PCG64(904))
    router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=8) as m:
        m.load_layer(0, router, M.F16, gate, gt, up, gt, down, dt)
        # the second call is smaller: whatever the first left in the static array must not leak in; one token takes the
        # two-launch form, whose logit table and epoch live in the static array as well
        for n in (8, 3, 1, 1):
            x = g.standard_normal((n, H), dtype=np.float32)
            xd = M.DeviceBuffer.from_array(x)
            want_d, got_d = M.DeviceBuffer(x.nbytes), M.DeviceBuffer(x.nbytes)
            got_d.upload(np.full((n, H), np.nan, np.float32))
            m.forward_device(0, xd, n, k, False, want_d)
            m.check()
            want = want_d.download(np.float32, (n, H))
            m.forward_device_noalloc(0, xd, n, k, False, got_d)
            m.check()
            got = got_d.download(np.float32, (n, H))
            assert np.all(np.isfinite(got))
            assert np.array_equal(bits(got), bits(want)), f"{n} tokens"
            assert np.array_equal(bits(want), bits(m.forward(x, k, False)))


def test_noalloc_forward_with_the_logit_table_at_every_offset_under_graph_capture_and_on_two_handles():
    # The static array is carved per call: with the two-launch form forced at every size, the router's logit table lands
    # behind buffers whose size follows the token count and top_k, on bytes that earlier calls used for activations.
    # Calls captured into a graph (what the entry point is for) and two handles taking turns on one stream share it too.
    H, I, E = 1024, 512, 32
    g = np.random.Generator(np.random.PCG64(911))
    handles = []
    for j in range(2):
        gate = synth.random_bank_fast(M.Q4_K, [H, I, E], 920 + 3 * j)
        up = synth.random_bank_fast(M.Q4_K, [H, I, E], 921 + 3 * j)
        down = synth.random_bank_fast(M.Q4_K, [I, H, E], 922 + 3 * j)
        router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.05)).astype(np.float16)
        m = M.SparseMoe(M.SparseMoeConfig(H, I, E, 8), max_tokens=8)
        m.load_layer(0, router, M.F16, gate, M.Q4_K, up, M.Q4_K, down, M.Q4_K)
        handles.append(m)
    try:
        a, b = handles
        for m in handles:
            m.set_router_exchange(2)
        for n, k in ((8, 8), (3, 4), (1, 8), (5, 2), (1, 4)):
            x = g.standard_normal((n, H), dtype=np.float32)
            xd = M.DeviceBuffer.from_array(x)
            for m in (a, b, a):  # taking turns: each call finds the other handle's data in the array
                got_d = M.DeviceBuffer(x.nbytes)
                got_d.upload(np.full((n, H), np.nan, np.float32))
                m.forward_device_noalloc(0, xd, n, k, False, got_d)
                m.check()
                assert np.array_equal(bits(got_d.download(np.float32, (n, H))), bits(m.forward(x, k, False))), (n, k)
        assert a.router_exchange_state()[1] == 0 and b.router_exchange_state()[1] == 0
        # captured: three calls of different sizes in one graph, replayed with fresh inputs
        shapes = ((1, 8), (4, 8), (2, 4))
        xs = [g.standard_normal((n, H), dtype=np.float32) for n, _ in shapes]
        xd = [M.DeviceBuffer.from_array(x) for x in xs]
        od = [M.DeviceBuffer(x.nbytes) for x in xs]
        a.graph_begin()
        for (n, k), x, o in zip(shapes, xd, od):
            a.forward_device_noalloc(0, x, n, k, False, o)
        graph = a.graph_end()
        for rep in range(3):
            for o, x in zip(od, xs):
                o.upload(np.full(x.shape, np.nan, np.float32))
            graph.launch()
            a.check()
            for (n, k), x, o in zip(shapes, xs, od):
                assert np.array_equal(bits(o.download(np.float32, (n, H))), bits(a.forward(x, k, False))), (rep, n, k)
            xs = [g.standard_normal((n, H), dtype=np.float32) for n, _ in shapes]
            for d, x in zip(xd, xs):
                d.upload(x)
        graph.close()
    finally:
        for m in handles:
            m.close()


def test_noalloc_forward_refuses_what_it_cannot_hold():
    H, I, E, k = 256, 64, 8, 2
    rng = synth.SplitMix64(5)
    q = [synth.synth_bank(synth.Q8_0, ne, rng) for ne in ([H, I, E], [H, I, E], [I, H, E])]
    f = [synth.dense_bank(synth.F16, ne, rng) for ne in ([H, I, E], [H, I, E], [I, H, E])]
    router = rng.normal(E * H, 0.0, 0.05).astype(np.float16).reshape(E, H)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=2, max_tokens=16) as m:
        m.load_layer(0, router, M.F16, q[0], M.Q8_0, q[1], M.Q8_0, q[2], M.Q8_0)
        m.load_layer(1, router, M.F16, f[0], M.F16, f[1], M.F16, f[2], M.F16)
        xd, od = M.DeviceBuffer(16 * H * 4), M.DeviceBuffer(16 * H * 4)
        with pytest.raises(M.MoeError, match="at most 8 tokens") as e:
            m.forward_device_noalloc(0, xd, 9, k, False, od)
        assert e.value.code == _lib.ERR_TOKENS
        with pytest.raises(M.MoeError, match="decode form only") as e:
            m.forward_device_noalloc(1, xd, 2, k, False, od)  # float banks
        assert e.value.code == _lib.ERR_CONFIG
        m.forward_device_noalloc(0, xd, 0, k, False, od)  # nothing to do
        with pytest.raises(M.MoeError):
            m.forward_device_noalloc(0, xd, 2, 0, False, od)
