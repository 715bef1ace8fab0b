"""The fused decode launches (one launch per layer, or router + gate/up in one) start a slot's rows on the expert whose LOGIT has the slot's rank and confirms that pick
against the routing proper (softmax -> top-8 on probabilities, the lower id on a tie: experts.rs:557-573,
nn/moe.rs:2143-2144) while the rows are on their way.  Logits built so that the two orders differ - two different
logits whose probabilities round to the same float, inside the top eight and across its boundary - must take the
slot's second pass and still give the routing and the output bits of the three-launch form, which routes first."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth

pytestmark = pytest.mark.gpu

H, I, E, K = 2048, 256, 64, 8


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def logit_order(l):
    """The eight largest logits, larger first, the lower id on equal values: the early pick."""
    return sorted(range(len(l)), key=lambda e: (-float(l[e]), e))[:8]


def softmax_order(l):
    """Top-8 of the f32 softmax, the lower id on equal probabilities (what the routing does)."""
    l = np.asarray(l, dtype=np.float32)
    p = np.exp((l - l.max()).astype(np.float32)).astype(np.float32)
    return sorted(range(len(l)), key=lambda e: (-float(p[e]), e))[:8]


def cases():
    tiny, tiny2 = np.float32(1e-30), np.float32(2e-30)
    out = {}
    # inside the top eight: expert 40 has the larger logit, expert 10 the same probability and the lower id
    l = np.full(E, -6.0, np.float32)
    l[[3, 7, 21, 33, 50, 63]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75]
    l[10], l[40] = tiny, tiny2
    out["order inside the eight"] = l
    # across the boundary: seven clear winners, then 40 (larger logit) against 10 (same probability, lower id)
    l = np.full(E, -6.0, np.float32)
    l[[3, 7, 21, 33, 50, 63, 12]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75, 0.5]
    l[10], l[40] = tiny, tiny2
    out["the eighth place"] = l
    # three of them, two places left
    l = np.full(E, -6.0, np.float32)
    l[[3, 7, 21, 33, 50, 63]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75]
    l[9], l[30], l[55] = tiny, np.float32(3e-30), tiny2
    out["three for two places"] = l
    # plain ties (equal logits): both orders agree, no second pass
    l = np.full(E, 0.25, np.float32)
    out["all equal"] = l
    return out


@pytest.mark.parametrize("flavour", [0, 1])
def test_the_early_pick_is_corrected_where_probabilities_tie(flavour):
    g = np.random.Generator(np.random.PCG64(9900 + flavour))
    table = cases()
    # precondition: the crafted logits really separate the two orders (but for the plain ties)
    for name, l in table.items():
        assert (logit_order(l) != softmax_order(l)) == (name != "all equal"), name
    m = M.SparseMoe(M.SparseMoeConfig(H, I, E, K), num_layers=1, max_tokens=8, rms_norm_eps=1e-5, router_flavour=flavour)
    gate = synth.random_bank_fast(M.Q4_K, [H, I, E], 9901)
    up = synth.random_bank_fast(M.Q4_K, [H, I, E], 9902)
    down = synth.random_bank_fast(M.Q4_K, [I, H, E], 9903)
    # an F32 router whose column j holds case j's logits: the one-hot token e_j gets exactly them
    router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.05)).astype(np.float32)
    names = list(table)
    for j, name in enumerate(names):
        router[:, 100 + j] = table[name]
    m.load_layer(0, router, M.F32, gate, M.Q4_K, up, M.Q4_K, down, M.Q4_K)
    with m:
        for j, name in enumerate(names):
            x = np.zeros((1, H), np.float32)
            x[0, 100 + j] = 1.0
            for norm in (False, True):
                m.set_router_exchange(False)      # three launches: routes first
                want = m.forward(x, K, norm)
                ids3, w3 = m.last_routing(1, K)
                assert list(ids3[0]) == softmax_order(table[name]), name
                m.set_router_exchange(True)
                m.set_layer_fusion(2)             # one launch, its sum as a launch of its own
                got = m.forward(x, K, norm)
                ids1, w1 = m.last_routing(1, K)
                assert np.array_equal(ids1, ids3), name
                assert np.array_equal(bits(w1), bits(w3)), name
                assert np.array_equal(bits(got), bits(want)), name
                m.set_layer_fusion(0)             # two launches: the fused gate/up kernel makes the same early pick
                got2 = m.forward(x, K, norm)
                ids2, w2 = m.last_routing(1, K)
                m.set_layer_fusion(2)
                assert np.array_equal(ids2, ids3) and np.array_equal(bits(w2), bits(w3)), name
                assert np.array_equal(bits(got2), bits(want)), name
                # and in a chain of deferred sums, where the weights reach the output through the next launch
                m.set_deferred_combine(True)
                a, o1, o2 = M.DeviceBuffer.from_array(x), M.DeviceBuffer(H * 4), M.DeviceBuffer(H * 4)
                m.forward_device(0, a, 1, K, norm, o1)
                m.forward_device(0, a, 1, K, norm, o2)
                m.check()
                assert np.array_equal(bits(o1.download(np.float32, (1, H))), bits(want)), name
                assert np.array_equal(bits(o2.download(np.float32, (1, H))), bits(want)), name
                m.set_deferred_combine(False)
                m.set_layer_fusion(1)
        assert m.router_exchange_state()[1] == 0


def test_random_tokens_route_alike_with_and_without_the_early_pick():
    g = np.random.Generator(np.random.PCG64(9950))
    m = M.SparseMoe(M.SparseMoeConfig(H, I, E, K), num_layers=1, max_tokens=8, rms_norm_eps=1e-5)
    gate = synth.random_bank_fast(M.Q8_0, [H, I, E], 9951)
    up = synth.random_bank_fast(M.Q8_0, [H, I, E], 9952)
    down = synth.random_bank_fast(M.Q8_0, [I, H, E], 9953)
    # a coarse router (few distinct values) makes equal and near-equal logits common
    router = (np.round(g.standard_normal((E, H)) * 2.0) / 64.0).astype(np.float16)
    m.load_layer(0, router, M.F16, gate, M.Q8_0, up, M.Q8_0, down, M.Q8_0)
    with m:
        for rep in range(24):
            x = np.round(g.standard_normal((1, H)) * 2.0).astype(np.float32)
            m.set_router_exchange(False)
            want = m.forward(x, K, True)
            ids3, w3 = m.last_routing(1, K)
            m.set_router_exchange(True)
            m.set_layer_fusion(2)
            got = m.forward(x, K, True)
            ids1, w1 = m.last_routing(1, K)
            m.set_layer_fusion(0)
            got2 = m.forward(x, K, True)
            ids2, w2 = m.last_routing(1, K)
            m.set_layer_fusion(1)
            assert np.array_equal(ids2, ids3) and np.array_equal(bits(w2), bits(w3)) and np.array_equal(bits(got2), bits(want)), rep
            assert np.array_equal(ids1, ids3), rep
            assert np.array_equal(bits(w1), bits(w3)), rep
            assert np.array_equal(bits(got), bits(want)), rep
        assert m.router_exchange_state()[1] == 0
