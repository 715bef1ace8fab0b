"""The decode launches that route by themselves (gate/up with the routing inside, router + gate/up in one launch, the
whole layer in one launch) start a slot's rows on the expert whose LOGIT has the slot's rank and confirm that pick
against the routing proper (softmax -> top-8 on probabilities, the lower id on a tie: experts.rs:557-573,
nn/moe.rs:2143-2144) while the rows are on their way.  Logits built so that the two orders differ - different logits
whose probabilities round to the same float, inside the top eight and across its last place - must take the slot's
second pass and still give the routing and the output bits of a handle that routes first (MUMMU_EARLY_IDS=0), in the
three-, two- and one-launch forms, one token at a time and as a decode batch."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth

pytestmark = pytest.mark.gpu

H, I, K = 2048, 256, 8


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


def cases(E):
    f = E // 64   # (with 128 experts the same places doubled: both experts of a routing lane take part)
    tiny, tiny2 = np.float32(1e-30), np.float32(2e-30)
    out = {}
    # inside the top eight: expert 40 has the larger logit, expert 10 the same probability and the lower id
    l = np.full(E, -6.0, np.float32)
    l[[3 * f, 7 * f, 21 * f, 33 * f, 50 * f, 63 * f]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75]
    l[10 * f], l[40 * f] = tiny, tiny2
    out["order inside the eight"] = l
    # across the boundary: seven clear winners, then 40 (larger logit) against 10 (same probability, lower id)
    l = np.full(E, -6.0, np.float32)
    l[[3 * f, 7 * f, 21 * f, 33 * f, 50 * f, 63 * f, 12 * f]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75, 0.5]
    l[10 * f], l[40 * f] = tiny, tiny2
    out["the eighth place"] = l
    # three of them, two places left
    l = np.full(E, -6.0, np.float32)
    l[[3 * f, 7 * f, 21 * f, 33 * f, 50 * f, 63 * f]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75]
    l[9 * f], l[30 * f], l[55 * f] = tiny, np.float32(3e-30), tiny2
    out["three for two places"] = l
    # plain ties (equal logits): both orders agree, no second pass
    l = np.full(E, 0.25, np.float32)
    out["all equal"] = l
    return out


def near_ties(E):
    """Logits a few units in the last place apart, the larger one at the higher id: the early pick, which tells experts
    apart by id below 2^7 units in the last place, may take them in the other order than the routing does - or not;
    either way the routing's answer has to come out."""
    f = E // 64
    out = {}
    for name, places, gap in (("one ulp inside", [3, 7, 21, 33, 50, 63], 1), ("forty ulps at the eighth place", [3, 7, 21, 33, 50, 63, 12], 40)):
        l = np.full(E, -6.0, np.float32)
        l[[p * f for p in places]] = [2.0, 1.75, 1.5, 1.25, 1.0, 0.75, 0.5][:len(places)]
        lo = np.float32(0.3)
        hi = lo
        for _ in range(gap):
            hi = np.nextafter(hi, np.float32(1.0))
        l[10 * f], l[40 * f] = lo, hi
        out[name] = l
    return out


def make(flavour, gt, router, rt, seed, early, E):
    """A one-layer handle; early = False: created with MUMMU_EARLY_IDS=0, every launch routes first."""
    import os
    old = os.environ.get("MUMMU_EARLY_IDS")
    os.environ["MUMMU_EARLY_IDS"] = "1" if early else "0"
    try:
        m = M.SparseMoe(M.SparseMoeConfig(H, I, E, K), num_layers=1, max_tokens=8, rms_norm_eps=1e-5, router_flavour=flavour)
    finally:
        if old is None:
            del os.environ["MUMMU_EARLY_IDS"]
        else:
            os.environ["MUMMU_EARLY_IDS"] = old
    gate = synth.random_bank_fast(gt, [H, I, E], seed + 1)
    up = synth.random_bank_fast(gt, [H, I, E], seed + 2)
    down = synth.random_bank_fast(gt, [I, H, E], seed + 3)
    m.load_layer(0, router, rt, gate, gt, up, gt, down, gt)
    return m


def forms(m, x, norm):
    """(name, output, ids, weights) of a call in the three-, two- and one-launch forms."""
    n = x.shape[0]
    out = []
    for name, exchange, fusion in (("three launches", False, 1), ("two launches", 2, 0), ("one launch", 2, 2)):
        m.set_router_exchange(exchange)
        m.set_layer_fusion(fusion)
        y = m.forward(x, K, norm)
        ids, w = m.last_routing(n, K)
        out.append((name, y, ids, w))
    m.set_router_exchange(True)
    m.set_layer_fusion(1)
    return out


@pytest.mark.parametrize("flavour,E", [(0, 64), (1, 64), (0, 128), (1, 128)])
def test_the_early_pick_is_corrected_where_probabilities_tie(flavour, E):
    g = np.random.Generator(np.random.PCG64(9900 + flavour + E))
    table = cases(E)
    # precondition: the crafted logits really separate the two orders (but for the plain ties)
    for name, l in table.items():
        assert (logit_order(l) != softmax_order(l)) == (name != "all equal"), name
    # an F32 router whose column j holds case j's logits: the one-hot token e_j gets exactly them
    router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.05)).astype(np.float32)
    extra = near_ties(E)
    table = dict(table, **extra)
    names = list(table)
    for j, name in enumerate(names):
        router[:, 100 + j] = table[name]
    ref = make(flavour, M.Q4_K, router, M.F32, 9900, False, E)
    m = make(flavour, M.Q4_K, router, M.F32, 9900, True, E)
    with ref, m:
        xs = np.zeros((len(names), H), np.float32)
        for j in range(len(names)):
            xs[j, 100 + j] = 1.0
        # one token at a time, then all of them as one decode batch (the multi-token launches)
        batches = [(name, xs[j:j + 1]) for j, name in enumerate(names)] + [("batch", xs), ("batch of eight", np.concatenate([xs[:4], xs[::-1][:4]]))]
        for name, x in batches:
            n = x.shape[0]
            for norm in (False, True):
                ref.set_router_exchange(False)
                want = ref.forward(x, K, norm)
                ids0, w0 = ref.last_routing(n, K)
                if n == 1 and name not in extra:
                    assert list(ids0[0]) == softmax_order(table[name]), name
                for form, y, ids, w in forms(m, x, norm):
                    assert np.array_equal(ids, ids0), (name, form)
                    assert np.array_equal(bits(w), bits(w0)), (name, form)
                    assert np.array_equal(bits(y), bits(want)), (name, form)
                if n > 1:
                    continue
                # and in a chain of deferred sums, where the weights reach the output through the next launch
                m.set_deferred_combine(True)
                a, o1, o2 = M.DeviceBuffer.from_array(x), M.DeviceBuffer(H * 4), M.DeviceBuffer(H * 4)
                m.forward_device(0, a, 1, K, norm, o1)
                m.forward_device(0, a, 1, K, norm, o2)
                m.check()
                assert np.array_equal(bits(o1.download(np.float32, (1, H))), bits(want)), name
                assert np.array_equal(bits(o2.download(np.float32, (1, H))), bits(want)), name
                m.set_deferred_combine(False)
        assert m.router_exchange_state()[1] == 0


@pytest.mark.parametrize("E", [64, 128])
def test_random_tokens_route_alike_with_and_without_the_early_pick(E):
    g = np.random.Generator(np.random.PCG64(9950 + E))
    # a coarse router (few distinct values) makes equal and near-equal logits common
    router = (np.round(g.standard_normal((E, H)) * 2.0) / 64.0).astype(np.float16)
    ref = make(0, M.Q8_0, router, M.F16, 9950, False, E)
    m = make(0, M.Q8_0, router, M.F16, 9950, True, E)
    with ref, m:
        for rep in range(24):
            n = 1 + rep % 8
            x = np.round(g.standard_normal((n, H)) * 2.0).astype(np.float32)
            ref.set_router_exchange(False)
            want = ref.forward(x, K, True)
            ids0, w0 = ref.last_routing(n, K)
            for form, y, ids, w in forms(m, x, True):
                assert np.array_equal(ids, ids0), (rep, form)
                assert np.array_equal(bits(w), bits(w0)), (rep, form)
                assert np.array_equal(bits(y), bits(want)), (rep, form)
        assert m.router_exchange_state()[1] == 0
