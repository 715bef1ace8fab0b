"""Pins the oracle's router (softmax / top-k / renorm), its dot products and its expf against
the reference's own known answers (models/qwen4exp/experts.rs:1365-1427), brute force on
tiny inputs, and higher-precision arithmetic."""
import math

import numpy as np
import pytest

from mummu_amd import synth
from oracle import binding as orc
from tests.helpers import ulp_diff


# --- expf -------------------------------------------------------------------------------

def test_expf_is_within_2_ulp_of_exact_over_a_dense_sweep():
    xs = np.concatenate([np.linspace(-104.5, 89.0, 40001), np.linspace(-1.0, 1.0, 20001),
                         np.array([0.0, -0.0, 1e-8, -1e-8, 88.72, -87.3, -87.4, -100.0, -103.9])]).astype(np.float32)
    got = orc.expf_array(xs)
    want64 = np.exp(xs.astype(np.float64))
    want = want64.astype(np.float32)
    fin = np.isfinite(want) & (want64 > 2e-38)  # normal results
    assert ulp_diff(got[fin], want[fin]).max() <= 2
    sub = (want64 <= 2e-38) & (want64 > 0)
    assert np.all(np.abs(got[sub].astype(np.float64) - want64[sub]) <= 3 * 1.4e-45)  # subnormal grid
    assert orc.expf(0.0) == 1.0
    assert orc.expf(89.0) == math.inf and orc.expf(-104.0) == 0.0 and math.isnan(orc.expf(math.nan))
    assert orc.expf(math.inf) == math.inf and orc.expf(-math.inf) == 0.0


def test_expf_is_monotone_on_the_softmax_range():
    xs = np.linspace(-30.0, 0.0, 200001).astype(np.float32)
    got = orc.expf_array(xs)
    assert np.all(np.diff(got) >= 0)


def test_silu_matches_the_closed_form_and_saturates_cleanly():
    # experts.rs:480-487: very negative x gives a clean -0.0, never NaN
    for x in [-20.0, -1.0, -0.1, 0.0, 0.3, 2.0, 15.0]:
        want = x / (1.0 + math.exp(-x))
        assert abs(orc.silu(x) - want) <= 1e-6 * max(1.0, abs(want))
    v = orc.silu(-200.0)
    assert v == 0.0 and math.copysign(1.0, v) == -1.0


# --- the 8-lane dot (experts.rs:463-478) --------------------------------------------------

def py_dot(a, b):
    f = np.float32
    acc = [f(0)] * 8
    n = len(a)
    for c in range(n // 8):
        for l in range(8):
            acc[l] = f(acc[l] + f(a[c * 8 + l] * b[c * 8 + l]))
    s = f(f(f(acc[0] + acc[4]) + f(acc[1] + acc[5])) + f(f(acc[2] + acc[6]) + f(acc[3] + acc[7])))
    for i in range(n // 8 * 8, n):
        s = f(s + f(a[i] * b[i]))
    return s


@pytest.mark.parametrize("n", [1, 7, 8, 9, 64, 100, 259])
def test_dot_follows_the_fixed_eight_lane_order(n):
    rng = synth.SplitMix64(n)
    a, b = rng.uniform_vec(n), rng.uniform_vec(n)
    assert np.float32(orc.dot(a, b)).view(np.uint32) == py_dot(a, b).view(np.uint32)


def py_router_dot(x, w):
    f = np.float32
    acc = [0.0] * 512  # fma emulated exactly: f64 product of two f32 is exact, one rounding to f32
    for i in range(len(x)):
        acc[i % 512] = float(f(float(x[i]) * float(w[i]) + acc[i % 512]))
    s = []
    for l in range(64):
        a = [f(v) for v in acc[l * 8:l * 8 + 8]]
        s.append(f(f(f(a[0] + a[4]) + f(a[1] + a[5])) + f(f(a[2] + a[6]) + f(a[3] + a[7]))))
    off = 1
    while off < 64:  # pairwise tree over adjacent group sums
        for l in range(0, 64, 2 * off):
            s[l] = f(s[l] + s[l + off])
        off *= 2
    return s[0]


@pytest.mark.parametrize("n", [4, 256, 512, 520, 2048])
def test_router_dot_order_and_value(n):
    rng = synth.SplitMix64(100 + n)
    x = rng.normal(n)
    w = rng.normal(n, 0.0, 0.02)
    got = np.float32(orc.router_dot(x, w, orc.F32))
    # the f64 product of two f32 values is exact and |acc| is far smaller than 2^29 ulps of
    # it, so rounding (product + acc) from f64 to f32 equals the single rounding of an fma
    # except on double-rounding ties, which these inputs do not hit
    assert got.view(np.uint32) == py_router_dot(x, w).view(np.uint32)
    exact = float(np.dot(x.astype(np.float64), w.astype(np.float64)))
    rss = float(np.sqrt(np.sum((x.astype(np.float64) * w.astype(np.float64)) ** 2)))
    assert abs(float(got) - exact) <= 1e-6 * max(abs(exact), rss)


def test_router_dot_converts_f16_and_bf16_weights_exactly():
    rng = synth.SplitMix64(5)
    x = rng.normal(2048)
    w = rng.normal(2048, 0.0, 0.02)
    w16 = w.astype(np.float16)
    assert orc.router_dot(x, w16, orc.F16) == orc.router_dot(x, w16.astype(np.float32), orc.F32)
    bf = synth.encode_float(w, synth.BF16).view(np.uint16)
    back = (bf.astype(np.uint32) << 16).view(np.float32)
    assert orc.router_dot(x, bf, orc.BF16) == orc.router_dot(x, back, orc.F32)


# --- qwen4exp router known answers (experts.rs:1365-1427) ----------------------------------

def test_the_router_picks_the_most_probable_and_renormalizes_without_scale():
    ids, w = orc.route_ggml([0.0, 3.0, 1.0, 2.5, -2.0, 2.0, 0.5, 2.9], 1, 8, 3)
    assert ids[0].tolist() == [1, 7, 3]
    z = math.exp(3.0) + math.exp(2.9) + math.exp(2.5)
    for g, l in zip(w[0], [3.0, 2.9, 2.5]):
        assert abs(float(g) - math.exp(l) / z) < 1e-6
    assert abs(float(w[0].sum()) - 1.0) < 1e-6


def test_router_ties_go_to_the_lowest_expert_id():
    ids, w = orc.route_ggml([0.5] * 8, 1, 8, 3)
    assert ids[0].tolist() == [0, 1, 2]
    assert np.all(np.abs(w - 1.0 / 3.0) < 1e-6)
    ids, _ = orc.route_ggml([1.0, 0.0, 2.0, 1.0], 1, 4, 2)
    assert ids[0].tolist() == [2, 0]
    ids, _ = orc.route_olmoe([1.0, 0.0, 2.0, 1.0], 1, 4, 2, False)
    assert ids[0].tolist() == [2, 0]


def test_router_is_stable_for_huge_logits_and_many_tokens():
    lg = np.full(3 * 16, -1000.0, dtype=np.float32)
    lg[5] = 1000.0
    lg[16 + 9] = 999.0
    lg[16 + 3] = 998.0
    lg[32 + 15] = 30.0
    ids, w = orc.route_ggml(lg, 3, 16, 2)
    assert ids[0, 0] == 5 and ids[1].tolist() == [9, 3] and ids[2, 0] == 15
    assert np.all(np.isfinite(w)) and np.all(np.abs(w.sum(axis=1) - 1.0) < 1e-6)
    e = math.e
    assert abs(float(w[1, 0]) - e / (e + 1.0)) < 1e-6


def test_router_refuses_non_finite_logits_and_bad_k():
    with pytest.raises(orc.OracleError, match="token 0 expert 1"):
        orc.route_ggml([0.0, math.nan, 1.0, 2.0], 2, 2, 1)
    for k in (0, 5):
        with pytest.raises(orc.OracleError):
            orc.route_ggml([0.0] * 4, 1, 4, k)
    with pytest.raises(orc.OracleError):
        orc.route_ggml([0.0] * 5, 1, 4, 2)
    with pytest.raises(orc.OracleError):
        orc.route_olmoe([0.0, math.inf, 1.0, 2.0], 1, 4, 2, False)


def test_a_vanishing_weight_sum_is_clamped_like_llama_cpp():
    # experts.rs:1419-1427
    w = orc.renormalize_ggml([1e-6, 2e-6])
    assert abs(float(w[0]) - 1e-6 / (1.0 / 16384.0)) < 1e-9
    assert orc.renormalize_ggml([0.25, 0.25]).tolist() == [0.5, 0.5]


# --- brute force on small random inputs ----------------------------------------------------

@pytest.mark.parametrize("flavour", ["ggml", "olmoe", "olmoe_norm"])
def test_routing_matches_an_argsort_brute_force(flavour):
    rng = synth.SplitMix64(77)
    n, e, k = 200, 16, 4
    lg = rng.uniform(-3.0, 3.0, n * e).reshape(n, e)
    lg[::7, 3] = lg[::7, 9]  # plant exact ties
    if flavour == "ggml":
        ids, w = orc.route_ggml(lg, n, e, k)
    else:
        ids, w = orc.route_olmoe(lg, n, e, k, flavour == "olmoe_norm")
    p = np.exp(lg.astype(np.float64) - lg.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    for t in range(n):
        order = sorted(range(e), key=lambda a: (-lg[t, a], a))  # exp is monotone: same order, lower id first
        assert ids[t].tolist() == order[:k], t
        sel = p[t, order[:k]]
        want = sel / sel.sum() if flavour != "olmoe" else sel
        assert np.allclose(w[t], want, rtol=2e-6, atol=1e-9)
        assert len(set(ids[t].tolist())) == k
        assert np.all(np.diff(w[t]) <= 0)
