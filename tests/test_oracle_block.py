"""Pins the oracle's expert products, routed combine and whole block against the reference's
own test oracles: the closed-form toy block and its hand-rolled scalar reference
(nn/moe.rs:1617-1651, 2088-2352) and the synthetic quantized toy layers with their f64
dense-mask reference (models/qwen4exp/experts.rs:1244-1353, 1429-1563)."""
import numpy as np
import pytest

from mummu_amd import synth
from oracle import binding as orc
from tests.helpers import TOY_A, TOY_D, toy_a_input, toy_a_scalar_reference, toy_a_weights, toy_d_layers


def toy_a_banks():
    router, gate, up, down = toy_a_weights()
    banks = orc.LayerBanks(TOY_A["hidden"], TOY_A["inter"], TOY_A["experts"], gate, up, down, orc.F32)
    return router, gate, up, down, banks


@pytest.mark.parametrize("t", [5, 1])
@pytest.mark.parametrize("norm", [False, True])
def test_forward_matches_the_hand_rolled_sparse_reference(t, norm):
    # nn/moe.rs:2177-2202, tolerance 1e-5 absolute as there
    router, gate, up, down, banks = toy_a_banks()
    x = toy_a_input(t, 2.0)
    got, ids, w, _ = orc.moe_forward(banks, router, orc.F32, x, TOY_A["top_k"], norm)
    want = toy_a_scalar_reference(router, gate, up, down, x, TOY_A["top_k"], norm)
    assert np.max(np.abs(got - want)) < 1e-5
    dense = orc.moe_forward_dense_mask(banks, router, orc.F32, x, TOY_A["top_k"], norm)
    assert np.max(np.abs(dense - want)) < 1e-5  # nn/moe.rs:1655-1700: routed == dense-mask


def test_top_k_equal_to_num_experts_uses_every_expert():
    # nn/moe.rs:2204-2230
    router, gate, up, down, banks = toy_a_banks()
    x = toy_a_input(3, 0.5)
    got, ids, _, _ = orc.moe_forward(banks, router, orc.F32, x, TOY_A["experts"], False)
    want = toy_a_scalar_reference(router, gate, up, down, x, TOY_A["experts"], False)
    assert np.max(np.abs(got - want)) < 1e-5
    assert all(sorted(r.tolist()) == [0, 1, 2, 3] for r in ids)


def test_norm_topk_weights_change_the_mixture():
    # nn/moe.rs:2297-2316
    router, _, _, _, banks = toy_a_banks()
    x = toy_a_input(4, 7.0)
    a = orc.moe_forward(banks, router, orc.F32, x, 2, False)[0]
    b = orc.moe_forward(banks, router, orc.F32, x, 2, True)[0]
    assert np.any(np.abs(a - b) > 1e-7)


def test_forward_is_position_independent_bitwise():
    # nn/moe.rs:2318-2338
    router, _, _, _, banks = toy_a_banks()
    row = toy_a_input(1, 11.0)
    s = orc.moe_forward(banks, router, orc.F32, row, 2, False)[0]
    d = orc.moe_forward(banks, router, orc.F32, np.concatenate([row, row]), 2, False)[0]
    assert np.array_equal(s[0].view(np.uint32), d[0].view(np.uint32))
    assert np.array_equal(s[0].view(np.uint32), d[1].view(np.uint32))


def test_zero_input_gives_zero_output():
    # nn/moe.rs:2340-2352
    router, _, _, _, banks = toy_a_banks()
    out = orc.moe_forward(banks, router, orc.F32, np.zeros((2, 4), dtype=np.float32), 2, False)[0]
    assert np.all(out == 0.0)


def test_bad_top_k_is_refused():
    # nn/moe.rs:2354-2374
    router, _, _, _, banks = toy_a_banks()
    for k in (0, 5):
        with pytest.raises(orc.OracleError):
            orc.moe_forward(banks, router, orc.F32, toy_a_input(1, 0.0), k, False)


# --- quantized expert products (experts.rs) ------------------------------------------------

@pytest.mark.parametrize("dtype,in_dim", [(orc.Q8_0, 96), (orc.Q5_1, 64), (orc.Q4_K, 512), (orc.Q5_K, 256)])
def test_matvec_equals_dequantize_then_matmul(dtype, in_dim):
    # experts.rs:1273-1314: f64 reference, 1e-5 against max(|want|, rss)
    rng = synth.SplitMix64(0x5EED ^ in_dim ^ (orc.block_bytes(dtype) << 20))
    out_dim = (1 << 16) // in_dim * 2 + 3
    blocks = in_dim // orc.block_size(dtype) * out_dim
    per_expert = [synth.synth_blocks(dtype, blocks, rng) for _ in range(3)]
    n = 4
    xs = rng.uniform_vec(n * in_dim).reshape(n, in_dim)
    for e in (0, 2):
        w = orc.dequantize(dtype, per_expert[e]).reshape(out_dim, in_dim).astype(np.float64)
        assert np.all(np.isfinite(w))
        terms = w[None, :, :] * xs.astype(np.float64)[:, None, :]
        want = terms.sum(axis=2)
        mag = np.sqrt((terms ** 2).sum(axis=2))
        got = orc.matvec(dtype, per_expert[e], in_dim, out_dim, xs)
        assert orc.rel_err(got, want, mag).max() <= 1e-5


def test_matvec_element_is_one_fixed_order_dot_of_one_row():
    # experts.rs:1316-1353: every output is dot(row r, x_t), whatever the chunking
    rng = synth.SplitMix64(7)
    in_dim, out_dim, n = 256, 37, 3
    bank = synth.synth_bank(synth.Q4_K, [in_dim, out_dim, 2], rng)
    xs = rng.uniform_vec(n * in_dim).reshape(n, in_dim)
    e1 = bank[out_dim * 144:]
    got = orc.matvec(orc.Q4_K, e1, in_dim, out_dim, xs)
    w = orc.dequantize(orc.Q4_K, e1).reshape(out_dim, in_dim)
    for t in range(n):
        for r in (0, 5, 36):
            assert np.float32(orc.dot(w[r], xs[t])).view(np.uint32) == got[t, r].view(np.uint32)
    with pytest.raises(orc.OracleError):  # experts.rs:1355-1363: 640-wide rows cannot be K-quant
        orc.matvec(orc.Q4_K, np.zeros(1024, dtype=np.uint8), 640, 4, np.zeros((1, 640), dtype=np.float32))


def toy_d_banks(seed):
    return [orc.LayerBanks(TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"], l["gate"], l["up"], l["down"],
                           l["gate_type"], l["up_type"], l["down_type"]) for l in toy_d_layers(seed)]


def test_routed_moe_equals_the_dense_mask_reference():
    # experts.rs:1466-1532, rebuilt with numpy f64 over the whole dequantized matrices
    layers = toy_d_banks(11)
    raw = toy_d_layers(11)
    rng = synth.SplitMix64(12)
    n, H, F, E = 5, TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    xs = rng.uniform_vec(n * H).reshape(n, H)
    logits = rng.uniform(-2.0, 2.0, n * E).reshape(n, E)
    for li, (banks, r) in enumerate(zip(layers, raw)):
        ids, w = orc.route_ggml(logits, n, E, 2)
        got = orc.apply_routing(banks, ids, w, xs)
        wg = orc.dequantize(r["gate_type"], r["gate"]).reshape(E, F, H).astype(np.float64)
        wu = orc.dequantize(r["up_type"], r["up"]).reshape(E, F, H).astype(np.float64)
        wd = orc.dequantize(r["down_type"], r["down"]).reshape(E, H, F).astype(np.float64)
        want = np.zeros((n, H))
        mag = np.zeros((n, H))
        for tok in range(n):
            p = np.exp(logits[tok].astype(np.float64))
            p /= p.sum()
            order = sorted(range(E), key=lambda e: (-p[e], e))[:2]
            top = p[order].sum()
            x = xs[tok].astype(np.float64)
            for e in order:
                g = wg[e] @ x
                u = wu[e] @ x
                hid = (g / (1.0 + np.exp(-g)) * u).astype(np.float32).astype(np.float64)
                terms = wd[e] * hid[None, :]
                want[tok] += p[e] / top * terms.sum(axis=1)
                mag[tok] += p[e] / top * np.sqrt((terms ** 2).sum(axis=1))
        assert orc.rel_err(got, want, mag).max() <= 1e-5, li
        # the oracle's own f64 reference is the same computation: pin it too
        w64, m64 = orc.moe_ref_f64(banks, ids, w, xs)
        # (it takes the f32 routing weights, the numpy one f64 probabilities: 1e-6 covers that)
        assert orc.rel_err(w64, want, mag).max() <= 1e-6 and np.allclose(m64, mag, rtol=1e-6, atol=1e-12)


def test_a_token_routes_bit_identically_alone_or_in_a_batch():
    # experts.rs:1534-1563
    banks = toy_d_banks(21)[0]
    rng = synth.SplitMix64(22)
    n, H, E = 6, TOY_D["hidden"], TOY_D["experts"]
    xs = rng.uniform_vec(n * H).reshape(n, H)
    logits = rng.uniform(-3.0, 3.0, n * E).reshape(n, E)
    ids, w = orc.route_ggml(logits, n, E, 3)
    batch = orc.apply_routing(banks, ids, w, xs)
    for t in range(n):
        i1, w1 = orc.route_ggml(logits[t], 1, E, 3)
        one = orc.apply_routing(banks, i1, w1, xs[t:t + 1])
        assert np.array_equal(one[0].view(np.uint32), batch[t].view(np.uint32))


def test_hits_count_rows_served_and_combine_is_ascending_expert_two_roundings():
    # nn/moe.rs:1562-1564 (hit counters), :1590-1601 and experts.rs:1137-1148 (combine order)
    banks = toy_d_banks(31)[1]
    rng = synth.SplitMix64(33)
    n, H, E, k = 7, TOY_D["hidden"], TOY_D["experts"], 3
    xs = rng.uniform_vec(n * H).reshape(n, H)
    logits = rng.uniform(-2.0, 2.0, n * E).reshape(n, E)
    ids, w = orc.route_ggml(logits, n, E, k)
    hits = np.zeros(E, dtype=np.uint64)
    got = orc.apply_routing(banks, ids, w, xs, hits)
    assert int(hits.sum()) == n * k
    assert hits.tolist() == np.bincount(ids.reshape(-1), minlength=E).tolist()
    want = np.zeros((n, H), dtype=np.float32)
    for e in range(E):
        for t in range(n):
            for s in range(k):
                if ids[t, s] == e:
                    y = orc.expert_ffn(banks, e, xs[t:t + 1])[0]
                    want[t] = want[t] + (w[t, s] * y).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_e2_k2_norm_reduces_to_a_softmax_weighted_pair():
    # special case: two experts, both picked, renormalised -> weights are the softmax itself
    rng = synth.SplitMix64(41)
    H, I = 64, 32
    gate = synth.dense_bank(synth.F32, [H, I, 2], rng, 0.3)
    up = synth.dense_bank(synth.F32, [H, I, 2], rng, 0.3)
    down = synth.dense_bank(synth.F32, [I, H, 2], rng, 0.3)
    router = rng.normal(2 * H, 0.0, 0.3).reshape(2, H)
    banks = orc.LayerBanks(H, I, 2, gate, up, down, orc.F32)
    x = rng.normal(3 * H).reshape(3, H)
    out, ids, w, lg = orc.moe_forward(banks, router, orc.F32, x, 2, True)
    g = gate.view(np.float32).reshape(2, I, H).astype(np.float64)
    u = up.view(np.float32).reshape(2, I, H).astype(np.float64)
    d = down.view(np.float32).reshape(2, H, I).astype(np.float64)
    for t in range(3):
        l = router.astype(np.float64) @ x[t].astype(np.float64)
        p = np.exp(l - l.max())
        p /= p.sum()
        want = np.zeros(H)
        for e in range(2):
            a = g[e] @ x[t]
            hid = a / (1 + np.exp(-a)) * (u[e] @ x[t])
            want += p[e] * (d[e] @ hid)
        assert np.allclose(out[t], want, rtol=2e-4, atol=2e-5)
        assert np.allclose(lg[t], l, rtol=1e-5, atol=1e-6)


def test_rmsnorm_and_layer_stack():
    # models/olmoe.rs:566-572: x = x + moe(rmsnorm(x)); closed form for the norm
    rng = synth.SplitMix64(51)
    H, I, E, k, n, L = 256, 32, 8, 2, 3, 2
    x = rng.normal(n * H).reshape(n, H)
    gamma = (1.0 + 0.1 * rng.normal(H)).astype(np.float32)
    got = orc.rmsnorm(x, gamma, 1e-5)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * gamma
    assert np.allclose(got, want, rtol=2e-6, atol=1e-7)
    raw = toy_d_layers(52)
    layers = [orc.LayerBanks(H, I, E, r["gate"], r["up"], r["down"], r["gate_type"], r["up_type"], r["down_type"]) for r in raw]
    routers = [rng.normal(E * H, 0.0, 0.05).reshape(E, H) for _ in range(L)]
    gammas = [gamma, gamma[::-1].copy()]
    out, ids = orc.layer_stack(layers, routers, orc.F32, gammas, 1e-5, x, k, False)
    cur = x.copy()
    for l in range(L):
        h2 = orc.rmsnorm(cur, gammas[l], 1e-5)
        moe, i_l, _, _ = orc.moe_forward(layers[l], routers[l], orc.F32, h2, k, False)
        assert np.array_equal(i_l, ids[l])
        cur = (cur + moe).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), cur.view(np.uint32))


# --- gate energy (nn/moe.rs:508-521) --------------------------------------------------------

def energy_f64(gate_f32, xs):
    """sum_i silu(x . g_i)^2 in f64 on the dequantized gate rows [I, H]."""
    pre = xs.astype(np.float64) @ gate_f32.astype(np.float64).T
    s = pre / (1.0 + np.exp(-pre))
    return (s * s).sum(axis=1)


@pytest.mark.parametrize("which", [0, 1])
def test_gate_energy_is_the_sum_of_squared_silu_gate_activations(which):
    raw = toy_d_layers(11)[which]
    H, F, E = TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    banks = orc.LayerBanks(H, F, E, raw["gate"], raw["up"], raw["down"], raw["gate_type"], raw["up_type"], raw["down_type"])
    xs = synth.SplitMix64(21).uniform_vec(6 * H).reshape(6, H)
    gate = orc.dequantize(raw["gate_type"], raw["gate"]).reshape(E, F, H)
    for e in (0, E - 1):
        got = orc.gate_energy(banks, e, xs)
        want = energy_f64(gate[e], xs)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(want, 1e-30))
    # an expert's energy does not depend on which rows share the call, and zero rows have none
    assert np.array_equal(orc.gate_energy(banks, 2, xs[3:4]), orc.gate_energy(banks, 2, xs)[3:4])
    assert orc.gate_energy(banks, 2, np.zeros((2, H), np.float32)).tolist() == [0.0, 0.0]
    with pytest.raises(orc.OracleError):
        orc.gate_energy(banks, E, xs)


def test_gate_energy_on_the_closed_form_toy_block():
    # the f32 toy layer of nn/moe.rs:1617-1651: the same sum written out in plain Python
    _, gate, _, _, banks = toy_a_banks()
    x = toy_a_input(3, 0.5)
    g = np.asarray(gate, np.float32).reshape(TOY_A["experts"], TOY_A["inter"], TOY_A["hidden"])
    for e in range(TOY_A["experts"]):
        want = []
        for t in range(3):
            tot = 0.0
            for i in range(TOY_A["inter"]):
                pre = sum(float(g[e, i, c]) * float(x[t, c]) for c in range(TOY_A["hidden"]))
                tot += (pre / (1.0 + np.exp(-pre))) ** 2
            want.append(tot)
        assert np.allclose(orc.gate_energy(banks, e, x), want, rtol=1e-5, atol=1e-12)
