"""GPU parity: every call goes through the C ABI (mummu_amd.moe over libmummu_moe.so) and is
compared with the CPU oracle on the same seeded inputs.

Bars: routing ids and dequantized weights bit-exact; block outputs within 1e-5 (f32 weights)
or 2e-3 (f16 / quantized weights), relative error measured as the reference measures it
(models/qwen4exp/experts.rs:1264-1271): |got - want| / max(|want|, rss of the terms).
"""
import math

import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc
from tests.helpers import TOY_A, TOY_D, toy_a_input, toy_a_scalar_reference, toy_a_weights, toy_d_layers

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5
TOL_QUANT = 2e-3


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---------------------------------------------------------------------------------------------
# codec
# ---------------------------------------------------------------------------------------------

def test_f16_bf16_f32_dequantize_exactly_for_every_bit_pattern():
    b16 = np.arange(65536, dtype=np.uint16)
    for t in (M.F16, M.BF16):
        got, want = M.dequantize(t, b16), orc.dequantize(t, b16)
        nan = np.isnan(want)
        assert np.array_equal(bits(got)[~nan], bits(want)[~nan]) and np.all(np.isnan(got[nan]))
    f = synth.SplitMix64(3).normal(4096)
    assert np.array_equal(bits(M.dequantize(M.F32, f)), bits(f))


@pytest.mark.parametrize("dtype,blocks", [(M.Q4_K, 777), (M.Q8_0, 3001)])
def test_quantized_blocks_dequantize_bit_exactly(dtype, blocks):
    raw = synth.synth_blocks(dtype, blocks, synth.SplitMix64(0xD0 + dtype))
    assert np.array_equal(bits(M.dequantize(dtype, raw)), bits(orc.dequantize(dtype, raw)))
    # arbitrary bytes: every 6-bit scale pattern and f16 scale, finite outputs compared by bits
    g = np.random.Generator(np.random.PCG64(dtype))
    raw = g.integers(0, 256, size=orc.block_bytes(dtype) * 512, dtype=np.uint8)
    got, want = M.dequantize(dtype, raw), orc.dequantize(dtype, raw)
    fin = np.isfinite(want)
    assert np.array_equal(bits(got)[fin], bits(want)[fin]) and np.array_equal(np.isnan(got), np.isnan(want))


def test_reference_known_answer_blocks_on_the_gpu():
    # gguf.rs:2395-2429
    blk = np.concatenate([np.array([0.5], np.float16).view(np.uint8), (np.arange(32, dtype=np.int8) - 16).view(np.uint8)])
    out = M.dequantize(M.Q8_0, blk)
    assert out[0] == -8.0 and out[16] == 0.0 and out[31] == 7.5
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([1.0], np.float16).view(np.uint8)
    b[2:4] = np.array([0.5], np.float16).view(np.uint8)
    b[4], b[5], b[8], b[12], b[16], b[80] = 2, 3, 1, 0x21, 0x51, 0x04
    out = M.dequantize(M.Q4_K, b)
    assert out[0] == 1.5 and out[1] == -0.5 and out[32] == 15.0 and out[128] == 3.0
    with pytest.raises(M.MoeError):
        M.dequantize(M.Q8_0, np.zeros(33, np.uint8))


# ---------------------------------------------------------------------------------------------
# router
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def toy():
    router, gate, up, down = toy_a_weights()
    m = M.SparseMoe(M.SparseMoeConfig(TOY_A["hidden"], TOY_A["inter"], TOY_A["experts"], TOY_A["top_k"]), max_tokens=8)
    m.load_layer(0, router, M.F32, gate, M.F32, up, M.F32, down, M.F32)
    banks = orc.LayerBanks(TOY_A["hidden"], TOY_A["inter"], TOY_A["experts"], gate, up, down, orc.F32)
    yield m, router, gate, up, down, banks
    m.close()


def test_router_known_answers_qwen4exp(toy):
    m = toy[0]
    # experts.rs:1365-1408
    ids, w = M.route(m, [0.0, 3.0, 1.0, 2.5, -2.0, 2.0, 0.5, 2.9], 1, 8, 3)
    assert ids[0].tolist() == [1, 7, 3]
    z = math.exp(3.0) + math.exp(2.9) + math.exp(2.5)
    assert all(abs(float(g) - math.exp(l) / z) < 1e-6 for g, l in zip(w[0], [3.0, 2.9, 2.5]))
    ids, w = M.route(m, [0.5] * 8, 1, 8, 3)
    assert ids[0].tolist() == [0, 1, 2] and np.all(np.abs(w - 1 / 3) < 1e-6)
    assert M.route(m, [1.0, 0.0, 2.0, 1.0], 1, 4, 2)[0][0].tolist() == [2, 0]
    lg = np.full(48, -1000.0, np.float32)
    lg[5], lg[16 + 9], lg[16 + 3], lg[32 + 15] = 1000.0, 999.0, 998.0, 30.0
    ids, w = M.route(m, lg, 3, 16, 2)
    assert ids[0, 0] == 5 and ids[1].tolist() == [9, 3] and ids[2, 0] == 15
    assert np.all(np.isfinite(w)) and np.all(np.abs(w.sum(axis=1) - 1) < 1e-6)
    assert abs(float(w[1, 0]) - math.e / (math.e + 1)) < 1e-6


def test_router_refuses_non_finite_logits_and_bad_k(toy):
    m = toy[0]
    # experts.rs:1410-1417
    with pytest.raises(M.MoeError, match="token 0 expert 1"):
        M.route(m, [0.0, math.nan, 1.0, 2.0], 2, 2, 1)
    for k in (0, 5):
        with pytest.raises(M.MoeError):
            M.route(m, [0.0] * 4, 1, 4, k)
    with pytest.raises(M.MoeError):
        M.route(m, [0.0] * 5, 1, 4, 2)
    # and the handle still works afterwards
    assert M.route(m, [1.0, 0.0, 2.0, 1.0], 1, 4, 2)[0][0].tolist() == [2, 0]


@pytest.mark.parametrize("flavour,norm", [(M.ROUTER_QWEN4EXP, True), (M.ROUTER_SPARSE_MOE, False), (M.ROUTER_SPARSE_MOE, True)])
@pytest.mark.parametrize("n_experts,k", [(8, 3), (64, 8), (128, 8), (130, 130), (512, 5), (512, 10), (300, 16)])
@pytest.mark.parametrize("spread", [4.0, 14.0])
def test_routing_of_random_logits_is_bit_exact(toy, flavour, norm, n_experts, k, spread):
    # spread 4: every probability stays above 2^-20 of the largest (the f64 normaliser may be
    # summed as a tree); spread 14: some fall below it (the sum must run in expert order)
    m = toy[0]
    rng = synth.SplitMix64(n_experts * 31 + k)
    n = 37
    lg = rng.uniform(-spread, spread, n * n_experts).reshape(n, n_experts)
    lg[::5, 1] = lg[::5, n_experts - 1]  # exact ties, some at the selection boundary
    lg[3] = 0.25                        # a fully tied row
    ids, w = M.route(m, lg, n, n_experts, k, flavour, norm)
    if flavour == M.ROUTER_QWEN4EXP:
        oi, ow = orc.route_ggml(lg, n, n_experts, k)
    else:
        oi, ow = orc.route_olmoe(lg, n, n_experts, k, norm)
    assert np.array_equal(ids, oi.astype(np.int32))
    assert np.array_equal(bits(w), bits(ow))


# ---------------------------------------------------------------------------------------------
# the block on the reference's closed-form toy (nn/moe.rs:1617-1651, 2088-2374)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("t", [5, 1])
@pytest.mark.parametrize("norm", [False, True])
def test_forward_matches_the_hand_rolled_sparse_reference(toy, t, norm):
    m, router, gate, up, down, banks = toy
    x = toy_a_input(t, 2.0)
    got = m.forward(x.reshape(1, t, 4), 2, norm)
    assert got.shape == (1, t, 4)
    want = toy_a_scalar_reference(router, gate, up, down, x, 2, norm)
    assert np.max(np.abs(got.reshape(t, 4) - want)) < 1e-5
    o_out, o_ids, o_w, o_lg = orc.moe_forward(banks, router, orc.F32, x, 2, norm)
    r, lg = m.route(x, 2, norm, return_logits=True)
    assert np.array_equal(bits(lg), bits(o_lg))
    assert np.array_equal(r.ids, o_ids.astype(np.int32)) and np.array_equal(bits(r.weights), bits(o_w))
    assert np.max(np.abs(got.reshape(t, 4) - o_out)) < 1e-5


def test_top_k_equal_to_num_experts_uses_every_expert(toy):
    m, router, gate, up, down, _ = toy
    x = toy_a_input(3, 0.5)
    got = m.forward(x, 4, False)
    want = toy_a_scalar_reference(router, gate, up, down, x, 4, False)
    assert np.max(np.abs(got - want)) < 1e-5


def test_norm_topk_weights_change_the_mixture(toy):
    m = toy[0]
    x = toy_a_input(4, 7.0)
    assert np.any(np.abs(m.forward(x, 2, False) - m.forward(x, 2, True)) > 1e-7)


def test_forward_is_position_independent_bitwise(toy):
    m = toy[0]
    row = toy_a_input(1, 11.0)
    s = m.forward(row, 2, False)
    d = m.forward(np.concatenate([row, row]), 2, False)
    assert np.array_equal(bits(s[0]), bits(d[0])) and np.array_equal(bits(s[0]), bits(d[1]))


def test_zero_input_gives_zero_output_and_empty_input_is_fine(toy):
    m = toy[0]
    assert np.all(m.forward(np.zeros((2, 4), np.float32), 2, False) == 0.0)
    assert m.forward(np.zeros((0, 4), np.float32), 2, False).shape == (0, 4)


def test_forward_rejects_bad_top_k_and_hidden_mismatch(toy):
    m = toy[0]
    with pytest.raises(M.MoeError, match="top_k"):
        m.forward(toy_a_input(1, 0.0), 5, False)
    with pytest.raises(M.MoeError, match="top_k"):
        m.forward(toy_a_input(1, 0.0), 0, False)
    with pytest.raises(M.MoeError, match="hidden"):
        m.forward(np.zeros((1, 5), np.float32), 2, False)
    with pytest.raises(M.MoeError):
        m.forward(toy_a_input(1, 0.0), 2, False, layer=3)
    with pytest.raises(M.MoeError, match="not finite"):
        m.forward(np.full((1, 4), np.inf, np.float32), 2, False)
    assert np.all(np.isfinite(m.forward(toy_a_input(2, 1.0), 2, False)))


def test_routed_equals_run_local_and_hits_count_rows(toy):
    # nn/moe.rs:1655-1700 (routed == dense) and :1976-1979 (hit count = tokens * k)
    m, router, *_rest, banks = toy
    m.take_hits()
    x = toy_a_input(5, 7.0)
    full = m.forward(x, 2, True)
    r = m.route(x, 2, True)
    assert sum(len(rows) for rows, _ in r.per_expert) == 10
    for rows, _ in r.per_expert:
        assert np.all(np.diff(rows) >= 0)
    hits = m.take_hits()
    assert int(hits.sum()) == 10 and hits.tolist() == np.bincount(r.ids.reshape(-1), minlength=4).tolist()
    again = m.run_local(x, r)
    assert np.array_equal(bits(full), bits(again))
    assert int(m.take_hits().sum()) == 10
    dense = orc.moe_forward_dense_mask(banks, router, orc.F32, x, 2, True)
    assert np.max(np.abs(full - dense)) < 1e-5


# ---------------------------------------------------------------------------------------------
# quantized toy layers (experts.rs:1429-1563): gate/up Q4_K, down Q5_1 (layer 0) / Q8_0 (layer 1)
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module", params=[0, 1], ids=["down_q5_1", "down_q8_0"])
def toy_q(request):
    raw = toy_d_layers(11)[request.param]
    H, F, E = TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    m = M.SparseMoe(M.SparseMoeConfig(H, F, E, 2), max_tokens=16, router_flavour=M.ROUTER_QWEN4EXP, norm_topk_prob=True)
    router = synth.SplitMix64(5).normal(E * H, 0.0, 0.05).reshape(E, H)
    m.load_layer(0, router, M.F32, raw["gate"], raw["gate_type"], raw["up"], raw["up_type"], raw["down"], raw["down_type"])
    banks = orc.LayerBanks(H, F, E, raw["gate"], raw["up"], raw["down"], raw["gate_type"], raw["up_type"], raw["down_type"])
    yield m, raw, banks, router
    m.close()


def test_resident_bytes_dequantize_to_the_reference_weights(toy_q):
    m, raw, banks, _ = toy_q
    H, F, E = TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    for which, t, shape in (("gate", raw["gate_type"], (E, F, H)), ("up", raw["up_type"], (E, F, H)), ("down", raw["down_type"], (E, H, F))):
        want = orc.dequantize(t, raw[which]).reshape(shape)
        for e in (0, 3, 7):
            assert np.array_equal(bits(m.dequantize_expert(0, which, e)), bits(want[e]))


def test_routed_moe_equals_the_dense_mask_reference(toy_q):
    # experts.rs:1466-1532 with this build's tolerance for quantized banks
    m, raw, banks, _ = toy_q
    rng = synth.SplitMix64(12)
    n, H, E = 5, TOY_D["hidden"], TOY_D["experts"]
    xs = rng.uniform_vec(n * H).reshape(n, H)
    logits = rng.uniform(-2.0, 2.0, n * E).reshape(n, E)
    got = m.routed_moe(0, logits, xs, n, 2)
    ids, w = orc.route_ggml(logits, n, E, 2)
    want, mag = orc.moe_ref_f64(banks, ids, w, xs)
    assert orc.rel_err(got, want, mag).max() <= TOL_QUANT
    cpu = orc.apply_routing(banks, ids, w, xs)
    assert orc.rel_err(got, cpu.astype(np.float64), mag).max() <= TOL_QUANT


def test_a_token_routes_bit_identically_alone_or_in_a_batch(toy_q):
    # experts.rs:1534-1563
    m = toy_q[0]
    rng = synth.SplitMix64(22)
    n, H, E = 6, TOY_D["hidden"], TOY_D["experts"]
    xs = rng.uniform_vec(n * H).reshape(n, H)
    logits = rng.uniform(-3.0, 3.0, n * E).reshape(n, E)
    batch = m.routed_moe(0, logits, xs, n, 3)
    for t in range(n):
        one = m.routed_moe(0, logits[t], xs[t], 1, 3)
        assert np.array_equal(bits(one[0]), bits(batch[t])), t


def test_expert_run_is_the_single_expert_swiglu(toy_q):
    # ExpertExec::run, nn/moe.rs:353-357; expert_ffn experts.rs:1015-1057
    m, raw, banks, _ = toy_q
    rng = synth.SplitMix64(77)
    H = TOY_D["hidden"]
    x = rng.uniform_vec(3 * H).reshape(3, H)
    got = m.expert_run(0, 5, x)
    ids = np.full((3, 1), 5, np.uint32)
    want, mag = orc.moe_ref_f64(banks, ids, np.ones((3, 1), np.float32), x)
    assert orc.rel_err(got, want, mag).max() <= TOL_QUANT
    with pytest.raises(M.MoeError, match="out of range"):
        m.expert_run(0, 8, x)
    with pytest.raises(M.MoeError, match="hidden"):
        m.expert_run(0, 0, np.zeros((1, 128), np.float32))
    with pytest.raises(M.MoeError, match="out of range"):
        m.apply_routing(0, np.array([[1, 9]], np.int32), np.ones((1, 2), np.float32), x[:1])


def test_unsupported_bank_types_and_ragged_rows_are_refused():
    raw = toy_d_layers(11)[0]
    H, F, E = TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    with M.SparseMoe(M.SparseMoeConfig(H, F, E, 2)) as m:
        router = np.zeros((E, H), np.float32)
        for no_kernel in (10, 11, 15, 20):  # Q2_K, Q3_K, Q8_K, IQ4_NL: container types without an expert kernel
            with pytest.raises(M.MoeError, match="type"):
                m.load_layer(0, router, M.F32, raw["gate"], raw["gate_type"], raw["up"], raw["up_type"], raw["down"], no_kernel)
        with pytest.raises(M.MoeError, match="share one type"):
            m.load_layer(0, router, M.F32, raw["gate"], M.Q4_K, np.zeros(E * F * (H // 256) * 176, np.uint8), M.Q5_K,
                         raw["down"], raw["down_type"])
        with pytest.raises(M.MoeError):
            m.forward(np.zeros((1, H), np.float32), 2, False)  # nothing loaded
    # experts.rs:1355-1363: 640-wide rows cannot be K-quant
    with M.SparseMoe(M.SparseMoeConfig(640, 32, 2, 1)) as m:
        with pytest.raises(M.MoeError, match="whole blocks"):
            m.load_layer(0, np.zeros((2, 640), np.float32), M.F32, np.zeros(10, np.uint8), M.Q4_K, np.zeros(10, np.uint8),
                         M.Q4_K, np.zeros(2 * 640 * 34, np.uint8), M.Q8_0)


# ---------------------------------------------------------------------------------------------
# ExpertExec::gate_energy (nn/moe.rs:411-418, 508-521)
# ---------------------------------------------------------------------------------------------

def test_gate_energy_matches_the_oracle_and_the_f64_sum(toy_q):
    m, raw, banks, _ = toy_q
    H, F, E = TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]
    xs = synth.SplitMix64(31).uniform_vec(9 * H).reshape(9, H)
    gate = orc.dequantize(raw["gate_type"], raw["gate"]).reshape(E, F, H).astype(np.float64)
    for e in (0, 3, E - 1):
        got = m.gate_energy(0, e, xs)
        pre = xs.astype(np.float64) @ gate[e].T
        want = ((pre / (1.0 + np.exp(-pre))) ** 2).sum(axis=1)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(want, 1e-30)), e
        assert np.allclose(got, orc.gate_energy(banks, e, xs), rtol=1e-5, atol=0)
    # a row's energy does not depend on the rows beside it; zero rows have none; bad arguments are refused
    assert np.array_equal(bits(m.gate_energy(0, 2, xs[4:5])), bits(m.gate_energy(0, 2, xs)[4:5]))
    assert m.gate_energy(0, 2, np.zeros((3, H), np.float32)).tolist() == [0.0, 0.0, 0.0]
    with pytest.raises(M.MoeError, match="out of range"):
        m.gate_energy(0, E, xs)
    with pytest.raises(M.MoeError, match="hidden"):
        m.gate_energy(0, 0, np.zeros((2, H + 32), np.float32))


def test_gate_energy_on_float_banks_and_many_rows(toy):
    m, router, gate, up, down, banks = toy
    x = np.tile(toy_a_input(4, 0.25), (5, 1))[:8]  # max_tokens of the fixture is 8
    g = np.asarray(gate, np.float64).reshape(TOY_A["experts"], TOY_A["inter"], TOY_A["hidden"])
    for e in range(TOY_A["experts"]):
        pre = x.astype(np.float64) @ g[e].T
        want = ((pre / (1.0 + np.exp(-pre))) ** 2).sum(axis=1)
        assert np.allclose(m.gate_energy(0, e, x), want, rtol=1e-5, atol=1e-12)


def test_expert_run_device_leaves_the_same_bits_on_the_device(toy_q):
    # ExpertExec::run_tensor_resident (nn/moe.rs:360-371): rows already on the device, the result left there
    m = toy_q[0]
    H = TOY_D["hidden"]
    xs = synth.SplitMix64(41).uniform_vec(7 * H).reshape(7, H)
    xd, od = M.DeviceBuffer.from_array(xs), M.DeviceBuffer(xs.nbytes)
    for e in (1, 5):
        m.expert_run_device(0, e, xd, 7, od)
        m.check()
        assert np.array_equal(bits(od.download(np.float32, (7, H))), bits(m.expert_run(0, e, xs)))
    with pytest.raises(M.MoeError, match="out of range"):
        m.expert_run_device(0, 99, xd, 7, od)
    with pytest.raises(M.MoeError, match="exceeds the workspace"):
        m.expert_run_device(0, 1, xd, 17, od)


def test_config_init_draws_fan_in_bounded_uniform_weights_and_checks_like_the_reference():
    # nn/moe.rs:61-99
    cfg = M.SparseMoeConfig(64, 32, 4, 2)
    with cfg.init(seed=3, max_tokens=4) as m:
        g, d = m.dequantize_expert(0, "gate", 1), m.dequantize_expert(0, "down", 3)
        assert g.shape == (32, 64) and d.shape == (64, 32)
        assert np.abs(g).max() <= 1 / 8 and np.abs(g).max() > 0.9 / 8          # 1/sqrt(64)
        assert np.abs(d).max() <= 1 / np.sqrt(32) and np.abs(d).max() > 0.9 / np.sqrt(32)
        x = synth.SplitMix64(1).uniform_vec(3 * 64).reshape(3, 64)
        assert np.all(np.isfinite(m.forward(x, 2, False))) and np.any(m.forward(x, 2, False) != 0)
    with cfg.init(seed=3, max_tokens=4) as a, cfg.init(seed=4, max_tokens=4) as b:
        assert not np.array_equal(a.dequantize_expert(0, "up", 0), b.dequantize_expert(0, "up", 0))
    for bad in (M.SparseMoeConfig(64, 32, 1, 1), M.SparseMoeConfig(64, 32, 4, 5), M.SparseMoeConfig(0, 32, 4, 2)):
        with pytest.raises(M.MoeError):
            bad.init()


@pytest.mark.parametrize("dtype", [M.F16, M.BF16])
def test_forward_in_the_ambient_dtype_is_the_f32_block_between_exact_widening_and_nearest_even_narrowing(toy_q, dtype):
    # nn/moe.rs:116-135: the block works in f32 and hands the result back in the input's dtype
    m = toy_q[0]
    H = TOY_D["hidden"]
    x32 = synth.SplitMix64(51).uniform_vec(6 * H).reshape(6, H)
    bits16 = synth.encode_float(x32, dtype).view(np.uint16).reshape(6, H)
    widened = (bits16.astype(np.uint32) << 16).view(np.float32) if dtype == M.BF16 else bits16.view(np.float16).astype(np.float32)
    want = synth.encode_float(m.forward(widened, 2, True), dtype).view(np.uint16).reshape(6, H)
    got = m.forward_typed(bits16, dtype, 2, True)
    assert got.dtype == np.uint16 and np.array_equal(got, want)
    # F32 through the same entry point is the plain forward
    assert np.array_equal(bits(m.forward_typed(x32, M.F32, 2, True)), bits(m.forward(x32, 2, True)))
    with pytest.raises(M.MoeError, match="F32, F16 or BF16"):
        m._check(m._lib.mummu_moe_forward_typed(m._h, 0, bits16.ctypes.data, M.Q8_0, 6, 2, 1, got.ctypes.data))


def test_gate_energy_with_rows_wider_than_the_default_lds_window():
    # 4 rows of 4096 f32 are 64 KB of LDS: above the 48 KB a launch gets without asking
    H, I, E = 4096, 64, 2
    g = np.random.Generator(np.random.PCG64(5))
    gate = (g.standard_normal((E, I, H), dtype=np.float32) * 0.02).astype(np.float32)
    up, down = gate.copy(), (g.standard_normal((E, H, I), dtype=np.float32) * 0.02).astype(np.float32)
    router = (g.standard_normal((E, H), dtype=np.float32) * 0.02).astype(np.float32)
    x = g.standard_normal((5, H), dtype=np.float32)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, 1), max_tokens=8) as m:
        m.load_layer(0, router, M.F32, gate, M.F32, up, M.F32, down, M.F32)
        got = m.gate_energy(0, 1, x)
    pre = x.astype(np.float64) @ gate[1].astype(np.float64).T
    want = ((pre / (1.0 + np.exp(-pre))) ** 2).sum(axis=1)
    assert np.all(np.abs(got - want) <= 1e-5 * want)


def test_a_graph_is_refused_once_the_buffers_it_points_into_are_gone():
    # a captured graph holds raw workspace and weight pointers: a host call that regrows the workspace, or a reload
    # of the layer, must make launch fail with MUMMU_ERR_STALE instead of replaying over freed memory
    from mummu_amd import _lib
    H, I, E, k = 256, 64, 8, 2
    rng = synth.SplitMix64(77)
    banks = [synth.synth_bank(synth.Q8_0, ne, rng) for ne in ([H, I, E], [H, I, E], [I, H, E])]
    router = rng.normal(E * H, 0.0, 0.05).astype(np.float16).reshape(E, H)
    x = rng.normal(2 * H).reshape(2, H)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=4) as m:
        m.load_layer(0, router, M.F16, banks[0], M.Q8_0, banks[1], M.Q8_0, banks[2], M.Q8_0)
        want = m.forward(x, k, False)
        xd, od = M.DeviceBuffer.from_array(x), M.DeviceBuffer(x.nbytes)

        def capture():
            m.graph_begin()
            m.forward_device(0, xd, 2, k, False, od)
            return m.graph_end()

        g = capture()
        g.launch()
        m.check()
        assert np.array_equal(bits(od.download(np.float32, x.shape)), bits(want))
        ms = g.launch_timed(3)
        assert ms.shape == (3,) and np.all(ms > 0)
        m.forward(rng.normal(64 * H).reshape(64, H), k, False)  # 64 tokens > max_tokens: the workspace is regrown
        with pytest.raises(M.MoeError) as e:
            g.launch()
        assert e.value.code == _lib.ERR_STALE
        with pytest.raises(M.MoeError):
            g.launch_timed(2)
        g.close()
        g = capture()  # captured again, it runs
        g.launch()
        m.check()
        assert np.array_equal(bits(od.download(np.float32, x.shape)), bits(want))
        m.load_layer(0, router, M.F16, banks[0], M.Q8_0, banks[1], M.Q8_0, banks[2], M.Q8_0)  # same bytes, new buffers
        with pytest.raises(M.MoeError) as e:
            g.launch()
        assert e.value.code == _lib.ERR_STALE
        g.close()


def test_the_read_probe_runs_every_pattern_and_refuses_the_others():
    # mummu_probe_read drops what it reads: all there is to check is that every pattern launches and finishes over a
    # buffer of exactly two slabs, and that a piece size without a kernel is refused
    row_bytes = 1152
    buf = M.DeviceBuffer(2 * 128 * row_bytes)
    buf.upload(np.zeros(2 * 128 * row_bytes // 4, dtype=np.int32))
    for piece in (0, 32, 64, 128):
        M.probe_read(buf, 2 * 128 * row_bytes, row_bytes, piece)
    M.synchronize()
    with pytest.raises(M.MoeError):
        M.probe_read(buf, 2 * 128 * row_bytes, row_bytes, 48)

