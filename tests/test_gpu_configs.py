"""GPU parity at the benchmark configurations' full shapes (OLMoE-1B-7B and Qwen3-30B-A3B
expert geometry), through the C ABI, against the CPU oracle on the same seeded inputs.

  C1  OLMoE f32, 16 tokens                      (float GEMV path, tolerance 1e-5)
  C2  OLMoE f16, 512 tokens, uniform router      (dispatch + grouped MFMA GEMM, 2e-3)
  C3  OLMoE Q4_K experts, f16 router, 1/4/8 tok  (packed integer GEMV, 2e-3)
  C4  16-layer OLMoE stack, RmsNorm + residual, Q8_0, decode 1 token and prefill 256 tokens
  C5  Qwen3-A3B shape, Q4_K, 64 tokens, Zipf-skewed routing, norm_topk_prob=true

Routing ids must be bit-exact; outputs are held to the stated relative error measured as the
reference measures it (experts.rs:1264-1271), every token and every element against the f64
product of the dequantized weights.
"""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from oracle import binding as orc

pytestmark = pytest.mark.gpu

OLMOE = dict(H=2048, I=1024, E=64, k=8)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def normal(shape, seed, std=1.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def float_bank(dtype, in_dim, out_dim, E, seed):
    w = normal(E * out_dim * in_dim, seed, 0.02)
    return synth.encode_float(w, dtype)


def check_rows(got, banks, ids, w, xs, rows, tol):
    want, mag = orc.moe_ref_f64(banks, ids[rows], w[rows], xs[rows])
    err = orc.rel_err(got[rows], want, mag).max()
    assert err <= tol, f"max relative error {err:.3e} > {tol}"
    return err


def test_c1_olmoe_f32_16_tokens():
    H, I, E, k = OLMOE["H"], OLMOE["I"], OLMOE["E"], OLMOE["k"]
    gate, up, down = (float_bank(synth.F32, H, I, E, 11), float_bank(synth.F32, H, I, E, 12), float_bank(synth.F32, I, H, E, 13))
    router = normal((E, H), 14, 0.02)
    x = normal((16, H), 15)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=16) as m:
        m.load_layer(0, router, M.F32, gate, M.F32, up, M.F32, down, M.F32)
        got = m.forward(x, k, False)
        r, lg = m.route(x, k, False, return_logits=True)
        assert m.resident_bytes() == 64 * 25_165_824 + E * H * 4
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.F32)
    out, ids, w, olg = orc.moe_forward(banks, router, orc.F32, x, k, False)
    assert np.array_equal(bits(lg), bits(olg))
    assert np.array_equal(r.ids, ids.astype(np.int32)) and np.array_equal(bits(r.weights), bits(w))
    check_rows(got, banks, ids, w, x, slice(0, 16), 1e-5)
    assert orc.rel_err(out, *orc.moe_ref_f64(banks, ids, w, x)).max() <= 1e-5  # the oracle's own f32 path


def test_c2_olmoe_f16_prefill_512_tokens_grouped_gemm():
    H, I, E, k = OLMOE["H"], OLMOE["I"], OLMOE["E"], OLMOE["k"]
    n = 512
    gate, up, down = (float_bank(synth.F16, H, I, E, 21), float_bank(synth.F16, H, I, E, 22), float_bank(synth.F16, I, H, E, 23))
    g = np.random.Generator(np.random.PCG64(24))
    router = g.uniform(-0.05, 0.05, size=(E, H)).astype(np.float16)  # uniform-random router: ~64 tokens per expert
    x = normal((n, H), 25)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n) as m:
        m.load_layer(0, router, M.F16, gate, M.F16, up, M.F16, down, M.F16)
        got = m.forward(x, k, False)
        r = m.route(x, k, False)
        hits = m.take_hits()
        # ragged batch sizes around the tile edges take the same path
        got_97 = m.forward(x[:97], k, False)
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.F16)
    out, ids, w, _ = orc.moe_forward(banks, router, orc.F16, x, k, False)
    assert np.array_equal(r.ids, ids.astype(np.int32)) and np.array_equal(bits(r.weights), bits(w))
    assert int(hits.sum()) == n * k and hits.tolist() == np.bincount(ids.reshape(-1), minlength=E).tolist()
    # every token, every element, by the reference's measure: all 4096 assignments, so every row position of
    # every tile of the grouped GEMM is checked
    check_rows(got, banks, ids, w, x, slice(0, n), 2e-3)
    check_rows(got_97, banks, ids, w, x, slice(0, 97), 2e-3)
    # and against the oracle's f32 result, scaled by the row's magnitude
    scale = np.sqrt((out.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert (np.abs(got - out) / scale).max() <= 2e-2
    assert np.abs(got - out).mean() / np.abs(out).mean() <= 2e-3
    assert (np.abs(got_97 - out[:97]) / scale[:97]).max() <= 2e-2


@pytest.fixture(scope="module")
def c3():
    H, I, E, k = OLMOE["H"], OLMOE["I"], OLMOE["E"], OLMOE["k"]
    gate = synth.random_bank_fast(synth.Q4_K, [H, I, E], 31)
    up = synth.random_bank_fast(synth.Q4_K, [H, I, E], 32)
    down = synth.random_bank_fast(synth.Q4_K, [I, H, E], 33)
    router = normal((E, H), 34, 0.02).astype(np.float16)
    m = M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=8)
    m.load_layer(0, router, M.F16, gate, M.Q4_K, up, M.Q4_K, down, M.Q4_K)
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.Q4_K)
    yield m, banks, router
    m.close()


@pytest.mark.parametrize("bt", [1, 4, 8])
def test_c3_olmoe_q4k_decode(c3, bt):
    m, banks, router = c3
    H, k = OLMOE["H"], OLMOE["k"]
    x = normal((bt, H), 40 + bt)
    got = m.forward(x, k, False)
    r = m.route(x, k, False)
    out, ids, w, _ = orc.moe_forward(banks, router, orc.F16, x, k, False)
    assert np.array_equal(r.ids, ids.astype(np.int32)) and np.array_equal(bits(r.weights), bits(w))
    err = check_rows(got, banks, ids, w, x, slice(0, bt), 2e-3)
    assert err <= 5e-4  # 16-bit activations: well inside the bar
    # the device-pointer entry point gives the same bits as the host one
    xd, od = M.DeviceBuffer.from_array(x), M.DeviceBuffer(x.nbytes)
    m.forward_device(0, xd, bt, k, False, od)
    m.check()
    assert np.array_equal(bits(od.download(np.float32, x.shape)), bits(got))
    gi, gw = m.last_routing(bt, k)
    assert np.array_equal(gi, r.ids) and np.array_equal(bits(gw), bits(r.weights))


def test_c3_expert_weights_resident_in_hbm_are_the_gguf_bytes(c3):
    m, banks, _ = c3
    H, I = OLMOE["H"], OLMOE["I"]
    for which, arr, shape in (("gate", banks.gate, (I, H)), ("down", banks.down, (H, I))):
        per = arr.size // OLMOE["E"]
        for e in (0, 63):
            want = orc.dequantize(orc.Q4_K, arr[e * per:(e + 1) * per]).reshape(shape)
            assert np.array_equal(bits(m.dequantize_expert(0, which, e)), bits(want))
    assert m.resident_bytes() == 64 * 3_538_944 + 64 * 2048 * 2


def test_c3_graph_replays_match_eager(c3):
    m, banks, router = c3
    H, k = OLMOE["H"], OLMOE["k"]
    xs = [normal((1, H), 60 + i) for i in range(3)]
    xd = [M.DeviceBuffer.from_array(x) for x in xs]
    od = [M.DeviceBuffer(H * 4) for _ in xs]
    eager = []
    for x, o in zip(xd, od):
        m.forward_device(0, x, 1, k, False, o)
    m.check()
    eager = [o.download(np.float32, (1, H)) for o in od]
    m.graph_begin()
    for x, o in zip(xd, od):
        m.forward_device(0, x, 1, k, False, o)
    graph = m.graph_end()
    for rep in range(4):
        for o in od:
            o.upload(np.zeros((1, H), np.float32))
        graph.launch()
        m.check()
        for o, want in zip(od, eager):
            assert np.array_equal(bits(o.download(np.float32, (1, H))), bits(want)), rep
        # eager work between replays
        m.forward(xs[rep % 3], k, False)
    graph.close()


def c4_layers(L, seed):
    H, I, E = OLMOE["H"], OLMOE["I"], OLMOE["E"]
    layers = []
    for l in range(L):
        gate = synth.random_bank_fast(synth.Q8_0, [H, I, E], seed + 10 * l)
        up = synth.random_bank_fast(synth.Q8_0, [H, I, E], seed + 10 * l + 1)
        down = synth.random_bank_fast(synth.Q8_0, [I, H, E], seed + 10 * l + 2)
        router = normal((E, H), seed + 10 * l + 3, 0.02).astype(np.float16)
        gamma = (1.0 + 0.05 * normal(H, seed + 10 * l + 4)).astype(np.float32)
        layers.append((router, gate, up, down, gamma))
    return layers


def run_c4(L, n, seed, layer_tol=None):
    """GPU stack vs the oracle run layer by layer.  With `layer_tol` every layer is also run on its own
    on the ORACLE's input to that layer and every element of its output is held to `layer_tol` of the f64
    reference by the reference's measure (experts.rs:1264-1271) - identical inputs, so no error carried
    over from the layers before.  Returns (got, gpu ids [L,n,k], want, oracle ids,
    oracle routing margins [L,n]): margin = the smallest relative gap (p_j - p_{j+1}) / p_j between
    neighbours among the oracle's k+1 most probable experts - the slack before either the selected
    set or the slot order can change."""
    H, I, E, k = OLMOE["H"], OLMOE["I"], OLMOE["E"], OLMOE["k"]
    layers = c4_layers(L, seed)
    x = normal((n, H), seed + 999)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=L, max_tokens=n, rms_norm_eps=1e-5) as m:
        for l, (router, gate, up, down, gamma) in enumerate(layers):
            m.load_layer(l, router, M.F16, gate, M.Q8_0, up, M.Q8_0, down, M.Q8_0, rms_gamma=gamma)
        got, gids = m.stack_forward(x, k, False, return_ids=True)
        # every layer on the ORACLE's input to that layer: identical inputs, so routing must be exact
        cur = x.copy()
        oids, margins = [], []
        for l, (router, gate, up, down, gamma) in enumerate(layers):
            banks = orc.LayerBanks(H, I, E, gate, up, down, orc.Q8_0)
            h2 = orc.rmsnorm(cur, gamma, 1e-5)
            moe, ids, w, lg = orc.moe_forward(banks, router, orc.F16, h2, k, False)
            r = m.route(h2, k, False, layer=l)
            assert np.array_equal(r.ids, ids.astype(np.int32)), f"layer {l}: routing differs on identical input"
            assert np.array_equal(bits(r.weights), bits(w))
            p = np.sort(np.exp(lg.astype(np.float64) - lg.max(axis=1, keepdims=True)), axis=1)[:, ::-1]
            margins.append(((p[:, :k] - p[:, 1:k + 1]) / p[:, :k]).min(axis=1))
            if layer_tol is not None:
                check_rows(m.forward(h2, k, False, layer=l), banks, ids, w, h2, slice(0, n), layer_tol)
            oids.append(ids.astype(np.int32))
            cur = (cur + moe).astype(np.float32)
    return got, gids, cur, np.stack(oids), np.stack(margins)


def check_stack(got, gids, want, oids, margins, tol, max_flips, max_margin):
    # A layer routes the GPU's own residual stream, which differs from the oracle's by the
    # expert products' rounding: a token whose closest pair among its top k+1 probabilities is
    # nearer than that noise may legitimately swap two slots or pick the other expert.  Such
    # tokens must be rare and near-tied; every other token must route identically in every layer.
    # `tol` bounds max|got - want| over a row in units of the row's rms (over 2048 elements the
    # maximum of an error with relative rms r is about 4.5 r).  The three bounds are set about 1.5x
    # above what this configuration measures (printed below; run with -s to see them), so that a
    # regression of the arithmetic shows here long before it reaches the 2e-3 bar of a single layer.
    L, n, _ = gids.shape
    same = np.array([[np.array_equal(gids[l, t], oids[l, t]) for t in range(n)] for l in range(L)])
    assert same[0].all(), "layer 0 sees the same input: routing must be exact"
    flipped = ~same
    first = np.argmax(flipped, axis=0)  # first layer at which each flipped token departs
    departed = np.nonzero(flipped.any(axis=0))[0]
    worst_margin = max((float(margins[first[t], t]) for t in departed), default=0.0)
    same_set = np.array([[sorted(gids[l, t]) == sorted(oids[l, t]) for t in range(n)] for l in range(L)]).all(axis=0)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    err = float((np.abs(got - want) / scale)[same_set].max())
    print(f"\nstack of {L} layers x {n} tokens: {int(flipped.sum())} of {L * n} (layer, token) routings differ from the oracle's, "
          f"{departed.size} tokens depart (largest margin at the departure {worst_margin:.3e}), {int((~same_set).sum())} tokens end "
          f"on another expert set, residual stream off by {err:.3e} of the row rms")
    assert flipped.sum() <= max_flips, f"{flipped.sum()} of {L * n} (layer, token) routings differ (bound {max_flips})"
    assert worst_margin <= max_margin, f"a token departed with margin {worst_margin:.3e} (bound {max_margin:.1e})"
    assert same_set.mean() >= 0.95
    assert err <= tol, f"residual stream off by {err:.3e} (bound {tol:.1e})"


def test_c4_sixteen_layer_q8_0_stack_decode():
    # integer GEMV with 16-bit activations; measured: no routing differs, residual stream off by 8.5e-4 of the row rms
    check_stack(*run_c4(16, 1, 400), tol=1.3e-3, max_flips=0, max_margin=0.0)


def test_c4_sixteen_layer_q8_0_stack_prefill_256_tokens():
    # the configuration as stated: 16 layers, 256 tokens.  Layer by layer on identical inputs every element is
    # inside 2e-3 by the reference's measure (layer_tol); the residual stream after 16 layers, where each layer's
    # rounding feeds the next, is held per row (see check_stack for the unit).  Measured: 21 of 4096 routings differ
    # (14 tokens depart, the least tied of them at a margin of 4.9e-4, 3 end on another expert set), residual stream
    # off by 2.03e-3 of the row rms
    check_stack(*run_c4(16, 256, 500, layer_tol=2e-3), tol=3e-3, max_flips=32, max_margin=8e-4)


@pytest.mark.parametrize("H,I,E,k,gt", [(2048, 256, 64, 8, M.Q4_K), (512, 128, 8, 2, M.Q8_0), (1280, 128, 16, 4, M.Q5_0),
                                        (2560, 128, 16, 4, M.Q8_0)],
                         ids=["2048", "512", "1280-ragged-chunk", "2560-too-wide-to-fuse"])
def test_decode_stack_with_the_norm_inside_the_router_launch_equals_the_separate_norm(H, I, E, k, gt):
    # up to 8 tokens the stack applies RmsNorm inside the router launch; from 9 on a kernel of its own
    # writes the normalised rows first.  Both must give a token the same bits, layer after layer (the
    # decode kernels serve both sizes, and a token's result does not depend on its batch), and the
    # first layer must agree with the oracle's RmsNorm + routing exactly.
    L = 3
    g = np.random.Generator(np.random.PCG64(H + E))
    layers = []
    for l in range(L):
        gate = synth.random_bank_fast(gt, [H, I, E], 10 * l + 1)
        up = synth.random_bank_fast(gt, [H, I, E], 10 * l + 2)
        down = synth.random_bank_fast(gt, [I, H, E], 10 * l + 3)
        router = normal((E, H), 10 * l + 4, 0.05).astype(np.float16)
        gamma = (1.0 + 0.2 * g.standard_normal(H)).astype(np.float32)
        layers.append((router, gate, up, down, gamma))
    x = normal((12, H), 77, 3.0)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=L, max_tokens=12, rms_norm_eps=1e-6) as m:
        for l, (router, gate, up, down, gamma) in enumerate(layers):
            m.load_layer(l, router, M.F16, gate, gt, up, gt, down, gt, rms_gamma=gamma)
        many, many_ids = m.stack_forward(x, k, True, return_ids=True)
        for n in (1, 3, 8):
            few, few_ids = m.stack_forward(x[:n], k, True, return_ids=True)
            assert np.array_equal(few_ids, many_ids[:, :n])
            assert np.array_equal(bits(few), bits(many[:n])), f"{n} tokens"
    router, gate, up, down, gamma = layers[0]
    h2 = orc.rmsnorm(x, gamma, 1e-6)
    _, ids, _, _ = orc.moe_forward(orc.LayerBanks(H, I, E, gate, up, down, gt), router, orc.F16, h2, k, True)
    assert np.array_equal(many_ids[0], ids.astype(np.int32))


def test_c4_q8_0_prefill_layer_against_the_f64_reference():
    # one full-size Q8_0 layer at 256 tokens (grouped GEMM), per element, the reference's measure
    H, I, E, k = OLMOE["H"], OLMOE["I"], OLMOE["E"], OLMOE["k"]
    router, gate, up, down, _ = c4_layers(1, 600)[0]
    x = normal((256, H), 601)
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=256) as m:
        m.load_layer(0, router, M.F16, gate, M.Q8_0, up, M.Q8_0, down, M.Q8_0)
        got = m.forward(x, k, False)
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.Q8_0)
    _, ids, w, _ = orc.moe_forward(banks, router, orc.F16, x, k, False)
    check_rows(got, banks, ids, w, x, slice(0, 256), 2e-3)


def test_c5_qwen3_a3b_shape_q4k_zipf_routing():
    H, I, E, k, n = 2048, 768, 128, 8, 64
    gate = synth.random_bank_fast(synth.Q4_K, [H, I, E], 71)
    up = synth.random_bank_fast(synth.Q4_K, [H, I, E], 72)
    down = synth.random_bank_fast(synth.Q4_K, [I, H, E], 73)
    router = normal((E, H), 74, 0.02)
    x = normal((n, H), 75)
    # router logits = x.W + b_e with b_e = log of a Zipf(1.1) pmf over a fixed random expert permutation
    g = np.random.Generator(np.random.PCG64(76))
    pmf = 1.0 / np.arange(1, E + 1) ** 1.1
    bias = np.log(pmf / pmf.sum())[g.permutation(E)].astype(np.float32)
    logits = orc.router_logits(x, router, orc.F32, E) + bias[None, :]
    with M.SparseMoe(M.SparseMoeConfig(H, I, E, k), max_tokens=n, router_flavour=M.ROUTER_QWEN4EXP, norm_topk_prob=True) as m:
        m.load_layer(0, router, M.F32, gate, M.Q4_K, up, M.Q4_K, down, M.Q4_K)
        ids, w = M.route(m, logits, n, E, k)
        got = m.routed_moe(0, logits, x, n, k)
        m.take_hits()
        one = m.routed_moe(0, logits[:3], x[:3], 3, k)  # small batch: the GEMV path
        # the block's own router (no bias) with norm_topk_prob: the fused top-2-per-lane kernel
        r = m.route(x, k, True)
    oi, ow = orc.route_ggml(logits, n, E, k)
    assert np.array_equal(ids, oi.astype(np.int32)) and np.array_equal(bits(w), bits(ow))
    counts = np.bincount(oi.reshape(-1), minlength=E)
    assert counts.max() >= 4 * max(1, int(np.median(counts)))  # the routing really is skewed
    banks = orc.LayerBanks(H, I, E, gate, up, down, orc.Q4_K)
    err = check_rows(got, banks, oi, ow, x, slice(0, n), 2e-3)
    check_rows(one, banks, oi, ow, x, slice(0, 3), 2e-3)
    o2 = orc.moe_forward(banks, router, orc.F32, x, k, True, flavour=1)
    assert np.array_equal(r.ids, o2[1].astype(np.int32)) and np.array_equal(bits(r.weights), bits(o2[2]))
