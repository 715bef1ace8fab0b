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
