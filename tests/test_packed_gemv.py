"""Q4GemvOps::q4s_gemv (nn/packed_gemv.rs) on burn's packed block-32 layout: the oracle's restatement of the
reference kernel against an independent f64 evaluation of x . dequantize(w) - the comparison the reference's own
test makes, to its bar of 1e-4 of the largest output (nn/packed_gemv.rs:1593-1624) and to a tighter one - and the
HIP kernel against both."""
import numpy as np
import pytest

from oracle import binding as orc
from tests.packed_helpers import pack_words, quantize_block32, reference_f64


def case(k, n, bits, m, seed):
    g = np.random.Generator(np.random.PCG64(seed))
    w = g.uniform(-1.0, 1.0, (k, n)).astype(np.float32)
    x = g.uniform(-1.0, 1.0, (m, k)).astype(np.float32)
    codes, scales = quantize_block32(w, bits)
    return codes, scales, pack_words(codes, bits), x


def judge(got, want):
    peak = max(float(np.abs(want).max()), 1e-6)
    return float(np.abs(got - want).max()) / peak


def test_packing_puts_element_j_at_bits_4j_in_twos_complement():
    codes = np.zeros((1, 32), np.int8)
    codes[0, :8] = [-8, -1, 0, 1, 7, -3, 2, -7]
    words = pack_words(codes, 4)
    fields = [(int(words[0, 0]) >> (4 * j)) & 0xF for j in range(8)]
    assert fields == [8, 15, 0, 1, 7, 13, 2, 9]


@pytest.mark.parametrize("k,n,bits,m", [(192, 160, 4, 1), (64, 32, 4, 3), (100, 96, 8, 2), (7, 64, 4, 1)])
def test_oracle_packed_gemv_equals_dequantize_then_matmul(k, n, bits, m):
    codes, scales, words, x = case(k, n, bits, m, 100 + k)
    got = orc.q4s_gemv(words, scales, k, n, bits, x)
    want = reference_f64(codes, scales, x)
    assert judge(got, want) < 1e-5
    # every code value, the most negative included, decodes as two's complement: a weight of one repeated code
    for code in (-8, -1, 7) if bits == 4 else (-128, -1, 127):
        c = np.full((k, n), code, np.int8)
        s = np.ones((k, n // 32), np.float32)
        y = orc.q4s_gemv(pack_words(c, bits), s, k, n, bits, np.ones((1, k), np.float32))
        assert np.all(y == np.float32(code * k))


def test_oracle_packed_gemv_rounds_each_term_twice_in_k_order():
    # one column, three terms chosen so that fused or reordered arithmetic gives other bits
    k, n = 3, 32
    codes = np.zeros((k, n), np.int8)
    codes[:, 0] = [7, -5, 3]
    scales = np.array([[0.1], [0.3], [0.7]], np.float32)
    x = np.array([[1.1, 2.3, -0.9]], np.float32)
    f = np.float32
    acc = f(0)
    for i in range(k):
        xs = f(x[0, i] * scales[i, 0])
        acc = f(acc + f(f(codes[i, 0]) * xs))
    got = orc.q4s_gemv(pack_words(codes, 4), scales, k, n, 4, x)
    assert got[0, 0].view(np.uint32) == acc.view(np.uint32) and np.all(got[0, 1:] == 0)


def test_oracle_packed_gemv_refuses_other_layouts():
    with pytest.raises(orc.OracleError):
        orc.q4s_gemv(np.zeros(8, np.uint32), np.zeros(2, np.float32), 2, 32, 2, np.zeros((1, 2), np.float32))
    with pytest.raises(orc.OracleError):
        orc.q4s_gemv(np.zeros(8, np.uint32), np.zeros(2, np.float32), 2, 48, 4, np.zeros((1, 2), np.float32))


# --- the HIP kernel through the C ABI ----------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("k,n,bits,m", [(192, 160, 4, 1), (2048, 1024, 4, 1), (1024, 2048, 4, 5), (5120, 1088, 4, 1),
                                        (100, 96, 8, 2), (7, 64, 4, 1), (4096, 32, 8, 64), (333, 2080, 4, 3)])
def test_gpu_packed_gemv_matches_the_oracle_and_the_f64_product(k, n, bits, m):
    from mummu_amd import moe as M
    codes, scales, words, x = case(k, n, bits, m, 7 * k + n)
    want = reference_f64(codes, scales, x)
    with M.PackedWeight(words, scales, k, n, bits) as w:
        assert w.resident_bytes() == k * n * bits // 8 + k * (n // 32) * 4
        got = w.gemv(x)
        again = w.gemv(x)
        one = w.gemv(x[m - 1])
        xd, yd = M.DeviceBuffer.from_array(x), M.DeviceBuffer(4 * m * n)
        w.gemv_device(xd, m, yd)
        dev = yd.download(np.float32, (m, n))
    assert got.shape == (m, n)
    assert judge(got, want) < 1e-5                                   # the reference's own bar is 1e-4
    assert judge(got, orc.q4s_gemv(words, scales, k, n, bits, x)) < 1e-5
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))            # call to call
    assert np.array_equal(one.view(np.uint32), got[m - 1:].view(np.uint32))      # a row alone or in a batch
    assert np.array_equal(dev.view(np.uint32), got.view(np.uint32))              # device pointers


@pytest.mark.gpu
def test_gpu_packed_gemv_decodes_every_code_and_checks_its_arguments():
    from mummu_amd import moe as M
    k, n = 64, 64
    for bits, vals in ((4, (-8, -1, 0, 7)), (8, (-128, -1, 127))):
        for code in vals:
            c = np.full((k, n), code, np.int8)
            with M.PackedWeight(pack_words(c, bits), np.ones((k, n // 32), np.float32), k, n, bits) as w:
                assert np.all(w.gemv(np.ones((1, k), np.float32)) == np.float32(code * k))
    c = np.zeros((k, n), np.int8)
    with M.PackedWeight(pack_words(c, 4), np.ones((k, 2), np.float32), k, n, 4) as w:
        with pytest.raises(M.MoeError, match="does not match the weight's K"):
            w.gemv(np.zeros((1, k + 1), np.float32))
        with pytest.raises(M.MoeError, match="0 to 64 rows"):
            w.gemv(np.zeros((65, k), np.float32))
        assert w.gemv(np.zeros((0, k), np.float32)).shape == (0, n)
    with pytest.raises(M.MoeError, match="not supported"):
        M.PackedWeight(np.zeros(k * n // 16, np.uint32), np.ones((k, 2), np.float32), k, n, 2)
    with pytest.raises(M.MoeError):
        M.PackedWeight(np.zeros(k * 6, np.uint32), np.ones((k, 1), np.float32), k, 48, 4)


@pytest.mark.gpu
def test_gpu_packed_gemv_on_a_weight_that_is_already_in_device_memory():
    from mummu_amd import moe as M
    k, n = 1024, 2048
    codes, scales, words, x = case(k, n, 4, 3, 77)
    wd, sd = M.DeviceBuffer.from_array(words), M.DeviceBuffer.from_array(scales)
    with M.PackedWeight(words, scales, k, n, 4) as own, M.PackedWeight.wrap_device(wd, sd, k, n, 4) as borrowed:
        assert np.array_equal(own.gemv(x).view(np.uint32), borrowed.gemv(x).view(np.uint32))
    # the borrowed buffers are still the caller's after the handle is gone
    assert np.array_equal(wd.download(np.uint32, words.shape), words)
