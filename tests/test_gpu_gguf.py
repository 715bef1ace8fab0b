"""A model file written to disk, opened through the GGUF reader and loaded through the
expert-bank locator must behave exactly like the same bytes handed to load_layer directly:
the payload reaches the kernels unchanged, so the outputs are bit-identical.  Covers a single
file with pre-norm weights (stack forward), a two-shard split set, and 256-byte alignment."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd import synth
from mummu_amd.gguf import GgufError, GgufFile
from tests import gguf_writer as W
from tests.test_gguf_reader import write_set

pytestmark = pytest.mark.gpu

CASE = dict(hidden=512, inter=256, experts=8, top_k=2, router_type=1, gate_type=12, up_type=12, down_type=8, norm=True)


def weights(case, layers, seed):
    H, I, E = case["hidden"], case["inter"], case["experts"]
    g = np.random.Generator(np.random.PCG64(seed))
    out = []
    for l in range(layers):
        out.append(dict(router=(g.standard_normal(E * H, dtype=np.float32) * 0.05).astype(np.float16),
                        gate=synth.random_bank_fast(case["gate_type"], [H, I, E], seed + 10 * l + 1),
                        up=synth.random_bank_fast(case["up_type"], [H, I, E], seed + 10 * l + 2),
                        down=synth.random_bank_fast(case["down_type"], [I, H, E], seed + 10 * l + 3),
                        gamma=(1.0 + 0.1 * g.standard_normal(H, dtype=np.float32)).astype(np.float32)))
    return out


def direct(case, lw, max_tokens):
    m = M.SparseMoe(M.SparseMoeConfig(case["hidden"], case["inter"], case["experts"], case["top_k"]),
                    num_layers=len(lw), max_tokens=max_tokens, rms_norm_eps=case.get("eps", 1e-5))
    for l, w in enumerate(lw):
        m.load_layer(l, w["router"], case["router_type"], w["gate"], case["gate_type"], w["up"], case["up_type"],
                     w["down"], case["down_type"], w["gamma"])
    return m


@pytest.mark.parametrize("alignment", [32, 256])
def test_a_gguf_file_loads_to_the_same_bits_as_load_layer(tmp_path, alignment):
    lw = weights(CASE, 3, 5)
    path = W.moe_gguf(CASE, lw, alignment=alignment, norm_gamma=[w["gamma"] for w in lw]).write(tmp_path / "m.gguf")
    g = np.random.Generator(np.random.PCG64(99))
    x = g.standard_normal((70, CASE["hidden"]), dtype=np.float32)
    with GgufFile.open(path) as f, direct(CASE, lw, 128) as ref:
        cfg = f.moe_config()
        assert cfg.norm_topk_prob == 1 and cfg.num_layers == 3
        with f.load_moe(max_tokens=128) as m:
            assert m.resident_bytes() == ref.resident_bytes()
            for n in (1, 5, 70):
                for l in range(3):
                    a = m.forward(x[:n], 2, True, layer=l)
                    b = ref.forward(x[:n], 2, True, layer=l)
                    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n, l)
            a = m.stack_forward(x[:4], 2, True)
            b = ref.stack_forward(x[:4], 2, True)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
            assert np.array_equal(m.dequantize_expert(1, "gate", 3), ref.dequantize_expert(1, "gate", 3))
        # a window of layers: file layers 1..3 become handle layers 0..2
        with f.load_moe(1, 2, max_tokens=8) as m:
            assert np.array_equal(m.forward(x[:3], 2, True, layer=0), ref.forward(x[:3], 2, True, layer=1))
            assert np.array_equal(m.forward(x[:3], 2, True, layer=1), ref.forward(x[:3], 2, True, layer=2))
        with pytest.raises(GgufError, match="layer 3"):
            f.load_moe(2, 2, max_tokens=8)


def test_a_split_set_loads_each_bank_from_its_own_shard(tmp_path):
    lw = weights(CASE, 2, 21)
    whole = W.moe_gguf(CASE, lw)
    s0 = W.GgufWriter()
    s0.kvs = list(whole.kvs) + [("split.count", W.U32, 2), ("split.no", W.U32, 0), ("split.tensors.count", W.U32, 10)]
    s1 = W.GgufWriter().kv_u32("split.count", 2).kv_u32("split.no", 1)
    H, I, E = CASE["hidden"], CASE["inter"], CASE["experts"]
    for l, dst in ((0, s0), (1, s1)):  # both shards' first tensor sits at offset 0 of its own payload
        dst.add(f"blk.{l}.ffn_gate_exps.weight", [H, I, E], CASE["gate_type"], lw[l]["gate"])
        dst.add(f"blk.{l}.ffn_gate_inp.weight", [H, E], CASE["router_type"], lw[l]["router"])
        dst.add(f"blk.{l}.ffn_norm.weight", [H], 0, lw[l]["gamma"])
        dst.add(f"blk.{l}.ffn_up_exps.weight", [H, I, E], CASE["up_type"], lw[l]["up"])
        dst.add(f"blk.{l}.ffn_down_exps.weight", [I, H, E], CASE["down_type"], lw[l]["down"])
    paths = write_set(tmp_path, [s0, s1], base="toy-of-two")
    g = np.random.Generator(np.random.PCG64(3))
    x = g.standard_normal((9, H), dtype=np.float32)
    with GgufFile.open(paths[0]) as f, direct(CASE, lw, 16) as ref, f.load_moe(max_tokens=16) as m:
        for l in range(2):
            assert np.array_equal(m.forward(x, 2, True, layer=l).view(np.uint32), ref.forward(x, 2, True, layer=l).view(np.uint32))
        assert np.array_equal(m.stack_forward(x, 2, True).view(np.uint32), ref.stack_forward(x, 2, True).view(np.uint32))


def test_a_bank_type_without_a_kernel_is_refused_with_the_tensor_named(tmp_path):
    case = dict(CASE, down_type=10)  # Q2_K (84-byte super-blocks) parses as a container type but has no expert kernel here
    lw = weights(CASE, 1, 8)
    lw[0]["down"] = np.zeros(CASE["experts"] * CASE["hidden"] * (CASE["inter"] // 256) * 84, np.uint8)
    with GgufFile.open(W.moe_gguf(case, lw).write(tmp_path / "q2.gguf")) as f:
        with pytest.raises(GgufError, match="blk.0") as e:
            f.load_moe(max_tokens=8)
        assert e.value.code == M._lib.ERR_TYPE


def test_a_file_of_another_geometry_is_refused_by_an_existing_handle(tmp_path):
    lw = weights(CASE, 1, 11)
    path = W.moe_gguf(CASE, lw).write(tmp_path / "m.gguf")
    with GgufFile.open(path) as f:
        for H, I, E in [(1024, 256, 8), (512, 512, 8), (512, 256, 16)]:
            with M.SparseMoe(M.SparseMoeConfig(H, I, E, 2), max_tokens=4) as m:
                with pytest.raises(GgufError, match="the handle was created for"):
                    f.load_into(m)
        with M.SparseMoe(M.SparseMoeConfig(512, 256, 8, 2), max_tokens=4) as m:
            with pytest.raises(GgufError, match="do not fit the handle"):
                f.load_into(m, 0, 2)
            f.load_into(m)
            x = np.random.Generator(np.random.PCG64(1)).standard_normal((3, 512), dtype=np.float32)
            with direct(CASE, lw, 4) as ref:
                assert np.array_equal(m.forward(x, 2, True).view(np.uint32), ref.forward(x, 2, True).view(np.uint32))
