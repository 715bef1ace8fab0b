"""An HF-style checkpoint directory (per-expert tensors, scrambled over shards, BF16 / F16 / F32)
loaded through the fuse must behave exactly like the same weights stacked by hand and given to
load_layer: bit-identical outputs, and within 1e-5 of the oracle on the stacked banks."""
import numpy as np
import pytest

from mummu_amd import moe as M
from mummu_amd.safetensors import Checkpoint, SafetensorsError
from oracle import binding as orc
from tests import safetensors_writer as SW

pytestmark = pytest.mark.gpu

H, I, E, K, L = 256, 96, 8, 2, 2


def make_layers(seed):
    g = np.random.Generator(np.random.PCG64(seed))
    return [dict(router=(g.standard_normal((E, H), dtype=np.float32) * 0.05), gate=g.standard_normal((E, I, H), dtype=np.float32) * 0.05,
                 up=g.standard_normal((E, I, H), dtype=np.float32) * 0.05, down=g.standard_normal((E, H, I), dtype=np.float32) * 0.05,
                 gamma=(1.0 + 0.1 * g.standard_normal(H, dtype=np.float32)).astype(np.float32)) for _ in range(L)]


@pytest.mark.parametrize("dtype,shards", [("BF16", 3), ("F16", 1), ("F32", 2)])
def test_the_fused_checkpoint_equals_hand_stacked_banks(tmp_path, dtype, shards):
    lw = make_layers(3)
    mt = {"BF16": M.BF16, "F16": M.F16, "F32": M.F32}[dtype]
    d = SW.write_checkpoint(tmp_path / "ck", SW.olmoe_config(H, I, E, K, L, norm_topk_prob=True), lw, dtype, shards=shards)
    x = np.random.Generator(np.random.PCG64(9)).standard_normal((11, H), dtype=np.float32)
    with Checkpoint.open(d) as ck, ck.load_moe(max_tokens=16) as m, \
            M.SparseMoe(M.SparseMoeConfig(H, I, E, K), num_layers=L, max_tokens=16) as ref:
        assert ck.moe_config().norm_topk_prob == 1
        enc = lambda a: SW.encode(a, dtype)
        stored_gamma = lambda w: (enc(w["gamma"]).astype(np.uint32) << 16).view(np.float32) if dtype == "BF16" else enc(w["gamma"]).astype(np.float32)
        for l, w in enumerate(lw):
            ref.load_layer(l, enc(w["router"]), mt, enc(w["gate"]), mt, enc(w["up"]), mt, enc(w["down"]), mt, stored_gamma(w))
        assert m.resident_bytes() == ref.resident_bytes()
        for l in range(L):
            for n in (1, 11):
                a, b = m.forward(x[:n], K, True, layer=l), ref.forward(x[:n], K, True, layer=l)
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (l, n)
        assert np.array_equal(m.stack_forward(x, K, True).view(np.uint32), ref.stack_forward(x, K, True).view(np.uint32))
        got = m.forward(x, K, True, layer=1)
        ot = {"BF16": orc.BF16, "F16": orc.F16, "F32": orc.F32}[dtype]
        w = lw[1]
        banks = orc.LayerBanks(H, I, E, enc(w["gate"]), enc(w["up"]), enc(w["down"]), ot)
        want, ids, _, _ = orc.moe_forward(banks, enc(w["router"]), ot, x, K, True)
        assert np.abs(got - want).max() <= 1e-5
        # a window of layers
        with ck.load_moe(1, 1, max_tokens=16) as one:
            assert np.array_equal(one.forward(x, K, True, layer=0), got)
        with pytest.raises(SafetensorsError, match="layer 2"):
            ck.load_moe(1, 2, max_tokens=16)


def test_a_short_group_is_refused_before_anything_is_loaded(tmp_path):
    lw = make_layers(4)
    d = SW.write_checkpoint(tmp_path / "short", SW.olmoe_config(H, I, E, K, L), lw, "BF16",
                            skip=("model.layers.1.mlp.experts.5.gate_proj.weight",))
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="7 of 8 members present"):
            ck.load_moe(max_tokens=8)
        with ck.load_moe(0, 1, max_tokens=8) as m:  # layer 0 alone is whole
            assert m.resident_bytes() > 0


def test_a_checkpoint_of_another_geometry_is_refused_by_an_existing_handle(tmp_path):
    d = SW.write_checkpoint(tmp_path / "ck", SW.olmoe_config(H, I, E, K, L), make_layers(4), "BF16")
    with Checkpoint.open(d) as ck:
        for h, i, e in [(2 * H, I, E), (H, 2 * I, E), (H, I, 2 * E)]:
            with M.SparseMoe(M.SparseMoeConfig(h, i, e, K), num_layers=L, max_tokens=4) as m:
                with pytest.raises(SafetensorsError, match="the handle was created for"):
                    ck.load_into(m, 0, L)
        with M.SparseMoe(M.SparseMoeConfig(H, I, E, K), num_layers=1, max_tokens=4) as m:
            with pytest.raises(SafetensorsError, match="do not fit the handle"):
                ck.load_into(m, 0, 2)
            ck.load_into(m, 1, 1)
