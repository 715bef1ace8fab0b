"""The GGUF container reader, restating the reference's own reader tests (gguf.rs:2105-2378,
2796-2823, 2961-2985) over the C ABI: header round trip, every refusal (magic, version,
truncation, bounds, unknown type ids, misaligned offsets, partial blocks, duplicate names,
overlapping payloads), split sets (merged namespace, per-shard payload base, missing shard,
duplicate across shards, tensor-count cross-check), and the MoE configuration keys
(models/olmoe.rs:116-179).  No device work: these run without a GPU."""
import os
import struct

import numpy as np
import pytest

from mummu_amd import _lib
from mummu_amd.gguf import GgufError, GgufFile
from tests import gguf_writer as W
from tests.gguf_writer import GgufWriter


def open_bytes(tmp_path, data: bytes, name="t.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return GgufFile.open(p)


def refused(tmp_path, data: bytes, code, needle=None):
    with pytest.raises(GgufError) as e:
        open_bytes(tmp_path, data)
    assert e.value.code == code, str(e.value)
    if needle:
        assert needle in str(e.value), str(e.value)
    return str(e.value)


def test_minimal_file_round_trips(tmp_path):
    data = (GgufWriter().kv_str("general.architecture", "qwen2").kv_u32("qwen2.block_count", 28)
            .kv_str_array("tokenizer.ggml.tokens", ["a", "b", "c"])
            .tensor("token_embd.weight", [64, 2], 0, 0).tensor("blk.0.attn_q.weight", [256], 12, 512).build())
    with open_bytes(tmp_path, data) as f:
        assert f.version == 3 and f.architecture() == "qwen2"
        assert f.get_u64("qwen2.block_count") == 28
        assert f.kv_count() == 3 and f.tensor_count() == 2 and f.shard_count() == 1
        embd = f.tensor("token_embd.weight")
        assert embd.dims == (64, 2) and embd.dtype == 0 and embd.nbytes == 64 * 2 * 4
        q = f.tensor("blk.0.attn_q.weight")
        assert q.dtype == 12 and q.nbytes == 144
        assert f.alignment == 32
        data_offset = embd.file_offset
        assert data_offset % 32 == 0 and data_offset >= len(data) and data_offset - len(data) < 32
        assert q.file_offset == data_offset + 512
        assert f.tensor("missing") is None and f.get_u64("missing") is None
        assert f.get_str("qwen2.block_count") is None and f.get_u64("general.architecture") is None


def test_version_2_is_accepted_and_every_scalar_type_reads_back(tmp_path):
    w = GgufWriter(version=2)
    w.kv("a.u8", W.U8, 200).kv("a.i8", W.I8, -3).kv("a.u16", W.U16, 60000).kv("a.i16", W.I16, -300)
    w.kv("a.u32", W.U32, 4000000000).kv("a.i32", W.I32, -7).kv("a.f32", W.F32, 0.25).kv("a.bool", W.BOOL, 1)
    w.kv("a.u64", W.U64, 1 << 40).kv("a.i64", W.I64, -(1 << 40)).kv("a.f64", W.F64, 1e-300)
    w.kv("a.nested", W.ARRAY, (W.ARRAY, [(W.U8, [1, 2]), (W.U8, [3])]))
    with open_bytes(tmp_path, w.build()) as f:
        assert f.version == 2
        assert [f.get_u64(k) for k in ("a.u8", "a.u16", "a.u32", "a.u64", "a.bool")] == [200, 60000, 4000000000, 1 << 40, 1]
        # as_u64 takes unsigned types only (gguf.rs:149-157)
        assert f.get_u64("a.i32") is None and f.get_u64("a.i8") is None and f.get_u64("a.f32") is None
        assert f.get_f64("a.f32") == 0.25 and f.get_f64("a.f64") == 1e-300 and f.get_f64("a.u8") is None


def test_bad_magic_version_and_truncation_are_refused(tmp_path):
    good = GgufWriter().kv_str("general.architecture", "qwen2").build()
    refused(tmp_path, b"FUGG" + good[4:], _lib.ERR_GGUF, "not a GGUF file")
    for v in (1, 4):
        refused(tmp_path, good[:4] + struct.pack("<I", v) + good[8:], _lib.ERR_GGUF, f"version {v}")
    refused(tmp_path, good[:-3], _lib.ERR_IO)
    refused(tmp_path, good[:10], _lib.ERR_IO)
    refused(tmp_path, b"", _lib.ERR_IO)
    with pytest.raises(GgufError) as e:
        GgufFile.open(tmp_path / "absent.gguf")
    assert e.value.code == _lib.ERR_IO


def test_oversized_counts_strings_and_arrays_are_refused_before_allocation(tmp_path):
    base = GgufWriter().build()
    refused(tmp_path, base[:8] + struct.pack("<Q", 65537) + base[16:], _lib.ERR_GGUF, "tensor count")
    refused(tmp_path, base[:16] + struct.pack("<Q", 4097) + base[24:], _lib.ERR_GGUF, "kv count")
    # a key string that claims more than 1 MiB, an array that claims more than 2^22 items
    head = b"GGUF" + struct.pack("<IQQ", 3, 0, 1)
    refused(tmp_path, head + struct.pack("<Q", (1 << 20) + 1) + b"x" * 64, _lib.ERR_GGUF, "exceeds the bound")
    arr = head + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", W.ARRAY, W.U8, (1 << 22) + 1)
    refused(tmp_path, arr, _lib.ERR_GGUF, "exceeds the bound")
    # exactly at the bounds the counts pass and the reader then runs out of file
    refused(tmp_path, base[:8] + struct.pack("<Q", 65536) + base[16:], _lib.ERR_IO)


def test_unknown_value_type_and_ggml_type_are_refused(tmp_path):
    with_kv = bytearray(GgufWriter().kv_u32("some.key", 1).build())
    with_kv[40:44] = struct.pack("<I", 99)  # magic 4 + version 4 + counts 16 + key length 8 + key 8
    refused(tmp_path, bytes(with_kv), _lib.ERR_GGUF, "unknown value type 99")
    refused(tmp_path, GgufWriter().tensor("t", [32], 63, 0).build(), _lib.ERR_GGUF, "unknown ggml type id 63")
    refused(tmp_path, GgufWriter().tensor("t", [32], 4, 0).build(), _lib.ERR_GGUF, "unknown ggml type id 4")  # removed Q4_2


def test_bool_bytes_utf8_and_array_depth_are_checked(tmp_path):
    refused(tmp_path, GgufWriter().kv("b", W.BOOL, 2).build(), _lib.ERR_GGUF, "bool byte 2")
    refused(tmp_path, GgufWriter().kv_str("s", b"\xff\xfe").build(), _lib.ERR_GGUF, "UTF-8")
    refused(tmp_path, GgufWriter().kv_str("s", b"\xc0\x80").build(), _lib.ERR_GGUF, "UTF-8")   # overlong NUL
    refused(tmp_path, GgufWriter().kv_str("s", b"\xed\xa0\x80").build(), _lib.ERR_GGUF, "UTF-8")  # surrogate
    refused(tmp_path, GgufWriter().kv_str("s", b"ab\xe2\x82").build(), _lib.ERR_GGUF, "UTF-8")  # cut short
    with open_bytes(tmp_path, GgufWriter().kv_str("s", "héllo € \U0001f600").build()) as f:
        assert f.get_str("s") == "héllo € \U0001f600"
    deep = (W.ARRAY, [(W.ARRAY, [(W.U8, [1])])])
    refused(tmp_path, GgufWriter().kv("deep", W.ARRAY, deep).build(), _lib.ERR_GGUF, "nested")


def test_alignment_must_be_a_power_of_two_and_moves_the_payload_base(tmp_path):
    refused(tmp_path, GgufWriter().kv_u32("general.alignment", 48).build(), _lib.ERR_GGUF, "48 is not a power of two")
    refused(tmp_path, GgufWriter().kv_u32("general.alignment", 0).build(), _lib.ERR_GGUF, "power of two")
    w = GgufWriter(alignment=256).kv_u32("general.alignment", 256)
    a = np.arange(8, dtype=np.float32)
    b = np.arange(8, dtype=np.float32) + 50
    w.add("a", [8], 0, a).add("b", [8], 0, b)
    data = w.build()
    with open_bytes(tmp_path, data) as f:
        assert f.alignment == 256
        ta, tb = f.tensor("a"), f.tensor("b")
        assert ta.file_offset % 256 == 0 and tb.file_offset == ta.file_offset + 256
        assert np.array_equal(f.tensor_bytes("a").view(np.float32), a)
        assert np.array_equal(f.tensor_bytes("b").view(np.float32), b)
    # an offset that is aligned for 32 but not for the declared 256
    refused(tmp_path, GgufWriter().kv_u32("general.alignment", 256).tensor("t", [8], 0, 32).build(), _lib.ERR_GGUF,
            "not 256-aligned")


def test_misaligned_offsets_partial_blocks_dims_and_duplicates_are_refused(tmp_path):
    refused(tmp_path, GgufWriter().tensor("t", [32], 8, 7).build(), _lib.ERR_GGUF, "offset 7 not 32-aligned")
    refused(tmp_path, GgufWriter().tensor("t", [100], 12, 0).build(), _lib.ERR_GGUF, "not whole blocks")
    refused(tmp_path, GgufWriter().tensor("t", [0], 0, 0).build(), _lib.ERR_GGUF, "0 elements")
    refused(tmp_path, GgufWriter().tensor("t", [], 0, 0).build(), _lib.ERR_GGUF, "0 dims")
    refused(tmp_path, GgufWriter().tensor("t", [2, 2, 2, 2, 2], 0, 0).build(), _lib.ERR_GGUF, "5 dims")
    refused(tmp_path, GgufWriter().tensor("t", [1 << 40, 1 << 40], 0, 0).build(), _lib.ERR_GGUF, "overflows")
    refused(tmp_path, GgufWriter().tensor("t", [32], 8, 0).tensor("t", [32], 8, 64).build(), _lib.ERR_GGUF,
            "duplicate tensor name")


def test_overlapping_tensor_payloads_are_refused(tmp_path):
    # a 32-element Q8_0 tensor is 34 bytes; a second tensor at the next aligned offset lands inside it
    msg = refused(tmp_path, GgufWriter().kv_str("general.architecture", "qwen2").tensor("a.weight", [32], 8, 0)
                  .tensor("b.weight", [8], 0, 32).build(), _lib.ERR_GGUF, "overlaps")
    assert "a.weight" in msg and "b.weight" in msg
    with open_bytes(tmp_path, GgufWriter().tensor("a.weight", [32], 8, 0).tensor("b.weight", [8], 0, 64).build()) as f:
        assert f.tensor_count() == 2
    # table order does not matter, only payload order
    refused(tmp_path, GgufWriter().tensor("late", [8], 0, 32).tensor("early", [32], 8, 0).build(), _lib.ERR_GGUF, "overlaps")


def test_a_payload_that_runs_past_the_end_of_the_file_is_refused_on_read(tmp_path):
    w = GgufWriter().add("t", [8], 0, np.arange(8, dtype=np.float32))
    data = w.build()
    with open_bytes(tmp_path, data[:-4]) as f:  # the header is whole, the payload is not
        with pytest.raises(GgufError, match="past the end"):
            f.tensor_bytes("t")


# ---- split sets (gguf.rs:2105-2240) ----------------------------------------------------------

def two_shard_set():
    a = np.arange(8, dtype=np.float32)
    b = np.arange(8, dtype=np.float32) + 100
    s0 = (GgufWriter().kv_str("general.architecture", "qwen4exp").kv_u32("split.count", 2).kv_u32("split.no", 0)
          .kv_u32("split.tensors.count", 2).add("a.weight", [8], 0, a))
    s1 = GgufWriter().kv_u32("split.count", 2).kv_u32("split.no", 1).add("b.weight", [8], 0, b)  # stub metadata
    return [s0, s1]


def write_set(tmp_path, shards, base="m", total=None):
    total = len(shards) if total is None else total
    paths = []
    for i, s in enumerate(shards):
        p = tmp_path / f"{base}-{i + 1:05d}-of-{total:05d}.gguf"
        s.write(p)
        paths.append(p)
    return paths


def test_a_split_set_opens_as_one_namespace_from_any_member(tmp_path):
    paths = write_set(tmp_path, two_shard_set())
    for member in paths:
        with GgufFile.open(member) as f:
            assert f.shard_count() == 2 and f.tensor_count() == 2
            assert f.architecture() == "qwen4exp"  # metadata from the richest shard, not shard order
            a, b = f.tensor("a.weight"), f.tensor("b.weight")
            assert a.shard == 0 and b.shard == 1 and a.path.endswith("00001-of-00002.gguf") and b.path.endswith("00002-of-00002.gguf")
            # both sit at offset 0 of their OWN shard: resolving against the wrong base reads the wrong bytes
            assert f.tensor_bytes("a.weight").view(np.float32)[0] == 0.0
            assert f.tensor_bytes("b.weight").view(np.float32)[0] == 100.0
            assert f.tensor_bytes("b.weight").view(np.float32).tolist() == [100.0 + i for i in range(8)]


def test_a_model_name_that_contains_of_still_splits_from_the_right(tmp_path):
    paths = write_set(tmp_path, two_shard_set(), base="best-of-breed-7b")
    with GgufFile.open(paths[0]) as f:
        assert f.shard_count() == 2 and f.tensor("b.weight") is not None


def test_a_single_file_is_unchanged_by_the_sharded_path(tmp_path):
    w = GgufWriter().kv_str("general.architecture", "qwen2").add("only.weight", [8], 0, np.arange(8, dtype=np.float32))
    with open_bytes(tmp_path, w.build(), "m-00001-of-00001.gguf") as f:
        assert f.shard_count() == 1 and f.tensor_bytes("only.weight").view(np.float32)[0] == 0.0
    w.kv_u32("split.count", 1)
    with open_bytes(tmp_path, w.build(), "plain.gguf") as f:
        assert f.shard_count() == 1


def test_a_missing_shard_is_refused_by_name(tmp_path):
    p = tmp_path / "m-00001-of-00002.gguf"
    two_shard_set()[0].write(p)
    with pytest.raises(GgufError, match="missing shard") as e:
        GgufFile.open(p)
    assert "m-00002-of-00002.gguf" in str(e.value)


def test_split_names_without_an_index_and_too_many_shards_are_refused(tmp_path):
    p = tmp_path / "model.gguf"
    two_shard_set()[0].write(p)
    with pytest.raises(GgufError, match="-of-"):
        GgufFile.open(p)
    p = tmp_path / "m-00001-of-00065.gguf"
    GgufWriter().kv_u32("split.count", 65).write(p)
    with pytest.raises(GgufError, match="64"):
        GgufFile.open(p)


def test_a_duplicate_tensor_name_across_shards_is_refused(tmp_path):
    dup = GgufWriter().kv_u32("split.count", 2).kv_u32("split.no", 1).add("a.weight", [8], 0, np.zeros(8, np.float32))
    paths = write_set(tmp_path, [two_shard_set()[0], dup])
    with pytest.raises(GgufError, match="more than one shard"):
        GgufFile.open(paths[0])


def test_a_tensor_count_that_disagrees_with_the_shards_is_refused(tmp_path):
    s = two_shard_set()
    s[0] = (GgufWriter().kv_str("general.architecture", "qwen4exp").kv_u32("split.count", 2).kv_u32("split.no", 0)
            .kv_u32("split.tensors.count", 3).add("a.weight", [8], 0, np.zeros(8, np.float32)))
    paths = write_set(tmp_path, s)
    with pytest.raises(GgufError, match="declares 3"):
        GgufFile.open(paths[0])


def test_a_broken_shard_reports_its_own_path(tmp_path):
    s = two_shard_set()
    paths = write_set(tmp_path, s)
    paths[1].write_bytes(b"FUGG" + paths[1].read_bytes()[4:])
    with pytest.raises(GgufError, match="00002-of-00002") as e:
        GgufFile.open(paths[0])
    assert "not a GGUF file" in str(e.value)


# ---- the MoE block's configuration (models/olmoe.rs:116-179, 210-215) -------------------------

def olmoe_header(**over):
    kv = {"olmoe.block_count": 16, "olmoe.embedding_length": 2048, "olmoe.feed_forward_length": 1024,
          "olmoe.expert_count": 64, "olmoe.expert_used_count": 8}
    kv.update(over)
    w = GgufWriter().kv_str("general.architecture", "olmoe")
    for k, v in kv.items():
        if v is not None:
            w.kv_u32(k, v)
    w.kv_f32("olmoe.attention.layer_norm_rms_epsilon", 1e-5)
    return w


def test_the_moe_configuration_is_read_from_the_architectures_keys(tmp_path):
    with open_bytes(tmp_path, olmoe_header().build()) as f:
        c = f.moe_config()
        assert (c.hidden_size, c.expert_intermediate_size, c.num_experts, c.num_experts_per_tok, c.num_layers) == (2048, 1024, 64, 8, 16)
        assert c.norm_topk_prob == 0 and abs(c.rms_norm_eps - 1e-5) < 1e-12
    # expert_feed_forward_length wins over feed_forward_length; expert_weights_norm is honoured
    w = olmoe_header(**{"olmoe.expert_feed_forward_length": 512}).kv_bool("olmoe.expert_weights_norm", True)
    with open_bytes(tmp_path, w.build()) as f:
        c = f.moe_config()
        assert c.expert_intermediate_size == 512 and c.norm_topk_prob == 1
    # any architecture prefix works the same way (qwen3moe files use the same key names)
    w = GgufWriter().kv_str("general.architecture", "qwen3moe")
    for k, v in (("block_count", 2), ("embedding_length", 64), ("expert_feed_forward_length", 32), ("expert_count", 4),
                 ("expert_used_count", 2)):
        w.kv_u32(f"qwen3moe.{k}", v)
    w.kv_f32("qwen3moe.attention.layer_norm_rms_epsilon", 1e-6)
    with open_bytes(tmp_path, w.build()) as f:
        assert f.moe_config().num_experts == 4


@pytest.mark.parametrize("over,needle", [
    ({"olmoe.embedding_length": None}, "olmoe.embedding_length"),
    ({"olmoe.feed_forward_length": None}, "olmoe.feed_forward_length"),
    ({"olmoe.expert_count": None}, "olmoe.expert_count"),
    ({"olmoe.expert_used_count": None}, "olmoe.expert_used_count"),
    ({"olmoe.block_count": None}, "olmoe.block_count"),
    ({"olmoe.expert_count": 1}, "num_experts must be >= 2"),
    ({"olmoe.expert_used_count": 0}, "num_experts_per_tok"),
    ({"olmoe.expert_used_count": 65}, "num_experts_per_tok"),
])
def test_missing_or_unusable_configuration_keys_are_refused(tmp_path, over, needle):
    with open_bytes(tmp_path, olmoe_header(**over).build()) as f:
        with pytest.raises(GgufError, match=needle):
            f.moe_config()


def test_a_signed_count_and_a_missing_architecture_are_refused(tmp_path):
    w = GgufWriter().kv_str("general.architecture", "olmoe").kv("olmoe.embedding_length", W.I32, 2048)
    with open_bytes(tmp_path, w.build()) as f:
        with pytest.raises(GgufError, match="olmoe.embedding_length"):
            f.moe_config()
    with open_bytes(tmp_path, GgufWriter().kv_u32("olmoe.embedding_length", 8).build()) as f:
        with pytest.raises(GgufError, match="general.architecture"):
            f.moe_config()


def test_null_arguments_are_errors_not_crashes():
    lib = _lib.load()
    assert lib.mummu_gguf_open(None, None) == _lib.ERR_ARG
    assert lib.mummu_gguf_tensor_count(None) == -1 and lib.mummu_gguf_find_tensor(None, b"x") == -1
    assert lib.mummu_gguf_moe_config(None, None) == _lib.ERR_ARG
    assert lib.mummu_moe_load_gguf(None, None, 0, 1) == _lib.ERR_ARG
    lib.mummu_gguf_close(None)
    assert os.path.exists(_lib.LIB_PATH)


# ---- the expert-bank locator (models/olmoe.rs:325-347, experts.rs:869-911) ----------------------

TOY = dict(hidden=256, inter=32, experts=4, top_k=2, router_type=0, gate_type=12, up_type=8, down_type=8)


def toy_weights(case, layers=2):
    from mummu_amd import synth
    H, I, E = case["hidden"], case["inter"], case["experts"]
    out = []
    for l in range(layers):
        rng = synth.SplitMix64(900 + l)
        out.append(dict(router=rng.normal(E * H, 0.0, 0.05),
                        gate=synth.random_bank_fast(case["gate_type"], [H, I, E], 10 + l),
                        up=synth.random_bank_fast(case["up_type"], [H, I, E], 20 + l),
                        down=synth.random_bank_fast(case["down_type"], [I, H, E], 30 + l)))
    return out


def test_the_locator_finds_every_bank_with_its_bytes_unchanged(tmp_path):
    lw = toy_weights(TOY)
    gamma = [np.full(TOY["hidden"], 1.0 + l, np.float32) for l in range(2)]
    p = W.moe_gguf(TOY, lw, norm_gamma=gamma).write(tmp_path / "toy.gguf")
    with GgufFile.open(p) as f:
        for l in range(2):
            at = f.locate_moe_layer(l)
            assert at["router"].name == f"blk.{l}.ffn_gate_inp.weight" and at["router"].dims == (256, 4)
            assert at["gate"].dims == (256, 32, 4) and at["gate"].dtype == 12 and at["gate"].nbytes == 4 * 32 * 144
            assert at["down"].dims == (32, 256, 4) and at["down"].dtype == 8 and at["down"].nbytes == 4 * 256 * 34
            assert at["norm"].dims == (256,)
            for k, name in (("gate", "ffn_gate_exps"), ("up", "ffn_up_exps"), ("down", "ffn_down_exps")):
                assert np.array_equal(f.tensor_bytes(f"blk.{l}.{name}.weight"), lw[l][k].view(np.uint8).reshape(-1))
            assert np.array_equal(f.tensor_bytes(f"blk.{l}.ffn_norm.weight").view(np.float32), gamma[l])
        with pytest.raises(GgufError, match="layer 2"):
            f.locate_moe_layer(2)
    with GgufFile.open(W.moe_gguf(TOY, lw).write(tmp_path / "nonorm.gguf")) as f:
        assert f.locate_moe_layer(0)["norm"] is None


def test_the_locator_refuses_missing_banks_wrong_dims_and_rows_of_partial_blocks(tmp_path):
    lw = toy_weights(TOY, 1)
    w = W.moe_gguf(TOY, lw)
    w.tensors = [t for t in w.tensors if "ffn_up_exps" not in t[0]]
    with GgufFile.open(w.write(tmp_path / "a.gguf")) as f:
        with pytest.raises(GgufError, match="GGUF has no blk.0.ffn_up_exps.weight"):
            f.locate_moe_layer(0)
    # gate stored [I, H, E] instead of [H, I, E]
    w = W.moe_gguf(TOY, lw)
    w.tensors = [(n, (d[1], d[0], d[2]) if "ffn_gate_exps" in n else d, t, o) for n, d, t, o in w.tensors]
    with GgufFile.open(w.write(tmp_path / "b.gguf")) as f:
        with pytest.raises(GgufError, match="ffn_gate_exps.weight: dim 0 is 32") as e:
            f.locate_moe_layer(0)
        assert e.value.code == _lib.ERR_SHAPE
    # a 2-dim bank
    w = W.moe_gguf(TOY, lw)
    w.tensors = [(n, (d[0], d[1] * d[2]) if "ffn_down_exps" in n else d, t, o) for n, d, t, o in w.tensors]
    with GgufFile.open(w.write(tmp_path / "c.gguf")) as f:
        with pytest.raises(GgufError, match="has 2 dims, want 3"):
            f.locate_moe_layer(0)
    # the down bank's row is the 32-wide intermediate: whole Q8_0 blocks but not whole Q4_K
    # superblocks, although the tensor as a whole is (experts.rs:150-154)
    case = dict(TOY, down_type=12)
    lw2 = toy_weights(dict(TOY), 1)
    lw2[0]["down"] = np.zeros(4 * 256 * 32 // 256 * 144, np.uint8)
    with GgufFile.open(W.moe_gguf(case, lw2).write(tmp_path / "d.gguf")) as f:
        with pytest.raises(GgufError, match="a row of 32 elements is not whole blocks") as e:
            f.locate_moe_layer(0)
        assert e.value.code == _lib.ERR_BLOCKS
    # an F16 pre-norm weight
    w = W.moe_gguf(TOY, lw, norm_gamma=[np.ones(256, np.float16)])
    w.tensors = [(n, d, 1 if "ffn_norm" in n else t, o) for n, d, t, o in w.tensors]
    with GgufFile.open(w.write(tmp_path / "e.gguf")) as f:
        with pytest.raises(GgufError, match="must be F32"):
            f.locate_moe_layer(0)


def test_banks_split_over_shards_are_located_in_their_own_files(tmp_path):
    lw = toy_weights(TOY, 2)
    whole = W.moe_gguf(TOY, lw)
    s0 = GgufWriter()
    s0.kvs = list(whole.kvs) + [("split.count", W.U32, 2), ("split.no", W.U32, 0), ("split.tensors.count", W.U32, 8)]
    s1 = GgufWriter().kv_u32("split.count", 2).kv_u32("split.no", 1)
    for l, dst in ((0, s0), (1, s1)):
        dst.add(f"blk.{l}.ffn_gate_inp.weight", [256, 4], 0, lw[l]["router"])
        dst.add(f"blk.{l}.ffn_gate_exps.weight", [256, 32, 4], 12, lw[l]["gate"])
        dst.add(f"blk.{l}.ffn_up_exps.weight", [256, 32, 4], 8, lw[l]["up"])
        dst.add(f"blk.{l}.ffn_down_exps.weight", [32, 256, 4], 8, lw[l]["down"])
    paths = write_set(tmp_path, [s0, s1], base="toy")
    with GgufFile.open(paths[1]) as f:
        assert f.shard_count() == 2 and f.moe_config().num_layers == 2
        a0, a1 = f.locate_moe_layer(0), f.locate_moe_layer(1)
        assert a0["gate"].shard == 0 and a1["gate"].shard == 1
        assert np.array_equal(f.tensor_bytes("blk.1.ffn_gate_exps.weight"), lw[1]["gate"].view(np.uint8).reshape(-1))
        assert np.array_equal(f.tensor_bytes("blk.0.ffn_down_exps.weight"), lw[0]["down"].view(np.uint8).reshape(-1))
