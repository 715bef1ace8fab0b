"""The HF-checkpoint side of the MoE block without a device: config.json parsing and validation
(models/olmoe.rs:52-226), safetensors header rules (safetensors.rs:180-320), shard discovery
(:377-430) and the expert group rules of the fuse (:600-740; models/olmoe.rs:405-430)."""
import json
import os
import struct

import numpy as np
import pytest

from mummu_amd import _lib
from mummu_amd.safetensors import Checkpoint, SafetensorsError, olmoe_config_from_json
from tests import safetensors_writer as SW

H, I, E, K = 8, 6, 4, 2


def layers(n=2, seed=0):
    g = np.random.Generator(np.random.PCG64(seed))
    return [dict(router=g.standard_normal((E, H), dtype=np.float32), gate=g.standard_normal((E, I, H), dtype=np.float32),
                 up=g.standard_normal((E, I, H), dtype=np.float32), down=g.standard_normal((E, H, I), dtype=np.float32),
                 gamma=np.ones(H, np.float32)) for _ in range(n)]


# ---- config.json ---------------------------------------------------------------------------------

def test_config_fields_defaults_and_validation():
    base = SW.olmoe_config(2048, 1024, 64, 8, 16)
    c = olmoe_config_from_json(json.dumps(base))
    assert (c.hidden_size, c.expert_intermediate_size, c.num_experts, c.num_experts_per_tok, c.num_layers) == (2048, 1024, 64, 8, 16)
    assert c.norm_topk_prob == 0 and abs(c.rms_norm_eps - 1e-5) < 1e-12
    assert olmoe_config_from_json(json.dumps(dict(base, norm_topk_prob=True))).norm_topk_prob == 1
    no_norm = {k: v for k, v in base.items() if k != "norm_topk_prob"}  # #[serde(default)]
    assert olmoe_config_from_json(json.dumps(no_norm)).norm_topk_prob == 0
    for over, needle in [
        (dict(num_experts=1), "num_experts (1) must be >= 2"),
        (dict(num_experts_per_tok=0), "in 1..=num_experts"),
        (dict(num_experts_per_tok=65), "in 1..=num_experts"),
        (dict(num_hidden_layers=0), "must be positive"),
        (dict(vocab_size=0), "must be positive"),
        (dict(num_key_value_heads=0), "positive multiple"),
        (dict(num_attention_heads=6, num_key_value_heads=4), "positive multiple"),
        (dict(hidden_size=2046), "split evenly"),
        (dict(num_attention_heads=2048, num_key_value_heads=2048), "even-sized heads"),
    ]:
        with pytest.raises(SafetensorsError, match=needle.replace("(", r"\(").replace(")", r"\)")) as e:
            olmoe_config_from_json(json.dumps(dict(base, **over)))
        assert e.value.code == _lib.ERR_CONFIG
    for missing in ("hidden_size", "intermediate_size", "num_experts", "num_experts_per_tok", "rms_norm_eps", "num_hidden_layers"):
        with pytest.raises(SafetensorsError, match=missing):
            olmoe_config_from_json(json.dumps({k: v for k, v in base.items() if k != missing}))
    with pytest.raises(SafetensorsError, match="not an unsigned integer"):
        olmoe_config_from_json(json.dumps(dict(base, num_experts=64.5)))
    with pytest.raises(SafetensorsError, match="not an unsigned integer"):
        olmoe_config_from_json(json.dumps(dict(base, hidden_size=-2048)))
    for broken in ('{"hidden_size": 1,}', '{"a": tru}', '[1, 2', '{"a": "\\q"}', '{"a": 1} x', ""):
        with pytest.raises(SafetensorsError):
            olmoe_config_from_json(broken)
    # string escapes and nesting in fields the block ignores do not disturb it
    odd = dict(base, note="café \\ \"q\" 😀", rope_scaling=None, nested={"a": [1, 2.5e3, {"b": []}]})
    assert olmoe_config_from_json(json.dumps(odd)).num_experts == 64
    assert olmoe_config_from_json(json.dumps(odd, ensure_ascii=False).encode("utf-8")).num_experts == 64


# ---- headers and shards --------------------------------------------------------------------------

def test_a_checkpoint_directory_opens_single_file_or_sharded(tmp_path):
    lw = layers()
    for shards in (1, 3):
        d = SW.write_checkpoint(tmp_path / f"ckpt{shards}", SW.olmoe_config(H, I, E, K, 2), lw, "BF16", shards=shards)
        with Checkpoint.open(d) as ck:
            assert ck.shard_count() == shards
            assert ck.tensor_count() == 2 * (3 + 3 * E)
            t = ck.tensor("model.layers.1.mlp.experts.3.down_proj.weight")
            assert t.dtype == "BF16" and t.shape == (H, I) and t.nbytes == H * I * 2
            raw = np.fromfile(t.path, dtype=np.uint16, count=H * I, offset=t.file_offset)
            assert np.array_equal(raw, SW.to_bf16(lw[1]["down"][3]).reshape(-1))
            assert ck.tensor("nope") is None
            c = ck.moe_config()
            assert (c.hidden_size, c.num_experts, c.num_layers) == (H, E, 2)
            ck.check_moe_layer(0)
            ck.check_moe_layer(1)
            with pytest.raises(SafetensorsError, match="layer 2"):
                ck.check_moe_layer(2)


def test_missing_checkpoint_and_missing_shards_are_named(tmp_path):
    d = tmp_path / "empty"
    d.mkdir()
    with pytest.raises(SafetensorsError, match="neither model.safetensors nor") as e:
        Checkpoint.open(d)
    assert e.value.code == _lib.ERR_IO
    d = SW.write_checkpoint(tmp_path / "c", SW.olmoe_config(H, I, E, K, 2), layers(), shards=3)
    victim = d / "model-00002-of-00003.safetensors"
    victim.rename(str(victim) + ".part")
    with pytest.raises(SafetensorsError, match="missing shard model-00002-of-00003.safetensors") as e:
        Checkpoint.open(d)
    assert "interrupted" in str(e.value)
    os.remove(str(victim) + ".part")
    with pytest.raises(SafetensorsError, match="missing shard") as e:
        Checkpoint.open(d)
    assert "interrupted" not in str(e.value)
    (d / "model.safetensors.index.json").write_text('{"metadata": {}}')
    with pytest.raises(SafetensorsError, match="weight_map"):
        Checkpoint.open(d)
    (d / "model.safetensors.index.json").write_text('{"weight_map": {"a": "../evil.safetensors"}}')
    with pytest.raises(SafetensorsError, match="plain file name"):
        Checkpoint.open(d)


def broken(tmp_path, patch=None, tensors=None, raw=None):
    d = tmp_path / "b"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(SW.olmoe_config(H, I, E, K, 1)))
    p = d / "model.safetensors"
    if raw is not None:
        p.write_bytes(raw)
    else:
        SW.write_file(p, tensors or [("t", "F32", np.zeros((2, 3), np.float32))], patch=patch)
    with pytest.raises(SafetensorsError) as e:
        Checkpoint.open(d)
    return e.value


def test_every_header_rule_is_enforced(tmp_path):
    def edit(**kw):
        def patch(h):
            h["t"].update(kw)
        return patch
    assert "unsupported dtype 'F128'" in str(broken(tmp_path, edit(dtype="F128")))
    assert "implies 24 bytes, header claims 20" in str(broken(tmp_path, edit(data_offsets=[0, 20])))
    assert "outside the 24-byte payload" in str(broken(tmp_path, edit(data_offsets=[0, 28])))
    assert "outside the" in str(broken(tmp_path, edit(data_offsets=[8, 4])))
    assert "data_offsets has 3 entries" in str(broken(tmp_path, edit(data_offsets=[0, 24, 30])))
    assert "non-integer dim" in str(broken(tmp_path, edit(shape=[2, 3.5])))
    assert "non-integer dim" in str(broken(tmp_path, edit(shape=[2, -3])))
    assert "non-integer data_offset" in str(broken(tmp_path, edit(data_offsets=[0, "24"])))
    assert "overflows" in str(broken(tmp_path, edit(shape=[1 << 40, 1 << 40])))

    def drop(key):
        def patch(h):
            del h["t"][key]
        return patch
    for key in ("dtype", "shape", "data_offsets"):
        assert f"missing '{key}'" in str(broken(tmp_path, drop(key)))

    def not_object(h):
        h["t"] = [1, 2]
    assert "entry is not an object" in str(broken(tmp_path, not_object))
    # the container itself
    assert broken(tmp_path, raw=b"\x01\x02").code == _lib.ERR_IO
    assert "header bytes" in str(broken(tmp_path, raw=struct.pack("<Q", 1 << 40) + b"{}"))
    assert "header bytes" in str(broken(tmp_path, raw=struct.pack("<Q", 100) + b"{}"))
    assert "not a JSON object" in str(broken(tmp_path, raw=struct.pack("<Q", 2) + b"[]"))
    assert "bad header" in str(broken(tmp_path, raw=struct.pack("<Q", 3) + b"{,}"))


def test_metadata_is_skipped_and_duplicate_names_across_shards_are_refused(tmp_path):
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(SW.olmoe_config(H, I, E, K, 1)))
    SW.write_file(d / "model.safetensors", [("a", "F16", np.zeros(4, np.float16))], metadata={"format": "pt", "x": "y"})
    with Checkpoint.open(d) as ck:
        assert ck.tensor_count() == 1 and ck.tensor("__metadata__") is None
    os.remove(d / "model.safetensors")
    SW.write_file(d / "s1.safetensors", [("a", "F16", np.zeros(4, np.float16))])
    SW.write_file(d / "s2.safetensors", [("a", "F16", np.zeros(4, np.float16))])
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    with pytest.raises(SafetensorsError, match="more than one shard"):
        Checkpoint.open(d)


# ---- the expert groups (safetensors.rs:600-740) ----------------------------------------------------

def test_a_short_group_a_stray_member_and_mixed_layouts_are_refused(tmp_path):
    lw = layers(1)
    cfg = SW.olmoe_config(H, I, E, K, 1)
    d = SW.write_checkpoint(tmp_path / "short", cfg, lw, skip=("model.layers.0.mlp.experts.2.up_proj.weight",))
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="mlp.experts.up: 3 of 4 members present") as e:
            ck.check_moe_layer(0)
        assert e.value.code == _lib.ERR_SAFETENSORS
    stray = ("model.layers.0.mlp.experts.4.gate_proj.weight", "BF16", np.zeros((I, H), np.uint16))
    d = SW.write_checkpoint(tmp_path / "stray", cfg, lw, extra=(stray,))
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="member index 4 outside 0..4"):
            ck.check_moe_layer(0)
    odd = ("model.layers.0.mlp.experts.1.down_proj.weight", "F16", np.zeros((H, I), np.float16))
    d = SW.write_checkpoint(tmp_path / "mixed", cfg, lw, skip=(odd[0],), extra=(odd,))
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="members disagree on layout"):
            ck.check_moe_layer(0)
    d = SW.write_checkpoint(tmp_path / "norouter", cfg, lw, skip=("model.layers.0.mlp.gate.weight",))
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="no model.layers.0.mlp.gate.weight"):
            ck.check_moe_layer(0)


def test_shapes_must_match_the_config_and_dtypes_must_be_float(tmp_path):
    lw = layers(1)
    d = SW.write_checkpoint(tmp_path / "wide", SW.olmoe_config(H, I + 2, E, K, 1), lw)
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="does not match the config") as e:
            ck.check_moe_layer(0)
        assert e.value.code == _lib.ERR_SHAPE
    d = SW.write_checkpoint(tmp_path / "moreexperts", SW.olmoe_config(H, I, E + 1, K, 1), lw)
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError):
            ck.check_moe_layer(0)
    ints = [("model.layers.0.mlp.gate.weight", "I64", np.zeros((E, H), np.int64))]
    d = SW.write_checkpoint(tmp_path / "ints", SW.olmoe_config(H, I, E, K, 1), lw, skip=(ints[0][0],), extra=ints)
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="not a float type") as e:
            ck.check_moe_layer(0)
        assert e.value.code == _lib.ERR_TYPE


def test_a_bad_config_json_is_reported_when_the_block_is_asked_for(tmp_path):
    d = SW.write_checkpoint(tmp_path / "badcfg", SW.olmoe_config(H, I, 1, 1, 1), layers(1))
    with Checkpoint.open(d) as ck:  # the tensors are readable; the config is not usable
        assert ck.tensor_count() > 0
        with pytest.raises(SafetensorsError, match="num_experts"):
            ck.moe_config()
        with pytest.raises(SafetensorsError, match="num_experts"):
            ck.check_moe_layer(0)
    os.remove(d / "config.json")
    with Checkpoint.open(d) as ck:
        with pytest.raises(SafetensorsError, match="config.json"):
            ck.moe_config()


def test_null_arguments_are_errors_not_crashes():
    lib = _lib.load()
    assert lib.mummu_st_open(None, None) == _lib.ERR_ARG
    assert lib.mummu_st_tensor_count(None) == -1 and lib.mummu_st_find_tensor(None, b"x") == -1
    assert lib.mummu_st_moe_config(None, None) == _lib.ERR_ARG
    assert lib.mummu_moe_load_safetensors(None, None, 0, 1) == _lib.ERR_ARG
    assert lib.mummu_olmoe_config_from_json(None, 0, None) == _lib.ERR_ARG
    lib.mummu_st_close(None)
