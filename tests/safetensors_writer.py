"""A small safetensors writer for test fixtures: header JSON + payload, with hooks for writing
broken headers on purpose, and an OLMoE-named HF checkpoint directory (config.json, shards,
index) for the MoE block."""
import json
import os
import struct

import numpy as np

DTYPES = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I64": np.int64, "U8": np.uint8}


def to_bf16(x: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((b >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    return ((b + r) >> np.uint32(16)).astype(np.uint16)


def encode(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "BF16":
        return to_bf16(x)
    return np.ascontiguousarray(x, dtype=DTYPES[dtype])


def write_file(path, tensors, metadata=None, patch=None):
    """tensors: list of (name, dtype, array).  patch(header_dict) may edit the header before it is written."""
    header, payload = {}, bytearray()
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, dtype, arr in tensors:
        raw = np.ascontiguousarray(arr).tobytes()
        header[name] = {"dtype": dtype, "shape": list(arr.shape), "data_offsets": [len(payload), len(payload) + len(raw)]}
        payload += raw
    if patch:
        patch(header)
    text = json.dumps(header, separators=(",", ":")).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text + bytes(payload))
    return path


def olmoe_config(hidden, inter, experts, top_k, layers, **over):
    cfg = dict(vocab_size=100, hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers, num_attention_heads=4,
               num_key_value_heads=2, num_experts=experts, num_experts_per_tok=top_k, norm_topk_prob=False, rms_norm_eps=1e-5,
               rope_theta=10000.0, model_type="olmoe")
    cfg.update(over)
    return {k: v for k, v in cfg.items() if v is not None}


def write_checkpoint(directory, cfg, layers, dtype="BF16", shards=1, skip=(), extra=()):
    """layers[l] = dict(router [E,H], gate/up [E,I,H], down [E,H,I], gamma [H]) as float32 arrays.
    Experts are written one tensor each, interleaved over `shards` files in a scrambled order."""
    os.makedirs(directory, exist_ok=True)
    with open(os.path.join(directory, "config.json"), "w") as f:
        json.dump(cfg, f)
    per_shard = [[] for _ in range(shards)]
    n = 0
    for l, w in enumerate(layers):
        base = f"model.layers.{l}."
        items = [(base + "mlp.gate.weight", w["router"]), (base + "post_attention_layernorm.weight", w["gamma"]),
                 (base + "self_attn.q_proj.weight", np.zeros((4, 4), np.float32))]
        E = w["gate"].shape[0]
        for e in reversed(range(E)):  # reverse order: the fuse must sort numerically, not by file order
            for proj in ("down", "gate", "up"):
                items.append((f"{base}mlp.experts.{e}.{proj}_proj.weight", w[proj][e]))
        for name, arr in items:
            if name in skip:
                continue
            per_shard[n % shards].append((name, dtype, encode(arr, dtype)))
            n += 1
    for name, dt, arr in extra:
        per_shard[0].append((name, dt, arr))
    if shards == 1:
        write_file(os.path.join(directory, "model.safetensors"), per_shard[0], metadata={"format": "pt"})
    else:
        weight_map = {}
        for s, tensors in enumerate(per_shard):
            fname = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
            write_file(os.path.join(directory, fname), tensors, metadata={"format": "pt"})
            for name, _, _ in tensors:
                weight_map[name] = fname
        with open(os.path.join(directory, "model.safetensors.index.json"), "w") as f:
            json.dump({"metadata": {"total_size": 0}, "weight_map": weight_map}, f)
    return directory
