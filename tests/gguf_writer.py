"""A small GGUF v3 writer for test fixtures (the counterpart of the reference's in-test
`TestGguf` builder, gguf.rs:1970-2100): typed metadata, a tensor table with caller-chosen type
ids and offsets (so that broken tables can be written too), and an optional payload."""
import struct
from typing import List, Sequence, Tuple

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}

# ggml type id -> (elements per block, bytes per block) for the types the fixtures use
BLOCKS = {0: (1, 4), 1: (1, 2), 30: (1, 2), 8: (32, 34), 12: (256, 144), 14: (256, 210)}


def _string(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype: int, v) -> bytes:
    if vtype == STR:
        return _string(v)
    if vtype == ARRAY:
        elem, items = v
        return struct.pack("<IQ", elem, len(items)) + b"".join(_value(elem, i) for i in items)
    return struct.pack(_FMT[vtype], v)


class GgufWriter:
    def __init__(self, version: int = 3, alignment: int = 32):
        self.version, self.alignment = version, alignment
        self.kvs: List[Tuple[str, int, object]] = []
        self.tensors: List[Tuple[str, Sequence[int], int, int]] = []
        self.payload = bytearray()

    def kv(self, key: str, vtype: int, value) -> "GgufWriter":
        self.kvs.append((key, vtype, value))
        return self

    def kv_str(self, key, v):
        return self.kv(key, STR, v)

    def kv_u32(self, key, v):
        return self.kv(key, U32, v)

    def kv_f32(self, key, v):
        return self.kv(key, F32, v)

    def kv_bool(self, key, v):
        return self.kv(key, BOOL, int(v))

    def kv_str_array(self, key, items):
        return self.kv(key, ARRAY, (STR, list(items)))

    def tensor(self, name: str, dims: Sequence[int], ggml_type: int, offset: int) -> "GgufWriter":
        """A table entry only, at a caller-chosen offset (may be wrong on purpose)."""
        self.tensors.append((name, tuple(dims), ggml_type, offset))
        return self

    def add(self, name: str, dims: Sequence[int], ggml_type: int, data) -> "GgufWriter":
        """A table entry plus its payload bytes, placed at the next aligned offset."""
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1).tobytes()
        pad = (-len(self.payload)) % self.alignment
        self.payload += b"\0" * pad
        self.tensors.append((name, tuple(dims), ggml_type, len(self.payload)))
        self.payload += raw
        return self

    def header(self) -> bytes:
        out = bytearray(b"GGUF")
        out += struct.pack("<IQQ", self.version, len(self.tensors), len(self.kvs))
        for key, vtype, v in self.kvs:
            out += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
        for name, dims, t, off in self.tensors:
            out += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
            out += struct.pack("<IQ", t, off)
        return bytes(out)

    def build(self, payload: bytes = None) -> bytes:
        """Header only when there is no payload; otherwise header, padding to the alignment, payload."""
        head = self.header()
        body = bytes(self.payload) if payload is None else bytes(payload)
        if not body:
            return head
        return head + b"\0" * ((-len(head)) % self.alignment) + body

    def write(self, path, payload: bytes = None):
        with open(path, "wb") as f:
            f.write(self.build(payload))
        return path


def moe_gguf(case, weights_per_layer, arch: str = "olmoe", alignment: int = 32, norm_gamma=None,
             expert_ffn_key: bool = True, extra=()) -> GgufWriter:
    """A model file holding only what the MoE blocks need.  `case` has hidden, inter, experts,
    top_k and the per-tensor ggml types; weights_per_layer[l] has the encoded router / gate /
    up / down byte arrays."""
    w = GgufWriter(alignment=alignment)
    w.kv_str("general.architecture", arch)
    if alignment != 32:
        w.kv_u32("general.alignment", alignment)
    w.kv_u32(f"{arch}.block_count", len(weights_per_layer))
    w.kv_u32(f"{arch}.embedding_length", case["hidden"])
    w.kv_u32(f"{arch}.feed_forward_length", 4 * case["inter"])
    if expert_ffn_key:
        w.kv_u32(f"{arch}.expert_feed_forward_length", case["inter"])
    else:
        w.kvs[-1] = (f"{arch}.feed_forward_length", U32, case["inter"])
    w.kv_u32(f"{arch}.expert_count", case["experts"])
    w.kv_u32(f"{arch}.expert_used_count", case["top_k"])
    w.kv_f32(f"{arch}.attention.layer_norm_rms_epsilon", case.get("eps", 1e-5))
    if case.get("norm") is not None:
        w.kv_bool(f"{arch}.expert_weights_norm", case["norm"])
    w.kv_str_array("tokenizer.ggml.tokens", ["<s>", "a", "b"])
    for key, vtype, v in extra:
        w.kv(key, vtype, v)
    H, I, E = case["hidden"], case["inter"], case["experts"]
    for l, lw in enumerate(weights_per_layer):
        if norm_gamma is not None:
            w.add(f"blk.{l}.ffn_norm.weight", [H], 0, norm_gamma[l])
        w.add(f"blk.{l}.ffn_gate_inp.weight", [H, E], case["router_type"], lw["router"])
        w.add(f"blk.{l}.ffn_gate_exps.weight", [H, I, E], case["gate_type"], lw["gate"])
        w.add(f"blk.{l}.ffn_up_exps.weight", [H, I, E], case["up_type"], lw["up"])
        w.add(f"blk.{l}.ffn_down_exps.weight", [I, H, E], case["down_type"], lw["down"])
    return w
