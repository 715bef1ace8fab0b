"""Host-side mirror of the reference's GGUF reader over the C ABI (gguf.rs:538-714, 1062-1122):
``GgufFile.open`` parses and validates a file or a split set, ``tensor`` / ``get`` look things
up, ``moe_config`` reads the MoE block's configuration (models/olmoe.rs:116-179) and
``load_moe`` hands the located expert banks to a ``SparseMoe`` with their bytes unchanged
(models/qwen4exp/experts.rs:869-911).  Parsing happens in the C++ library, not here.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np

from . import _lib
from .moe import MoeError, SparseMoe, SparseMoeConfig


class GgufError(MoeError):
    """GgufError (gguf.rs:65-118): Io, BadMagic, BadVersion, OverBound, BadValue, BadTensor."""


@dataclass
class GgufTensorInfo:
    """GgufTensorInfo (gguf.rs:403-430) and its payload location (gguf.rs:1096)."""
    name: str
    dims: Tuple[int, ...]  # GGUF order: fastest-varying first
    dtype: int             # ggml type id
    shard: int
    path: str
    file_offset: int
    nbytes: int


class GgufFile:
    def __init__(self, handle, lib):
        self._h, self._lib = handle, lib

    @staticmethod
    def open(path) -> "GgufFile":
        """GgufFile::open_sharded (gguf.rs:628): a single file, or any member of a split set."""
        lib = _lib.load()
        h = C.c_void_p()
        rc = lib.mummu_gguf_open(os.fsencode(path), C.byref(h))
        if rc:
            raise GgufError(rc, lib.mummu_gguf_last_error().decode("utf-8", "replace"))
        return GgufFile(h, lib)

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self._lib.mummu_gguf_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc: int):
        if rc:
            raise GgufError(rc, self._lib.mummu_gguf_last_error().decode("utf-8", "replace"))

    # -- header -----------------------------------------------------------------------------
    @property
    def version(self) -> int:
        return self._lib.mummu_gguf_version(self._h)

    @property
    def alignment(self) -> int:
        return self._lib.mummu_gguf_alignment(self._h)

    def shard_count(self) -> int:
        return self._lib.mummu_gguf_shard_count(self._h)

    def tensor_count(self) -> int:
        return self._lib.mummu_gguf_tensor_count(self._h)

    def kv_count(self) -> int:
        return self._lib.mummu_gguf_kv_count(self._h)

    def architecture(self) -> Optional[str]:
        return self.get_str("general.architecture")

    # -- metadata ---------------------------------------------------------------------------
    def get_u64(self, key: str) -> Optional[int]:
        v = C.c_uint64()
        rc = self._lib.mummu_gguf_get_u64(self._h, key.encode(), C.byref(v))
        return None if rc else int(v.value)

    def get_f64(self, key: str) -> Optional[float]:
        v = C.c_double()
        rc = self._lib.mummu_gguf_get_f64(self._h, key.encode(), C.byref(v))
        return None if rc else float(v.value)

    def get_str(self, key: str) -> Optional[str]:
        s = self._lib.mummu_gguf_get_str(self._h, key.encode())
        return None if s is None else s.decode()

    # -- tensors ----------------------------------------------------------------------------
    def tensor_index(self, name: str) -> Optional[int]:
        i = self._lib.mummu_gguf_find_tensor(self._h, name.encode())
        return None if i < 0 else i

    def tensor_at(self, index: int) -> GgufTensorInfo:
        t = _lib.GgufTensor()
        self._check(self._lib.mummu_gguf_tensor_info(self._h, index, C.byref(t)))
        return GgufTensorInfo(t.name.decode(), tuple(t.dims[:t.n_dims]), t.ggml_type, t.shard, os.fsdecode(t.path),
                              int(t.file_offset), int(t.nbytes))

    def tensor(self, name: str) -> Optional[GgufTensorInfo]:
        i = self.tensor_index(name)
        return None if i is None else self.tensor_at(i)

    def tensor_bytes(self, name: str) -> np.ndarray:
        """A copy of the payload bytes of one tensor."""
        i = self.tensor_index(name)
        if i is None:
            raise GgufError(_lib.ERR_GGUF, f"GGUF has no {name}")
        p, n = C.c_void_p(), C.c_uint64()
        self._check(self._lib.mummu_gguf_tensor_data(self._h, i, C.byref(p), C.byref(n)))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n.value,)).copy()

    # -- the MoE block ------------------------------------------------------------------------
    def moe_config(self) -> _lib.Config:
        cfg = _lib.Config()
        self._check(self._lib.mummu_gguf_moe_config(self._h, C.byref(cfg)))
        return cfg

    def locate_moe_layer(self, layer: int) -> dict:
        """The layer's router / gate / up / down / norm tensors (norm is None when absent)."""
        at = _lib.GgufMoeLayer()
        self._check(self._lib.mummu_gguf_locate_moe_layer(self._h, layer, C.byref(at)))
        return {k: (self.tensor_at(getattr(at, k)) if getattr(at, k) >= 0 else None)
                for k in ("router", "gate", "up", "down", "norm")}

    def load_into(self, moe: SparseMoe, first_layer: int = 0, n_layers: int = 1) -> None:
        """Layers [first_layer, first_layer + n_layers) of the file into layers 0.. of an existing handle; refused when
        the handle was created for another geometry than the file's."""
        self._check(self._lib.mummu_moe_load_gguf(moe._h, self._h, first_layer, n_layers))

    def load_moe(self, first_layer: int = 0, n_layers: Optional[int] = None, *, max_tokens: int = 64,
                 router_flavour: int = _lib.ROUTER_SPARSE_MOE) -> SparseMoe:
        """A SparseMoe holding the MoE blocks of layers [first_layer, first_layer + n_layers)."""
        cfg = self.moe_config()
        n_layers = cfg.num_layers - first_layer if n_layers is None else n_layers
        moe = SparseMoe(SparseMoeConfig(cfg.hidden_size, cfg.expert_intermediate_size, cfg.num_experts,
                                        cfg.num_experts_per_tok),
                        num_layers=max(n_layers, 1), max_tokens=max_tokens, norm_topk_prob=bool(cfg.norm_topk_prob),
                        router_flavour=router_flavour, rms_norm_eps=cfg.rms_norm_eps)
        try:
            self._check(self._lib.mummu_moe_load_gguf(moe._h, self._h, first_layer, n_layers))
        except Exception:
            moe.close()
            raise
        moe.norm_topk_prob = bool(cfg.norm_topk_prob)
        return moe
