"""Host-side mirror of the reference's HF-checkpoint path for the MoE block over the C ABI:
``Checkpoint.open(dir)`` discovers and validates the safetensors shards (safetensors.rs:180-430),
``moe_config`` parses ``config.json`` (models/olmoe.rs:52-226) and ``load_moe`` fuses the
per-expert projections into ``[E, out, in]`` banks and loads them (models/olmoe.rs:405-500).
Parsing and fusing happen in the C++ library, not here.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Optional, Tuple

from . import _lib
from .moe import MoeError, SparseMoe, SparseMoeConfig


class SafetensorsError(MoeError):
    """SafetensorsError (safetensors.rs:62-118) and the config errors of OlmoeConfig::from_json_bytes."""


@dataclass
class TensorEntry:
    """TensorEntry (safetensors.rs:122-148) and where its payload lies."""
    name: str
    dtype: str
    shape: Tuple[int, ...]
    shard: int
    path: str
    file_offset: int
    nbytes: int


def olmoe_config_from_json(text) -> _lib.Config:
    """OlmoeConfig::from_json_bytes (models/olmoe.rs:104-108), the MoE block's fields."""
    lib = _lib.load()
    raw = text if isinstance(text, bytes) else text.encode()
    cfg = _lib.Config()
    rc = lib.mummu_olmoe_config_from_json(raw, len(raw), C.byref(cfg))
    if rc:
        raise SafetensorsError(rc, lib.mummu_st_last_error().decode("utf-8", "replace"))
    return cfg


class Checkpoint:
    def __init__(self, handle, lib):
        self._h, self._lib = handle, lib

    @staticmethod
    def open(directory) -> "Checkpoint":
        lib = _lib.load()
        h = C.c_void_p()
        rc = lib.mummu_st_open(os.fsencode(directory), C.byref(h))
        if rc:
            raise SafetensorsError(rc, lib.mummu_st_last_error().decode("utf-8", "replace"))
        return Checkpoint(h, lib)

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self._lib.mummu_st_close(self._h)
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
            raise SafetensorsError(rc, self._lib.mummu_st_last_error().decode("utf-8", "replace"))

    def shard_count(self) -> int:
        return self._lib.mummu_st_shard_count(self._h)

    def tensor_count(self) -> int:
        return self._lib.mummu_st_tensor_count(self._h)

    def tensor(self, name: str) -> Optional[TensorEntry]:
        i = self._lib.mummu_st_find_tensor(self._h, name.encode())
        if i < 0:
            return None
        t = _lib.StTensor()
        self._check(self._lib.mummu_st_tensor_info(self._h, i, C.byref(t)))
        return TensorEntry(t.name.decode(), t.dtype.decode(), tuple(t.dims[:t.n_dims]), t.shard, os.fsdecode(t.path),
                           int(t.file_offset), int(t.nbytes))

    def moe_config(self) -> _lib.Config:
        cfg = _lib.Config()
        self._check(self._lib.mummu_st_moe_config(self._h, C.byref(cfg)))
        return cfg

    def check_moe_layer(self, layer: int):
        """The fuse's planning pass for one layer: names, completeness, dtypes and shapes."""
        self._check(self._lib.mummu_st_check_moe_layer(self._h, layer))

    def load_into(self, moe: SparseMoe, first_layer: int = 0, n_layers: int = 1) -> None:
        """Layers [first_layer, first_layer + n_layers) of the checkpoint into layers 0.. of an existing handle; refused
        when the handle was created for another geometry than the checkpoint's."""
        self._check(self._lib.mummu_moe_load_safetensors(moe._h, self._h, first_layer, n_layers))

    def load_moe(self, first_layer: int = 0, n_layers: Optional[int] = None, *, max_tokens: int = 64) -> SparseMoe:
        cfg = self.moe_config()
        n_layers = cfg.num_layers - first_layer if n_layers is None else n_layers
        moe = SparseMoe(SparseMoeConfig(cfg.hidden_size, cfg.expert_intermediate_size, cfg.num_experts,
                                        cfg.num_experts_per_tok),
                        num_layers=max(n_layers, 1), max_tokens=max_tokens, norm_topk_prob=bool(cfg.norm_topk_prob),
                        rms_norm_eps=cfg.rms_norm_eps)
        try:
            self._check(self._lib.mummu_moe_load_safetensors(moe._h, self._h, first_layer, n_layers))
        except Exception:
            moe.close()
            raise
        moe.norm_topk_prob = bool(cfg.norm_topk_prob)
        return moe
