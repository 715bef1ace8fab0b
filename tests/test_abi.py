"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and refuses bad configurations before it ever touches a device (nn/moe.rs:62-76, 2363-2374)."""
import ctypes as C
import os
import re

import pytest

from mummu_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "mummu_moe.h")).read()
    return sorted(set(re.findall(r"MUMMU_API[^;(]*?\b(mummu_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mummu_moe.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "the ctypes signature table and the header disagree"


def test_every_declaration_cites_the_reference_or_says_it_has_none():
    text = open(os.path.join(ROOT, "include", "mummu_moe.h")).read()
    assert "nn/moe.rs:116" in text and "experts.rs:1066" in text and "gguf.rs:1403" in text


def _create(**kw):
    lib = _lib.load()
    base = dict(hidden_size=4, expert_intermediate_size=3, num_experts=4, num_experts_per_tok=2, norm_topk_prob=0,
                router_flavour=0, num_layers=1, max_tokens=8, rms_norm_eps=1e-5)
    base.update(kw)
    cfg = _lib.Config(**base)
    h = C.c_void_p()
    rc = lib.mummu_moe_create(C.byref(cfg), C.byref(h))
    msg = lib.mummu_moe_last_error(None).decode()
    if rc == 0:
        lib.mummu_moe_destroy(h)
    return rc, msg


def test_config_rejects_zero_top_k():
    # nn/moe.rs:2363-2374 expects the message to name num_experts_per_tok
    rc, msg = _create(num_experts_per_tok=0)
    assert rc == _lib.ERR_CONFIG and "num_experts_per_tok" in msg


@pytest.mark.parametrize("kw,needle", [
    (dict(num_experts=1, num_experts_per_tok=1), "num_experts must be >= 2"),
    (dict(num_experts_per_tok=5), "must be in 1..=num_experts"),
    (dict(hidden_size=0), "must be >= 1"),
    (dict(expert_intermediate_size=0), "must be >= 1"),
    (dict(num_experts=1024, num_experts_per_tok=8), "at most 512"),
    (dict(router_flavour=7), "router_flavour"),
])
def test_config_validation_matches_the_reference_asserts(kw, needle):
    rc, msg = _create(**kw)
    assert rc == _lib.ERR_CONFIG and needle in msg, msg


def test_null_arguments_are_errors_not_crashes():
    lib = _lib.load()
    assert lib.mummu_moe_create(None, None) == _lib.ERR_ARG
    assert lib.mummu_moe_forward(None, 0, None, 1, 1, 0, None) == _lib.ERR_ARG
    assert lib.mummu_moe_last_error(None) is not None
    lib.mummu_moe_destroy(None)
    # partial blocks are refused before any device work (gguf.rs:2654-2662)
    buf = (C.c_uint8 * 33)()
    out = (C.c_float * 64)()
    assert lib.mummu_dequantize(_lib.Q8_0, buf, 33, out) == _lib.ERR_BLOCKS
    assert lib.mummu_dequantize(_lib.Q8_0, buf, 0, out) == _lib.ERR_BLOCKS
    assert lib.mummu_dequantize(15, buf, 33, out) == _lib.ERR_TYPE
    # the read probe checks its arguments before it launches anything
    assert lib.mummu_probe_read(None, 1 << 20, 1152, 32, None) == _lib.ERR_ARG
    assert lib.mummu_probe_read(C.c_void_p(4096), 1 << 20, 100, 32, None) == _lib.ERR_ARG     # a row that is no multiple of 128 bytes
    assert lib.mummu_probe_read(C.c_void_p(4096), 1000, 1152, 32, None) == _lib.ERR_ARG       # less than one slab of 128 rows


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmummu_moe.so")
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.load()
