"""ctypes binding of the CPU oracle (``moe_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Nothing here computes: every function forwards numpy buffers to the C restatement of the
reference's algorithms and returns numpy arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")

F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 2, 3, 6, 7, 8, 12, 13, 14, 30

OK, ERR_TYPE, ERR_BLOCKS, ERR_TOPK, ERR_NONFINITE, ERR_RANGE, ERR_SHAPE = range(7)


class OracleError(RuntimeError):
    def __init__(self, code: int, what: str, detail: str = ""):
        self.code = code
        names = ["ok", "type", "blocks", "topk", "nonfinite", "range", "shape"]
        super().__init__(f"oracle {what}: error {names[code] if code < len(names) else code} {detail}")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a second or two)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "moe_oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True, capture_output=not force)
    return _SO


class Banks(C.Structure):
    _fields_ = [
        ("hidden", C.c_int), ("inter", C.c_int), ("n_experts", C.c_int),
        ("gate_type", C.c_int), ("up_type", C.c_int), ("down_type", C.c_int),
        ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_expf.restype = C.c_float
        L.orc_expf.argtypes = [C.c_float]
        L.orc_silu.restype = C.c_float
        L.orc_silu.argtypes = [C.c_float]
        L.orc_dot.restype = C.c_float
        L.orc_dot.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_router_dot.restype = C.c_float
        L.orc_router_dot.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_size_t]
        L.orc_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_route_ggml.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_route_olmoe.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_router_logits.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_int, C.c_void_p]
        L.orc_matvec.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_expert_ffn.argtypes = [C.POINTER(Banks), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_q4s_gemv.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_gate_energy.argtypes = [C.POINTER(Banks), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_apply_routing.argtypes = [C.POINTER(Banks), C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_moe_forward.argtypes = [C.POINTER(Banks), C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                      C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_moe_forward_dense_mask.argtypes = [C.POINTER(Banks), C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                                 C.c_size_t, C.c_void_p]
        L.orc_rmsnorm.restype = None
        L.orc_rmsnorm.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_size_t, C.c_size_t, C.c_void_p]
        L.orc_layer_stack.argtypes = [C.POINTER(Banks), C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_void_p), C.c_float,
                                      C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_moe_ref_f64.argtypes = [C.POINTER(Banks), C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p,
                                      C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(-1)


def block_size(t: int) -> int:
    return lib().orc_block_size(t)


def block_bytes(t: int) -> int:
    return lib().orc_block_bytes(t)


def row_bytes(t: int, in_dim: int) -> int:
    return in_dim // block_size(t) * block_bytes(t)


def f16_to_f32(bits: int) -> float:
    return lib().orc_f16_to_f32(bits)


def expf(x: float) -> float:
    return lib().orc_expf(x)


def expf_array(x) -> np.ndarray:
    x = _f32(x).reshape(-1)
    f = lib().orc_expf
    return np.array([f(float(v)) for v in x], dtype=np.float32)


def silu(x: float) -> float:
    return lib().orc_silu(x)


def dot(a, b) -> float:
    a, b = _f32(a), _f32(b)
    assert a.size == b.size
    return lib().orc_dot(_p(a), _p(b), a.size)


def router_dot(x, w, wtype: int) -> float:
    x = _f32(x)
    w = np.ascontiguousarray(w)
    return lib().orc_router_dot(_p(x), _p(w), wtype, 0, x.size)


def dequantize(t: int, data) -> np.ndarray:
    b = _u8(data)
    bs, bb = block_size(t), block_bytes(t)
    if bb == 0:
        raise OracleError(ERR_TYPE, "dequantize")
    out = np.empty(max(b.size // bb, 1) * bs, dtype=np.float32)
    rc = lib().orc_dequantize(t, _p(b), b.size, _p(out))
    if rc:
        raise OracleError(rc, "dequantize", f"({b.size} bytes of type {t})")
    return out


def renormalize_ggml(top) -> np.ndarray:
    w = _f32(top).copy()
    lib().orc_renormalize_ggml.restype = None
    lib().orc_renormalize_ggml(_p(w), C.c_int(w.size))
    return w


def route_ggml(logits, n: int, n_experts: int, k: int):
    """experts.rs `route`: returns (ids uint32 [n,k], weights f32 [n,k])."""
    lg = _f32(logits).reshape(-1)
    if lg.size != n * n_experts:
        raise OracleError(ERR_SHAPE, "route_ggml", f"{lg.size} logits is not {n} rows x {n_experts}")
    ids = np.zeros((n, max(k, 1)), dtype=np.uint32)
    w = np.zeros((n, max(k, 1)), dtype=np.float32)
    bad = C.c_int64(-1)
    rc = lib().orc_route_ggml(_p(lg), n, n_experts, k, _p(ids), _p(w), C.byref(bad))
    if rc:
        d = f"token {bad.value // n_experts} expert {bad.value % n_experts}" if rc == ERR_NONFINITE else ""
        raise OracleError(rc, "route_ggml", d)
    return ids, w


def route_olmoe(logits, n: int, n_experts: int, k: int, norm: bool):
    lg = _f32(logits).reshape(-1)
    if lg.size != n * n_experts:
        raise OracleError(ERR_SHAPE, "route_olmoe")
    ids = np.zeros((n, max(k, 1)), dtype=np.uint32)
    w = np.zeros((n, max(k, 1)), dtype=np.float32)
    bad = C.c_int64(-1)
    rc = lib().orc_route_olmoe(_p(lg), n, n_experts, k, int(norm), _p(ids), _p(w), C.byref(bad))
    if rc:
        raise OracleError(rc, "route_olmoe")
    return ids, w


def router_logits(x, w, wtype: int, n_experts: int) -> np.ndarray:
    x = _f32(x)
    n, h = x.shape
    w = np.ascontiguousarray(w)
    out = np.empty((n, n_experts), dtype=np.float32)
    rc = lib().orc_router_logits(_p(x), _p(w), wtype, n, h, n_experts, _p(out))
    if rc:
        raise OracleError(rc, "router_logits")
    return out


def matvec(t: int, expert_bytes, in_dim: int, out_dim: int, xs) -> np.ndarray:
    xs = _f32(xs).reshape(-1, in_dim)
    b = _u8(expert_bytes)
    out = np.empty((xs.shape[0], out_dim), dtype=np.float32)
    rc = lib().orc_matvec(t, _p(b), in_dim, out_dim, _p(xs), xs.shape[0], _p(out))
    if rc:
        raise OracleError(rc, "matvec")
    return out


class LayerBanks:
    """One layer's expert banks in GGUF order, kept alive for the C struct."""

    def __init__(self, hidden, inter, n_experts, gate, up, down, gate_type, up_type=None, down_type=None):
        self.gate, self.up, self.down = _u8(gate), _u8(up), _u8(down)
        up_type = gate_type if up_type is None else up_type
        down_type = gate_type if down_type is None else down_type
        self.hidden, self.inter, self.n_experts = hidden, inter, n_experts
        self.types = (gate_type, up_type, down_type)
        for arr, t, i, o in ((self.gate, gate_type, hidden, inter), (self.up, up_type, hidden, inter),
                             (self.down, down_type, inter, hidden)):
            bs = block_size(t)
            if bs and i % bs == 0:
                want = n_experts * o * row_bytes(t, i)
                if arr.size != want:
                    raise OracleError(ERR_SHAPE, "banks", f"bank is {arr.size} bytes, want {want}")
        self.c = Banks(hidden, inter, n_experts, gate_type, up_type, down_type,
                       self.gate.ctypes.data, self.up.ctypes.data, self.down.ctypes.data)

    def expert_bytes(self, e: int) -> int:
        h, i = self.hidden, self.inter
        g, u, d = self.types
        return i * row_bytes(g, h) + i * row_bytes(u, h) + h * row_bytes(d, i)


def expert_ffn(banks: LayerBanks, expert: int, xs) -> np.ndarray:
    xs = _f32(xs).reshape(-1, banks.hidden)
    out = np.empty_like(xs)
    rc = lib().orc_expert_ffn(C.byref(banks.c), expert, _p(xs), xs.shape[0], _p(out))
    if rc:
        raise OracleError(rc, "expert_ffn")
    return out


def q4s_gemv(words, scales, k: int, n: int, bits: int, xs) -> np.ndarray:
    """nn/packed_gemv.rs:370-451 at split 1: x . w over burn's packed block-32 layout, sequential in k."""
    words = np.ascontiguousarray(words, dtype=np.uint32)
    scales = _f32(scales)
    xs = _f32(xs).reshape(-1, k)
    out = np.empty((xs.shape[0], n), dtype=np.float32)
    rc = lib().orc_q4s_gemv(_p(words), _p(scales), k, n, bits, _p(xs), xs.shape[0], _p(out))
    if rc:
        raise OracleError(rc, "q4s_gemv")
    return out


def gate_energy(banks: LayerBanks, expert: int, xs) -> np.ndarray:
    """nn/moe.rs:508-521: per row, sum over the intermediate width of silu(x . gate_i)^2."""
    xs = _f32(xs).reshape(-1, banks.hidden)
    out = np.empty(xs.shape[0], dtype=np.float32)
    rc = lib().orc_gate_energy(C.byref(banks.c), expert, _p(xs), xs.shape[0], _p(out))
    if rc:
        raise OracleError(rc, "gate_energy")
    return out


def apply_routing(banks: LayerBanks, ids, weights, xs, hits=None) -> np.ndarray:
    xs = _f32(xs).reshape(-1, banks.hidden)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    weights = _f32(weights)
    n, k = ids.shape
    assert xs.shape[0] == n and weights.shape == ids.shape
    out = np.empty_like(xs)
    rc = lib().orc_apply_routing(C.byref(banks.c), _p(ids), _p(weights), n, k, _p(xs), _p(out),
                                 _p(hits) if hits is not None else None)
    if rc:
        raise OracleError(rc, "apply_routing")
    return out


def moe_forward(banks: LayerBanks, router_w, router_type: int, xs, k: int, norm: bool, flavour: int = 0, hits=None):
    """Returns (out [n,H], ids [n,k] uint32, weights [n,k], logits [n,E])."""
    xs = _f32(xs).reshape(-1, banks.hidden)
    n = xs.shape[0]
    rw = np.ascontiguousarray(router_w)
    out = np.empty_like(xs)
    ids = np.zeros((n, max(k, 1)), dtype=np.uint32)
    w = np.zeros((n, max(k, 1)), dtype=np.float32)
    lg = np.zeros((n, banks.n_experts), dtype=np.float32)
    rc = lib().orc_moe_forward(C.byref(banks.c), _p(rw), router_type, flavour, k, int(norm), _p(xs), n, _p(out),
                               _p(ids), _p(w), _p(lg), _p(hits) if hits is not None else None)
    if rc:
        raise OracleError(rc, "moe_forward")
    return out, ids, w, lg


def moe_forward_dense_mask(banks: LayerBanks, router_w, router_type: int, xs, k: int, norm: bool) -> np.ndarray:
    xs = _f32(xs).reshape(-1, banks.hidden)
    rw = np.ascontiguousarray(router_w)
    out = np.empty_like(xs)
    rc = lib().orc_moe_forward_dense_mask(C.byref(banks.c), _p(rw), router_type, k, int(norm), _p(xs), xs.shape[0], _p(out))
    if rc:
        raise OracleError(rc, "moe_forward_dense_mask")
    return out


def rmsnorm(x, gamma, eps: float) -> np.ndarray:
    x = _f32(x)
    gamma = _f32(gamma)
    out = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(gamma), eps, x.shape[0], x.shape[1], _p(out))
    return out


def layer_stack(layers, routers, router_type: int, gammas, eps: float, xs, k: int, norm: bool, flavour: int = 0):
    """x <- x + MoE(RmsNorm(x)) through every layer.  Returns (x_out, ids [L,n,k])."""
    x = _f32(xs).copy()
    n = x.shape[0]
    nl = len(layers)
    arr = (Banks * nl)(*[l.c for l in layers])
    routers = [np.ascontiguousarray(r) for r in routers]
    gammas = [_f32(g) for g in gammas]
    rp = (C.c_void_p * nl)(*[r.ctypes.data for r in routers])
    gp = (C.c_void_p * nl)(*[g.ctypes.data for g in gammas])
    ids = np.zeros((nl, n, k), dtype=np.uint32)
    rc = lib().orc_layer_stack(arr, rp, router_type, gp, eps, nl, flavour, k, int(norm), _p(x), n, _p(ids))
    if rc:
        raise OracleError(rc, "layer_stack")
    return x, ids


def moe_ref_f64(banks: LayerBanks, ids, weights, xs):
    """The f64 tolerance reference for a given routing: (want, mag), both [n,H] float64."""
    xs = _f32(xs).reshape(-1, banks.hidden)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    weights = _f32(weights)
    n, k = ids.shape
    want = np.empty(xs.shape, dtype=np.float64)
    mag = np.empty(xs.shape, dtype=np.float64)
    rc = lib().orc_moe_ref_f64(C.byref(banks.c), _p(ids), _p(weights), n, k, _p(xs), _p(want), _p(mag))
    if rc:
        raise OracleError(rc, "moe_ref_f64")
    return want, mag


def rel_err(got, want, mag) -> np.ndarray:
    """Relative closeness as the reference measures it (experts.rs:1264-1271): against the
    larger of |want| and the root-sum-square magnitude of the terms."""
    got = np.asarray(got, dtype=np.float64)
    scale = np.maximum(np.maximum(np.abs(want), mag), 1e-30)
    return np.abs(got - want) / scale
