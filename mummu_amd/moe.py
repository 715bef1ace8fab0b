"""Host-side mirror of the reference's sparse-MoE module interface over the C ABI.

Names, argument meaning and error behaviour follow the reference (physics515/Mummu,
crates/mummu/src/):

  SparseMoeConfig / SparseMoe.forward(x, top_k, norm_topk_prob)   nn/moe.rs:42-177
  SparseMoePerExpert.route -> Routing, run_local                   nn/moe.rs:247-337
  ExpertExec.run (expert_run), ExpertPool hits (take_hits)         nn/moe.rs:348-419, 857-874
  route(), RoutedExperts.{routed_moe, apply_routing, expert_ffn}   models/qwen4exp/experts.rs:541-582, 1015-1150
  gguf::dequantize                                                 gguf.rs:1403

Where the reference panics (a contract violation) or returns Err(String), these raise
``MoeError`` carrying the library's status code and message.  Every computation happens in the
HIP library; numpy is only the container for host buffers.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _lib
from ._lib import (BF16, F16, F32, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, ROUTER_QWEN4EXP,  # noqa: F401
                   ROUTER_SPARSE_MOE)


class MoeError(RuntimeError):
    def __init__(self, code: int, message: str):
        self.code = code
        name = _lib.STATUS_NAMES[code] if 0 <= code < len(_lib.STATUS_NAMES) else str(code)
        super().__init__(f"[{name}] {message}")


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _bytes(a) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


@dataclass
class SparseMoeConfig:
    """nn/moe.rs:42-50."""
    hidden_size: int
    expert_intermediate_size: int
    num_experts: int
    num_experts_per_tok: int

    def init(self, seed: int = 0, **handle_args) -> "SparseMoe":
        """SparseMoeConfig::init (nn/moe.rs:61-99): a block with Linear-style uniform weights, every projection
        bounded by 1/sqrt(its fan-in) (router and gate/up: hidden, down: intermediate), as f32 banks.  The
        reference draws from burn's generator; here the draws are SplitMix64 of `seed`.  The same checks refuse
        fewer than two experts, a top-k outside 1..=num_experts and zero widths."""
        from . import synth
        moe = SparseMoe(self, **handle_args)
        h, i, e = self.hidden_size, self.expert_intermediate_size, self.num_experts
        rng = synth.SplitMix64(seed)
        bh, bi = 1.0 / np.sqrt(float(h)), 1.0 / np.sqrt(float(i))
        router = rng.uniform(-bh, bh, e * h)
        gate, up = rng.uniform(-bh, bh, e * i * h), rng.uniform(-bh, bh, e * i * h)
        down = rng.uniform(-bi, bi, e * h * i)
        moe.load_layer(0, router, F32, gate, F32, up, F32, down, F32)
        return moe


@dataclass
class Routing:
    """nn/moe.rs:333-337: for every expert, the token rows it serves (ascending) and their
    weights; plus the raw per-token view the device produced."""
    tokens: int
    per_expert: List[Tuple[np.ndarray, np.ndarray]]
    ids: np.ndarray      # int32 [tokens, k], slot order (descending probability)
    weights: np.ndarray  # f32   [tokens, k]

    @staticmethod
    def from_slots(ids: np.ndarray, weights: np.ndarray, num_experts: int) -> "Routing":
        n, k = ids.shape
        flat_e = ids.reshape(-1)
        rows = np.repeat(np.arange(n, dtype=np.int32), k)
        order = np.argsort(flat_e, kind="stable")  # token-major, slot-minor within an expert
        bounds = np.searchsorted(flat_e[order], np.arange(num_experts + 1))
        wf = weights.reshape(-1)
        per = [(rows[order[bounds[e]:bounds[e + 1]]], wf[order[bounds[e]:bounds[e + 1]]]) for e in range(num_experts)]
        return Routing(n, per, ids, weights)


class SparseMoe:
    """The router + expert bank of one or more layers, resident on the GPU."""

    def __init__(self, config: SparseMoeConfig, *, num_layers: int = 1, max_tokens: int = 64,
                 norm_topk_prob: bool = False, router_flavour: int = ROUTER_SPARSE_MOE, rms_norm_eps: float = 1e-5):
        self.config = config
        self.num_layers = num_layers
        self._lib = _lib.load()
        self._h = C.c_void_p()
        cfg = _lib.Config(config.hidden_size, config.expert_intermediate_size, config.num_experts,
                          config.num_experts_per_tok, int(norm_topk_prob), router_flavour, num_layers, max_tokens,
                          rms_norm_eps)
        rc = self._lib.mummu_moe_create(C.byref(cfg), C.byref(self._h))
        if rc:
            raise MoeError(rc, self._lib.mummu_moe_last_error(None).decode())

    # -- lifetime --------------------------------------------------------------------------
    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self._lib.mummu_moe_destroy(self._h)
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
            raise MoeError(rc, self._lib.mummu_moe_last_error(self._h).decode())

    # -- weights ---------------------------------------------------------------------------
    def load_layer(self, layer: int, router, router_type: int, gate, gate_type: int, up, up_type: int, down,
                   down_type: int, rms_gamma=None):
        """GGUF payload bytes in GGUF order (models/olmoe.rs:338-345).  Sizes are checked here,
        where the byte counts are known (ExpertBank::from_bytes, experts.rs:167-183)."""
        c = self.config
        router, gate, up, down = _bytes(router), _bytes(gate), _bytes(up), _bytes(down)

        def want(t, in_dim, out_dim):
            bs = _lib.BLOCKS.get(t)
            if bs is None or in_dim % bs[0]:
                return None  # the library reports the precise error
            return c.num_experts * out_dim * (in_dim // bs[0]) * bs[1]

        for name, arr, t, i, o in (("gate", gate, gate_type, c.hidden_size, c.expert_intermediate_size),
                                   ("up", up, up_type, c.hidden_size, c.expert_intermediate_size),
                                   ("down", down, down_type, c.expert_intermediate_size, c.hidden_size)):
            w = want(t, i, o)
            if w is not None and arr.size != w:
                raise MoeError(_lib.ERR_SHAPE, f"expert bank {name} is {w} bytes, got {arr.size}")
        rw = {F32: 4, F16: 2, BF16: 2}.get(router_type)
        if rw is not None and router.size != c.num_experts * c.hidden_size * rw:
            raise MoeError(_lib.ERR_SHAPE, f"router is {c.num_experts * c.hidden_size * rw} bytes, got {router.size}")
        g = None if rms_gamma is None else _f32(rms_gamma)
        if g is not None and g.size != c.hidden_size:
            raise MoeError(_lib.ERR_SHAPE, "rms_gamma must have hidden_size entries")
        self._check(self._lib.mummu_moe_load_layer(self._h, layer, _ptr(router), router_type, _ptr(gate), gate_type,
                                                   _ptr(up), up_type, _ptr(down), down_type, _ptr(g)))

    def load_shared_expert(self, layer: int, inter: int, gate, gate_type: int, up, up_type: int, down, down_type: int,
                           gate_vec=None, gate_vec_type: int = F32):
        """The always-on shared expert of a Qwen-style block and its sigmoid gate vector
        (models/qwen4exp/model.rs:786-804): gate/up [inter, hidden], down [hidden, inter] as GGUF
        payload bytes, gate_vec [hidden] or None."""
        c = self.config
        gate, up, down = _bytes(gate), _bytes(up), _bytes(down)
        for name, arr, t, i, o in (("gate", gate, gate_type, c.hidden_size, inter), ("up", up, up_type, c.hidden_size, inter),
                                   ("down", down, down_type, inter, c.hidden_size)):
            bs = _lib.BLOCKS.get(t)
            if bs is not None and i % bs[0] == 0 and arr.size != o * (i // bs[0]) * bs[1]:
                raise MoeError(_lib.ERR_SHAPE, f"shared expert {name} is {o * (i // bs[0]) * bs[1]} bytes, got {arr.size}")
        gv = None if gate_vec is None else _bytes(gate_vec)
        vw = {F32: 4, F16: 2, BF16: 2}.get(gate_vec_type)
        if gv is not None and vw is not None and gv.size != c.hidden_size * vw:
            raise MoeError(_lib.ERR_SHAPE, f"shared expert gate vector is {c.hidden_size * vw} bytes, got {gv.size}")
        self._check(self._lib.mummu_moe_load_shared_expert(self._h, layer, inter, _ptr(gate), gate_type, _ptr(up), up_type,
                                                           _ptr(down), down_type, _ptr(gv), gate_vec_type))

    def resident_bytes(self) -> int:
        return int(self._lib.mummu_moe_resident_bytes(self._h))

    def batched_from(self, layer: int = 0) -> int:
        """Smallest token count that takes dispatch + grouped GEMM on this layer (2**31 - 1: never)."""
        return int(self._lib.mummu_moe_batched_from(self._h, layer))

    # -- the block -------------------------------------------------------------------------
    def _rows(self, x) -> Tuple[np.ndarray, tuple]:
        x = _f32(x)
        if x.shape[-1] != self.config.hidden_size:
            raise MoeError(_lib.ERR_SHAPE, f"MoE forward: input hidden {x.shape[-1]} does not match expert hidden "
                                           f"{self.config.hidden_size}")
        return x.reshape(-1, self.config.hidden_size), x.shape

    def forward(self, x, top_k: int, norm_topk_prob: bool, layer: int = 0) -> np.ndarray:
        """[b, t, hidden] -> [b, t, hidden] (nn/moe.rs:116)."""
        xt, shape = self._rows(x)
        out = np.empty_like(xt)
        self._check(self._lib.mummu_moe_forward(self._h, layer, _ptr(xt), xt.shape[0], top_k, int(norm_topk_prob), _ptr(out)))
        return out.reshape(shape)

    def forward_typed(self, x_bits, dtype: int, top_k: int, norm_topk_prob: bool, layer: int = 0) -> np.ndarray:
        """forward on activations in their ambient dtype (nn/moe.rs:116-135): `x_bits` holds [tokens, hidden] values
        as float32 (F32) or as the uint16 bit patterns of F16 / BF16; the result comes back in the same form."""
        want = np.float32 if dtype == F32 else np.uint16
        xb = np.ascontiguousarray(x_bits, dtype=want).reshape(-1, self.config.hidden_size)
        out = np.empty_like(xb)
        self._check(self._lib.mummu_moe_forward_typed(self._h, layer, _ptr(xb), dtype, xb.shape[0], top_k, int(norm_topk_prob),
                                                      _ptr(out)))
        return out

    def route(self, xt, top_k: int, norm_topk_prob: bool, layer: int = 0, return_logits: bool = False):
        """nn/moe.rs:247-290."""
        xt, _ = self._rows(xt)
        n = xt.shape[0]
        ids = np.zeros((n, max(top_k, 1)), dtype=np.int32)
        w = np.zeros((n, max(top_k, 1)), dtype=np.float32)
        lg = np.zeros((n, self.config.num_experts), dtype=np.float32) if return_logits else None
        self._check(self._lib.mummu_moe_route(self._h, layer, _ptr(xt), n, top_k, int(norm_topk_prob), _ptr(ids), _ptr(w), _ptr(lg)))
        r = Routing.from_slots(ids, w, self.config.num_experts)
        return (r, lg) if return_logits else r

    def run_local(self, xt, routing: Routing, layer: int = 0) -> np.ndarray:
        """nn/moe.rs:296-328 / ExpertPool::run_layer :1545-1607."""
        return self.apply_routing(layer, routing.ids, routing.weights, xt)

    def apply_routing(self, layer: int, ids, weights, xs) -> np.ndarray:
        """experts.rs:1092-1150."""
        xs, shape = self._rows(xs)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        weights = _f32(weights)
        if ids.ndim != 2 or ids.shape != weights.shape or ids.shape[0] != xs.shape[0]:
            raise MoeError(_lib.ERR_SHAPE, f"routing ids {ids.shape} / weights {weights.shape} do not match {xs.shape[0]} rows")
        out = np.empty_like(xs)
        self._check(self._lib.mummu_moe_apply_routing(self._h, layer, _ptr(ids), _ptr(weights), _ptr(xs), xs.shape[0],
                                                      ids.shape[1], _ptr(out)))
        return out.reshape(shape)

    def routed_moe(self, layer: int, router_logits, xs, n: int, k: int) -> np.ndarray:
        """experts.rs:1066-1076."""
        lg = _f32(router_logits).reshape(-1)
        xs = _f32(xs).reshape(-1)
        if lg.size != n * self.config.num_experts:
            raise MoeError(_lib.ERR_SHAPE, f"router logits: {lg.size} values is not {n} rows x {self.config.num_experts}")
        if xs.size != n * self.config.hidden_size:
            raise MoeError(_lib.ERR_SHAPE, f"moe input: {xs.size} values is not {n} rows x {self.config.hidden_size}")
        out = np.empty(n * self.config.hidden_size, dtype=np.float32)
        self._check(self._lib.mummu_moe_routed(self._h, layer, _ptr(lg), _ptr(xs), n, k, _ptr(out)))
        return out.reshape(n, self.config.hidden_size)

    def expert_run(self, layer: int, expert: int, x, rows: Optional[int] = None, hidden: Optional[int] = None) -> np.ndarray:
        """ExpertExec::run (nn/moe.rs:357) / expert_ffn (experts.rs:1015)."""
        x = _f32(x)
        hidden = x.shape[-1] if hidden is None else hidden
        rows = x.size // max(hidden, 1) if rows is None else rows
        if rows * hidden != x.size:
            raise MoeError(_lib.ERR_SHAPE, f"expert input: {x.size} values is not {rows} rows x {hidden}")
        out = np.empty((rows, hidden), dtype=np.float32)
        self._check(self._lib.mummu_expert_run(self._h, layer, expert, _ptr(x), rows, hidden, _ptr(out)))
        return out

    def gate_energy(self, layer: int, expert: int, x) -> np.ndarray:
        """ExpertExec::gate_energy (nn/moe.rs:411-418, 508-521): per row, sum_i silu(x . gate_i)^2."""
        x = _f32(x)
        hidden = x.shape[-1]
        rows = x.size // max(hidden, 1)
        out = np.empty(rows, dtype=np.float32)
        self._check(self._lib.mummu_expert_gate_energy(self._h, layer, expert, _ptr(x), rows, hidden, _ptr(out)))
        return out

    def take_hits(self, layer: int = 0) -> np.ndarray:
        hits = np.zeros(self.config.num_experts, dtype=np.uint64)
        self._check(self._lib.mummu_moe_take_hits(self._h, layer, _ptr(hits)))
        return hits

    def stack_forward(self, x, top_k: int, norm_topk_prob: bool, return_ids: bool = False):
        """x <- x + MoE_l(RmsNorm_l(x)) through every layer (models/olmoe.rs:566-572)."""
        xt, shape = self._rows(x)
        n = xt.shape[0]
        out = np.empty_like(xt)
        ids = np.zeros((self.num_layers, n, top_k), dtype=np.int32) if return_ids else None
        self._check(self._lib.mummu_moe_stack_forward(self._h, _ptr(xt), n, top_k, int(norm_topk_prob), _ptr(out), _ptr(ids)))
        return (out.reshape(shape), ids) if return_ids else out.reshape(shape)

    def dequantize_expert(self, layer: int, which: str, expert: int) -> np.ndarray:
        """One expert matrix dequantized from the device-resident bytes: [out_dim, in_dim] f32."""
        c = self.config
        w = {"gate": 0, "up": 1, "down": 2}[which]
        shape = (c.hidden_size, c.expert_intermediate_size) if w == 2 else (c.expert_intermediate_size, c.hidden_size)
        out = np.empty(shape, dtype=np.float32)
        self._check(self._lib.mummu_moe_dequantize_expert(self._h, layer, w, expert, _ptr(out)))
        return out

    # -- device-resident calls (benchmarks, serving loops) -----------------------------------
    def forward_device(self, layer: int, x_dev: "DeviceBuffer", n: int, top_k: int, norm_topk_prob: bool,
                       out_dev: "DeviceBuffer"):
        self._check(self._lib.mummu_moe_forward_device(self._h, layer, x_dev.ptr, n, top_k, int(norm_topk_prob),
                                                       out_dev.ptr, self.stream))

    def forward_device_noalloc(self, layer: int, x_dev: "DeviceBuffer", n: int, top_k: int, norm_topk_prob: bool,
                               out_dev: "DeviceBuffer"):
        """forward_device through the entry point that allocates nothing: the kernels' intermediate data lives in the
        library's static device array (decode form only; see include/mummu_moe.h)."""
        self._check(self._lib.mummu_moe_forward_device_noalloc(self._h, layer, x_dev.ptr, n, top_k, int(norm_topk_prob),
                                                               out_dev.ptr, self.stream))

    def set_router_exchange(self, enable, spin_ticks: int = 5000):
        """Two-launch decode form: 0 / False off, 1 / True at one token (default), 2 at every size it takes; and the
        bound (10 ns units) of a workgroup's wait for the others' logits."""
        self._check(self._lib.mummu_moe_set_router_exchange(self._h, int(enable), spin_ticks))

    def set_layer_fusion(self, enable):
        """Whether a decode step on block-quantized banks with top-8 routing runs its experts in ONE launch (router,
        routing, gate/up and the down product): 0 / False never, 1 / True (default) in chains of deferred sums only,
        2 wherever the kernel serves."""
        self._check(self._lib.mummu_moe_set_layer_fusion(self._h, int(enable)))

    def set_deferred_combine(self, enable):
        """With the one-launch decode form: leave the sum over a token's eight weighted rows to the launch of the next
        forward_device call (off by default).  out of a call is complete after the next call, flush() or check()."""
        self._check(self._lib.mummu_moe_set_deferred_combine(self._h, int(bool(enable))))

    def set_tile_order(self, enable):
        """Decode steps of several tokens fetch the rows of an expert that several tokens share once: None = from six
        tokens on (the default: there it is also the faster order), True = from two (a third less HBM traffic, 1 - 6 %
        more time at two to four tokens), False = never.  Same bits in every case."""
        self._check(self._lib.mummu_moe_set_tile_order(self._h, -1 if enable is None else int(bool(enable))))

    def flush(self):
        """Enqueues the sum a deferred decode step left pending; does not synchronise."""
        self._check(self._lib.mummu_moe_flush(self._h))

    def router_exchange_state(self):
        """(two-launch form in use on this device, workgroups that gave up waiting since the last call)."""
        usable, fb = C.c_int(0), C.c_uint64(0)
        self._check(self._lib.mummu_moe_router_exchange_state(self._h, C.byref(usable), C.byref(fb)))
        return bool(usable.value), int(fb.value)

    def expert_run_device(self, layer: int, expert: int, x_dev: "DeviceBuffer", rows: int, out_dev: "DeviceBuffer"):
        """ExpertExec::run_tensor_resident (nn/moe.rs:360-371): rows already on the device, result left there."""
        self._check(self._lib.mummu_expert_run_device(self._h, layer, expert, x_dev.ptr, rows, self.config.hidden_size,
                                                      out_dev.ptr, self.stream))

    def stack_forward_device(self, x_dev: "DeviceBuffer", n: int, top_k: int, norm_topk_prob: bool, out_dev: "DeviceBuffer"):
        self._check(self._lib.mummu_moe_stack_forward_device(self._h, x_dev.ptr, n, top_k, int(norm_topk_prob),
                                                             out_dev.ptr, self.stream))

    @property
    def stream(self):
        return self._lib.mummu_moe_stream(self._h)

    def check(self):
        self._check(self._lib.mummu_moe_check(self._h, self.stream))

    def last_routing(self, n: int, top_k: int):
        ids = np.zeros((n, top_k), dtype=np.int32)
        w = np.zeros((n, top_k), dtype=np.float32)
        self._check(self._lib.mummu_moe_last_routing(self._h, n, top_k, _ptr(ids), _ptr(w)))
        return ids, w

    def graph_begin(self):
        self._check(self._lib.mummu_graph_begin(self._h))

    def graph_end(self) -> "Graph":
        g = C.c_void_p()
        self._check(self._lib.mummu_graph_end(self._h, C.byref(g)))
        return Graph(self, g)

    def timer_start(self):
        self._check(self._lib.mummu_timer_start(self._h))

    def timer_stop(self) -> float:
        ms = C.c_float()
        self._check(self._lib.mummu_timer_stop(self._h, C.byref(ms)))
        return ms.value

    def kernel_timing(self, enable: bool):
        self._check(self._lib.mummu_moe_kernel_timing(self._h, int(enable)))

    def kernel_times(self) -> dict:
        """{kernel: (total_ms, launches)} since the last call."""
        n = 16
        names = (C.c_char_p * n)()
        ms = (C.c_double * n)()
        cnt = (C.c_int64 * n)()
        got = self._lib.mummu_moe_kernel_times(self._h, names, ms, cnt, n)
        if got < 0:
            raise MoeError(_lib.ERR_DEVICE, "kernel_times failed")
        return {names[i].decode(): (ms[i], cnt[i]) for i in range(got)}


# SparseMoePerExpert (nn/moe.rs:202-329) has the same forward/route/run_local surface; on this
# backend both module flavours are the same routed implementation over GGUF-layout banks.
SparseMoePerExpert = SparseMoe


class Graph:
    def __init__(self, moe: SparseMoe, handle):
        self._moe, self._g = moe, handle

    def launch(self):
        self._moe._check(self._moe._lib.mummu_graph_launch(self._moe._h, self._g))

    def launch_timed(self, reps: int) -> np.ndarray:
        """`reps` replays back to back, device milliseconds of each (HIP events between neighbours)."""
        ms = np.zeros(reps, dtype=np.float32)
        self._moe._check(self._moe._lib.mummu_graph_launch_timed(self._moe._h, self._g, reps,
                                                                 ms.ctypes.data_as(C.POINTER(C.c_float))))
        return ms

    def close(self):
        if self._g:
            self._moe._lib.mummu_graph_destroy(self._g)
            self._g = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def probe_copy(dst: "DeviceBuffer", src: "DeviceBuffer", nbytes: int, stream=None):
    """Launch the library's plain copy kernel over nbytes (the known-size dispatch that HBM
    traffic counters are calibrated against)."""
    lib = _lib.load()
    rc = lib.mummu_probe_copy(dst.ptr, src.ptr, nbytes, stream)
    if rc:
        raise MoeError(rc, lib.mummu_moe_last_error(None).decode())


def probe_read(src: "DeviceBuffer", nbytes: int, row_bytes: int, piece_bytes: int, stream=None, offset: int = 0):
    """Launch the library's read-only stream over nbytes (from byte `offset` of src) seen as rows of row_bytes:
    piece_bytes of each of a workgroup's 128 rows per step (the grouped GEMMs' walk of a weight slab), or front to
    back (0)."""
    lib = _lib.load()
    rc = lib.mummu_probe_read(C.c_void_p(int(src.ptr) + offset), nbytes, row_bytes, piece_bytes, stream)
    if rc:
        raise MoeError(rc, lib.mummu_moe_last_error(None).decode())


class PackedWeight:
    """A weight in burn's packed block-32 layout, resident in HBM, behind Q4GemvOps::q4s_gemv
    (nn/packed_gemv.rs:248-260): `words` [K, N*bits/32] u32 (element j of a word at bits j*bits), `scales`
    [K, N/32] f32 (pack.rs:940-985)."""

    def __init__(self, words, scales, k: int, n: int, value_bits: int = 4):
        self._lib = _lib.load()
        self._h = None
        words = np.ascontiguousarray(words, dtype=np.uint32)
        scales = _f32(scales)
        if words.size != k * n * value_bits // 32 or scales.size != k * (n // 32):
            raise MoeError(_lib.ERR_SHAPE, f"packed weight: {words.size} words / {scales.size} scales do not make [{k}, {n}] "
                                           f"at {value_bits} bits")
        h = C.c_void_p()
        rc = self._lib.mummu_packed_weight_create(_ptr(words), _ptr(scales), k, n, value_bits, C.byref(h))
        if rc:
            raise MoeError(rc, self._lib.mummu_packed_last_error().decode())
        self._h, self.k, self.n, self.value_bits = h, k, n, value_bits

    @classmethod
    def wrap_device(cls, words_dev: "DeviceBuffer", scales_dev: "DeviceBuffer", k: int, n: int, value_bits: int = 4):
        """A weight whose words and scales already lie in device memory (borrowed; keep the buffers alive)."""
        self = cls.__new__(cls)
        self._lib = _lib.load()
        h = C.c_void_p()
        rc = self._lib.mummu_packed_weight_wrap_device(words_dev.ptr, scales_dev.ptr, k, n, value_bits, C.byref(h))
        if rc:
            self._h = None
            raise MoeError(rc, self._lib.mummu_packed_last_error().decode())
        self._h, self.k, self.n, self.value_bits = h, k, n, value_bits
        self._keep = (words_dev, scales_dev)
        return self

    def _check(self, rc: int):
        if rc:
            raise MoeError(rc, self._lib.mummu_packed_last_error().decode())

    def resident_bytes(self) -> int:
        return int(self._lib.mummu_packed_weight_bytes(self._h))

    def gemv(self, x) -> np.ndarray:
        """try_q4s_gemv (nn/packed_gemv.rs:98-152): x [m, K] -> [m, N], m <= 64."""
        x = _f32(x)
        k = x.shape[-1] if x.ndim else 0
        m = x.size // max(k, 1)
        y = np.empty((m, self.n), dtype=np.float32)
        self._check(self._lib.mummu_q4s_gemv(self._h, _ptr(x), m, k, _ptr(y)))
        return y

    def gemv_device(self, x_dev: "DeviceBuffer", m: int, y_dev: "DeviceBuffer", stream=None):
        self._check(self._lib.mummu_q4s_gemv_device(self._h, x_dev.ptr, m, self.k, y_dev.ptr, stream))

    def close(self):
        if self._h:
            self._lib.mummu_packed_weight_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        self.close()


class DeviceBuffer:
    """A plain HIP allocation (hipMalloc) addressed through the library."""

    def __init__(self, nbytes: int):
        self._lib = _lib.load()
        self.nbytes = nbytes
        self.ptr = self._lib.mummu_device_alloc(nbytes)
        if not self.ptr:
            raise MoeError(_lib.ERR_DEVICE, f"hipMalloc({nbytes}) failed")

    @staticmethod
    def from_array(a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = DeviceBuffer(a.nbytes)
        b.upload(a)
        return b

    def upload(self, a: np.ndarray):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        rc = self._lib.mummu_copy_to_device(self.ptr, _ptr(a), a.nbytes)
        if rc:
            raise MoeError(rc, self._lib.mummu_moe_last_error(None).decode())

    def download(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        rc = self._lib.mummu_copy_to_host(_ptr(out), self.ptr, out.nbytes)
        if rc:
            raise MoeError(rc, self._lib.mummu_moe_last_error(None).decode())
        return out

    def close(self):
        if self.ptr:
            self._lib.mummu_device_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def synchronize():
    rc = _lib.load().mummu_device_synchronize()
    if rc:
        raise MoeError(rc, _lib.load().mummu_moe_last_error(None).decode())


def device_name() -> str:
    buf = C.create_string_buffer(256)
    rc = _lib.load().mummu_device_name(buf, 256)
    if rc:
        raise MoeError(rc, _lib.load().mummu_moe_last_error(None).decode())
    return buf.value.decode()


def dequantize(dtype: int, data) -> np.ndarray:
    """gguf::dequantize (gguf.rs:1403) on the GPU, bit-exact."""
    b = _bytes(data)
    geom = _lib.BLOCKS.get(dtype, (1, 1))
    out = np.empty(max(b.size // geom[1], 1) * geom[0], dtype=np.float32)
    lib = _lib.load()
    rc = lib.mummu_dequantize(dtype, _ptr(b), b.size, _ptr(out))
    if rc:
        raise MoeError(rc, lib.mummu_moe_last_error(None).decode())
    return out


def route(moe: SparseMoe, logits, n: int, n_experts: int, k: int, flavour: int = ROUTER_QWEN4EXP,
          norm_topk_prob: bool = True):
    """experts.rs:541-582 `route` (or the SparseMoe router, by flavour) on given logits.
    Returns (ids int32 [n,k], weights f32 [n,k])."""
    lg = _f32(logits).reshape(-1)
    if lg.size != n * n_experts:
        raise MoeError(_lib.ERR_SHAPE, f"router logits: {lg.size} values is not {n} rows x {n_experts}")
    ids = np.zeros((n, max(k, 1)), dtype=np.int32)
    w = np.zeros((n, max(k, 1)), dtype=np.float32)
    moe._check(moe._lib.mummu_route_logits(moe._h, _ptr(lg), n, n_experts, k, flavour, int(norm_topk_prob), _ptr(ids), _ptr(w)))
    return ids, w
