"""Shared fixtures for the parity tests: the reference's closed-form toy block
(nn/moe.rs:1617-1651, 2088-2175) and its synthetic quantized toy layers
(models/qwen4exp/experts.rs:1429-1447), rebuilt from their formulas and seeds."""
from __future__ import annotations

import math

import numpy as np

from mummu_amd import synth

# nn/moe.rs:1617-1620
TOY_A = dict(hidden=4, inter=3, experts=4, top_k=2)


def _sin_fill(seed: float, n: int) -> np.ndarray:
    # f32_from_usize(i).mul_add(0.37, seed).sin() * 0.5  (nn/moe.rs:1627-1629)
    i = np.arange(n, dtype=np.float64)
    arg = (i * float(np.float32(0.37)) + float(np.float32(seed))).astype(np.float32)
    return (np.sin(arg.astype(np.float64)).astype(np.float32) * np.float32(0.5)).astype(np.float32)


def toy_a_weights():
    """Returns (router [E,H] f32 -- the transpose of the reference's [H,E] Linear weight --,
    gate [E,I,H], up [E,I,H], down [E,H,I])."""
    h, i, e = TOY_A["hidden"], TOY_A["inter"], TOY_A["experts"]
    idx = np.arange(h * e, dtype=np.float64)
    arg = (idx * float(np.float32(0.61)) + 1.0).astype(np.float32)
    router_he = (np.cos(arg.astype(np.float64)).astype(np.float32) * np.float32(0.5)).reshape(h, e)
    gate = _sin_fill(0.1, e * i * h).reshape(e, i, h)
    up = _sin_fill(1.7, e * i * h).reshape(e, i, h)
    down = _sin_fill(3.3, e * h * i).reshape(e, h, i)
    return np.ascontiguousarray(router_he.T), gate, up, down


def toy_a_input(t: int, seed: float) -> np.ndarray:
    # ((i + seed) * 0.9).sin()  (nn/moe.rs:2088-2093)
    h = TOY_A["hidden"]
    i = np.arange(t * h, dtype=np.float32)
    arg = ((i + np.float32(seed)) * np.float32(0.9)).astype(np.float32)
    return np.sin(arg.astype(np.float64)).astype(np.float32).reshape(t, h)


def toy_a_scalar_reference(router_eh, gate, up, down, xs, top_k: int, norm: bool) -> np.ndarray:
    """The reference's hand-rolled f32 block (nn/moe.rs:2101-2175), restated with Python
    loops and numpy float32 scalars: sequential sums, max-shifted softmax, stable
    descending sort, two-rounding combine in picked (descending-probability) order."""
    f = np.float32
    e_n, i_n, h_n = gate.shape
    t_n = xs.shape[0]
    out = np.zeros((t_n, h_n), dtype=np.float32)
    for tok in range(t_n):
        x = xs[tok]
        logits = []
        for e in range(e_n):
            s = f(0)
            for i in range(h_n):
                s = f(s + f(x[i] * router_eh[e, i]))
            logits.append(s)
        mx = max(logits)
        exps = [f(math.exp(float(f(l - mx)))) for l in logits]
        total = f(0)
        for v in exps:
            total = f(total + v)
        probs = [f(v / total) for v in exps]
        order = sorted(range(e_n), key=lambda a: -float(probs[a]))  # stable
        picked = order[:top_k]
        denom = f(1)
        if norm:
            denom = f(0)
            for e in picked:
                denom = f(denom + probs[e])
        for e in picked:
            weight = f(probs[e] / denom)
            act = []
            for j in range(i_n):
                g = f(0)
                u = f(0)
                for i in range(h_n):
                    g = f(g + f(x[i] * gate[e, j, i]))
                    u = f(u + f(x[i] * up[e, j, i]))
                silu = f(g / f(f(1) + f(math.exp(-float(g)))))
                act.append(f(silu * u))
            for i in range(h_n):
                d = f(0)
                for j in range(i_n):
                    d = f(d + f(act[j] * down[e, i, j]))
                out[tok, i] = f(out[tok, i] + f(weight * d))
    return out


# models/qwen4exp/experts.rs:1429-1431
TOY_D = dict(hidden=256, ffn=32, experts=8)


def toy_d_layers(seed: int):
    """experts.rs:1435-1447: two layers, gate/up Q4_K, down Q5_1 (layer 0) / Q8_0 (layer 1).
    Returns a list of dicts of raw bank bytes."""
    rng = synth.SplitMix64(seed)
    fwd = [TOY_D["hidden"], TOY_D["ffn"], TOY_D["experts"]]
    back = [TOY_D["ffn"], TOY_D["hidden"], TOY_D["experts"]]
    layers = []
    for down_t in (synth.Q5_1, synth.Q8_0):
        gate = synth.synth_bank(synth.Q4_K, fwd, rng)
        up = synth.synth_bank(synth.Q4_K, fwd, rng)
        down = synth.synth_bank(down_t, back, rng)
        layers.append(dict(gate=gate, up=up, down=down, gate_type=synth.Q4_K, up_type=synth.Q4_K, down_type=down_t))
    return layers


def ulp_diff(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in units of last place between two float32 arrays (finite values)."""
    ai = np.asarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    bi = np.asarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    return np.abs(ai - bi)
