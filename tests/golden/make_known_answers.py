"""Writes tests/golden/reference_known_answers.json: the known-answer vectors that the reference's own
unit tests hold for this path, as data (inputs and expected outputs, each with the reference file:line
it was read from).  The reference is Rust and cannot be built or run here, so the values were read
from its test sources as text; this script only lays the described fields out as block bytes and
writes the file.  Run it from the repository root:  python3 tests/golden/make_known_answers.py"""
import json
import os

import numpy as np


def f16(v):
    return np.array([v], dtype=np.float16).view(np.uint8).tolist()


def q8_0_block():
    # f16 d = 0.5, codes q[i] = i - 16
    return f16(0.5) + (np.arange(32, dtype=np.int8) - 16).view(np.uint8).tolist()


def q4_k_block():
    # d = 1, dmin = 0.5, scales[0] = 2, scales[1] = 3, scales[4] = 1, scales[8] = 0x21, qs[0] = 0x51, qs[64] = 0x04
    b = [0] * 144
    b[0:2], b[2:4] = f16(1.0), f16(0.5)
    b[4 + 0], b[4 + 1], b[4 + 4], b[4 + 8] = 2, 3, 1, 0x21
    b[16 + 0], b[16 + 64] = 0x51, 0x04
    return b


def q6_k_block():
    # ql[0] = 0x0F, qh[0] = 0b11, scales[0] = 2, scales[2] = 1, d = 1
    b = [0] * 210
    b[0], b[128], b[192], b[194] = 0x0F, 0b11, 2, 1
    b[208:210] = f16(1.0)
    return b


def q4_0_block():
    # f16 d = 2, qs[0] = 0x31 (low nibble 1 -> element 0, high nibble 3 -> element 16)
    return f16(2.0) + [0x31] + [0] * 15


def q4_1_block():
    # f16 d = 2, f16 m = 1, qs[0] = 0x31
    return f16(2.0) + f16(1.0) + [0x31] + [0] * 15


def q5_0_block():
    # f16 d = 1, qh = 1 | 1 << 16 (little endian), qs[0] = 0x21
    return f16(1.0) + [1, 0, 1, 0] + [0x21] + [0] * 15


def q5_1_block():
    # f16 d = 1, f16 m = 1, qh = 1, qs[0] = 0x01
    return f16(1.0) + f16(1.0) + [1, 0, 0, 0] + [0x01] + [0] * 15


def q5_k_block():
    # d = 1, dmin = 1, scales[0] = 2 (sub 0 scale), scales[1] = 3 (sub 1 scale), scales[4] = 1 (sub 0 min),
    # qh[0] = 1 (element 0 gets +16), ql[0] = 0x21 (low 1 -> element 0, high 2 -> element 32)
    b = [0] * 176
    b[0:2], b[2:4] = f16(1.0), f16(1.0)
    b[4], b[5], b[8], b[16], b[48] = 2, 3, 1, 1, 0x21
    return b


def main():
    stable = [-1000.0] * 48
    stable[5], stable[16 + 9], stable[16 + 3], stable[32 + 15] = 1000.0, 999.0, 998.0, 30.0
    doc = {
        "about": "Known answers held by the reference's own tests for the MoE block path; data only. "
                 "type = GGML tensor type id; expect maps element index -> exact f32 value.",
        "codec": [
            {"cite": "gguf.rs:2379-2393", "type": 0, "bytes": np.array([1.5], np.float32).view(np.uint8).tolist(), "expect": {"0": 1.5}},
            {"cite": "gguf.rs:2379-2393", "type": 1, "bytes": f16(-0.25), "expect": {"0": -0.25}},
            {"cite": "gguf.rs:2379-2393", "type": 30, "bytes": [0x00, 0x40], "expect": {"0": 2.0}},
            {"cite": "gguf.rs:2395-2405", "type": 8, "bytes": q8_0_block(), "count": 32, "expect": {"0": -8.0, "16": 0.0, "31": 7.5}},
            {"cite": "gguf.rs:2407-2429", "type": 12, "bytes": q4_k_block(), "count": 256,
             "expect": {"0": 1.5, "1": -0.5, "32": 15.0, "128": 3.0}},
            {"cite": "gguf.rs:2549-2560", "type": 2, "bytes": q4_0_block(), "count": 32, "expect": {"0": -14.0, "16": -10.0, "1": -16.0}},
            {"cite": "gguf.rs:2562-2569", "type": 3, "bytes": q4_1_block(), "count": 32, "expect": {"0": 3.0, "16": 7.0, "1": 1.0}},
            {"cite": "gguf.rs:2572-2582", "type": 6, "bytes": q5_0_block(), "count": 32, "expect": {"0": 1.0, "16": 2.0, "1": -16.0}},
            {"cite": "gguf.rs:2584-2592", "type": 7, "bytes": q5_1_block(), "count": 32, "expect": {"0": 18.0, "16": 1.0}},
            {"cite": "gguf.rs:2638-2652", "type": 13, "bytes": q5_k_block(), "count": 256, "expect": {"0": 33.0, "1": -1.0, "32": 6.0}},
            {"cite": "gguf.rs:2431-2447", "type": 14, "bytes": q6_k_block(), "count": 256, "expect": {"0": 62.0, "32": -32.0, "64": 0.0}},
        ],
        "codec_refused": [
            {"cite": "gguf.rs:2654-2662", "type": 8, "n_bytes": 33},
            {"cite": "gguf.rs:2654-2662", "type": 8, "n_bytes": 0},
        ],
        "router_qwen4exp": [
            {"cite": "experts.rs:1365-1378", "logits": [0.0, 3.0, 1.0, 2.5, -2.0, 2.0, 0.5, 2.9], "tokens": 1, "experts": 8, "k": 3,
             "ids": [[1, 7, 3]], "weights_softmax_of_selected_logits": True, "tol": 1e-6},
            {"cite": "experts.rs:1380-1388", "logits": [0.5] * 8, "tokens": 1, "experts": 8, "k": 3,
             "ids": [[0, 1, 2]], "weights": [[1 / 3, 1 / 3, 1 / 3]], "tol": 1e-6},
            {"cite": "experts.rs:1380-1388", "logits": [1.0, 0.0, 2.0, 1.0], "tokens": 1, "experts": 4, "k": 2, "ids": [[2, 0]]},
            {"cite": "experts.rs:1390-1408", "logits": stable, "tokens": 3, "experts": 16, "k": 2,
             "ids_prefix": [[5], [9, 3], [15]], "weights_finite_and_sum_to_one": True, "tol": 1e-6,
             "weight_at": {"token": 1, "slot": 0, "value": float(np.e / (np.e + 1.0))}},
        ],
        "router_refused": [
            {"cite": "experts.rs:1410-1417", "logits": [0.0, "nan", 1.0, 2.0], "tokens": 2, "experts": 2, "k": 1, "message": "token 0 expert 1"},
            {"cite": "experts.rs:1410-1417", "logits": [0.0, 0.0, 0.0, 0.0], "tokens": 1, "experts": 4, "k": 0},
            {"cite": "experts.rs:1410-1417", "logits": [0.0, 0.0, 0.0, 0.0], "tokens": 1, "experts": 4, "k": 5},
            {"cite": "experts.rs:1410-1417", "logits": [0.0, 0.0, 0.0, 0.0, 0.0], "tokens": 1, "experts": 4, "k": 2},
        ],
        "renormalize_qwen4exp": [
            {"cite": "experts.rs:1419-1427", "weights": [1e-6, 2e-6], "expect_first": 1e-6 / (1.0 / 16384.0), "tol": 1e-9},
            {"cite": "experts.rs:1419-1427", "weights": [0.25, 0.25], "expect": [0.5, 0.5]},
        ],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_known_answers.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
