"""Times the packed-GEMV op (Q4GemvOps::q4s_gemv, nn/packed_gemv.rs) on one GPU with device-resident inputs.

    python -m mummu_amd.bench_packed_gemv                      # Q4S [5120, 17408], 1 row
    python -m mummu_amd.bench_packed_gemv --k 4096 --n 14336 --bits 8 --rows 8

Several copies of the weight are used in rotation so that no call finds its weight in the 256 MB cache.  Prints one
JSON line: wall-clock microseconds per call (two launches: the product and the sum over the K split) and the packed
bytes (values + scales) per second."""
import argparse
import json
import time

import numpy as np

from . import _lib, moe as M, synth


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--k", type=int, default=5120)
    ap.add_argument("--n", type=int, default=17408)
    ap.add_argument("--bits", type=int, default=4, choices=[4, 8])
    ap.add_argument("--rows", type=int, default=1)
    ap.add_argument("--reps", type=int, default=50)
    args = ap.parse_args()
    lib = _lib.load()
    g = np.random.Generator(np.random.PCG64(1))
    lim = 1 << (args.bits - 1)
    codes = g.integers(-lim, lim, (args.k, args.n), dtype=np.int8)
    scales = g.uniform(0.001, 0.01, (args.k, args.n // 32)).astype(np.float32)
    words = synth.pack_words(codes, args.bits)
    copies = max(1, min(8, int(600e6 // (words.nbytes + scales.nbytes))))
    weights = [M.PackedWeight(words, scales, args.k, args.n, args.bits) for _ in range(copies)]
    x = g.standard_normal((args.rows, args.k)).astype(np.float32)
    xd, yd = M.DeviceBuffer.from_array(x), M.DeviceBuffer(4 * args.rows * args.n)
    for w in weights:
        w.gemv_device(xd, args.rows, yd)
    lib.mummu_device_synchronize()
    t0 = time.perf_counter()
    for _ in range(args.reps):
        for w in weights:
            w.gemv_device(xd, args.rows, yd)
    lib.mummu_device_synchronize()
    dt = (time.perf_counter() - t0) / (args.reps * copies)
    nbytes = weights[0].resident_bytes()
    print(json.dumps({"op": "q4s_gemv", "k": args.k, "n": args.n, "value_bits": args.bits, "rows": args.rows,
                      "us_per_call": round(dt * 1e6, 2), "packed_bytes": nbytes, "gb_per_s": round(nbytes / dt / 1e9, 1),
                      "weight_copies": copies, "calls": args.reps * copies}))
    for w in weights:
        w.close()


if __name__ == "__main__":
    main()
