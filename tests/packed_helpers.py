"""Weights in burn's packed block-32 layout (pack.rs:940-985) for the packed-GEMV tests - built by the package's
synthetic-data helpers - and an independent f64 evaluation of x . dequantize(w) to judge the op against, as
nn/packed_gemv.rs:1593-1624 does."""
import numpy as np

from mummu_amd.synth import pack_words, quantize_block32  # noqa: F401


def reference_f64(codes, scales, x):
    w = codes.astype(np.float64) * np.repeat(scales.astype(np.float64), 32, axis=1)
    return x.astype(np.float64) @ w
