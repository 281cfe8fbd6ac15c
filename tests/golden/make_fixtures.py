#!/usr/bin/env python3
"""Writes tests/golden/turq_vectors.npz: inputs and expected outputs of the quantized-linear path.

The expected values come from the NumPy restatement of the block formats (oracle/oracle_np.py, written per
output element from the format definitions) and, for the matmul, from a float64 product on the dequantized
weights computed here with plain NumPy.  The C oracle, the GPU kernels and later edits of either restatement
are all checked against these committed vectors (tests/test_golden_vectors.py), so a change in any of them
shows up as a difference from data that no longer depends on the code under test.

No reference implementation (candle) can be executed in the build environment; what these vectors pin is the
agreement of two independently written restatements at the time of writing, not candle itself.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle_np as onp  # noqa: E402
from tur_amd import synth  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "turq_vectors.npz")
DTYPES = {"q8_0": onp.Q8_0, "q4_k": onp.Q4_K, "q5_k": onp.Q5_K, "q6_k": onp.Q6_K}


def main() -> None:
    out = {}
    for name, dt in DTYPES.items():
        # a small weight [n, k] of seeded blocks (synth mixes in zero, subnormal and large f16 scales)
        n, k, m = 16, 512, 3
        raw = synth.random_weight(dt, n, k, seed=20240 + dt)
        deq = onp.dequantize(dt, raw)
        x = synth.random_activation(m, k, seed=77 + dt)
        dense = (x.astype(np.float64) @ deq.reshape(n, k).astype(np.float64).T).astype(np.float32)
        out[f"{name}_raw"] = raw
        out[f"{name}_shape"] = np.array([n, k, m], np.int64)
        out[f"{name}_dequant_bits"] = deq.view(np.uint32)
        out[f"{name}_x"] = x
        out[f"{name}_dense"] = dense
        out[f"{name}_cpu_qmatmul"] = onp.qmatmul(dt, x, raw, n, k)
    # activation quantisation: seeded rows plus ties, a zero block and a near-overflow block
    rng = np.random.default_rng(5)
    xq = rng.standard_normal((4, 512)).astype(np.float32)
    xq[1, :32] = 0.0
    xq[2, :8] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.0, -127.0], np.float32)
    xq[3] *= 1e6
    out["quant_x"] = xq
    out["quant_q8_0"] = onp.quantize_q8_0(xq)
    out["quant_q8_k"] = onp.quantize_q8_K(xq)
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT}: {os.path.getsize(OUT)} bytes, {len(out)} arrays")


if __name__ == "__main__":
    main()
