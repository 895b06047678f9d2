"""Writes the golden vectors of tests/golden/ with this repository's own oracle (no reference code is involved:
the reference holds no fixtures or known-answer vectors for this path).

    python tests/golden/make_golden.py

cfg1 (B=1, H=2, N=128, d=64, scale 1/8): q/k/v as e4m3 codes (uint8) from a recorded seed, the oracle output for
kv block 64 non-causal and causal (fp16 bits), and exact fp64 attention on the dequantised inputs (float32).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import fa8_oracle as fo  # noqa: E402
from oracle import np_restatement as nr  # noqa: E402


def main():
    rng = np.random.default_rng(20240601)
    shape = (1, 2, 128, 64)
    q, k, v = (nr.encode_rne_sat(rng.standard_normal(shape)) for _ in range(3))
    o = fo.forward(q, k, v, 0.125, kv_block=64)
    oc = fo.forward(q, k, v, 0.125, causal=True, kv_block=64)
    f64 = fo.attention_f64(q, k, v, 0.125).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "cfg1_golden.npz"), q=q, k=k, v=v, o_fp16_bits=o.view(np.uint16),
                        o_causal_fp16_bits=oc.view(np.uint16), o_exact_f32=f64, scale=np.float32(0.125),
                        kv_block=np.int32(64))
    print("wrote", os.path.join(HERE, "cfg1_golden.npz"))


if __name__ == "__main__":
    main()
