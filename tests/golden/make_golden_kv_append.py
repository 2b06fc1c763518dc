"""Writes tests/golden/kv_append_golden.npz: what oracle/kv_append.py answers for the cases of cases_kv_append.py
(q_out and the caches after the append, stored exactly as float32).  The reference holds no vectors for this
operator and its own oracle (flashinfer) is not available, so the vectors freeze this repo's oracle.

    python tests/golden/make_golden_kv_append.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

from cases_kv_append import KV_APPEND_CASES, as_f32, kv_append_case  # noqa: E402
from oracle import kv_append as okv  # noqa: E402


def main():
    blob = {}
    for name in KV_APPEND_CASES:
        c = kv_append_case(name)
        cos, sin = okv.cos_sin_tables(c["qkv"].shape[-1], c["max_positions"], c["rope_theta"])
        q_out = okv.kv_append(c["qkv"], c["k"], c["v"], c["table"], c["lens"], c["wq"], c["wk"], cos, sin, c["hq"],
                              k_scale=c["k_scale"], v_scale=c["v_scale"])
        blob[name + ".q_out"] = as_f32(q_out)
        blob[name + ".k"] = as_f32(c["k"])
        blob[name + ".v"] = as_f32(c["v"])
        blob[name + ".qkv_sum"] = np.float64(c["qkv"].double().sum().item())
    path = os.path.join(HERE, "kv_append_golden.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
