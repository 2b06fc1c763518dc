"""Writes tests/golden/decode_golden.npz: float64-oracle (out, lse) and the torch-restatement out for the
small seeded cases of cases.py.  The reference holds no golden vectors for this path and cannot be
imported here, so these vectors come from this repo's oracle (oracle/closed_form.py, oracle/paged_attn.py);
they freeze its answers so that oracle, fixtures and kernels are compared three ways.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

from cases import all_cases  # noqa: E402
from oracle.closed_form import attn_fp64  # noqa: E402
from oracle.paged_attn import ref_paged_attn  # noqa: E402


def main():
    blob = {}
    for name, c in all_cases():
        out, lse = attn_fp64(c["q"], c["k_cache"], c["v_cache"], c["block_table"], c["kv_lens"], c["sm_scale"],
                             c["soft_cap"])
        ref = ref_paged_attn(c["q"], c["k_cache"], c["v_cache"], c["kv_lens"], c["block_table"], c["sm_scale"],
                             c["soft_cap"])
        blob[name + ".out64"] = out.numpy().astype(np.float32)   # 24-bit mantissa is ample for a 2e-2 / 1e-3 bar
        blob[name + ".lse64"] = lse.numpy()
        blob[name + ".ref"] = ref.float().numpy()
        blob[name + ".q_sum"] = np.float64(c["q"].double().sum().item())   # guards the seeded inputs
    path = os.path.join(HERE, "decode_golden.npz")
    np.savez_compressed(path, **blob)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
