"""The committed golden vectors against the oracle (CPU).  The GPU tests compare the kernels with the same
vectors, so oracle, fixtures and kernels are checked three ways."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

from cases import EDGE_CASES, all_cases  # noqa: E402
from oracle.closed_form import attn_fp64  # noqa: E402
from oracle.paged_attn import ref_paged_attn  # noqa: E402

GOLDEN = np.load(os.path.join(ROOT, "tests", "golden", "decode_golden.npz"))
CASES = dict(all_cases())


def test_fixture_covers_all_cases():
    names = {k.split(".")[0] for k in GOLDEN.files}
    assert names == set(CASES) == {"tiny", *EDGE_CASES}


@pytest.mark.parametrize("name", list(CASES))
def test_oracle_reproduces_golden(name):
    c = CASES[name]
    assert abs(float(c["q"].double().sum()) - float(GOLDEN[name + ".q_sum"])) < 1e-9   # same seeded inputs
    out, lse = attn_fp64(c["q"], c["k_cache"], c["v_cache"], c["block_table"], c["kv_lens"], c["sm_scale"],
                         c["soft_cap"])
    np.testing.assert_allclose(out.numpy(), GOLDEN[name + ".out64"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(lse.numpy(), GOLDEN[name + ".lse64"], rtol=1e-12, atol=1e-12)
    ref = ref_paged_attn(c["q"], c["k_cache"], c["v_cache"], c["kv_lens"], c["block_table"], c["sm_scale"],
                         c["soft_cap"])
    # torch's CPU kernels may differ in accumulation order between builds: one low-precision ulp of slack
    np.testing.assert_allclose(ref.float().numpy(), GOLDEN[name + ".ref"], rtol=2e-2, atol=2e-3)
    # and the two oracles agree at the reference's own tolerance
    np.testing.assert_allclose(GOLDEN[name + ".ref"], GOLDEN[name + ".out64"], rtol=1e-2, atol=1e-2)


def test_tiny_config_shapes():
    c = CASES["tiny"]
    assert tuple(c["q"].shape) == (2, 8, 128) and tuple(c["k_cache"].shape) == (1024, 1, 2, 128)
    assert sorted(c["block_table"].flatten().tolist()) == list(range(1024))      # a permutation of the pool
    assert GOLDEN["tiny.out64"].shape == (2, 8, 128) and GOLDEN["tiny.lse64"].shape == (2, 8)


# ---- the RMSNorm + rotary + paged-append operator -----------------------------------------------------------------
from cases_kv_append import KV_APPEND_CASES, as_f32, kv_append_case  # noqa: E402
from oracle import kv_append as okv  # noqa: E402

KV_GOLDEN = np.load(os.path.join(ROOT, "tests", "golden", "kv_append_golden.npz"))


@pytest.mark.parametrize("name", list(KV_APPEND_CASES))
def test_kv_append_oracle_reproduces_golden(name):
    c = kv_append_case(name)
    assert abs(float(c["qkv"].double().sum()) - float(KV_GOLDEN[name + ".qkv_sum"])) < 1e-9
    cos, sin = okv.cos_sin_tables(c["qkv"].shape[-1], c["max_positions"], c["rope_theta"])
    q_out = okv.kv_append(c["qkv"], c["k"], c["v"], c["table"], c["lens"], c["wq"], c["wk"], cos, sin, c["hq"],
                          k_scale=c["k_scale"], v_scale=c["v_scale"])
    step = 2.0 ** -7 if c["qkv"].dtype == torch.bfloat16 else 2.0 ** -10
    # torch's CPU reductions may differ in the last fp32 bit between builds: at most one 16-bit rounding step
    # (for a rotated element: of its pair's magnitude; for an fp8 byte: one e4m3 code = 2^-3)
    pair = np.abs(KV_GOLDEN[name + ".q_out"]).max()
    np.testing.assert_allclose(as_f32(q_out), KV_GOLDEN[name + ".q_out"], rtol=step, atol=2.5 * step * pair)
    k_step = 2.0 ** -3 if c["k"].dtype == torch.float8_e4m3fn else step
    np.testing.assert_allclose(as_f32(c["k"]), KV_GOLDEN[name + ".k"], rtol=k_step, atol=2.5 * k_step * np.abs(KV_GOLDEN[name + ".k"]).max())
    np.testing.assert_array_equal(as_f32(c["v"]), KV_GOLDEN[name + ".v"])              # copies / exact quotients
    assert (as_f32(q_out) == KV_GOLDEN[name + ".q_out"]).mean() > 0.99                 # and in fact (almost) all equal
