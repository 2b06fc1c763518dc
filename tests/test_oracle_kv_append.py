"""Pins oracle/kv_append.py (CPU only) with checks that do not share its formulas: an independent float64 route
(numpy norm, complex rotation), invariants of a rotation, special positions, bit-exact copies and untouched rows.

A slip such as a swapped sign in the rotation, pairing (2i, 2i+1) instead of (i, i + D/2), the wrong table row,
mean over the wrong length, eps outside the root, a slot without the page factor or v taken from the k heads
fails at least one of them."""
import numpy as np
import pytest
import torch

from oracle import fp8 as ofp8
from oracle import kv_append as okv

TOL = dict(atol=1e-2, rtol=1e-2)          # the reference test's tolerance (test_qk_norm_rope.py:115-116)


def _setup(seed, b, t, hq, hkv, d, page, lens, dtype=torch.bfloat16, spare=3, theta=1000000.0):
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(b, t, hq + 2 * hkv, d, generator=g).to(dtype)
    wq = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    wk = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + spare
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.zeros(b, max(pages) + 1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    cos, sin = okv.cos_sin_tables(d, max(lens) + 1, theta)
    return qkv, wq, wk, table, k, v, cos, sin


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rows_agree_with_the_float64_route(d, dtype):
    g = torch.Generator().manual_seed(d)
    cos, sin = okv.cos_sin_tables(d, 5000)
    for pos in (0, 1, 17, 4095, 4999):
        x = torch.randn(d, generator=g).to(dtype)
        w = (1.0 + 0.3 * torch.randn(d, generator=g)).to(dtype)
        got = okv.norm_rope_row(x, w, 1e-6, cos[pos], sin[pos]).double()
        want = okv.norm_rope_fp64(x, w, 1e-6, pos)
        torch.testing.assert_close(got, want, **TOL)
        # tighter: the only roundings are 16-bit ones of values of size ~|w| (2 roundings, each 2^-8 relative for bf16)
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        assert (got - want).abs().max() <= 4 * ulp * want.abs().max() + 1e-6


def test_position_zero_is_the_identity_rotation_and_unit_weights_give_unit_rms():
    d = 128
    cos, sin = okv.cos_sin_tables(d, 4)
    x = torch.randn(d, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    w = torch.ones(d, dtype=torch.bfloat16)
    y = okv.norm_rope_row(x, w, 0.0, cos[0], sin[0]).double()
    # rmsnorm only: y = x / rms(x); mean(y^2) = 1; direction unchanged
    assert abs(float((y * y).mean()) - 1.0) < 1e-2
    torch.testing.assert_close(y, x.double() / x.double().pow(2).mean().sqrt(), atol=2e-2, rtol=1e-2)
    # constant rows normalise to +-1 exactly
    c = torch.full((d,), -3.0, dtype=torch.bfloat16)
    assert torch.equal(okv.norm_rope_row(c, w, 0.0, cos[0], sin[0]), torch.full((d,), -1.0, dtype=torch.bfloat16))
    # eps sits inside the root: a zero row stays zero (no division by zero), and a huge eps shrinks the row
    z = torch.zeros(d, dtype=torch.bfloat16)
    assert torch.equal(okv.norm_rope_row(z, w, 1e-6, cos[1], sin[1]), z)
    big = okv.norm_rope_row(x, w, 99.0, cos[0], sin[0]).double()
    torch.testing.assert_close(big, x.double() / (x.double().pow(2).mean() + 99.0).sqrt(), atol=1e-2, rtol=1e-2)


def test_rotation_preserves_pair_norms_and_composes():
    d = 128
    cos, sin = okv.cos_sin_tables(d, 3000, rope_theta=10000.0)
    x = torch.randn(d, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    w = torch.ones(d, dtype=torch.bfloat16)
    base = okv.norm_rope_row(x, w, 1e-6, cos[0], sin[0]).double()
    for pos in (1, 100, 2999):
        y = okv.norm_rope_row(x, w, 1e-6, cos[pos], sin[pos]).double()
        n0 = base[: d // 2] ** 2 + base[d // 2:] ** 2
        n1 = y[: d // 2] ** 2 + y[d // 2:] ** 2
        torch.testing.assert_close(n1, n0, atol=3e-2, rtol=3e-2)       # pair (i, i + D/2) is rotated, nothing else
        # the slowest pair (i = D/2 - 1) turns by pos * theta^(-(D-2)/D): check the angle itself
        i = d // 2 - 1
        ang = np.arctan2(float(y[d // 2 + i]), float(y[i])) - np.arctan2(float(base[d // 2 + i]), float(base[i]))
        want = pos * 10000.0 ** (-(d - 2) / d)
        assert abs((ang - want + np.pi) % (2 * np.pi) - np.pi) < 3e-2
    # <rope(q, m), rope(k, n)> depends on m - n only
    xq = torch.randn(d, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    dots = [float(okv.norm_rope_row(x, w, 1e-6, cos[m], sin[m]).double() @
                  okv.norm_rope_row(xq, w, 1e-6, cos[m + 7], sin[m + 7]).double()) for m in (0, 50, 1234)]
    assert max(dots) - min(dots) < 0.05 * d ** 0.5


@pytest.mark.parametrize("page", [1, 16, 6])
@pytest.mark.parametrize("t", [1, 3])
def test_append_touches_exactly_the_target_rows(page, t):
    b, hq, hkv, d = 3, 4, 2, 64
    lens = [t, 40 + t, 17 + t]                                   # lengths after the append
    qkv, wq, wk, table, k, v, cos, sin = _setup(5 + page, b, t, hq, hkv, d, page, lens)
    k0, v0 = k.clone(), v.clone()
    q_out = okv.kv_append(qkv, k, v, table, lens, wq, wk, cos, sin, hq)
    touched = torch.zeros(k.shape[0], page, dtype=torch.bool)
    for i in range(b):
        for j in range(t):
            pos = lens[i] - t + j
            pg, off = int(table[i, pos // page]), pos % page
            touched[pg, off] = True
            # v: bit-exact copy of the v heads (the last Hkv head rows), k: the normalised, rotated k heads
            assert torch.equal(v[pg, off], qkv[i, j, hq + hkv:])
            for h in range(hkv):
                want = okv.norm_rope_fp64(qkv[i, j, hq + h], wk, 1e-6, pos)
                torch.testing.assert_close(k[pg, off, h].double(), want, **TOL)
            for h in range(hq):
                want = okv.norm_rope_fp64(qkv[i, j, h], wq, 1e-6, pos)
                torch.testing.assert_close(q_out[i, j, h].double(), want, **TOL)
    assert int(touched.sum()) == b * t                           # distinct slots
    assert torch.equal(k[~touched], k0[~touched]) and torch.equal(v[~touched], v0[~touched])


def test_fp8_write_is_the_saturating_cast_of_the_quotient():
    b, t, hq, hkv, d, page = 2, 2, 4, 2, 128, 16
    lens = [2, 35]
    qkv, wq, wk, table, k, v, cos, sin = _setup(9, b, t, hq, hkv, d, page, lens)
    qkv[1, 1, hq + hkv] *= 50.0                                  # a v row far above the scale: must saturate
    k8 = torch.zeros(k.shape, dtype=torch.float8_e4m3fn)
    v8 = torch.zeros(v.shape, dtype=torch.float8_e4m3fn)
    ks = torch.tensor([0.01, 0.02], dtype=torch.float32)
    vs = torch.tensor([0.015, 0.005], dtype=torch.float32)
    kb, vb = k.clone(), v.clone()
    okv.kv_append(qkv, kb, vb, table, lens, wq, wk, cos, sin, hq)                      # 16-bit cache
    okv.kv_append(qkv, k8, v8, table, lens, wq, wk, cos, sin, hq, k_scale=ks, v_scale=vs)
    tab = torch.from_numpy(ofp8.e4m3fn_table())
    for i in range(b):
        for j in range(t):
            pos = lens[i] - t + j
            pg, off = int(table[i, pos // page]), pos % page
            for h in range(hkv):
                for c8, cb, sc in ((k8, kb, ks), (v8, vb, vs)):
                    want = cb[pg, off, h].float() / sc[h]
                    got = tab[c8[pg, off, h].view(torch.uint8).long()]
                    assert torch.isfinite(got).all()
                    inside = want.abs() <= 448
                    # nearest e4m3 value: within half a step (2^-4 relative) of the quotient; saturated outside
                    assert ((got - want).abs()[inside] <= want.abs()[inside] * 2.0 ** -4 + 2.0 ** -10).all()
                    assert (got[~inside].abs() == 448).all() and (torch.sign(got[~inside]) == torch.sign(want[~inside])).all()
    assert (tab[v8.view(torch.uint8).long()].abs() == 448).any()
