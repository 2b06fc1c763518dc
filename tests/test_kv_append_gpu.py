"""Parity of the RMSNorm + rotary + paged-append kernel with its oracle, on a real MI355X, through the C ABI.

Bars: q_out and the appended K rows within one rounding step of the 16-bit dtype of the oracle (and within the
reference test's atol = rtol = 1e-2 of the independent float64 route, test_qk_norm_rope.py:115-116); V rows and every
cache row that is not a target bit-exact; fp8 bytes equal to the oracle's except where the quotient sits on a
rounding boundary (at most one code apart, rare)."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

import triton_distributed_amd as tda  # noqa: E402
from oracle import closed_form as cf  # noqa: E402
from oracle import fp8 as ofp8  # noqa: E402
from oracle import kv_append as okv  # noqa: E402

from cases_kv_append import KV_APPEND_CASES, as_f32, kv_append_case  # noqa: E402

pytestmark = pytest.mark.gpu
KV_GOLDEN = __import__("numpy").load(os.path.join(ROOT, "tests", "golden", "kv_append_golden.npz"))


def _setup(seed, lens, t, hq, hkv, d, page, dtype, spare=3, theta=1000000.0, poison=True):
    g = torch.Generator().manual_seed(seed)
    b = len(lens)
    qkv = torch.randn(b, t, hq + 2 * hkv, d, generator=g).to(dtype)
    wq = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    wk = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + spare
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((b, max(pages) + 2), 2 ** 31 - 1 if poison else 0, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    cos, sin = okv.cos_sin_tables(d, max(lens) + 1, theta)
    return qkv, wq, wk, table, k, v, cos, sin


def _ulp_close(got, want, dtype, tag, rotated=True):
    """The kernel and the oracle round at the same two points (the normalised halves, the result) but their fp32
    arithmetic differs in the last bit (reduction order, fused multiply-add), which can flip either rounding by
    one step: |got - want| <= step * (|result| + 1.5 * |pair|), |pair| = norm of the rotary pair (i, i + D/2) the
    element belongs to (a flipped input half moves the rotated result by up to its own step)."""
    step = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    g, w = got.double(), want.double()
    half = g.shape[-1] // 2
    pair = (w[..., :half] ** 2 + w[..., half:] ** 2).sqrt()
    pair = torch.cat((pair, pair), dim=-1) if rotated else torch.zeros_like(w)
    bound = step * (torch.maximum(g.abs(), w.abs()) + 1.5 * pair) + 1e-6
    bad = (g - w).abs() > bound
    assert not bad.any(), f"{tag}: {int(bad.sum())} elements beyond one rounding step; worst {float((g - w).abs().max())}"
    assert (g != w).double().mean() < 0.05, f"{tag}: {float((g != w).double().mean()):.3f} of the elements differ"


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page,t", [(1, 1), (16, 1), (16, 5), (6, 3)])
def test_append_matches_the_oracle(cuda_device, d, dtype, page, t):
    print(f"case append D={d} {dtype} P={page} T={t}", flush=True)
    hq, hkv = 8, 2
    lens = [t, 40 + t, 17 + t, 16 * 9 + t]                          # lengths after the append
    qkv, wq, wk, table, k, v, cos, sin = _setup(11 + d + page, lens, t, hq, hkv, d, page, dtype)
    k_ref, v_ref = k.clone(), v.clone()
    q_ref = okv.kv_append(qkv, k_ref, v_ref, table, lens, wq, wk, cos, sin, hq)
    dev = cuda_device
    kd, vd = k.to(dev), v.to(dev)
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), kd, vd, table.to(dev),
                                            torch.tensor(lens, dtype=torch.int32, device=dev), wq.to(dev), wk.to(dev),
                                            cos.to(dev), sin.to(dev))
    torch.cuda.synchronize()
    _ulp_close(q_out.cpu(), q_ref, dtype, "q_out")
    kd, vd = kd.cpu(), vd.cpu()
    assert torch.equal(vd, v_ref)                                     # v: copies, everything else untouched
    _ulp_close(kd, k_ref, dtype, "k_cache")
    untouched = (k_ref == k).all(dim=-1).all(dim=-1)                   # rows the oracle left alone ...
    assert torch.equal(kd[untouched], k[untouched])                    # ... are bit-identical on the GPU too
    # independent float64 route, the reference test's tolerance
    for b, n in enumerate(lens):
        for j in range(t):
            pos = n - t + j
            for h in (0, hq - 1):
                want = okv.norm_rope_fp64(qkv[b, j, h], wq, 1e-6, pos)
                torch.testing.assert_close(q_out[b, j, h].cpu().double(), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("name", list(KV_APPEND_CASES))
def test_append_matches_the_committed_vectors(cuda_device, name):
    c = kv_append_case(name)
    dev = cuda_device
    cos, sin = okv.cos_sin_tables(c["qkv"].shape[-1], c["max_positions"], c["rope_theta"])
    kd, vd = c["k"].to(dev), c["v"].to(dev)
    sc = {} if c["k_scale"] is None else dict(k_scale=c["k_scale"].to(dev), v_scale=c["v_scale"].to(dev))
    q_out = tda.qk_norm_rope_update_kvcache(c["qkv"].to(dev), kd, vd, c["table"].to(dev),
                                            torch.tensor(c["lens"], dtype=torch.int32, device=dev), c["wq"].to(dev),
                                            c["wk"].to(dev), cos.to(dev), sin.to(dev), **sc)
    torch.cuda.synchronize()
    dtype = c["qkv"].dtype
    _ulp_close(q_out.float().cpu(), torch.from_numpy(KV_GOLDEN[name + ".q_out"]), dtype, "q_out vs golden")
    assert (as_f32(vd.cpu()) == KV_GOLDEN[name + ".v"]).all()
    if c["k_scale"] is None:
        _ulp_close(kd.float().cpu(), torch.from_numpy(KV_GOLDEN[name + ".k"]), dtype, "k vs golden")
    else:
        got, want = torch.from_numpy(as_f32(kd.cpu())), torch.from_numpy(KV_GOLDEN[name + ".k"])
        assert ((got - want).abs() <= 0.126 * torch.maximum(got.abs(), want.abs()) + 2.0 ** -9).all()
        assert (got != want).float().mean() < 0.02


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_appends_against_the_oracle(cuda_device, seed):
    import numpy as np
    rng = np.random.default_rng(300 + seed)
    d = int(rng.choice([64, 128, 256]))
    dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float16
    page = int(rng.choice([1, 2, 3, 8, 16, 64]))
    t = int(rng.choice([1, 1, 2, 7]))
    hkv = int(rng.choice([1, 2, 8]))
    hq = hkv * int(rng.choice([0, 1, 4, 5]))                      # 0: only the cache is updated
    batch = int(rng.choice([1, 3, 9]))
    lens = (rng.integers(0, 200, size=batch) + t).tolist()
    fp8 = bool(rng.random() < 0.3) and dtype == torch.bfloat16
    print(f"case random append seed={seed} B={batch} T={t} {hq}q/{hkv}kv D={d} P={page} {dtype} fp8={fp8}", flush=True)
    qkv, wq, wk, table, k, v, cos, sin = _setup(seed, lens, t, hq, hkv, d, page, dtype, theta=float(rng.choice([1e4, 1e6])))
    ks = vs = None
    if fp8:
        k = torch.zeros(k.shape, dtype=torch.float8_e4m3fn)
        v = torch.zeros(v.shape, dtype=torch.float8_e4m3fn)
        ks = torch.tensor(rng.uniform(0.01, 0.03, size=hkv), dtype=torch.float32)
        vs = torch.tensor(rng.uniform(0.01, 0.03, size=hkv), dtype=torch.float32)
    k_ref, v_ref = k.clone(), v.clone()
    q_ref = okv.kv_append(qkv, k_ref, v_ref, table, lens, wq, wk, cos, sin, hq, 1e-5, 1e-6, k_scale=ks, v_scale=vs)
    dev = cuda_device
    kd, vd = k.to(dev), v.to(dev)
    sc = {} if ks is None else dict(k_scale=ks.to(dev), v_scale=vs.to(dev))
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), kd, vd, table.to(dev),
                                            torch.tensor(lens, dtype=torch.int32, device=dev), wq.to(dev), wk.to(dev),
                                            cos.to(dev), sin.to(dev), None, 1e-5, 1e-6, **sc)
    torch.cuda.synchronize()
    if hq:
        _ulp_close(q_out.cpu(), q_ref, dtype, "q_out")
    else:
        assert q_out.numel() == 0
    if fp8:
        tab = torch.from_numpy(ofp8.e4m3fn_table())
        assert torch.equal(vd.cpu().view(torch.uint8), v_ref.view(torch.uint8))
        got, want = tab[kd.cpu().view(torch.uint8).long()], tab[k_ref.view(torch.uint8).long()]
        assert ((got - want).abs() <= 0.126 * torch.maximum(got.abs(), want.abs()) + 2.0 ** -9).all()
        assert (got != want).float().mean() < 0.03
    else:
        assert torch.equal(vd.cpu(), v_ref)
        _ulp_close(kd.cpu(), k_ref, dtype, "k_cache")


def test_positions_outside_the_table_and_poisoned_entries_are_not_written(cuda_device):
    dev = cuda_device
    hq, hkv, d, page, t = 4, 2, 128, 16, 2
    lens = [2, 50, 33]
    qkv, wq, wk, table, k, v, cos, sin = _setup(3, lens, t, hq, hkv, d, page, torch.bfloat16)
    bad_lens = torch.tensor([1, 50, 16 * table.shape[1] + 7], dtype=torch.int32)    # b=0: first token at pos -1; b=2: past the table
    table[1, 49 // page] = -5                                                        # b=1: its target page id is invalid
    kd, vd = k.to(dev), v.to(dev)
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), kd, vd, table.to(dev), bad_lens.to(dev), wq.to(dev), wk.to(dev),
                                            cos.to(dev), sin.to(dev))
    torch.cuda.synchronize()
    assert torch.isfinite(q_out.float()).all()
    changed = (kd.cpu() != k).any(dim=-1).any(dim=-1) | (vd.cpu() != v).any(dim=-1).any(dim=-1)
    # only b=0's second token (position 0) has a valid target
    assert int(changed.sum()) == 1 and bool(changed[int(table[0, 0]), 0])


@pytest.mark.parametrize("d", [128, 256])
def test_fp8_cache_receives_the_saturating_quantised_rows(cuda_device, d):
    dev = cuda_device
    hq, hkv, page, t = 8, 2, 16, 2
    lens = [2, 35, 100]
    qkv, wq, wk, table, k, v, cos, sin = _setup(9 + d, lens, t, hq, hkv, d, page, torch.bfloat16)
    qkv[1, 1, hq + hkv] *= 50.0                                      # a v row far above the scale: saturates
    ks = torch.tensor([0.01, 0.02], dtype=torch.float32)
    vs = torch.tensor([0.015, 0.005], dtype=torch.float32)
    k8 = torch.zeros(k.shape, dtype=torch.float8_e4m3fn)
    v8 = torch.zeros(v.shape, dtype=torch.float8_e4m3fn)
    k8_ref, v8_ref = k8.clone(), v8.clone()
    q_ref = okv.kv_append(qkv, k8_ref, v8_ref, table, lens, wq, wk, cos, sin, hq, k_scale=ks, v_scale=vs)
    k8d, v8d = k8.to(dev), v8.to(dev)
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), k8d, v8d, table.to(dev),
                                            torch.tensor(lens, dtype=torch.int32, device=dev), wq.to(dev), wk.to(dev),
                                            cos.to(dev), sin.to(dev), k_scale=ks.to(dev), v_scale=vs.to(dev))
    torch.cuda.synchronize()
    _ulp_close(q_out.cpu(), q_ref, torch.bfloat16, "q_out")
    assert torch.equal(v8d.cpu().view(torch.uint8), v8_ref.view(torch.uint8))       # v: same bf16 input, same bytes
    tab = torch.from_numpy(ofp8.e4m3fn_table())
    got, want = tab[k8d.cpu().view(torch.uint8).long()], tab[k8_ref.view(torch.uint8).long()]
    assert torch.isfinite(got).all()
    # k rows pass through a bf16 rounding that may differ by one step from the oracle's: the bytes then differ
    # by at most one e4m3 code (2^-3 relative), and almost all are equal
    assert ((got - want).abs() <= 0.126 * torch.maximum(got.abs(), want.abs()) + 2.0 ** -9).all()
    assert (got != want).float().mean() < 0.02
    assert (tab[v8d.cpu().view(torch.uint8).long()].abs() == 448).any()


def test_append_then_decode_equals_attention_over_the_grown_cache(cuda_device):
    # the two operators back to back, as the reference's attention layer runs them (models/layers/tp_attn.py:111-115):
    # the appended token must be attended by the decode that follows
    dev = cuda_device
    hq, hkv, d, page = 32, 8, 128, 16
    lens = [1, 200, 513, 4096]
    qkv, wq, wk, table, k, v, cos, sin = _setup(21, lens, 1, hq, hkv, d, page, torch.bfloat16, poison=False)
    k_ref, v_ref = k.clone(), v.clone()
    q_ref = okv.kv_append(qkv, k_ref, v_ref, table, lens, wq, wk, cos, sin, hq)
    kd, vd, td = k.to(dev), v.to(dev), table.to(dev)
    lens_t = torch.tensor(lens, dtype=torch.int32, device=dev)
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), kd, vd, td, lens_t, wq.to(dev), wk.to(dev), cos.to(dev), sin.to(dev))
    out, lse = tda.flash_decode(q_out[:, 0], kd, vd, td, lens_t, d ** -0.5)
    # the same through the mega-kernel builder's layout ([B, 1, Hq, D] in and out, default scale)
    out4 = torch.full((len(lens), 1, hq, d), float("nan"), dtype=torch.bfloat16, device=dev)
    assert tda.flash_decode_bsnh(q_out, kd, vd, td, lens_t, out4).data_ptr() == out4.data_ptr()
    torch.cuda.synchronize()
    assert torch.equal(out4[:, 0], out)
    o64, l64 = cf.attn_fp64(q_ref[:, 0], k_ref, v_ref, table, lens, d ** -0.5)
    torch.testing.assert_close(out.double().cpu(), o64, atol=1e-2, rtol=2e-2)
    torch.testing.assert_close(lse.double().cpu(), l64, atol=2e-2, rtol=0)     # q rows may differ by a 16-bit rounding step
    # sequence 0 holds exactly the appended token: the output is that token's v row
    assert torch.equal(out[0].cpu().view(hkv, hq // hkv, d), qkv[0, 0, hq + hkv:][:, None].expand(hkv, hq // hkv, d))


@pytest.mark.parametrize("hq,hkv,t", [(8, 1, 300), (16, 1, 301), (20, 1, 301)])
def test_prefill_sized_append_and_per_sequence_tables(cuda_device, hq, hkv, t):
    # many new tokens per sequence, cos / sin given per sequence ([B, S, D]); 9000 / 15351 / 19866 head rows: grids of
    # one, two and four rows per wavefront, the last wavefront of the larger two only partly filled
    dev = cuda_device
    d, page = 128, 16
    lens = [t, 1500, 777]
    qkv, wq, wk, table, k, v, cos, sin = _setup(31, lens, t, hq, hkv, d, page, torch.bfloat16)
    cos3 = cos[None].repeat(3, 1, 1).contiguous()
    sin3 = sin[None].repeat(3, 1, 1).contiguous()
    k_ref, v_ref = k.clone(), v.clone()
    q_ref = okv.kv_append(qkv, k_ref, v_ref, table, lens, wq, wk, cos, sin, hq)
    kd, vd = k.to(dev), v.to(dev)
    q_pre = torch.full((3, t, hq, d), float("nan"), dtype=torch.bfloat16, device=dev)
    q_out = tda.qk_norm_rope_update_kvcache(qkv.to(dev), kd, vd, table.to(dev),
                                            torch.tensor(lens, dtype=torch.int32, device=dev), wq.to(dev), wk.to(dev),
                                            cos3.to(dev), sin3.to(dev), q_pre, 1e-6, 1e-6)
    torch.cuda.synchronize()
    assert q_out.data_ptr() == q_pre.data_ptr()
    _ulp_close(q_out.cpu(), q_ref, torch.bfloat16, "q_out")
    _ulp_close(kd.cpu(), k_ref, torch.bfloat16, "k_cache")
    assert torch.equal(vd.cpu(), v_ref)


def test_host_rejects_what_the_kernel_cannot_take(cuda_device):
    dev = cuda_device
    qkv, wq, wk, table, k, v, cos, sin = _setup(1, [3], 1, 4, 2, 128, 16, torch.bfloat16)
    args = [x.to(dev) for x in (qkv, k, v, table, torch.tensor([3], dtype=torch.int32), wq, wk, cos, sin)]
    with pytest.raises(ValueError):
        tda.qk_norm_rope_update_kvcache(args[0].cpu(), *args[1:])                      # no CPU path
    with pytest.raises(ValueError):
        tda.qk_norm_rope_update_kvcache(args[0], args[1], args[2].half(), *args[3:])   # cache dtypes differ
    with pytest.raises(ValueError):
        tda.qk_norm_rope_update_kvcache(*args[:3], args[3].long(), *args[4:])          # int64 table
    with pytest.raises(ValueError):
        tda.qk_norm_rope_update_kvcache(*args[:7], args[7].half(), args[8].half())     # 16-bit cos / sin
    with pytest.raises(ValueError):
        tda.qk_norm_rope_update_kvcache(*args[:5], args[5][:64], *args[6:])            # short weight
    with pytest.raises(ValueError):                                                     # fp8 cache without scales
        tda.qk_norm_rope_update_kvcache(args[0], args[1].to(torch.float8_e4m3fn), args[2].to(torch.float8_e4m3fn), *args[3:])
