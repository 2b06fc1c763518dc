"""Parity of the HIP decode path with the oracle, on a real MI355X, through the C ABI.

Tolerances (the bar this path is held to):
  out  bf16/fp16: |out - ref| <= 2e-2 + 2e-2*|ref| against the torch restatement of the reference's
       torch implementation, and a tighter 8e-3 + 1e-2*|x| against the exact float64 answer;
  lse  fp32: |lse - lse64| <= 1e-3;
  block_table indexing: bit-exact where the mathematics allows it (single-token sequences, page
  permutations), no NaN/inf anywhere for kv_len >= 1."""
import math
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

import triton_distributed_amd as tda  # noqa: E402
from triton_distributed_amd import workloads as wl  # noqa: E402
from cases import EDGE_CASES, all_cases  # noqa: E402
from oracle import closed_form as cf  # noqa: E402
from oracle import fp8 as ofp8  # noqa: E402
from oracle.paged_attn import ref_paged_attn  # noqa: E402

pytestmark = pytest.mark.gpu

OUT_ATOL = OUT_RTOL = 2e-2
LSE_ATOL = 1e-3
GOLDEN = np.load(os.path.join(ROOT, "tests", "golden", "decode_golden.npz"))


def _dev(c, device):
    return {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}


def _lens_t(lens, device):
    return torch.as_tensor(list(lens), dtype=torch.int32, device=device)


def _check(out, lse, q, k, v, table, lens, scale, soft_cap=0.0, k_scale=None, v_scale=None, ref_kv=None, tag="",
           ref_tol=None):
    """Compare one result with both oracles (run on the tensors' own device).  ``ref_tol`` widens the comparison with
    the torch restatement only (it rounds its logits to 16 bits, so its own error grows with the logit scale)."""
    assert torch.isfinite(out.float()).all(), f"{tag}: non-finite out"
    assert torch.isfinite(lse).all(), f"{tag}: non-finite lse"
    rk, rv = ref_kv if ref_kv is not None else (k, v)
    ref = ref_paged_attn(q, rk, rv, lens, table, scale, soft_cap)
    torch.testing.assert_close(out.float(), ref.float(), atol=ref_tol or OUT_ATOL, rtol=ref_tol or OUT_RTOL,
                               msg=lambda m: f"{tag} vs torch ref: {m}")
    o64, l64 = cf.attn_fp64(q, rk, rv, table, lens, scale, soft_cap)
    # (P is rounded to the 16-bit dtype before the second product, as in the reference: with |v| ~ 3 a single
    # element can be off by 6e-3 from the exact answer)
    torch.testing.assert_close(out.double(), o64, atol=8e-3, rtol=1e-2, msg=lambda m: f"{tag} vs fp64: {m}")
    torch.testing.assert_close(lse.double(), l64, atol=LSE_ATOL, rtol=0, msg=lambda m: f"{tag} lse: {m}")


# ---- the reference's own test grid (test_decode_attn.py:123-162) ---------------------------------------------
@pytest.mark.parametrize("kv_lens", [[1320, 18, 463], [1, 54, 293, 70]])
@pytest.mark.parametrize("num_heads", [(16, 16), (32, 8), (64, 8), (6, 1)])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("soft_cap", [0, 30, 50])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_reference_grid(cuda_device, kv_lens, num_heads, block_size, dtype, soft_cap, algo):
    print(f"case lens={kv_lens} heads={num_heads} P={block_size} {dtype} cap={soft_cap} {algo}", flush=True)
    num_blocks = 1024
    g = torch.Generator(device="cpu").manual_seed(hash((tuple(kv_lens), num_heads, block_size, soft_cap)) & 0xFFFF)
    hq, hkv = num_heads
    d = 128
    scale = d ** -0.5
    q = torch.randn(len(kv_lens), hq, d, generator=g).to(dtype).to(cuda_device)
    kv = torch.randn(num_blocks + 1, 2, block_size, hkv, d, generator=g).to(dtype).to(cuda_device)
    k, v = kv[:, 0], kv[:, 1]                       # strided views: page stride is twice the page extent
    max_blocks = (max(kv_lens) + block_size - 1) // block_size
    table = torch.randint(0, num_blocks, (len(kv_lens), max_blocks), generator=g, dtype=torch.int32).to(cuda_device)
    lens_t = _lens_t(kv_lens, cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap), algo=algo)
    torch.cuda.synchronize()
    _check(out, lse, q, k, v, table, kv_lens, scale, float(soft_cap), tag="grid")
    if algo != tda.get_split_kv_plan(q, k, v, table, lens_t).algo:
        return                                      # the reference-named entry points use the default algorithm
    # the reference entry points: same numbers, reference layouts
    o2 = tda.gqa_fwd_batch_decode(q, k, v, None, [1] * len(kv_lens), lens_t, table, scale, float(soft_cap))
    packed = tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, [1] * len(kv_lens), lens_t, table, scale,
                                                 float(soft_cap), kv_split=32)
    torch.cuda.synchronize()
    assert torch.equal(o2, out)
    assert packed.shape == (len(kv_lens), hq, d + 1) and packed.dtype == dtype
    torch.testing.assert_close(packed[..., :d].float(), out.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(packed[..., d].float(), lse, atol=3e-2, rtol=1e-2)     # lse rounded to 16 bits


# ---- the reference's persistent entry point and its test grid (test_decode_attn.py:207-251, 254-296) --------------
@pytest.mark.parametrize("kv_lens", [[32], [1320], [18], [463], [1], [54], [293], [70], [1320, 18, 463, 1, 4000] * 8])
def test_persistent_entry_points(cuda_device, kv_lens):
    hq, hkv, d, block_size, dtype = 96, 12, 128, 1, torch.float16
    num_blocks = 8192
    g = torch.Generator().manual_seed(len(kv_lens) * 1000 + kv_lens[0])
    q = torch.randn(len(kv_lens), hq, d, generator=g).to(dtype).to(cuda_device)
    kv = torch.randn(num_blocks, 2, block_size, hkv, d, generator=g).to(dtype).to(cuda_device)
    k, v = kv[:, 0].contiguous(), kv[:, 1].contiguous()
    table = torch.randint(0, num_blocks, (len(kv_lens), max(kv_lens)), generator=g, dtype=torch.int32).to(cuda_device)
    lens_t = _lens_t(kv_lens, cuda_device)
    scale = d ** -0.5
    ws1 = torch.zeros([1], dtype=torch.int32, device=cuda_device)       # what the reference's test passes
    # any contents are fine for the reference's barrier (it only flips the top bit): the drop-in never uses it
    ws4 = torch.tensor([7, -3, 1 << 30, -(1 << 31)], dtype=torch.int32, device=cuda_device)
    out = tda.gqa_fwd_batch_decode_persistent(q, k, v, ws1, [1] * len(kv_lens), lens_t, table, scale, 0)
    out4 = tda.gqa_fwd_batch_decode_persistent(q, k, v, ws4, [1] * len(kv_lens), lens_t, table, scale, 0)
    out_aot = tda.gqa_fwd_batch_decode_persistent_aot(torch.cuda.current_stream(), q, k, v, ws1, [1] * len(kv_lens),
                                                      lens_t, table, scale, 0, kv_split=16)
    torch.cuda.synchronize()
    assert out.shape == (len(kv_lens), hq, d) and out.dtype == dtype
    ref = ref_paged_attn(q, k, v, kv_lens, table, scale, 0.0)
    for o in (out, out4, out_aot):
        torch.testing.assert_close(o.float(), ref.float(), atol=1e-2, rtol=1e-2)        # the reference test's bar
    assert torch.equal(out, out4) and int(ws1.abs().sum()) == 0
    assert ws4.tolist() == [7, -3, 1 << 30, -(1 << 31)]                 # left alone


def test_large_pool_index_arithmetic(cuda_device):
    # NUM_BLOCKS = 32000 "large enough to test overflow in index calculation" (test_decode_attn.py:120):
    # here the pool is made large enough that element offsets pass 2^31 and 2^32
    hq, hkv, d, page = 32, 8, 128, 16
    num_blocks = 140_000                       # 140000*16*8*128 = 2.29e9 elements (> 2^31), 4.6e9 bytes (> 2^32)
    g = torch.Generator(device=cuda_device).manual_seed(5)
    k = torch.randn(num_blocks, page, hkv, d, generator=g, device=cuda_device, dtype=torch.bfloat16)
    v = torch.randn(num_blocks, page, hkv, d, generator=g, device=cuda_device, dtype=torch.bfloat16)
    q = torch.randn(3, hq, d, generator=g, device=cuda_device, dtype=torch.bfloat16)
    lens = [700, 16, 1]
    table = torch.tensor([[num_blocks - 1 - 3 * i for i in range(44)],
                          [num_blocks - 2] * 44, [70_000] * 44], dtype=torch.int32, device=cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, _lens_t(lens, cuda_device), d ** -0.5)
    torch.cuda.synchronize()
    _check(out, lse, q, k, v, table, lens, d ** -0.5, tag="bigpool")


def test_unbuilt_head_dims_are_rejected(cuda_device):
    tbl = torch.zeros(1, 1, dtype=torch.int32, device=cuda_device)
    for d, algo in ((96, "auto"), (512, "auto"), (256, "valu"), (64, "valu")):
        q = torch.zeros(1, 8, d, dtype=torch.float16, device=cuda_device)
        k = torch.zeros(4, 16, 8, d, dtype=torch.float16, device=cuda_device)
        with pytest.raises(ValueError, match="head_dim"):
            tda.flash_decode(q, k, k, tbl, _lens_t([1], cuda_device), 1.0, algo=algo)


# ---- head sizes other than 128: 256 is in the reference's grid (test_decode_attn.py:125), 64 is built as well ----
@pytest.mark.parametrize("head_size", [64, 256])
@pytest.mark.parametrize("kv_lens", [[1320, 18, 463], [1, 54, 293, 70]])
@pytest.mark.parametrize("num_heads", [(16, 16), (32, 8), (64, 8), (6, 1)])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("soft_cap", [0, 50])
def test_reference_grid_other_head_sizes(cuda_device, head_size, kv_lens, num_heads, block_size, dtype, soft_cap):
    print(f"case D={head_size} lens={kv_lens} heads={num_heads} P={block_size} {dtype} cap={soft_cap}", flush=True)
    num_blocks = 512
    g = torch.Generator(device="cpu").manual_seed(hash((head_size, tuple(kv_lens), num_heads, block_size)) & 0xFFFF)
    hq, hkv = num_heads
    d = head_size
    scale = d ** -0.5
    q = torch.randn(len(kv_lens), hq, d, generator=g).to(dtype).to(cuda_device)
    kv = torch.randn(num_blocks + 1, 2, block_size, hkv, d, generator=g).to(dtype).to(cuda_device)
    k, v = kv[:, 0], kv[:, 1]
    max_blocks = (max(kv_lens) + block_size - 1) // block_size
    table = torch.randint(0, num_blocks, (len(kv_lens), max_blocks), generator=g, dtype=torch.int32).to(cuda_device)
    lens_t = _lens_t(kv_lens, cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap))
    out1, lse1 = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap), kv_split=1)
    out9, lse9 = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap), kv_split=9)
    packed = tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, [1] * len(kv_lens), lens_t, table, scale,
                                                 float(soft_cap), kv_split=32)
    torch.cuda.synchronize()
    for o, l, tag in ((out, lse, "auto"), (out1, lse1, "S=1"), (out9, lse9, "S=9")):
        _check(o, l, q, k, v, table, kv_lens, scale, float(soft_cap), tag=f"D={d} {tag}")
    assert packed.shape == (len(kv_lens), hq, d + 1) and packed.dtype == dtype
    torch.testing.assert_close(packed[..., :d].float(), out.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(packed[..., d].float(), lse, atol=3e-2, rtol=1e-2)


@pytest.mark.parametrize("head_size", [64, 256])
@pytest.mark.parametrize("page", [16, 4, 6, 64])
def test_other_head_sizes_fp8_pages_and_rank_merge(cuda_device, head_size, page):
    d = head_size
    cfg = wl.DecodeConfig("fp8_d", 57 + d + page, 5, 32, 8, d, page, kv_len_range=(1, 1500), kv_dtype="fp8_e4m3",
                          spare_pages=4)
    inp = wl.make_inputs(cfg, cuda_device, poison_tail=True)
    out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                k_scale=inp.k_scale, v_scale=inp.v_scale)
    torch.cuda.synchronize()
    kd = ofp8.dequant_per_head(inp.k_cache, inp.k_scale)
    vd = ofp8.dequant_per_head(inp.v_cache, inp.v_scale)
    _check(out, lse, inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens_host, inp.sm_scale,
           ref_kv=(kd, vd), tag=f"fp8 D={d} P={page}")
    # bf16 cache of the same shape, then the cross-rank merge of two copies of the result: merging a result
    # with itself leaves out unchanged and adds ln 2 to lse
    o2, l2 = tda.flash_decode(inp.q, kd, vd, inp.block_table, inp.kv_lens, inp.sm_scale)
    torch.cuda.synchronize()
    _check(o2, l2, inp.q, kd, vd, inp.block_table, inp.kv_lens_host, inp.sm_scale, tag=f"bf16 D={d} P={page}")
    both = torch.stack([tda.pack_out_lse(o2, l2, torch.float32)] * 2)
    gl = inp.kv_lens[None].repeat(2, 1)
    lse_m = torch.empty_like(l2)
    merged = tda.inter_rank_combine(both, gl, lse_out=lse_m)
    torch.cuda.synchronize()
    torch.testing.assert_close(merged.float(), o2.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse_m, l2 + math.log(2.0), atol=1e-4, rtol=0)


# ---- q / K rows of two segments and V rows of their own length: the reference's BLOCK_HEAD_DIM + BLOCK_DPE and V_DIM
# (flash_decode.py:103-109,187-191,210-214): 192 = 128 + 64 with V rows of 192 or 128, 576 = 512 + 64 with V rows of 512 ----
TWO_SEGMENT_DIMS = [(192, 192), (192, 128), (576, 512)]


def _two_segment_inputs(device, dims, lens, heads, page, dtype, seed, spare_pages=3, table_extra=0):
    """q [B,Hq,Dk], K pool [pages,P,Hkv,Dk], V pool [pages,P,Hkv,Dv], a table of distinct pages in random order (columns
    past a sequence's pages point at a page of NaN), lengths."""
    dk, dv = dims
    hq, hkv = heads
    g = torch.Generator(device="cpu").manual_seed(seed)
    per_seq = [(n + page - 1) // page for n in lens]
    width = max(max(per_seq), 1) + table_extra
    n_pages = sum(per_seq) + spare_pages + 1
    q = torch.randn(len(lens), hq, dk, generator=g).to(dtype).to(device)
    k = torch.randn(n_pages, page, hkv, dk, generator=g).to(dtype).to(device)
    v = torch.randn(n_pages, page, hkv, dv, generator=g).to(dtype).to(device)
    k[n_pages - 1] = float("nan")
    v[n_pages - 1] = float("nan")
    perm = torch.randperm(n_pages - 1, generator=g).to(torch.int32)
    table = torch.full((len(lens), width), n_pages - 1, dtype=torch.int32)
    at = 0
    for b, n in enumerate(per_seq):
        table[b, :n] = perm[at:at + n]
        at += n
    return q, k, v, table.to(device), _lens_t(lens, device)


@pytest.mark.parametrize("dims", TWO_SEGMENT_DIMS)
@pytest.mark.parametrize("kv_lens", [[1320, 18, 463], [1, 54, 293, 70]])
@pytest.mark.parametrize("num_heads", [(16, 16), (32, 8), (64, 8), (6, 1)])
@pytest.mark.parametrize("block_size", [1, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("soft_cap", [0, 50])
def test_reference_grid_two_segment_head_dims(cuda_device, dims, kv_lens, num_heads, block_size, dtype, soft_cap):
    print(f"case dims={dims} lens={kv_lens} heads={num_heads} P={block_size} {dtype} cap={soft_cap}", flush=True)
    dk, dv = dims
    num_blocks = 256
    g = torch.Generator(device="cpu").manual_seed(hash((dims, tuple(kv_lens), num_heads, block_size)) & 0xFFFF)
    hq, hkv = num_heads
    scale = dk ** -0.5
    q = torch.randn(len(kv_lens), hq, dk, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(num_blocks + 1, block_size, hkv, dk, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(num_blocks + 1, block_size, hkv, dv, generator=g).to(dtype).to(cuda_device)
    max_blocks = (max(kv_lens) + block_size - 1) // block_size
    table = torch.randint(0, num_blocks, (len(kv_lens), max_blocks), generator=g, dtype=torch.int32).to(cuda_device)
    lens_t = _lens_t(kv_lens, cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap))
    out1, lse1 = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap), kv_split=1)
    out9, lse9 = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=float(soft_cap), kv_split=9)
    o2 = tda.gqa_fwd_batch_decode(q, k, v, None, [1] * len(kv_lens), lens_t, table, scale, float(soft_cap))
    packed = tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, [1] * len(kv_lens), lens_t, table, scale,
                                                 float(soft_cap), kv_split=32)
    torch.cuda.synchronize()
    assert out.shape == (len(kv_lens), hq, dv) and out.dtype == dtype
    for o, l, tag in ((out, lse, "auto"), (out1, lse1, "S=1"), (out9, lse9, "S=9")):
        _check(o, l, q, k, v, table, kv_lens, scale, float(soft_cap), tag=f"dims={dims} {tag}")
    assert torch.equal(o2, out)
    assert packed.shape == (len(kv_lens), hq, dv + 1) and packed.dtype == dtype
    torch.testing.assert_close(packed[..., :dv].float(), out.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(packed[..., dv].float(), lse, atol=3e-2, rtol=1e-2)


@pytest.mark.parametrize("dims", TWO_SEGMENT_DIMS)
@pytest.mark.parametrize("page", [16, 64, 4, 6, 1])
def test_two_segment_head_dims_in_every_plan(cuda_device, dims, page):
    """Ragged batches through equal shares, own-length chunks, the work queue and a single pass; page sizes whose page
    numbers come one per tile (16, 64) and one per row (4, 6, 1); empty sequences; fp32 output; the rank merge."""
    dk, dv = dims
    scale = dk ** -0.5
    g = torch.Generator().manual_seed(dk + dv + page)
    lens = [int(x) for x in torch.randint(1, 3000, (12,), generator=g)]
    lens[3], lens[7] = 0, 1
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, dims, lens, (48, 2), page, torch.bfloat16, 77 + page, table_extra=2)   # two q-head tiles per kv head, the second half full
    ref_plan = tda.get_split_kv_plan(q, k, v, table, lens_t, scale)
    assert ref_plan.algo == "mfma"
    live = [i for i, n in enumerate(lens) if n > 0]

    def check(o, l, tag):
        assert torch.isfinite(o.float()).all() and float(o[3].abs().max()) == 0 and bool((l[3] == -math.inf).all()), tag
        _check(o[live], l[live], q[live], k, v, table[live], [lens[i] for i in live], scale, tag=f"dims={dims} P={page} {tag}")

    out_b, lse_b = tda.flash_decode(q, k, v, table, lens_t, scale, force_balanced=True)
    plan_b = tda.get_split_kv_plan(q, k, v, table, lens_t, scale, force_balanced=True)
    assert plan_b.balanced
    out_c, lse_c = tda.flash_decode(q, k, v, table, lens_t, scale, kv_split=5)
    out_q, lse_q = tda.flash_decode(q, k, v, table, lens_t, scale, kv_split=48)      # 12 x 48 pieces: more than are resident, a queue
    out_f = torch.empty(len(lens), 48, dv, dtype=torch.float32, device=cuda_device)
    _, lse_f = tda.flash_decode(q, k, v, table, lens_t, scale, out=out_f)
    torch.cuda.synchronize()
    check(out_b, lse_b, "equal shares")
    check(out_c, lse_c, "5 chunks")
    check(out_q, lse_q, "work queue")
    check(out_f, lse_f, "fp32 out")
    torch.testing.assert_close(out_f, out_b.float(), atol=1e-2, rtol=1e-2)
    # a batch that fills the GPU by itself: whole sequences per workgroup, in blocks of kv heads (one head per workgroup
    # where a token's K and V rows hold more than 512 values: the kernels whose wavefronts share the staged tiles)
    lens2 = [int(x) for x in torch.randint(40, 160, (130,), generator=g)]
    q2, k2, v2, table2, lens2_t = _two_segment_inputs(cuda_device, dims, lens2, (16, 8), page, torch.float16, 99 + page)
    plan2 = tda.get_split_kv_plan(q2, k2, v2, table2, lens2_t, scale, max_kv_len=max(lens2), min_kv_len=max(lens2))
    assert plan2.num_splits == 1 and plan2.kv_heads_per_wg == (1 if dk + dv > 512 else 4), plan2
    o2, l2 = tda.flash_decode(q2, k2, v2, table2, lens2_t, scale, max_kv_len=max(lens2), min_kv_len=max(lens2))
    torch.cuda.synchronize()
    _check(o2, l2, q2, k2, v2, table2, lens2, scale, tag=f"dims={dims} P={page} single pass")
    # the cross-rank merge on rows of dv values: a result merged with itself is itself, lse + ln 2
    both = torch.stack([tda.pack_out_lse(o2, l2, torch.float32)] * 2)
    lse_m = torch.empty_like(l2)
    merged = tda.inter_rank_combine(both, lens2_t[None].repeat(2, 1), lse_out=lse_m)
    torch.cuda.synchronize()
    torch.testing.assert_close(merged.float(), o2.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse_m, l2 + math.log(2.0), atol=1e-4, rtol=0)


@pytest.mark.parametrize("seed", list(range(30)))
def test_two_segment_head_dims_random_shapes(cuda_device, seed):
    g = torch.Generator().manual_seed(4000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    dims = TWO_SEGMENT_DIMS[seed % 3]
    hkv = [1, 2, 3, 4, 8][r(0, 4)]
    group = [1, 2, 4, 7, 8, 16, 20, 40, 64, 100, 128][r(0, 10)]
    page = [1, 2, 5, 8, 16, 32, 48, 128][r(0, 7)]
    batch = r(1, 20)
    top = [60, 700, 5000][r(0, 2)]
    lens = [r(0 if batch > 1 else 1, top) for _ in range(batch)]
    if max(lens) == 0:
        lens[0] = 17
    dtype = [torch.bfloat16, torch.float16][r(0, 1)]
    cap = [0.0, 20.0][r(0, 1)]
    split = [-1, -1, 1, 2, 7, 33][r(0, 5)]
    hints = r(0, 1)
    print(f"case seed={seed} dims={dims} heads=({hkv * group},{hkv}) P={page} B={batch} top={top} {dtype} cap={cap} "
          f"split={split} hints={hints}", flush=True)
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, dims, lens, (hkv * group, hkv), page, dtype, 5000 + seed,
                                                 table_extra=r(0, 3))
    scale = dims[0] ** -0.5 * [1.0, 0.5, 2.0][r(0, 2)]
    kw = dict(max_kv_len=max(lens), min_kv_len=min(lens)) if hints else {}
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, kv_split=split, **kw)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    for i, n in enumerate(lens):
        if n == 0:
            assert float(out[i].abs().max()) == 0 and bool((lse[i] == -math.inf).all())
    _check(out[live], lse[live], q[live], k, v, table[live], [lens[i] for i in live], scale, cap, tag=f"seed {seed}",
           ref_tol=4e-2 if scale > dims[0] ** -0.5 else None)


@pytest.mark.parametrize("dims,heads,fp8", [(d, (32, 2), False) for d in TWO_SEGMENT_DIMS] + [((576, 512), (128, 1), False),
                                                     ((192, 192), (24, 3), True), ((576, 512), (128, 1), True)])
def test_two_segment_head_dims_under_graph_capture_and_through_the_static_entry(cuda_device, dims, heads, fp8):
    """A captured call (the kernels of the widest rows ask for more LDS than the default limit at launch; 128 q heads on one
    kv head: the kernels whose wavefronts share the staged tiles) replayed on changed q and lengths, and the entry point
    that allocates nothing, against the eager call.  16-bit and e4m3 caches."""
    dk, dv = dims
    g = torch.Generator().manual_seed(dk * 3 + dv)
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, dims, [2500] * 4, heads, 16, torch.bfloat16, 31)   # pages for every length below
    ref_kv, kw8 = None, {}
    if fp8:
        k, ks, v, vs, kd, vd = _quantized_two_segment(k, v, torch.bfloat16)
        ref_kv, kw8 = (kd, vd), dict(k_scale=ks, v_scale=vs)
    lens_t.copy_(_lens_t([2500, 1, 900, 1800], cuda_device))
    scale = dk ** -0.5
    call = tda.prepare_decode(q, k, v, table, lens_t, scale, max_kv_len=2500, **kw8)
    assert call.plan.num_splits > 1
    call.run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call.run()
    for i, new_lens in enumerate(([2500, 1, 900, 1800], [7, 2400, 0, 333], [1200, 1200, 1200, 1200])):
        lens_t.copy_(_lens_t(new_lens, cuda_device))
        q.copy_(torch.randn(q.shape, generator=g).to(torch.bfloat16).to(cuda_device))
        call.out.fill_(float("nan"))
        call.lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_l = call.out.clone(), call.lse.clone()
        want_o, want_l = tda.flash_decode(q, k, v, table, lens_t, scale, max_kv_len=2500, **kw8)
        static = tda.prepare_decode(q, k, v, table, lens_t, scale, max_kv_len=2500, static_scratch=True, **kw8)
        if call.plan.workspace_bytes <= 32 << 20:
            st_o, st_l = static.run_static()
        else:                                   # (128 q heads x 32 splits x 512 values: beyond the 32 MiB the library holds)
            with pytest.raises(Exception, match="static scratch"):
                static.run_static()
            st_o, st_l = want_o, want_l
        torch.cuda.synchronize()
        assert torch.equal(got_o, want_o) and torch.equal(got_l, want_l), f"replay {i}"
        assert torch.equal(st_o, want_o) and torch.equal(st_l, want_l), f"static entry {i}"
        live = [j for j, n in enumerate(new_lens) if n > 0]
        _check(got_o[live], got_l[live], q[live], k, v, table[live], [new_lens[j] for j in live], scale, ref_kv=ref_kv,
               tag=f"dims={dims} fp8={fp8} graph replay {i}")


@pytest.mark.parametrize("heads", [(128, 1), (128, 2), (64, 1), (40, 1), (66, 2)])
@pytest.mark.parametrize("page", [64, 16, 6, 1])
def test_large_groups_on_one_kv_head_share_the_staged_tiles(cuda_device, heads, page):
    """More than 32 q heads per kv head with rows of 576 / 512 values (latent attention): the workgroups cover 64 q heads
    of a kv head and their wavefronts share every staged tile.  Every way of handing out the pieces, groups that fill
    the last workgroup or wavefront only partly, empty sequences, fp16, a soft cap."""
    dims = (576, 512)
    hq, hkv = heads
    scale = 576 ** -0.5
    g = torch.Generator().manual_seed(hq * 7 + hkv + page)
    lens = [int(x) for x in torch.randint(1, 2200, (7,), generator=g)]
    lens[2], lens[5] = 0, 1
    dtype = torch.float16 if page == 16 else torch.bfloat16
    cap = 25.0 if page == 6 else 0.0
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, dims, lens, heads, page, dtype, 300 + hq + page, table_extra=1)
    live = [i for i, n in enumerate(lens) if n > 0]

    def check(o, l, tag):
        assert o.shape == (len(lens), hq, 512)
        assert torch.isfinite(o.float()).all() and float(o[2].abs().max()) == 0 and bool((l[2] == -math.inf).all()), tag
        _check(o[live], l[live], q[live], k, v, table[live], [lens[i] for i in live], scale, cap, tag=f"heads={heads} P={page} {tag}")

    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, scale)
    assert plan.algo == "mfma" and plan.kv_heads_per_wg == 1
    out_a, lse_a = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap)
    out_1, lse_1 = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, kv_split=1)
    out_c, lse_c = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, kv_split=5)
    out_q, lse_q = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, kv_split=40)       # a work queue
    out_b, lse_b = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, force_balanced=True)
    assert tda.get_split_kv_plan(q, k, v, table, lens_t, scale, force_balanced=True).balanced
    out_h, lse_h = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, max_kv_len=max(lens), min_kv_len=max(lens))
    packed = tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, None, lens_t, table, scale, cap, kv_split=32)
    torch.cuda.synchronize()
    for o, l, tag in ((out_a, lse_a, "auto"), (out_1, lse_1, "single pass"), (out_c, lse_c, "5 chunks"), (out_q, lse_q, "queue"),
                      (out_b, lse_b, "equal shares"), (out_h, lse_h, "alike lengths")):
        check(o, l, tag)
    torch.testing.assert_close(packed[..., :512].float(), out_a.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(packed[live][..., 512].float(), lse_a[live], atol=3e-2, rtol=1e-2)


@pytest.mark.parametrize("heads", [(64, 1), (128, 2), (40, 1), (71, 1), (51, 3)])
@pytest.mark.parametrize("page", [16, 1, 6])
def test_large_groups_at_head_dim_128(cuda_device, heads, page):
    """More than 16 q heads per kv head with rows of 128 values (multi-query attention): the q-head tiles of a kv head run
    on one XCD and load with plain loads.  Every way of handing out the pieces, empty sequences, fp16, a soft cap, an
    e4m3 cache, the single-launch form (which stays with the other kernels)."""
    hq, hkv = heads
    scale = 128 ** -0.5
    g = torch.Generator().manual_seed(hq * 5 + hkv + page)
    lens = [int(x) for x in torch.randint(1, 2500, (6,), generator=g)]
    lens[1], lens[4] = 0, 1
    dtype = torch.float16 if page == 1 else torch.bfloat16
    cap = 30.0 if page == 6 else 0.0
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, (128, 128), lens, heads, page, dtype, 700 + hq + page, table_extra=1)
    live = [i for i, n in enumerate(lens) if n > 0]

    def check(o, l, tag, **kw):
        assert o.shape == (len(lens), hq, 128)
        assert torch.isfinite(o.float()).all() and float(o[1].abs().max()) == 0 and bool((l[1] == -math.inf).all()), tag
        _check(o[live], l[live], q[live], k, v, table[live], [lens[i] for i in live], scale, cap, tag=f"heads={heads} P={page} {tag}", **kw)

    for tag, kw in (("auto", {}), ("single pass", dict(kv_split=1)), ("5 chunks", dict(kv_split=5)), ("queue", dict(kv_split=40)),
                    ("equal shares", dict(force_balanced=True)), ("alike lengths", dict(max_kv_len=max(lens), min_kv_len=max(lens)))):
        o, l = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, **kw)
        torch.cuda.synchronize()
        check(o, l, tag)
    call = tda.prepare_decode(q, k, v, table, lens_t, scale, soft_cap=cap, kv_split=4, single_launch=True)
    call.run()
    torch.cuda.synchronize()
    check(call.out, call.lse, "single launch")
    k8, ks, v8, vs, kd, vd = _quantized_two_segment(k, v, dtype)
    for tag, kw in (("fp8 auto", {}), ("fp8 equal shares", dict(force_balanced=True)), ("fp8 3 chunks", dict(kv_split=3))):
        o, l = tda.flash_decode(q, k8, v8, table, lens_t, scale, soft_cap=cap, k_scale=ks, v_scale=vs, **kw)
        torch.cuda.synchronize()
        assert float(o[1].abs().max()) == 0 and bool((l[1] == -math.inf).all()), tag
        _check(o[live], l[live], q[live], k8, v8, table[live], [lens[i] for i in live], scale, cap, ref_kv=(kd, vd),
               tag=f"heads={heads} P={page} {tag}")


def _quantized_two_segment(k16, v16, dtype):
    """e4m3 caches with per-kv-head scales from the 16-bit caches of _two_segment_inputs (whose last page holds NaN for
    the unused table columns), and what they dequantise to in ``dtype``."""
    k16[-1], v16[-1] = 0, 0                          # (the page of NaN does not quantise)
    k8, ks = wl.quantize_kv_fp8(k16)
    v8, vs = wl.quantize_kv_fp8(v16)
    k8.view(torch.uint8)[-1] = 0x7F                  # unused table columns still point at NaN (0x7F in e4m3)
    v8.view(torch.uint8)[-1] = 0x7F
    return k8, ks, v8, vs, ofp8.dequant_per_head(k8, ks, dtype), ofp8.dequant_per_head(v8, vs, dtype)


@pytest.mark.parametrize("seed", list(range(24)))
def test_two_segment_head_dims_random_shapes_with_an_fp8_cache(cuda_device, seed):
    g = torch.Generator().manual_seed(7000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    dims = TWO_SEGMENT_DIMS[seed % 3]
    hkv = [1, 2, 3, 4, 8][r(0, 4)]
    group = [1, 2, 4, 7, 8, 16, 20, 40, 64, 100, 128][r(0, 10)]
    page = [1, 2, 5, 8, 16, 32, 48, 128][r(0, 7)]
    batch = r(1, 16)
    top = [60, 700, 4000][r(0, 2)]
    lens = [r(0 if batch > 1 else 1, top) for _ in range(batch)]
    if max(lens) == 0:
        lens[0] = 17
    dtype = [torch.bfloat16, torch.float16][r(0, 1)]
    cap = [0.0, 20.0][r(0, 1)]
    split = [-1, -1, 1, 2, 7, 33][r(0, 5)]
    hints = r(0, 1)
    print(f"case fp8 seed={seed} dims={dims} heads=({hkv * group},{hkv}) P={page} B={batch} top={top} {dtype} cap={cap} "
          f"split={split} hints={hints}", flush=True)
    q, k16, v16, table, lens_t = _two_segment_inputs(cuda_device, dims, lens, (hkv * group, hkv), page, dtype, 8000 + seed,
                                                     table_extra=r(0, 3))
    k8, ks, v8, vs, kd, vd = _quantized_two_segment(k16, v16, dtype)
    scale = dims[0] ** -0.5
    kw = dict(max_kv_len=max(lens), min_kv_len=min(lens)) if hints else {}
    out, lse = tda.flash_decode(q, k8, v8, table, lens_t, scale, soft_cap=cap, kv_split=split, k_scale=ks, v_scale=vs, **kw)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    for i, n in enumerate(lens):
        if n == 0:
            assert float(out[i].abs().max()) == 0 and bool((lse[i] == -math.inf).all())
    _check(out[live], lse[live], q[live], k8, v8, table[live], [lens[i] for i in live], scale, cap, ref_kv=(kd, vd),
           tag=f"fp8 seed {seed}")


@pytest.mark.parametrize("dims", TWO_SEGMENT_DIMS)
@pytest.mark.parametrize("heads,page", [((32, 8), 16), ((16, 2), 4), ((40, 1), 64), ((128, 1), 16), ((66, 2), 6), ((128, 2), 1)])
def test_two_segment_head_dims_with_an_fp8_cache(cuda_device, dims, heads, page):
    """e4m3 caches with per-kv-head scales behind rows of two segments: exact dequantisation (the decode over the
    dequantised cache) and the K scale folded into the logit scale, through a single pass, chunks, a work queue and equal
    shares; groups of more than 16 q heads on rows of 576 / 512 values run in the kernels that share the staged tiles.
    fp16 queries at page size 6."""
    dk, dv = dims
    hq, hkv = heads
    g = torch.Generator().manual_seed(dk + hq + page)
    lens = [int(x) for x in torch.randint(1, 1800, (5,), generator=g)]
    lens[1] = 0
    dtype = torch.float16 if page == 6 else torch.bfloat16
    q, k16, v16, table, lens_t = _two_segment_inputs(cuda_device, dims, lens, heads, page, dtype, 900 + hq + page)
    k8, ks, v8, vs, kd, vd = _quantized_two_segment(k16, v16, dtype)
    scale = dk ** -0.5
    live = [i for i, n in enumerate(lens) if n > 0]
    plan = tda.get_split_kv_plan(q, k8, v8, table, lens_t, scale)
    assert plan.algo == "mfma"
    for tag, kw in (("auto", {}), ("single pass", dict(kv_split=1)), ("3 chunks", dict(kv_split=3)), ("queue", dict(kv_split=40)),
                    ("equal shares", dict(force_balanced=True)), ("folded", dict(fp8_fold_k_scale=True))):
        out, lse = tda.flash_decode(q, k8, v8, table, lens_t, scale, k_scale=ks, v_scale=vs, **kw)
        torch.cuda.synchronize()
        assert out.shape == (len(lens), hq, dv)
        assert float(out[1].abs().max()) == 0 and bool((lse[1] == -math.inf).all()), tag
        name = f"fp8 dims={dims} heads={heads} P={page} {tag}"
        ll = [lens[i] for i in live]
        if tag != "folded":
            _check(out[live], lse[live], q[live], k8, v8, table[live], ll, scale, ref_kv=(kd, vd), tag=name)
            continue
        # the folded form evaluates the cache exactly: the standard bars hold against k8 * k_scale without the 16-bit
        # rounding of K, and lse is within 5e-3 of the dequantise-then-decode definition (as for one-segment rows)
        assert torch.isfinite(out.float()).all() and torch.isfinite(lse[live]).all(), name
        o64, l64 = cf.attn_fp64(q[live], k8.float(), v8.float(), table[live], ll, scale, k_scale=ks, v_scale=vs)
        _, l_deq = cf.attn_fp64(q[live], kd, vd, table[live], ll, scale)
        torch.testing.assert_close(out[live].float(), ref_paged_attn(q[live], kd, vd, ll, table[live], scale).float(),
                                   atol=OUT_ATOL, rtol=OUT_RTOL, msg=lambda m: f"{name} vs torch ref: {m}")
        torch.testing.assert_close(out[live].double(), o64, atol=8e-3, rtol=1e-2, msg=lambda m: f"{name} vs exact cache: {m}")
        torch.testing.assert_close(lse[live].double(), l64, atol=LSE_ATOL, rtol=0, msg=lambda m: f"{name} lse vs exact cache: {m}")
        torch.testing.assert_close(lse[live].double(), l_deq, atol=5e-3, rtol=0, msg=lambda m: f"{name} lse vs dequantised: {m}")


def test_what_is_not_built_for_two_segment_head_dims_is_refused(cuda_device):
    q, k, v, table, lens_t = _two_segment_inputs(cuda_device, (192, 128), [300, 20], (8, 2), 16, torch.bfloat16, 5)
    with pytest.raises(ValueError, match="matrix-core"):
        tda.flash_decode(q, k, v, table, lens_t, 1.0, algo="valu")
    with pytest.raises(ValueError, match="single-launch"):
        tda.prepare_decode(q, k, v, table, lens_t, 1.0, kv_split=4, single_launch=True).run()
    for dk, dv in ((192, 64), (128, 64), (576, 576), (256, 128)):
        qq = torch.zeros(2, 8, dk, dtype=torch.bfloat16, device=cuda_device)
        kk = torch.zeros(8, 16, 2, dk, dtype=torch.bfloat16, device=cuda_device)
        vv = torch.zeros(8, 16, 2, dv, dtype=torch.bfloat16, device=cuda_device)
        with pytest.raises(ValueError, match="head_dim"):
            tda.flash_decode(qq, kk, vv, table[:, :1], lens_t, 1.0)


# ---- golden vectors and edge cases -----------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["tiny", *EDGE_CASES])
@pytest.mark.parametrize("kv_split", [-1, 1, 3, 32])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_golden_cases(cuda_device, name, kv_split, algo):
    print(f"case golden {name} kv_split={kv_split} {algo}", flush=True)
    c = _dev(dict(all_cases())[name], cuda_device)
    lens_t = _lens_t(c["kv_lens"], cuda_device)
    out, lse = tda.flash_decode(c["q"], c["k_cache"], c["v_cache"], c["block_table"], lens_t, c["sm_scale"],
                                soft_cap=c["soft_cap"], kv_split=kv_split, algo=algo)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    np.testing.assert_allclose(out.float().cpu().numpy(), GOLDEN[name + ".ref"], atol=OUT_ATOL, rtol=OUT_RTOL)
    np.testing.assert_allclose(out.float().cpu().numpy(), GOLDEN[name + ".out64"], atol=5e-3, rtol=1e-2)
    np.testing.assert_allclose(lse.cpu().numpy(), GOLDEN[name + ".lse64"], atol=LSE_ATOL, rtol=0)


@pytest.mark.parametrize("page", [1, 16])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_single_token_sequences_are_bit_exact_gathers(cuda_device, page, algo):
    g = torch.Generator().manual_seed(31)
    b, hq, hkv, d, pool = 7, 8, 2, 128, 50
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.randint(0, pool, (b, 3), generator=g, dtype=torch.int32).to(cuda_device)
    table[:, 1:] = 2**31 - 1                                       # never read
    out, lse = tda.flash_decode(q, k, v, table, _lens_t([1] * b, cuda_device), d ** -0.5, algo=algo)
    torch.cuda.synchronize()
    for i in range(b):
        for h in range(hq):
            assert torch.equal(out[i, h], v[table[i, 0].item(), 0, h // 4]), (i, h)   # softmax of one logit == 1
            want = d ** -0.5 * float(torch.dot(q[i, h].double(), k[table[i, 0].item(), 0, h // 4].double()))
            assert abs(float(lse[i, h]) - want) < 1e-4


def test_zero_query_gives_mean_and_log_n(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=9, kv_len_range=(1, 3000)), cuda_device,
                         poison_tail=True)
    q = torch.zeros_like(inp.q)
    out, lse = tda.flash_decode(q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    torch.cuda.synchronize()
    for b, n in enumerate(inp.kv_lens_host):
        rows = cf.gather_kv(inp.v_cache, inp.block_table[b].cpu(), n).double()
        torch.testing.assert_close(out[b].double(), rows[:, 0].mean(0).expand(8, -1), atol=2e-3, rtol=1e-2)
        assert abs(float(lse[b, 0]) - math.log(n)) < 1e-4


def test_rows_that_encode_their_slot_catch_a_wrong_gather(cuda_device):
    # one sequence, V row r of the pool = r (spread over columns so that bf16 holds it exactly), K = 0:
    # the output must be the exact mean of the slots named by block_table
    page, hkv, d, pool = 16, 2, 128, 64
    v = torch.zeros(pool, page, hkv, d)
    idx = torch.arange(pool * page).view(pool, page)
    v[:, :, 0, 0] = (idx % 256).float()
    v[:, :, 0, 1] = (idx // 256).float()
    v[:, :, 1, 2] = (idx % 256).float()
    v[:, :, 1, 3] = (idx // 256).float()
    v = v.to(torch.bfloat16).to(cuda_device)
    k = torch.zeros_like(v)
    q = torch.randn(1, 4, d).to(torch.bfloat16).to(cuda_device)
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(1)).to(torch.int32)
    n = 37 * page + 5
    table = perm[None, :40].contiguous().to(cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, _lens_t([n], cuda_device), 1.0, out=torch.empty(1, 4, d, device=cuda_device))
    torch.cuda.synchronize()
    slots = torch.cat([perm[i].item() * page + torch.arange(page) for i in range(38)])[:n].double()
    lo, hi = (slots % 256).mean().item(), (slots // 256).float().mean().item()
    got = out[0].double().cpu()
    for h, (c0, c1) in enumerate([(0, 1), (0, 1), (2, 3), (2, 3)]):
        assert abs(got[h, c0].item() - lo) < 0.5 and abs(got[h, c1].item() - hi) < 0.01, (h, got[h, :4], lo, hi)
    assert abs(float(lse[0, 0]) - math.log(n)) < 1e-4


def test_permuting_pool_pages_with_the_table_changes_nothing(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=3, kv_len=1000), cuda_device)
    out0, lse0 = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    pool = inp.k_cache.shape[0]
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(9)).to(cuda_device)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(pool, device=cuda_device)
    k2, v2 = inp.k_cache[perm], inp.v_cache[perm]                 # new page i holds old page perm[i]
    table2 = inv[inp.block_table.long()].to(torch.int32)
    out1, lse1 = tda.flash_decode(inp.q, k2, v2, table2, inp.kv_lens, inp.sm_scale)
    torch.cuda.synchronize()
    assert torch.equal(out0, out1) and torch.equal(lse0, lse1)


def test_poisoned_table_tail_is_never_read(cuda_device):
    cfg = wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=12, kv_len_range=(1, 700))
    a = wl.make_inputs(cfg, cuda_device, poison_tail=False)
    b = wl.make_inputs(cfg, cuda_device, poison_tail=True)
    assert not torch.equal(a.block_table, b.block_table)
    oa, la = tda.flash_decode(a.q, a.k_cache, a.v_cache, a.block_table, a.kv_lens, a.sm_scale)
    ob, lb = tda.flash_decode(b.q, b.k_cache, b.v_cache, b.block_table, b.kv_lens, b.sm_scale)
    torch.cuda.synchronize()
    assert torch.equal(oa, ob) and torch.equal(la, lb)


@pytest.mark.parametrize("kv_split", [32, 64])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_short_sequences_and_empty_splits_stay_finite(cuda_device, kv_split, algo):
    lens = [1, 2, kv_split - 1, kv_split, kv_split + 1, 63, 64, 65, 255, 256, 257]
    g = torch.Generator().manual_seed(77)
    hq, hkv, d, page = 8, 2, 128, 16
    pool = 200
    q = torch.randn(len(lens), hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    # unused slots of live pages hold NaN: masked rows must not leak into the result
    table = torch.randperm(pool, generator=g)[:len(lens) * 17].view(len(lens), 17).to(torch.int32).to(cuda_device)
    for i, n in enumerate(lens):
        last = table[i, (n - 1) // page].item()
        if n % page:
            k[last, n % page:] = float("nan")
            v[last, n % page:] = float("nan")
    # force real splitting of short sequences: pretend the host bound is the table width
    out, lse = tda.flash_decode(q, k, v, table, _lens_t(lens, cuda_device), d ** -0.5, kv_split=kv_split, algo=algo)
    torch.cuda.synchronize()
    kc, vc = torch.nan_to_num(k), torch.nan_to_num(v)
    _check(out, lse, q, kc, vc, table, lens, d ** -0.5, tag=f"short S={kv_split}")


def test_split_invariance(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=5, kv_len_range=(1, 9000)), cuda_device)
    res = {}
    for s in (1, 2, 3, 32, 64):
        o = torch.empty(inp.q.shape, dtype=torch.float32, device=cuda_device)
        res[s] = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                  kv_split=s, out=o)
    torch.cuda.synchronize()
    for s in (2, 3, 32, 64):
        torch.testing.assert_close(res[s][0], res[1][0], atol=1e-3, rtol=5e-3)
        torch.testing.assert_close(res[s][1], res[1][1], atol=2e-5, rtol=0)


@pytest.mark.parametrize("algo", ["valu", "mfma"])
@pytest.mark.parametrize("kv_split", [-1, 1, 4])
def test_a_length_hint_that_is_too_small_loses_no_tokens(cuda_device, algo, kv_split):
    # max_kv_len only sizes the plan: the last split runs to the end of each sequence
    g = torch.Generator().manual_seed(91)
    lens, hq, hkv, d, page = [1000, 37, 2500, 640], 32, 8, 128, 16
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages)
    q = torch.randn(4, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.zeros((4, max(pages)), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, _lens_t(lens, cuda_device), d ** -0.5, max_kv_len=600, kv_split=kv_split,
                                algo=algo)
    torch.cuda.synchronize()
    _check(out, lse, q, k, v, table, lens, d ** -0.5, tag=f"small hint {algo} S={kv_split}")


@pytest.mark.parametrize("true_lens", [[24000] * 4, [24000, 23990, 24000, 23900], [24000, 37, 1, 9000]])
def test_the_lower_length_hint_selects_chunks_and_never_changes_results(cuda_device, true_lens):
    # min_kv_len close to max_kv_len: per-sequence chunks instead of balanced shares.  The hint may be wrong (third
    # case: the batch is ragged although the caller claims uniform lengths) - the result is the same, only slower.
    g = torch.Generator().manual_seed(93)
    hq, hkv, d, page = 32, 8, 128, 16
    pages = [(24000 + page - 1) // page] * 4
    pool = sum(pages)
    q = torch.randn(4, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.randperm(pool, generator=g).to(torch.int32).view(4, pages[0]).to(cuda_device)
    lens_t = _lens_t(true_lens, cuda_device)
    args = (q, k, v, table, lens_t, d ** -0.5)
    p_bal = tda.get_split_kv_plan(*args, max_kv_len=24000)
    p_uni = tda.get_split_kv_plan(*args, max_kv_len=24000, min_kv_len=24000)
    p_near = tda.get_split_kv_plan(*args, max_kv_len=24000, min_kv_len=23900)
    p_far = tda.get_split_kv_plan(*args, max_kv_len=24000, min_kv_len=20000)
    assert p_bal.balanced and p_far.balanced and not p_uni.balanced and not p_near.balanced
    assert p_uni.num_splits == 256 // (4 * 8 // p_uni.kv_heads_per_wg)          # one workgroup per compute unit
    out_b, lse_b = tda.flash_decode(*args, max_kv_len=24000)
    out_u, lse_u = tda.flash_decode(*args, max_kv_len=24000, min_kv_len=24000)
    torch.cuda.synchronize()
    _check(out_u, lse_u, q, k, v, table, true_lens, d ** -0.5, tag=f"uniform hint {true_lens}")
    torch.testing.assert_close(out_u.float(), out_b.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse_u, lse_b, atol=1e-4, rtol=1e-5)
    with pytest.raises(ValueError, match="min_kv_len"):
        tda.flash_decode(*args, max_kv_len=24000, min_kv_len=24001)


@pytest.mark.parametrize("page", [1, 16, 64])
def test_chunks_follow_each_sequences_own_length_when_the_host_gives_no_bounds(cuda_device, page):
    # No length bounds at all: the plan is sized for the table's capacity and the chunks are cut on the GPU from
    # kv_lens, as the reference cuts them (flash_decode.py:151-153).  Every row the combine merges must have been
    # written by this call: the workspace starts out as NaN.
    g = torch.Generator().manual_seed(97 + page)
    hq, hkv, d, cap = 32, 8, 128, 16384
    pages = cap // page
    q = torch.randn(1, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pages, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pages, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.randperm(pages, generator=g).to(torch.int32).view(1, pages).to(cuda_device)
    plan = tda.get_split_kv_plan(q, k, v, table, _lens_t([cap], cuda_device), d ** -0.5)
    assert not plan.balanced and plan.num_splits == 64 and plan.chunk_floor == 64 and plan.chunk_tokens == 256
    assert tda.get_split_kv_plan(q, k, v, table, _lens_t([cap], cuda_device), d ** -0.5, max_kv_len=cap,
                                 min_kv_len=cap).chunk_floor == 0        # lengths the host vouches for: fixed chunks
    assert tda.get_split_kv_plan(q, k, v, table, _lens_t([cap], cuda_device), d ** -0.5, kv_split=8).chunk_floor == 64
    ws = torch.empty(plan.workspace_bytes // 4, dtype=torch.float32, device=cuda_device)
    ws32 = torch.empty_like(ws)
    for n in (0, 1, 15, 16, 63, 64, 65, 1000, 64 * 64 - 1, 64 * 64, 64 * 64 + 1, 5000, 16383, cap, cap + 100):
        print(f"page {page} kv_len {n}", flush=True)
        ws.fill_(float("nan"))
        lens = _lens_t([n], cuda_device)
        out, lse = tda.flash_decode(q, k, v, table, lens, d ** -0.5, workspace=ws)
        out1, lse1 = tda.flash_decode(q, k, v, table, lens, d ** -0.5, kv_split=1)
        ws32.fill_(float("nan"))
        out32, lse32 = tda.flash_decode(q, k, v, table, lens, d ** -0.5, kv_split=32, workspace=ws32)   # the reference's count
        torch.cuda.synchronize()
        if n == 0:
            assert torch.all(out == 0) and torch.all(torch.isneginf(lse))
            assert torch.all(out32 == 0) and torch.all(torch.isneginf(lse32))
            continue
        torch.testing.assert_close(out32.float(), out1.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(lse32, lse1, atol=1e-4, rtol=1e-5)
        _check(out, lse, q, k, v, table, [min(n, cap)], d ** -0.5, tag=f"own-length chunks P={page} n={n}")
        torch.testing.assert_close(out.float(), out1.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(lse, lse1, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("single_launch", [False, True])
def test_own_length_chunks_of_a_short_ragged_batch_and_a_bound_that_is_too_small(cuda_device, single_launch):
    # batches whose shares would be too short for balanced mode are cut per sequence as well; a max_kv_len below
    # the real lengths caps the chunk, and the last split then runs to the end of its sequence
    g = torch.Generator().manual_seed(101)
    lens, hq, hkv, d, page = [1500, 0, 33, 700, 1], 16, 4, 128, 16
    cap_pages = 96
    pool = len(lens) * cap_pages
    q = torch.randn(len(lens), hq, d, generator=g).to(torch.float16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    table = torch.randperm(pool, generator=g).to(torch.int32).view(len(lens), cap_pages).to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    for hint in (None, 400):
        plan = tda.get_split_kv_plan(q, k, v, table, lens_t, d ** -0.5, max_kv_len=hint)
        assert not plan.balanced and plan.num_splits > 1 and plan.chunk_floor == 64
        call = tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, max_kv_len=hint, single_launch=single_launch)
        call.run()
        torch.cuda.synchronize()
        assert torch.all(call.out[1] == 0) and torch.all(torch.isneginf(call.lse[1]))
        keep = [0, 2, 3, 4]
        _check(call.out[keep], call.lse[keep], q[keep], k, v, table[keep], [lens[i] for i in keep], d ** -0.5,
               tag=f"ragged own-length chunks hint={hint} single_launch={single_launch}")


def test_length_feedback_reports_the_bounds_of_kv_lens_in_every_plan(cuda_device):
    # the last kernel of a call leaves {min, max of the clamped kv_lens, call count, batch} where the host can read it
    g = torch.Generator().manual_seed(103)
    hq, hkv, d, page, cap_pages = 32, 8, 128, 16, 160
    fb = tda.LengthFeedback()
    assert fb.read() == (0, 0, 0, 0) and fb.bounds(4) == (None, None)
    last_epoch = 0
    for batch, lens, kw, what in [
            (40, [2048] * 40, dict(max_kv_len=2048, min_kv_len=2048), "single pass"),
            (4, [2500, 37, 1, 900], dict(max_kv_len=2500, min_kv_len=2400), "chunks"),
            (4, [2500, 37, 0, 900], dict(), "equal shares"),
            (1, [777], dict(), "own-length chunks"),
            (3, [100, 5000, -3], dict(kv_split=7), "forced splits, lengths outside the table")]:
        pool = batch * cap_pages
        q = torch.randn(batch, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
        k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
        v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
        table = torch.randperm(pool, generator=g).to(torch.int32).view(batch, cap_pages).to(cuda_device)
        call = tda.prepare_decode(q, k, v, table, _lens_t(lens, cuda_device), d ** -0.5, length_feedback=fb, **kw)
        print(f"case length feedback: {what}, plan {call.plan}", flush=True)
        call.run()
        torch.cuda.synchronize()
        clamped = [min(max(n, 0), cap_pages * page) for n in lens]
        lo, hi, epoch, nb = fb.read()
        assert (lo, hi, nb) == (min(clamped), max(clamped), batch), what
        assert epoch > last_epoch
        last_epoch = epoch
        assert fb.bounds(batch) == ((lo, hi) if lo >= 1 else (None, None)) and fb.bounds(batch + 1) == (None, None)
        live = [i for i, n in enumerate(clamped) if n > 0]
        _check(call.out[live], call.lse[live], q[live], k, v, table[live], [clamped[i] for i in live], d ** -0.5,
               tag=f"length feedback {what}")
    fb.close()


def test_drop_in_entry_points_learn_the_length_bounds_from_the_previous_call(cuda_device):
    # the reference's signature has no host-side lengths: with a LengthFeedback the first call runs the plan for unknown
    # lengths, later calls the plan for the bounds the previous call left behind - same results, also after the
    # lengths behind the tensor have changed (the bounds are then out of date for one call)
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=32, kv_len=2304), cuda_device)
    args = (inp.q, inp.k_cache, inp.v_cache, None, None, inp.kv_lens, inp.block_table, inp.sm_scale)
    fb = tda.LengthFeedback()
    stateless = tda.gqa_fwd_batch_decode_intra_rank(*args, kv_split=32).clone()
    first = tda.gqa_fwd_batch_decode_intra_rank(*args, kv_split=32, length_feedback=fb).clone()
    torch.cuda.synchronize()
    assert torch.equal(first, stateless)                       # nothing known yet: the same plan
    assert fb.bounds(32) == (2304, 2304)
    plan_known = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                       max_kv_len=2304, min_kv_len=2304)
    plan_unknown = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    assert plan_known.num_splits == 1 and plan_unknown.balanced
    second = tda.gqa_fwd_batch_decode_intra_rank(*args, kv_split=32, length_feedback=fb).clone()
    torch.cuda.synchronize()
    known = torch.empty_like(second)
    tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale, max_kv_len=2304,
                       min_kv_len=2304, packed_out=known, want_lse=False).run()
    torch.cuda.synchronize()
    assert torch.equal(second, known)                          # the single pass of a caller who knows the lengths
    torch.testing.assert_close(first[..., :-1].float(), second[..., :-1].float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(first[..., -1].float(), second[..., -1].float(), atol=3e-2, rtol=1e-2)
    # the batch behind the tensor changes: ragged now, while the bounds still say alike
    new_lens = [2304 - 71 * i for i in range(32)]
    inp.kv_lens.copy_(_lens_t(new_lens, cuda_device))
    out_ref, lse_ref = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    third = tda.gqa_fwd_batch_decode_intra_rank(*args, kv_split=32, length_feedback=fb).clone()
    torch.cuda.synchronize()
    assert fb.bounds(32) == (min(new_lens), 2304)
    _check(out_ref, lse_ref, inp.q, inp.k_cache, inp.v_cache, inp.block_table, new_lens, inp.sm_scale, tag="ragged, no bounds")
    torch.testing.assert_close(third[..., :-1].float(), out_ref.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(third[..., -1].float(), lse_ref, atol=3e-2, rtol=1e-2)     # lse rounded to 16 bits
    fourth = tda.gqa_fwd_batch_decode(*args, kv_split=32, length_feedback=fb)
    torch.cuda.synchronize()
    torch.testing.assert_close(fourth.float(), out_ref.float(), atol=1e-2, rtol=1e-2)
    # the layer keeps a block of its own
    layer = tda.SpGQAFlashDecodeAttention(0, 0, 1, 1, 32, 8, 128, 128, page_size=16, scale=inp.sm_scale, max_allowed_batch=32)
    for _ in range(2):
        res = layer(inp.q, inp.k_cache, inp.v_cache, inp.kv_lens[None], inp.block_table)
        torch.cuda.synchronize()
        torch.testing.assert_close(res.float(), out_ref.float(), atol=1e-2, rtol=1e-2)
    assert layer._feedback.bounds(32) == (min(new_lens), 2304)


def test_zero_length_sequence_is_defined(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=3, kv_len=300), cuda_device)
    lens = _lens_t([300, 0, 17], cuda_device)
    for s in (1, 4):
        out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, lens, inp.sm_scale, kv_split=s)
        torch.cuda.synchronize()
        assert torch.all(out[1] == 0) and torch.all(torch.isneginf(lse[1]))
        assert torch.isfinite(out[0].float()).all() and torch.isfinite(lse[[0, 2]]).all()


@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_lengths_outside_the_table_are_clamped_and_negative_ones_are_empty(cuda_device, algo):
    # kv_lens is device data the host never sees: a length beyond the table attends the table's capacity, a
    # negative one nothing - in every plan mode, without reading outside the table
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=4, kv_len=320), cuda_device)
    cap = inp.block_table.shape[1] * 16
    lens = _lens_t([cap + 5000, -3, 17, 2 ** 31 - 1], cuda_device)
    for kw in (dict(kv_split=1), dict(kv_split=5), dict()):
        out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, lens, inp.sm_scale, algo=algo, **kw)
        torch.cuda.synchronize()
        assert torch.all(out[1] == 0) and torch.all(torch.isneginf(lse[1]))
        _check(out[[0, 2, 3]], lse[[0, 2, 3]], inp.q[[0, 2, 3]], inp.k_cache, inp.v_cache, inp.block_table[[0, 2, 3]],
               [cap, 17, cap], inp.sm_scale, tag=f"clamped {algo} {kw}")


def test_fp16_queries_with_an_fp8_cache(cuda_device):
    g = torch.Generator().manual_seed(97)
    lens, hq, hkv, d, page = [700, 3, 129, 2000], 32, 8, 128, 16
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 1
    q = torch.randn(4, hq, d, generator=g).to(torch.float16).to(cuda_device)
    k16 = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    v16 = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    table = torch.zeros((4, max(pages)), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    k8, ks = wl.quantize_kv_fp8(k16)
    v8, vs = wl.quantize_kv_fp8(v16)
    ref_kv = (ofp8.dequant_per_head(k8, ks, torch.float16), ofp8.dequant_per_head(v8, vs, torch.float16))
    for kw in (dict(), dict(kv_split=6), dict(algo="valu")):
        out, lse = tda.flash_decode(q, k8, v8, table, _lens_t(lens, cuda_device), d ** -0.5, k_scale=ks, v_scale=vs, **kw)
        torch.cuda.synchronize()
        assert out.dtype == torch.float16
        _check(out, lse, q, k8, v8, table, lens, d ** -0.5, ref_kv=ref_kv, tag=f"fp16 q / fp8 kv {kw}")


def test_split_then_combine_entry_points_equal_the_fused_call(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=4, kv_len=2048), cuda_device)
    for s in (1, 8):
        ref_o, ref_l = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                        kv_split=s)
        call = tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                  kv_split=s, always_workspace=True)
        call.out.zero_()
        call.run_splitkv()
        torch.cuda.synchronize()
        assert torch.all(call.out == 0)                     # the split entry point writes only the workspace
        o, l = call.run_combine()
        torch.cuda.synchronize()
        torch.testing.assert_close(o.float(), ref_o.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(l, ref_l, atol=1e-5, rtol=0)


@pytest.mark.parametrize("config,kw", [("ragged_g8", dict(batch=40, kv_len_range=(1, 6000))),
                                       ("llama3_8b_b32", dict(batch=3, kv_len=3000))])
def test_single_launch_form_equals_split_then_combine_and_restores_its_counters(cuda_device, config, kw):
    # with counters: one launch (the last workgroup of a unit merges; many pieces are pulled from a queue) against
    # one workgroup per piece followed by the combine kernel
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS[config], **kw), cuda_device, poison_tail=True)
    for kv_split in (-1, 7, 64):
        two = tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                 kv_split=kv_split, work_queue=False)
        ctr = torch.zeros(4096, dtype=torch.int32, device=cuda_device)
        one = tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                 kv_split=kv_split, counters=ctr, single_launch=True)
        assert one.plan.num_splits == two.plan.num_splits and one.args.counters and not two.args.counters
        o2, l2 = two.run()
        firsts = None
        for _ in range(3):                               # repeated calls reuse the same counters
            one.out.fill_(float("nan"))
            one.lse.fill_(float("nan"))
            o1, l1 = one.run()
            torch.cuda.synchronize()
            if firsts is None:
                firsts = (o1.clone(), l1.clone())
            assert torch.equal(o1, firsts[0]) and torch.equal(l1, firsts[1])      # whoever merges: same arithmetic
        # same pieces; the two merges differ in rounding only (at most one step of the 16-bit output)
        torch.testing.assert_close(o1.float(), o2.float(), atol=2e-3, rtol=2 ** -7)
        torch.testing.assert_close(l1, l2, atol=2e-6, rtol=1e-6)
        assert int(ctr.abs().sum()) == 0
        _check(o1, l1, inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens_host, inp.sm_scale,
               tag=f"work queue S={kv_split}")


def test_runs_on_a_side_stream_and_is_repeatable(cuda_device):
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=4, kv_len=1500), cuda_device)
    call = tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    o0, l0 = [t.clone() for t in call.run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(3):
            call.out.zero_()
            o1, l1 = call.run()
    side.synchronize()
    assert torch.equal(o0, o1) and torch.equal(l0, l1)      # deterministic: no atomics, fixed merge order


@pytest.mark.parametrize("mode", ["single_pass", "chunks_queue", "balanced"])
def test_hip_graph_replays_follow_the_inputs(cuda_device, mode):
    # A captured call holds only pointers: replays must follow in-place changes of q and kv_lens (also the
    # balanced partition, which the kernel derives from kv_lens), with eager work between the replays.
    g = torch.Generator().manual_seed(61)
    if mode == "single_pass":
        b, hq, hkv, n_max, kw = 40, 32, 8, 700, {}
    elif mode == "chunks_queue":
        b, hq, hkv, n_max, kw = 12, 32, 8, 3000, dict(kv_split=24)        # 12*24*4 items > 512 resident workgroups
    else:
        b, hq, hkv, n_max, kw = 3, 8, 1, 40000, dict(force_balanced=True)    # (a batch this small is cut into chunks otherwise)
    d, page = 128, 16
    pages = (n_max + page - 1) // page
    pool = b * pages
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.randperm(pool, generator=g).to(torch.int32).view(b, pages).to(cuda_device)
    lens_sets = [torch.randint(1, n_max + 1, (b,), generator=g).to(torch.int32) for _ in range(3)]
    lens_sets[1][0] = 0                                                        # an empty sequence in one replay
    lens_t = lens_sets[0].clone().to(cuda_device)
    fb = tda.LengthFeedback()           # the replays also report the bounds of the lengths they ran on
    call = tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, max_kv_len=n_max, length_feedback=fb, **kw)
    if mode == "balanced":
        assert call.plan.balanced
    elif mode == "single_pass":
        assert call.plan.num_splits == 1
    else:
        assert call.plan.num_splits == 24 and not call.plan.balanced
    call.run()                                                                  # warm up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call.run()
    for i, new_lens in enumerate(lens_sets):
        lens_t.copy_(new_lens.to(cuda_device))
        q.copy_(torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device))
        call.out.fill_(float("nan"))
        call.lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_l = call.out.clone(), call.lse.clone()
        want_o, want_l = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, max_kv_len=n_max, **kw)   # eager, own buffers
        torch.cuda.synchronize()
        assert torch.equal(got_o, want_o) and torch.equal(got_l, want_l), f"replay {i}"
        assert fb.read()[:2] == (int(new_lens.min()), int(new_lens.max())) and fb.read()[3] == b, f"replay {i}"
        live = [j for j in range(b) if int(new_lens[j]) > 0]
        rows = live[:4]
        _check(got_o[rows], got_l[rows], q[rows], k, v, table[rows], [int(new_lens[j]) for j in rows], d ** -0.5,
               tag=f"graph replay {i}")


def test_concurrent_host_threads_on_their_own_streams(cuda_device):
    # The library keeps no mutable state apart from a thread-local error string: four host threads, each with its
    # own stream, buffers and problem, call it at the same time (ctypes releases the GIL during the calls).
    import threading
    g = torch.Generator().manual_seed(71)
    problems = []
    for i, (b, hq, hkv, n, split) in enumerate([(3, 32, 8, 900, -1), (40, 32, 8, 300, -1), (2, 8, 1, 5000, 16), (5, 64, 8, 700, 3)]):
        page, d = 16, 128
        pages = (n + page - 1) // page
        q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
        k = torch.randn(b * pages, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
        v = torch.randn(b * pages, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
        table = torch.randperm(b * pages, generator=g).to(torch.int32).view(b, pages).to(cuda_device)
        lens = torch.randint(1, n + 1, (b,), generator=g).to(torch.int32).to(cuda_device)
        want = tda.flash_decode(q, k, v, table, lens, d ** -0.5, kv_split=split)
        problems.append((q, k, v, table, lens, d ** -0.5, split, want))
    torch.cuda.synchronize()
    errors = []

    def worker(idx):
        try:
            q, k, v, table, lens, scale, split, want = problems[idx]
            stream = torch.cuda.Stream(device=cuda_device)
            call = tda.prepare_decode(q, k, v, table, lens, scale, kv_split=split)
            for it in range(40):
                call.out.fill_(float("nan"))
                with torch.cuda.stream(stream):
                    call.out.record_stream(stream)
                    stream.wait_stream(torch.cuda.current_stream())
                    out, lse = call.run(stream)
                stream.synchronize()
                if not (torch.equal(out, want[0]) and torch.equal(lse, want[1])):
                    errors.append((idx, it))
                    return
            try:                                                  # a rejected call in one thread disturbs no other
                tda.flash_decode(q, k, v, table.long(), lens, scale)
                errors.append((idx, "int64 table accepted"))
            except ValueError:
                pass
        except Exception as exc:                                  # noqa: BLE001
            errors.append((idx, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(problems))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


def test_inter_rank_combine_equals_one_shot(cuda_device):
    # R ranks each hold a disjoint slice of every sequence (sequence parallel decode, one GPU stands in for all):
    # local decode per rank -> packed [R,B,Hq,D+1] -> merge == decode over the whole sequence
    r_, b, hq, hkv, d, page = 4, 3, 32, 8, 128, 16
    g = torch.Generator().manual_seed(13)
    shard_lens = torch.tensor([[512, 16, 0], [300, 0, 0], [0, 77, 0], [1, 1000, 5]], dtype=torch.int32)
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    pool = 200
    ks = [torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device) for _ in range(r_)]
    vs = [torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device) for _ in range(r_)]
    tables = [torch.randperm(pool, generator=g)[:b * 63].view(b, 63).to(torch.int32).to(cuda_device) for _ in range(r_)]
    packed = torch.full((r_, b, hq, d + 1), float("nan"), dtype=torch.float32, device=cuda_device)
    outs = torch.empty(r_, b, hq, d, dtype=torch.bfloat16, device=cuda_device)
    lses = torch.empty(r_, b, hq, dtype=torch.float32, device=cuda_device)
    for r in range(r_):
        lens_r = shard_lens[r].to(cuda_device)
        o, l = tda.flash_decode(q, ks[r], vs[r], tables[r], lens_r, d ** -0.5, out=outs[r], lse=lses[r])
        packed[r] = tda.pack_out_lse(o, l, torch.float32)
        packed[r][(shard_lens[r] == 0).to(cuda_device)] = float("nan")   # what the reference leaves there
    gl = shard_lens.to(cuda_device)
    final = tda.inter_rank_combine(packed, gl)
    final2 = tda.inter_rank_combine(outs, gl, all_ranks_lse=lses)
    torch.cuda.synchronize()
    # one-shot over the concatenation
    for i in range(b):
        kk = torch.cat([cf.gather_kv(ks[r], tables[r][i].cpu(), int(shard_lens[r, i])) for r in range(r_)])
        vv = torch.cat([cf.gather_kv(vs[r], tables[r][i].cpu(), int(shard_lens[r, i])) for r in range(r_)])
        n = kk.shape[0]
        o64, _ = cf.attn_fp64(q[i:i + 1], kk[:, None].contiguous(), vv[:, None].contiguous(),
                              torch.arange(n, dtype=torch.int32)[None], [n], d ** -0.5)
        torch.testing.assert_close(final[i].double(), o64[0], atol=5e-3, rtol=1e-2)
        torch.testing.assert_close(final2[i].double(), o64[0], atol=5e-3, rtol=1e-2)
    # against the oracle's restatement of the reference merge
    want = cf.combine_ranks(outs.cpu(), lses.cpu(), shard_lens)
    torch.testing.assert_close(final2.double().cpu(), want, atol=4e-3, rtol=1e-2)
    # the merged lse: the log-sum-exp of the ranks that hold tokens (sequence 2 has tokens on rank 3 only)
    lse_out = torch.full((b, hq), float("nan"), dtype=torch.float32, device=cuda_device)
    tda.inter_rank_combine(outs, gl, all_ranks_lse=lses, lse_out=lse_out)
    torch.cuda.synchronize()
    masked = torch.where((shard_lens > 0)[:, :, None].to(cuda_device), lses, torch.full_like(lses, float("-inf")))
    torch.testing.assert_close(lse_out, torch.logsumexp(masked.double(), dim=0).float(), atol=1e-4, rtol=0)
    # output tensors of the wrong dtype / shape / device are refused before anything is launched
    for bad in (torch.empty(b, hq, dtype=torch.bfloat16, device=cuda_device),
                torch.empty(b, hq - 1, dtype=torch.float32, device=cuda_device),
                torch.empty(b, hq, dtype=torch.float32)):
        with pytest.raises(ValueError):
            tda.inter_rank_combine(outs, gl, all_ranks_lse=lses, lse_out=bad)
    with pytest.raises(ValueError):
        tda.inter_rank_combine(outs, gl, torch.empty(b, hq, d - 1, dtype=torch.bfloat16, device=cuda_device),
                               all_ranks_lse=lses)


# ---- large batches: single pass with blocks of 4 or 8 kv heads per (eight-wave) workgroup ------------------------------
@pytest.mark.parametrize("heads,batch,want_nh", [((32, 8), 256, 8), ((32, 8), 128, 4), ((16, 4), 256, 4), ((48, 2), 300, 2),
                                                ((8, 8), 300, 8), ((96, 4), 130, 4), ((32, 8), 32, 1), ((24, 3), 100, 1)])
@pytest.mark.parametrize("d,dtype,fp8,page", [(128, torch.bfloat16, False, 16), (128, torch.float16, False, 1),
                                             (128, torch.bfloat16, True, 16), (64, torch.bfloat16, False, 6),
                                             (256, torch.float16, False, 16), (256, torch.bfloat16, True, 64)])
def test_large_batches_take_wide_head_blocks(cuda_device, heads, batch, want_nh, d, dtype, fp8, page):
    hq, hkv = heads
    print(f"case wide blocks heads={heads} B={batch} D={d} {dtype} fp8={fp8} P={page}", flush=True)
    g = torch.Generator().manual_seed(batch * 7 + d + page)
    lens = torch.randint(0, 150, (batch,), generator=g).tolist()
    lens[0], lens[1], lens[batch - 1] = 149, 0, 1
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 2
    q = torch.randn(batch, hq, d, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, max(pages) + 1), -7, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, dtype), ofp8.dequant_per_head(v, vs, dtype))
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t)
    assert plan.num_splits == 1 and plan.kv_heads_per_wg == want_nh, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    empty = [i for i, n in enumerate(lens) if n == 0]
    assert (out[empty] == 0).all() and (lse[empty] == float("-inf")).all()
    rows = [i for i, n in enumerate(lens) if n > 0][:: max(1, batch // 24)] + [batch - 1]
    _check(out[rows], lse[rows], q[rows], k, v, table[rows], [lens[i] for i in rows], d ** -0.5, ref_kv=ref_kv,
           tag=f"wide blocks nh={want_nh}")
    # the same call with the head block forced apart (a split count forces chunk mode with narrower blocks)
    out2, lse2 = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs, kv_split=2)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    torch.testing.assert_close(out[live].float(), out2[live].float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse[live], lse2[live], atol=1e-4, rtol=0)


# ---- single pass with one kv head per workgroup: the split kernel runs with one register buffer per wavefront ----------
@pytest.mark.parametrize("d,dtype,fp8,page", [(128, torch.bfloat16, False, 16), (128, torch.float16, False, 1),
                                             (128, torch.bfloat16, False, 8), (128, torch.bfloat16, False, 6),
                                             (128, torch.float16, True, 16), (128, torch.bfloat16, True, 1),
                                             (64, torch.bfloat16, False, 16), (64, torch.float16, True, 3)])
def test_single_pass_with_one_kv_head_per_workgroup(cuda_device, d, dtype, fp8, page):
    """Batch 32 x 8 kv heads gives exactly one workgroup per compute unit of a 256-unit GPU, each on one kv head: the
    plan of the headline configuration.  Lengths from 0 to 1500 tokens (up to 24 tiles per wavefront), every page mode."""
    batch, hq, hkv = 32, 32, 8
    print(f"case one head per workgroup D={d} {dtype} fp8={fp8} P={page}", flush=True)
    g = torch.Generator().manual_seed(d + page + (7 if fp8 else 0))
    lens = torch.randint(1, 1501, (batch,), generator=g).tolist()
    lens[0], lens[1], lens[2], lens[3], lens[batch - 1] = 1500, 0, 1, 16, 17
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 2
    q = torch.randn(batch, hq, d, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, max(pages) + 1), -7, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, dtype), ofp8.dequant_per_head(v, vs, dtype))
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t)
    from triton_distributed_amd import _lib
    if _lib.load().fdk_device_cus() == 256:
        assert plan.num_splits == 1 and plan.kv_heads_per_wg == 1, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    assert (out[1] == 0).all() and (lse[1] == float("-inf")).all()
    rows = [0, 2, 3, 4, 9, 17, 30, batch - 1]
    _check(out[rows], lse[rows], q[rows], k, v, table[rows], [lens[i] for i in rows], d ** -0.5, ref_kv=ref_kv,
           tag="one head per workgroup")
    # the same call cut into chunks (two register buffers, partial rows, combine launch)
    out2, lse2 = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs, kv_split=3)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    torch.testing.assert_close(out[live].float(), out2[live].float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse[live], lse2[live], atol=1e-4, rtol=0)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("hints", [True, False])
def test_kernel_shape_overrides_change_timing_only(cuda_device, fp8, hints):
    """wavefronts / buffers (measurement aids) select how the split kernel is shaped; every combination the kernel
    accepts gives the result of the library's own choice (same arithmetic per wavefront: bit-identical with the same
    number of wavefronts, within rounding otherwise), and combinations it cannot run are ignored."""
    batch, hq, hkv, d, page = 32, 32, 8, 128, 16
    g = torch.Generator().manual_seed(77)
    lens = [2100] * batch if hints else torch.randint(1, 2101, (batch,), generator=g).tolist()
    lens[0] = 2100
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 1
    q = torch.randn(batch, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.zeros((batch, max(pages)), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table, lens_t = table.to(cuda_device), _lens_t(lens, cuda_device)
    ks = vs = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
    kw = dict(k_scale=ks, v_scale=vs, max_kv_len=max(lens))
    if hints:
        kw["min_kv_len"] = min(lens)             # alike lengths: a single pass; without: equal shares
    base = tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, **kw)
    assert base.plan.balanced == (not hints)
    out0, lse0 = (t.clone() for t in base.run())
    torch.cuda.synchronize()
    for wf in (0, 4, 8):
        for nb in (0, 1, 2):
            print(f"case overrides fp8={fp8} hints={hints} wavefronts={wf} buffers={nb}", flush=True)
            out, lse = tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, wavefronts=wf, buffers=nb, **kw).run()
            torch.cuda.synchronize()
            torch.testing.assert_close(out.float(), out0.float(), atol=1e-2, rtol=1e-2)
            torch.testing.assert_close(lse, lse0, atol=1e-5, rtol=0)
    for spc in (1, 2, 3):                        # workgroups per compute unit of a balanced plan
        print(f"case overrides fp8={fp8} hints={hints} shares_per_cu={spc}", flush=True)
        call = tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, shares_per_cu=spc, **kw)
        # (three per compute unit would be shares below 512 tokens here: the plan then drops the equal shares)
        assert hints or call.plan.workgroups == (spc * base.plan.workgroups if spc < 3 else 0)
        out, lse = call.run()
        torch.cuda.synchronize()
        torch.testing.assert_close(out.float(), out0.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(lse, lse0, atol=1e-4, rtol=0)
    with pytest.raises(Exception):
        tda.prepare_decode(q, k, v, table, lens_t, d ** -0.5, wavefronts=3, **kw).run()


@pytest.mark.parametrize("name,batch,n,fp8,want_balanced", [("uneven_fill", 40, 2304, False, True),
                                                           ("fp8_chunks_one_workgroup_per_cu", 8, 4096, True, False),
                                                           ("fp8_uneven_fill", 40, 6144, True, True)])
def test_plans_for_alike_lengths_that_do_not_fill_the_gpu_evenly(cuda_device, name, batch, n, fp8, want_balanced):
    """Alike lengths (the host says so): 40 x 8 units on 256 compute units would leave a quarter of them with two
    workgroups, so the batch runs as equal shares; 8 x 4 head blocks are cut into per-sequence chunks, one workgroup
    per compute unit, which for an fp8 cache runs eight wavefronts with one buffer each."""
    hq, hkv, d, page = 32, 8, 128, 16
    print(f"case alike lengths {name}", flush=True)
    g = torch.Generator().manual_seed(batch + n)
    lens = [n - (i % 3) for i in range(batch)]                      # within 1/32 of each other
    pages = [(x + page - 1) // page for x in lens]
    pool = sum(pages) + 1
    q = torch.randn(batch, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.zeros((batch, max(pages)), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, x in enumerate(pages):
        table[i, :x] = perm[at:at + x]
        at += x
    table, lens_t = table.to(cuda_device), _lens_t(lens, cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, torch.bfloat16), ofp8.dequant_per_head(v, vs, torch.bfloat16))
    hints = dict(max_kv_len=max(lens), min_kv_len=min(lens))
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, **hints)
    assert plan.balanced == want_balanced and plan.num_splits > 1, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs, **hints)
    torch.cuda.synchronize()
    rows = list(range(0, batch, max(1, batch // 8)))
    _check(out[rows], lse[rows], q[rows], k, v, table[rows], [lens[i] for i in rows], d ** -0.5, ref_kv=ref_kv, tag=name)
    # and against the forced single pass
    out1, lse1 = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs, kv_split=1)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.float(), out1.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse, lse1, atol=1e-4, rtol=0)


# ---- balanced mode: the kernel cuts the batch's KV ranges into equal shares from kv_lens ---------------------------
BALANCED_CASES = {
    # name: (kv_lens, (Hq, Hkv), page, head_dim, fp8)
    "one_long_two_short": ([40000, 0, 777], (8, 1), 16, 128, False),
    "short_first": ([1, 39999, 64, 65], (8, 1), 16, 128, False),
    "all_heads_two_per_wg": ([30000, 12345, 5, 0, 20000], (32, 8), 16, 128, False),
    "group16_p64": ([50000, 3, 17000], (16, 1), 64, 128, False),
    "group24_two_tiles": ([40000, 30000], (24, 1), 16, 128, False),
    "page1": ([9000, 40000, 1], (8, 2), 1, 128, False),
    "fp8_d128": ([33000, 100, 8000], (16, 2), 16, 128, True),
    "d64": ([33000, 100, 8000], (8, 2), 16, 64, False),
    "d256": ([33000, 100, 8000], (8, 2), 16, 256, False),
    "odd_page24": ([40000, 4097, 23], (8, 1), 24, 128, False),
}


@pytest.mark.parametrize("name", list(BALANCED_CASES))
def test_balanced_mode_ragged_batches(cuda_device, name):
    lens, (hq, hkv), page, d, fp8 = BALANCED_CASES[name]
    print(f"case balanced {name}", flush=True)
    g = torch.Generator().manual_seed(hash(name) & 0xFFFF)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 3
    width = max(pages) + 2
    q = torch.randn(len(lens), hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((len(lens), width), 2 ** 31 - 1, dtype=torch.int32)      # poisoned beyond each sequence
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    ks = vs = None
    ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks), ofp8.dequant_per_head(v, vs))
    scale = d ** -0.5
    # (equal shares are the planner's own choice only for batches that stream for some tens of microseconds; these
    # small ones force them)
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, max_kv_len=max(lens), force_balanced=True)
    assert plan.balanced and plan.workgroups > 0, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, max_kv_len=max(lens), k_scale=ks, v_scale=vs,
                                force_balanced=True)
    # chunk mode on the same inputs (a forced split count)
    out_c, lse_c = tda.flash_decode(q, k, v, table, lens_t, scale, max_kv_len=max(lens), k_scale=ks, v_scale=vs,
                                    kv_split=7)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    empty = [i for i, n in enumerate(lens) if n == 0]
    for o, l, tag in ((out, lse, "balanced"), (out_c, lse_c, "chunks")):
        if empty:
            assert (o[empty] == 0).all() and torch.isinf(l[empty]).all() and (l[empty] < 0).all()
        _check(o[live], l[live], q[live], k, v, table[live], [lens[i] for i in live], scale, ref_kv=ref_kv,
               tag=f"{name} {tag}")
    torch.testing.assert_close(out.float(), out_c.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse[live], lse_c[live], atol=1e-4, rtol=0)


def test_balanced_mode_with_soft_cap_strides_and_output_forms(cuda_device):
    # fp16, soft cap, q / out taken as strided views, fp32 output, packed [B, Hq, D+1] output - all in balanced mode
    g = torch.Generator().manual_seed(83)
    lens, hq, hkv, d, page = [30000, 11, 17000], 16, 2, 128, 16
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 1
    q_big = torch.randn(3, hq, 2 * d, generator=g).to(torch.float16).to(cuda_device)
    q = q_big[:, :, :d]                                           # head stride 2 D, contiguous D
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.float16).to(cuda_device)
    table = torch.zeros((3, max(pages)), dtype=torch.int32)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    scale, cap = d ** -0.5, 30.0
    assert tda.get_split_kv_plan(q, k, v, table, lens_t, max_kv_len=max(lens), force_balanced=True).balanced
    out32 = torch.full((3, hq, d + 3), float("nan"), dtype=torch.float32, device=cuda_device)
    o, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=cap, max_kv_len=max(lens), out=out32[:, :, :d],
                              force_balanced=True)
    packed = torch.full((3, hq, d + 1), float("nan"), dtype=torch.float16, device=cuda_device)
    tda.prepare_decode(q, k, v, table, lens_t, scale, soft_cap=cap, max_kv_len=max(lens), packed_out=packed,
                       want_lse=False, force_balanced=True).run()
    torch.cuda.synchronize()
    assert o.data_ptr() == out32.data_ptr() and torch.isnan(out32[:, :, d:]).all()      # nothing written past D
    o64, l64 = cf.attn_fp64(q, k, v, table, lens, scale, cap)
    torch.testing.assert_close(o.double(), o64, atol=8e-3, rtol=1e-2)
    torch.testing.assert_close(lse.double(), l64, atol=LSE_ATOL, rtol=0)
    torch.testing.assert_close(packed[..., :d].float(), o, atol=2e-3, rtol=2e-3)        # fp16 rounding of the same result
    torch.testing.assert_close(packed[..., d].float(), lse, atol=1e-2, rtol=1e-3)
    ref = ref_paged_attn(q, k, v, lens, table, scale, cap)
    torch.testing.assert_close(packed[..., :d].float(), ref.float(), atol=OUT_ATOL, rtol=OUT_RTOL)


def test_balanced_mode_clamps_lengths_like_the_other_modes(cuda_device):
    g = torch.Generator().manual_seed(89)
    hq, hkv, d, page, width = 8, 1, 128, 16, 2600
    cap = width * page
    true_lens = [cap, 0, 30000]                                   # what the device lengths below amount to
    pool = width + 1875 + 2
    q = torch.randn(3, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((3, width), -9, dtype=torch.int32)
    table[0] = perm[:width]
    table[2, :1875] = perm[width:width + 1875]
    table = table.to(cuda_device)
    lens_t = _lens_t([cap + 1000, -1, 30000], cuda_device)
    assert tda.get_split_kv_plan(q, k, v, table, lens_t, force_balanced=True).balanced
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, force_balanced=True)
    torch.cuda.synchronize()
    assert torch.all(out[1] == 0) and torch.all(torch.isneginf(lse[1]))
    _check(out[[0, 2]], lse[[0, 2]], q[[0, 2]], k, v, table[[0, 2]], [cap, 30000], d ** -0.5, tag="balanced clamp")


def test_balanced_mode_many_sequences(cuda_device):
    # more than 64 sequences: the partition scan runs over several 64-lane chunks; includes empty sequences
    g = torch.Generator().manual_seed(77)
    b, hq, hkv, d, page = 150, 8, 1, 128, 16
    lens = torch.randint(0, 6001, (b,), generator=g).tolist()
    for i in (0, 63, 64, 65, 127, 128, 149):
        lens[i] = 0
    lens[1], lens[66], lens[148] = 6000, 1, 5999
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 1
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.zeros((b, max(pages)), dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, max_kv_len=6000)
    assert plan.balanced, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, max_kv_len=6000)
    torch.cuda.synchronize()
    live = [i for i, n in enumerate(lens) if n > 0]
    empty = [i for i, n in enumerate(lens) if n == 0]
    assert (out[empty] == 0).all() and (lse[empty] == float("-inf")).all()
    _check(out[live], lse[live], q[live], k, v, table[live], [lens[i] for i in live], d ** -0.5, tag="balanced b150")


def test_sequence_parallel_layer_mirror(cuda_device):
    # the reference's layer (sp_flash_decode_layer.py:83-185) on one GPU: R layer objects stand in for R ranks, the
    # exchange between them is a stack of their blocks
    r_, b, hq, hkv, d, page = 3, 4, 32, 8, 128, 16
    g = torch.Generator().manual_seed(19)
    shard_lens = torch.tensor([[700, 16, 0, 33], [300, 0, 0, 1], [1, 77, 0, 2000]], dtype=torch.int32)
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    pool = 4 * 130
    ks = [torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device) for _ in range(r_)]
    vs = [torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device) for _ in range(r_)]
    tables = [torch.randperm(pool, generator=g)[:b * 126].view(b, 126).to(torch.int32).to(cuda_device) for _ in range(r_)]
    gl = shard_lens.to(cuda_device)
    blocks = {}

    def gather_for(rank):
        def all_gather(block):
            blocks[rank] = block
            return torch.stack([blocks[i] for i in range(r_)]) if len(blocks) == r_ else None
        return all_gather

    layers = [tda.SpGQAFlashDecodeAttention(rk, 0, r_, 1, hq, hkv, d, d, page_size=page, scale=d ** -0.5,
                                            max_allowed_batch=b, all_gather=gather_for(rk)) for rk in range(r_)]
    for rk in range(r_ - 1):                       # the first ranks only deposit their block
        blocks[rk] = layers[rk].local_decode(q, ks[rk], vs[rk], gl, tables[rk])
    final = layers[r_ - 1](q, ks[r_ - 1], vs[r_ - 1], gl, tables[r_ - 1])
    torch.cuda.synchronize()
    assert final.shape == (b, hq, d) and final.dtype == torch.bfloat16
    for i in range(b):
        total = int(shard_lens[:, i].sum())
        if total == 0:
            assert (final[i] == 0).all()            # no rank holds tokens: defined as zero
            continue
        kk = torch.cat([cf.gather_kv(ks[rk], tables[rk][i].cpu(), int(shard_lens[rk, i])) for rk in range(r_)])
        vv = torch.cat([cf.gather_kv(vs[rk], tables[rk][i].cpu(), int(shard_lens[rk, i])) for rk in range(r_)])
        o64, _ = cf.attn_fp64(q[i:i + 1], kk[:, None].contiguous(), vv[:, None].contiguous(),
                              torch.arange(total, dtype=torch.int32)[None], [total], d ** -0.5)
        torch.testing.assert_close(final[i].double(), o64[0], atol=2e-2, rtol=2e-2)   # blocks travel in bf16
    # one rank: forward needs no exchange and equals the plain decode
    solo = tda.SpGQAFlashDecodeAttention(0, 0, 1, 1, hq, hkv, d, d, page_size=page, scale=d ** -0.5, max_allowed_batch=b)
    got = solo(q, ks[0], vs[0], gl[:1], tables[0])
    want, _ = tda.flash_decode(q, ks[0], vs[0], tables[0], gl[0], d ** -0.5)
    torch.cuda.synchronize()
    live = (shard_lens[0] > 0).to(cuda_device)
    torch.testing.assert_close(got[live].float(), want[live].float(), atol=1e-2, rtol=1e-2)
    with pytest.raises(ValueError):
        tda.SpGQAFlashDecodeAttention(0, 0, 2, 1, hq, hkv, d, d)            # more ranks need an exchange


@pytest.mark.parametrize("page", [6, 24])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_page_sizes_that_are_not_powers_of_two(cuda_device, page, algo):
    c = _dev(dict(all_cases())["odd_page6"], cuda_device) if page == 6 else None
    if c is None:
        g = torch.Generator().manual_seed(41)
        lens = [500, 23, 24, 25]
        pool = 100
        c = dict(q=torch.randn(4, 8, 128, generator=g).to(torch.bfloat16).to(cuda_device),
                 k_cache=torch.randn(pool, page, 2, 128, generator=g).to(torch.bfloat16).to(cuda_device),
                 v_cache=torch.randn(pool, page, 2, 128, generator=g).to(torch.bfloat16).to(cuda_device),
                 block_table=torch.randperm(pool, generator=g)[:4 * 21].view(4, 21).to(torch.int32).to(cuda_device),
                 kv_lens=lens, sm_scale=128 ** -0.5, soft_cap=0.0)
    out, lse = tda.flash_decode(c["q"], c["k_cache"], c["v_cache"], c["block_table"], _lens_t(c["kv_lens"], cuda_device),
                                c["sm_scale"], algo=algo)
    torch.cuda.synchronize()
    _check(out, lse, c["q"], c["k_cache"], c["v_cache"], c["block_table"], c["kv_lens"], c["sm_scale"], tag=f"P={page}")


# ---- seeded random sweep over the whole argument space -------------------------------------------------------------
@pytest.mark.parametrize("seed", list(range(96)))
def test_random_shapes_against_the_oracle(cuda_device, seed):
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.choice([64, 128, 128, 256]))
    hkv = int(rng.choice([1, 2, 3, 4, 8]))
    group = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 20]))
    hq = hkv * group
    page = int(rng.choice([1, 2, 3, 4, 8, 16, 16, 32, 64, 24]))
    batch = int(rng.choice([1, 2, 5, 17, 40, 90]))
    n_max = int(rng.choice([40, 300, 1500, 3000])) if batch <= 40 else int(rng.choice([40, 200]))
    dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float16
    fp8 = bool(rng.random() < 0.25)
    soft_cap = float(rng.choice([0.0, 0.0, 30.0]))
    kv_split = int(rng.choice([-1, -1, -1, 1, 2, 5, 32]))
    lens = rng.integers(0, n_max + 1, size=batch).tolist()
    lens[int(rng.integers(0, batch))] = n_max
    if rng.random() < 0.5:
        lens[int(rng.integers(0, batch))] = 1
    hint = None if rng.random() < 0.5 else int(n_max * rng.choice([0.5, 1.0, 2.0]))
    print(f"case random seed={seed} B={batch} {hq}q/{hkv}kv D={d} P={page} N<={n_max} {dtype} fp8={fp8} cap={soft_cap} "
          f"S={kv_split} hint={hint}", flush=True)
    g = torch.Generator().manual_seed(seed)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 3
    q = torch.randn(batch, hq, d, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, max(max(pages), 1) + int(rng.integers(0, 3))), int(rng.choice([-1, 2 ** 31 - 1, 0])), dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, dtype), ofp8.dequant_per_head(v, vs, dtype))
    scale_mult = float(rng.choice([0.5, 1.0, 1.0, 2.0]))
    scale = float(d ** -0.5) * scale_mult
    # hints may be wrong in either direction (an upper bound below the longest sequence, a lower bound above the
    # shortest): they cost balance, never tokens
    low = None if rng.random() < 0.6 else int((hint if hint is not None else n_max) * rng.choice([0.25, 0.98, 1.0]))
    out, lse = tda.flash_decode(q, k, v, table, _lens_t(lens, cuda_device), scale, soft_cap=soft_cap, kv_split=kv_split,
                                max_kv_len=hint, min_kv_len=low, k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    empty = [i for i, n in enumerate(lens) if n == 0]
    live = [i for i, n in enumerate(lens) if n > 0]
    if empty:
        assert (out[empty] == 0).all() and torch.isneginf(lse[empty]).all()
    # doubled logits double the 16-bit logit rounding of the torch restatement; the float64 comparison stays as tight
    _check(out[live], lse[live], q[live], k, v, table[live], [lens[i] for i in live], scale, soft_cap, ref_kv=ref_kv,
           tag=f"random seed {seed}", ref_tol=4e-2 if scale_mult > 1.0 else None)


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_short_sequences_in_wide_tables_against_the_oracle(cuda_device, seed):
    # no length bounds and a table far wider than the sequences: the plan is sized for the table, the chunks follow
    # kv_lens on the GPU (few sequences, every head size, page size and cache type)
    rng = np.random.default_rng(7000 + seed)
    d = int(rng.choice([64, 128, 256]))
    hkv = int(rng.choice([1, 2, 4, 8]))
    group = int(rng.choice([1, 4, 8, 16]))
    hq = hkv * group
    page = int(rng.choice([1, 8, 16, 64]))
    batch = int(rng.choice([1, 1, 2, 3]))
    cap = int(rng.choice([2048, 8192, 20000]))
    dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float16
    fp8 = bool(rng.random() < 0.3)
    lens = [int(rng.choice([1, 17, 64, 65, 500, 1023, 1024, 1800])) for _ in range(batch)]
    print(f"case wide table seed={seed} B={batch} {hq}q/{hkv}kv D={d} P={page} cap={cap} lens={lens} {dtype} fp8={fp8}", flush=True)
    g = torch.Generator().manual_seed(seed)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 2
    q = torch.randn(batch, hq, d, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, (cap + page - 1) // page), -1, dtype=torch.int32)     # unused columns: never followed
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, dtype), ofp8.dequant_per_head(v, vs, dtype))
    lens_t = _lens_t(lens, cuda_device)
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, d ** -0.5)
    assert plan.num_splits > 1 and (plan.balanced or plan.chunk_floor == 64)
    ws = torch.full((plan.workspace_bytes // 4,), float("nan"), dtype=torch.float32, device=cuda_device)
    out, lse = tda.flash_decode(q, k, v, table, lens_t, d ** -0.5, k_scale=ks, v_scale=vs, workspace=ws)
    torch.cuda.synchronize()
    _check(out, lse, q, k, v, table, lens, d ** -0.5, ref_kv=ref_kv, tag=f"wide table seed {seed}")


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_long_and_wide_batches_against_the_oracle(cuda_device, seed):
    # the plans the small sweep above rarely reaches: balanced mode (few long sequences) and single pass with wide
    # head blocks (many short sequences)
    rng = np.random.default_rng(5000 + seed)
    long_case = seed % 3 != 2
    d = int(rng.choice([64, 128, 128, 256]))
    page = int(rng.choice([1, 4, 16, 16, 64, 24]))
    dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float16
    fp8 = bool(rng.random() < 0.3)
    soft_cap = float(rng.choice([0.0, 0.0, 50.0]))
    if long_case:
        hkv = int(rng.choice([1, 2, 4]))
        group = int(rng.choice([1, 4, 8, 16, 24]))
        batch = int(rng.choice([1, 2, 3, 6]))
        n_max = int(rng.choice([20000, 33000, 48000])) // (2 if d == 256 or hkv == 4 else 1)
        lens = rng.integers(0, n_max + 1, size=batch).tolist()
        lens[int(rng.integers(0, batch))] = n_max
    else:
        hkv = int(rng.choice([4, 8]))
        group = int(rng.choice([1, 4, 8]))
        batch = int(rng.choice([260, 300, 520]))
        n_max = 70
        lens = rng.integers(0, n_max + 1, size=batch).tolist()
    hq = hkv * group
    print(f"case random2 seed={seed} B={batch} {hq}q/{hkv}kv D={d} P={page} N<={n_max} {dtype} fp8={fp8} cap={soft_cap}", flush=True)
    g = torch.Generator().manual_seed(seed)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 2
    q = torch.randn(batch, hq, d, generator=g).to(dtype).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype).to(cuda_device)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, max(max(pages), 1) + 1), -1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    table = table.to(cuda_device)
    ks = vs = ref_kv = None
    if fp8:
        k, ks = wl.quantize_kv_fp8(k)
        v, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k, ks, dtype), ofp8.dequant_per_head(v, vs, dtype))
    scale = float(d ** -0.5)
    lens_t = _lens_t(lens, cuda_device)
    plan = tda.get_split_kv_plan(q, k, v, table, lens_t, max_kv_len=n_max)
    if long_case:
        assert plan.balanced or plan.num_splits > 1, plan
    else:
        assert plan.num_splits == 1 and plan.kv_heads_per_wg >= 2, plan
    out, lse = tda.flash_decode(q, k, v, table, lens_t, scale, soft_cap=soft_cap, max_kv_len=n_max, k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    empty = [i for i, n in enumerate(lens) if n == 0]
    live = [i for i, n in enumerate(lens) if n > 0]
    if empty:
        assert (out[empty] == 0).all() and torch.isneginf(lse[empty]).all()
    rows = live if long_case else live[:: max(1, len(live) // 20)]
    _check(out[rows], lse[rows], q[rows], k, v, table[rows], [lens[i] for i in rows], scale, soft_cap, ref_kv=ref_kv,
           tag=f"random2 seed {seed} {plan}")


# ---- fp8 KV cache ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("heads", [(32, 8), (64, 8), (8, 8)])
@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_fp8_kv_cache_small(cuda_device, heads, algo):
    cfg = wl.DecodeConfig("fp8_small", 55, 5, heads[0], heads[1], 128, 16, kv_len_range=(1, 2000), kv_dtype="fp8_e4m3",
                          spare_pages=4)
    inp = wl.make_inputs(cfg, cuda_device, poison_tail=True)
    out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                k_scale=inp.k_scale, v_scale=inp.v_scale, algo=algo)
    torch.cuda.synchronize()
    # the workload's definition: dequantise to bf16, then the same decode
    kd = ofp8.dequant_per_head(inp.k_cache, inp.k_scale)
    vd = ofp8.dequant_per_head(inp.v_cache, inp.v_scale)
    _check(out, lse, inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens_host, inp.sm_scale,
           ref_kv=(kd, vd), tag="fp8")
    # the exact dequantisation in float64 (no bf16 rounding of k8*scale) is a different function of the bytes:
    # rounding K to bf16 moves single logits by ~2^-9 relative, i.e. lse by up to a few 1e-3
    o64, l64 = cf.attn_fp64(inp.q, inp.k_cache.float(), inp.v_cache.float(), inp.block_table, inp.kv_lens_host,
                            inp.sm_scale, k_scale=inp.k_scale, v_scale=inp.v_scale)
    torch.testing.assert_close(out.double(), o64, atol=5e-3, rtol=1e-2)
    torch.testing.assert_close(lse.double(), l64, atol=5e-3, rtol=0)


@pytest.mark.parametrize("heads,page,lens", [((32, 8), 16, (1, 2000)), ((64, 8), 16, (1, 2000)), ((8, 8), 1, (1, 700)),
                                             ((16, 2), 16, [33000, 100, 8000]), ((8, 1), 16, [1, 2, 17, 64, 65])])
def test_fp8_folded_k_scale(cuda_device, heads, page, lens):
    """FDK_FLAG_FP8_FOLD_K_SCALE: logits are (q . k8) * k_scale instead of q . round_bf16(k8 * k_scale).  That is the
    exact evaluation of what the cache holds: against the float64 attention over k8 * k_scale (no rounding of K) the
    bars of this path hold as they are (lse 1e-3).  Against the dequantise-to-bf16-then-decode definition - the oracle
    of the default form - single logits differ by the 16-bit rounding of K (about 1e-3 for 128 unit-variance terms),
    so lse is compared at 5e-3 there, out at the usual 2e-2; short and peaked sequences are where the two definitions
    are furthest apart, long diffuse ones agree to 1e-4 (the benchmark configuration is checked at the standard bars in
    test_config5_fp8_70b_b128_folded_k_scale)."""
    g = torch.Generator().manual_seed(91 + heads[0] + page)
    if isinstance(lens, tuple):
        lens = torch.randint(lens[0], lens[1] + 1, (5,), generator=g).tolist()
    hq, hkv, d = heads[0], heads[1], 128
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 3
    table = torch.full((len(lens), max(pages) + 2), 2 ** 31 - 1, dtype=torch.int32)      # poisoned beyond each sequence
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    k8, ks = wl.quantize_kv_fp8(torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device))
    v8, vs = wl.quantize_kv_fp8(torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device))

    class inp:                                          # the names the checks below use
        q = torch.randn(len(lens), hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
        k_cache, v_cache, k_scale, v_scale = k8, v8, ks, vs
        block_table = table.to(cuda_device)
        kv_lens, kv_lens_host, sm_scale = _lens_t(lens, cuda_device), list(lens), d ** -0.5
    results = {}
    for fold in (False, True):
        for kw in (dict(), dict(kv_split=1), dict(kv_split=5)):
            out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                        k_scale=inp.k_scale, v_scale=inp.v_scale, fp8_fold_k_scale=fold, **kw)
            torch.cuda.synchronize()
            results[(fold, tuple(kw.items()))] = (out.clone(), lse.clone())
    kd = ofp8.dequant_per_head(inp.k_cache, inp.k_scale)
    vd = ofp8.dequant_per_head(inp.v_cache, inp.v_scale)
    ref = ref_paged_attn(inp.q, kd, vd, inp.kv_lens_host, inp.block_table, inp.sm_scale)
    _, l_deq = cf.attn_fp64(inp.q, kd, vd, inp.block_table, inp.kv_lens_host, inp.sm_scale)
    o64, l64 = cf.attn_fp64(inp.q, inp.k_cache.float(), inp.v_cache.float(), inp.block_table, inp.kv_lens_host,
                            inp.sm_scale, k_scale=inp.k_scale, v_scale=inp.v_scale)
    for (fold, kw), (out, lse) in results.items():
        assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all(), (fold, kw)
        torch.testing.assert_close(out.float(), ref.float(), atol=OUT_ATOL, rtol=OUT_RTOL, msg=lambda m: f"fold={fold} {kw}: {m}")
        if fold:
            torch.testing.assert_close(lse.double(), l64, atol=LSE_ATOL, rtol=0, msg=lambda m: f"folded vs exact cache {kw}: {m}")
            torch.testing.assert_close(out.double(), o64, atol=8e-3, rtol=1e-2)
            torch.testing.assert_close(lse.double(), l_deq, atol=5e-3, rtol=0)
        else:
            torch.testing.assert_close(lse.double(), l_deq, atol=LSE_ATOL, rtol=0, msg=lambda m: f"default form {kw}: {m}")
    # the flag changes nothing for a 16-bit cache
    k16, v16 = kd.contiguous(), vd.contiguous()
    a = tda.flash_decode(inp.q, k16, v16, inp.block_table, inp.kv_lens, inp.sm_scale)
    b = tda.flash_decode(inp.q, k16, v16, inp.block_table, inp.kv_lens, inp.sm_scale, fp8_fold_k_scale=True)
    torch.cuda.synchronize()
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("algo", ["valu", "mfma"])
def test_fp8_every_byte_value_dequantises_exactly(cuda_device, algo):
    # 254 finite e4m3 codes as single-token V rows: out must equal table[code] * scale bit-exactly in fp32
    table = torch.from_numpy(ofp8.e4m3fn_table())
    codes = torch.tensor([c for c in range(256) if not math.isnan(table[c])], dtype=torch.uint8)
    n = codes.numel()
    v8 = codes.view(n, 1, 1, 1).expand(n, 1, 1, 128).contiguous().view(torch.float8_e4m3fn).to(cuda_device)
    k8 = torch.zeros_like(v8)
    q = torch.zeros(n, 1, 128, dtype=torch.bfloat16, device=cuda_device)
    scale = torch.tensor([0.75], device=cuda_device)
    bt = torch.arange(n, dtype=torch.int32, device=cuda_device)[:, None].contiguous()
    out = torch.empty(n, 1, 128, dtype=torch.float32, device=cuda_device)
    tda.flash_decode(q, k8, v8, bt, _lens_t([1] * n, cuda_device), 1.0, k_scale=scale, v_scale=scale, out=out, algo=algo)
    torch.cuda.synchronize()
    want = (table[codes.long()] * 0.75).to(cuda_device)
    assert torch.equal(out[:, 0, 0], want) and torch.equal(out[:, 0, 127], want)


@pytest.mark.parametrize("dims,heads", [((128, 128), (4, 1)), ((192, 128), (4, 2)), ((576, 512), (4, 1)), ((576, 512), (40, 1))])
@pytest.mark.parametrize("k_scale", [1.0, 0.5, 2.0 ** -7, 8.0, 0.75])
def test_fp8_k_scales_that_are_powers_of_two(cuda_device, dims, heads, k_scale):
    """A K scale that is a power of two goes into the conversion instruction as an exponent instead of a multiplication per
    value: the logit of a one-hot query over a single token is the dequantised K value, for every e4m3 code, in every
    kernel family (one-segment, two-segment, shared tiles); 0.75 takes the multiplications, as a control."""
    dk, dv = dims
    hq, hkv = heads
    table = torch.from_numpy(ofp8.e4m3fn_table())
    codes = torch.tensor([c for c in range(256) if not math.isnan(table[c])], dtype=torch.uint8)
    n = codes.numel()
    # sequence i: one token whose K row holds code i everywhere; q head h is one-hot at column 37 h + 5
    k8 = codes.view(n, 1, 1, 1).expand(n, 1, hkv, dk).contiguous().view(torch.float8_e4m3fn).to(cuda_device)
    v8 = torch.zeros(n, 1, hkv, dv, dtype=torch.uint8).view(torch.float8_e4m3fn).to(cuda_device)
    q = torch.zeros(n, hq, dk, dtype=torch.bfloat16)
    for h in range(hq):
        q[:, h, (37 * h + 5) % dk] = 1.0
    q = q.to(cuda_device)
    ks = torch.full((hkv,), k_scale, device=cuda_device)
    vs = torch.ones(hkv, device=cuda_device)
    bt = torch.arange(n, dtype=torch.int32, device=cuda_device)[:, None].contiguous()
    sm = 0.125
    out, lse = tda.flash_decode(q, k8, v8, bt, _lens_t([1] * n, cuda_device), sm, k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    want = (table[codes.long()].double() * k_scale).to(torch.bfloat16).double() * sm       # (exact in bf16 for powers of two)
    got = lse.double().cpu()
    assert float(out.abs().max()) == 0
    for h in (0, hq - 1):
        torch.testing.assert_close(got[:, h], want, atol=2e-6, rtol=2e-6, msg=lambda m: f"dims={dims} k_scale={k_scale} head {h}: {m}")


# ---- the five benchmark configurations at full size ----------------------------------------------------------------
_INPUT_CACHE = {}


def _full_config(name, cuda_device, algo="auto", **hints):
    if name not in _INPUT_CACHE:
        _INPUT_CACHE.clear()                         # one configuration resident at a time
        print(f"config {name}: generating", flush=True)
        _INPUT_CACHE[name] = wl.make_inputs(name, cuda_device)
    inp = _INPUT_CACHE[name]
    print(f"config {name}: decode ({algo})", flush=True)
    out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                k_scale=inp.k_scale, v_scale=inp.v_scale, algo=algo, **hints)
    torch.cuda.synchronize()
    assert out.shape == inp.q.shape and out.dtype == inp.q.dtype and lse.dtype == torch.float32
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    return inp, out, lse


def _check_rows(inp, out, lse, rows, tag):
    """Oracle comparison on a subset of sequences (the oracle runs on the GPU tensors, one sequence at a time)."""
    k, v = inp.k_cache, inp.v_cache
    for b in rows:
        sl = slice(b, b + 1)
        lens = [inp.kv_lens_host[b]]
        if inp.cfg.kv_dtype == "fp8_e4m3":
            # dequantise only the pages this sequence uses
            n_pg = (lens[0] + inp.cfg.page_size - 1) // inp.cfg.page_size
            ids = inp.block_table[b, :n_pg].long()
            kd = ofp8.dequant_per_head(k[ids], inp.k_scale)
            vd = ofp8.dequant_per_head(v[ids], inp.v_scale)
            tbl = torch.arange(n_pg, dtype=torch.int32, device=k.device)[None]
            _check(out[sl], lse[sl], inp.q[sl], kd, vd, tbl, lens, inp.sm_scale, tag=f"{tag} b={b}")
        else:
            _check(out[sl], lse[sl], inp.q[sl], k, v, inp.block_table[sl], lens, inp.sm_scale, tag=f"{tag} b={b}")


@pytest.mark.parametrize("algo", ["auto", "valu", "mfma"])
def test_config1_tiny(cuda_device, algo):
    inp, out, lse = _full_config("tiny", cuda_device, algo)
    assert out.shape == (2, 8, 128) and lse.shape == (2, 8)
    _check_rows(inp, out, lse, range(2), "tiny")


@pytest.mark.parametrize("algo", ["auto", "valu", "mfma"])
def test_config2_llama3_8b_b32(cuda_device, algo):
    inp, out, lse = _full_config("llama3_8b_b32", cuda_device, algo)
    _check_rows(inp, out, lse, range(32) if algo == "auto" else range(0, 32, 5), "cfg2")


def _hinted_single_pass(cuda_device, name, rows):
    # bench.py passes the host-known length bounds: equal bounds say that the sequences are alike, which is what a
    # single pass (whole sequences per workgroup, no partial rows, no combine launch) needs; without them the same
    # configuration runs as equal shares
    cfg = wl.CONFIGS[name]
    hints = dict(max_kv_len=cfg.kv_len, min_kv_len=cfg.kv_len)
    inp, out, lse = _full_config(name, cuda_device, **hints)
    plan = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, **hints)
    assert not plan.balanced and plan.num_splits == 1
    assert tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens).balanced
    _check_rows(inp, out, lse, rows, f"{name} hinted")


def test_config2_llama3_8b_b32_with_the_length_hints_of_the_benchmark(cuda_device):
    _hinted_single_pass(cuda_device, "llama3_8b_b32", range(0, 32, 3))


@pytest.mark.parametrize("algo", ["auto", "valu"])
def test_config3_ragged_g8(cuda_device, algo):
    inp, out, lse = _full_config("ragged_g8", cuda_device, algo)
    _check_rows(inp, out, lse, range(64) if algo == "auto" else range(0, 64, 7), "cfg3")


@pytest.mark.parametrize("algo", ["auto", "valu"])
def test_config4_long_131k(cuda_device, algo):
    inp, out, lse = _full_config("long_131k", cuda_device, algo)
    _check_rows(inp, out, lse, range(4) if algo == "auto" else [3], "cfg4")


@pytest.mark.parametrize("algo", ["auto", "valu"])
def test_config5_fp8_70b_b128(cuda_device, algo):
    inp, out, lse = _full_config("fp8_70b_b128", cuda_device, algo)
    _check_rows(inp, out, lse, range(0, 128, 9) if algo == "auto" else [5, 100], "cfg5")


def test_config5_fp8_70b_b128_folded_k_scale(cuda_device):
    # the folded form of the fp8 K scale against the SAME oracle and bars as the default form (dequantise to bf16, then
    # decode: out 2e-2, lse 1e-3): 8192 tokens per sequence average the 16-bit rounding of K away
    cfg = wl.CONFIGS["fp8_70b_b128"]
    for hints in (dict(), dict(max_kv_len=cfg.kv_len, min_kv_len=cfg.kv_len)):
        inp, out, lse = _full_config("fp8_70b_b128", cuda_device, fp8_fold_k_scale=True, **hints)
        _check_rows(inp, out, lse, range(0, 128, 13), f"cfg5 folded {hints}")


def test_config5_fp8_70b_b128_with_the_length_hints_of_the_benchmark(cuda_device):
    _hinted_single_pass(cuda_device, "fp8_70b_b128", range(0, 128, 11))


def test_config4_long_131k_with_the_length_hints_of_the_benchmark(cuda_device):
    # bench.py passes the host-known length bounds: equal bounds select per-sequence chunks instead of balanced shares
    cfg = wl.CONFIGS["long_131k"]
    hints = dict(max_kv_len=cfg.kv_len, min_kv_len=cfg.kv_len)
    inp, out, lse = _full_config("long_131k", cuda_device, **hints)
    plan = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, **hints)
    assert not plan.balanced and plan.num_splits > 1
    _check_rows(inp, out, lse, range(4), "cfg4 hinted")


# ---- the shape of the reference's published figure (README.md:200-202; test_sp_decode_attn.py:203-220):
# batch 1, 96 q / 12 kv heads, fp16, page size 1, local KV 8K ... 128K, at full size ----------------------------
@pytest.mark.parametrize("name", wl.REF_SHAPE_ORDER)
def test_reference_published_shape(cuda_device, name):
    inp, out, lse = _full_config(name, cuda_device)
    assert out.dtype == torch.float16 and out.shape == (1, 96, 128)
    _check_rows(inp, out, lse, [0], name)
    # what the reference's layer passes: 32 forced splits, packed output (sp_flash_decode_layer.py:62,100-110)
    packed = tda.gqa_fwd_batch_decode_intra_rank(inp.q, inp.k_cache, inp.v_cache, None, [1], inp.kv_lens,
                                                 inp.block_table, inp.sm_scale, kv_split=32)
    torch.cuda.synchronize()
    torch.testing.assert_close(packed[..., :128].float(), out.float(), atol=2e-3, rtol=1e-2)
    torch.testing.assert_close(packed[..., 128].float(), lse, atol=2e-2, rtol=1e-2)      # lse rounded to fp16


# ---- single launch: the last workgroup of a (sequence, head block, head tile) merges its pieces ----------------------
# (the reference's persistent kernel merges after a grid barrier, flash_decode.py:719-760)
FUSED_CASES = {
    # name: (batch, hq, hkv, head_dim, page, kv_lens or (lo, hi), kv dtype, kv_split)
    "chunks_short": (3, 32, 8, 128, 16, [700, 64, 1], torch.bfloat16, -1),
    "chunks_forced_32": (5, 32, 8, 128, 16, [4000, 1, 17, 2049, 333], torch.bfloat16, 32),
    "chunks_more_splits_than_tokens": (2, 8, 2, 128, 1, [5, 70], torch.float16, 64),
    "queue_many_items": (12, 32, 8, 128, 16, (1, 3000), torch.bfloat16, 24),
    "balanced_ragged": (9, 8, 1, 128, 16, [30000, 1, 0, 777, 12000, 64, 65, 0, 5000], torch.bfloat16, -1),
    "balanced_all_but_one_empty": (4, 16, 2, 128, 16, [0, 0, 70000, 0], torch.bfloat16, -1),
    "balanced_two_tiles_d64": (3, 48, 2, 64, 16, [40000, 60000, 40], torch.float16, -1),
    "balanced_fp8_d256": (2, 16, 4, 256, 16, [60000, 30000], "fp8", -1),
    "ref_shape_p1": (1, 96, 12, 128, 1, [6000], torch.float16, -1),
}


@pytest.mark.parametrize("name", list(FUSED_CASES))
def test_single_launch_decode_against_the_oracle_and_the_two_launch_form(cuda_device, name):
    batch, hq, hkv, d, page, lens, dt, kv_split = FUSED_CASES[name]
    g = torch.Generator().manual_seed(sum(map(ord, name)))
    if isinstance(lens, tuple):
        lens = torch.randint(lens[0], lens[1] + 1, (batch,), generator=g).tolist()
    fp8 = dt == "fp8"
    qdt = torch.bfloat16 if fp8 else dt
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 4
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((batch, max(max(pages), 1)), -1, dtype=torch.int32)        # poison: never used as a page
    pos = 0
    for b, n_pg in enumerate(pages):
        table[b, :n_pg] = perm[pos:pos + n_pg]
        pos += n_pg
    q = torch.randn(batch, hq, d, generator=g).to(qdt).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(qdt)
    v = torch.randn(pool, page, hkv, d, generator=g).to(qdt)
    ks = vs = None
    ref_kv = None
    if fp8:
        k8, ks = wl.quantize_kv_fp8(k)
        v8, vs = wl.quantize_kv_fp8(v)
        ref_kv = (ofp8.dequant_per_head(k8, ks).to(cuda_device), ofp8.dequant_per_head(v8, vs).to(cuda_device))
        k, v, ks, vs = k8, v8, ks.to(cuda_device), vs.to(cuda_device)
    k, v, table = k.to(cuda_device), v.to(cuda_device), table.to(cuda_device)
    lens_t = _lens_t(lens, cuda_device)
    scale = d ** -0.5
    kw = dict(kv_split=kv_split, k_scale=ks, v_scale=vs, max_kv_len=max(max(lens), 1),
              force_balanced=name.startswith("balanced"))
    two = tda.prepare_decode(q, k, v, table, lens_t, scale, work_queue=False, **kw)
    one = tda.prepare_decode(q, k, v, table, lens_t, scale, single_launch=True, **kw)
    assert one.plan.num_splits > 1 and one.args.counters and not two.args.counters, one.plan
    if name.startswith("balanced"):
        assert one.plan.balanced
    o2, l2 = [t.clone() for t in two.run()]
    first = None
    for it in range(25):                  # the merging workgroup changes from run to run; the result must not
        one.out.fill_(float("nan"))
        one.lse.fill_(float("nan"))
        o1, l1 = one.run()
        torch.cuda.synchronize()
        if first is None:
            first = (o1.clone(), l1.clone())
        assert torch.equal(o1, first[0]) and torch.equal(l1, first[1]), f"{name}: run {it} differs from run 0"
    live = [b for b in range(batch) if lens[b] > 0]
    dead = [b for b in range(batch) if lens[b] == 0]
    torch.testing.assert_close(o1[live].float(), o2[live].float(), atol=2e-3, rtol=2 ** -7)
    torch.testing.assert_close(l1[live], l2[live], atol=2e-6, rtol=1e-6)
    if dead:
        assert torch.all(o1[dead] == 0) and torch.all(l1[dead] == float("-inf"))
    _check(o1[live], l1[live], q[live], k, v, table[live], [lens[b] for b in live], scale, ref_kv=ref_kv, tag=name)
    assert int(one._keep[-1].abs().sum()) == 0                  # the counters are back at zero


def test_reference_entry_points_read_kv_split_as_an_upper_bound(cuda_device):
    # the reference's layer passes kv_split = 32 for every shape (sp_flash_decode_layer.py:62)
    import importlib
    fd = importlib.import_module("triton_distributed_amd.flash_decode")
    big = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=40, kv_len=600), cuda_device)
    one = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=1, kv_len=16000), cuda_device)
    args = lambda i: (i.q, i.k_cache, i.v_cache, i.block_table, i.kv_lens, i.sm_scale, 0.0)
    assert fd._reference_kv_split(32, *args(big))[0] == -1          # 40 x 8 units fill the GPU: one pass, no chunks
    assert fd._reference_kv_split(-1, *args(big)) == (-1, None)
    own = tda.get_split_kv_plan(one.q, one.k_cache, one.v_cache, one.block_table, one.kv_lens)
    assert own.num_splits > 4 and fd._reference_kv_split(4, *args(one)) == (4, None)       # fewer than the library would take: forced
    assert fd._reference_kv_split(1024, *args(one))[0] == -1
    for inp in (big, one):
        packed = tda.gqa_fwd_batch_decode_intra_rank(inp.q, inp.k_cache, inp.v_cache, None, None, inp.kv_lens,
                                                     inp.block_table, inp.sm_scale, kv_split=32)
        out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale, kv_split=32)
        torch.cuda.synchronize()
        torch.testing.assert_close(packed[..., :128].float(), out.float(), atol=4e-3, rtol=2 ** -7)


def test_load_only_probes_run_and_leave_the_inputs_alone(cuda_device):
    # measurement aids (bench.py --op ceiling): they produce no results, but must run on every plan mode and read only
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=9, kv_len_range=(1, 9000)), cuda_device)
    k0, v0, q0 = inp.k_cache.clone(), inp.v_cache.clone(), inp.q.clone()
    for kw in (dict(), dict(kv_split=8), dict(kv_split=1)):
        call = tda.prepare_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                  probe_loads=True, always_workspace=True, **kw)
        call.run()
        call.run_splitkv()
    buf = torch.arange(1 << 22, dtype=torch.int32, device=cuda_device)
    ref = buf.clone()
    tda.probe_linear_read(buf, nontemporal=True)
    tda.probe_linear_read(buf, nontemporal=False, workgroups=64)
    torch.cuda.synchronize()
    assert torch.equal(buf, ref) and torch.equal(inp.k_cache, k0) and torch.equal(inp.v_cache, v0) and torch.equal(inp.q, q0)
    # the real call right after a probe call on the same buffers is unaffected
    out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale)
    torch.cuda.synchronize()
    _check(out, lse, inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens_host, inp.sm_scale, tag="after probe")


def test_shared_scratch_of_a_foreign_stream_is_not_reused_by_the_current_one(cuda_device):
    # flash_decode(..., stream=side) keeps its split partials in a buffer shared by the calls of that stream and grows
    # it on demand.  The buffer belongs to the side stream's memory pool: while the side stream's kernels still write
    # partial rows, the default stream allocates and fills tensors of the very sizes that were just dropped - they must
    # never be handed the memory of a buffer that is still in use.
    side = torch.cuda.Stream(device=cuda_device)
    cases = []
    for i, (b, n) in enumerate([(1, 3000), (2, 9000), (3, 20000), (5, 40000)]):       # growing workspaces
        inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=b, kv_len_range=(n // 2, n)), cuda_device)
        plan = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens)
        assert plan.num_splits > 1, (b, n)
        cases.append((inp, plan.workspace_bytes))
    assert [w for _, w in cases] == sorted(w for _, w in cases) and cases[0][1] < cases[-1][1]
    torch.cuda.synchronize()
    results, hogs = [], []
    side.wait_stream(torch.cuda.current_stream())
    for rep in range(3):
        for inp, ws in cases:
            out, lse = tda.flash_decode(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, inp.sm_scale,
                                        stream=side)
            results.append((inp, out, lse))
            # the default stream, unsynchronised with the side stream: same-sized allocations, filled at once
            for nbytes in {w for _, w in cases}:
                hogs.append(torch.full((nbytes,), 0x7f, dtype=torch.uint8, device=cuda_device))
            hogs = hogs[-8:]
        import importlib
        fd = importlib.import_module("triton_distributed_amd.flash_decode")
        fd._SCRATCH_CACHE.clear()                  # the next round grows the buffer again from the smallest size
    side.synchronize()
    torch.cuda.synchronize()
    for i, (inp, out, lse) in enumerate(results):
        _check(out, lse, inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens_host, inp.sm_scale,
               tag=f"foreign stream call {i}")


def test_captured_drop_in_call_with_feedback_follows_grown_lengths(cuda_device):
    # A drop-in entry point that is given a LengthFeedback block plans with the bounds the previous call left there -
    # but not while its stream is capturing: a graph is replayed while kv_lens grows, and bounds baked into it (here
    # about 500 tokens) would size the chunks of every replay, the last chunk taking all the rest.  Capture at N,
    # replay at about 8 N: right result, and no slower than a few times the eager call planned for that length.
    import time
    b, hq, hkv, d, page, n0, n1 = 4, 32, 8, 128, 16, 500, 4000
    g = torch.Generator().manual_seed(77)
    pages = (n1 + page - 1) // page
    pool = b * pages
    q = torch.randn(b, hq, d, generator=g).to(torch.bfloat16).to(cuda_device)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16).to(cuda_device)
    table = torch.randperm(pool, generator=g).to(torch.int32).view(b, pages).to(cuda_device)
    lens = torch.full((b,), n0, dtype=torch.int32, device=cuda_device)
    fb = tda.LengthFeedback()
    oc = torch.empty(b, hq, d + 1, dtype=torch.bfloat16, device=cuda_device)
    call = lambda: tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, None, lens, table, d ** -0.5, output_combine=oc,
                                                       kv_split=32, length_feedback=fb)
    for _ in range(3):                                  # eager warm-up: the block now holds (n0, n0)
        call()
        torch.cuda.synchronize()
    assert fb.bounds(b) == (n0, n0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    lens.fill_(n1)
    oc.fill_(float("nan"))
    graph.replay()
    torch.cuda.synchronize()
    assert fb.bounds(b) == (n1, n1)                     # the replay still reports what it ran on
    out, lse = oc[..., :d].clone(), oc[..., d].float().clone()
    ref = ref_paged_attn(q, k, v, [n1] * b, table, d ** -0.5)
    torch.testing.assert_close(out.float(), ref.float(), atol=OUT_ATOL, rtol=OUT_RTOL)
    _, l64 = cf.attn_fp64(q, k, v, table, [n1] * b, d ** -0.5)
    torch.testing.assert_close(lse.double(), l64, atol=5e-2, rtol=1e-2)      # lse went through bf16 in the packed row

    def timed(fn, n=20):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n
    t_graph = timed(graph.replay)
    t_eager = timed(lambda: tda.flash_decode(q, k, v, table, lens, d ** -0.5, max_kv_len=n1, min_kv_len=n1))
    assert t_graph < 4 * t_eager + 50e-6, (t_graph, t_eager)
