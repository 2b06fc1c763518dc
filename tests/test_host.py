"""Host-side logic that needs no GPU: argument checks of the Python entry points, the packed layout helpers,
the workload generators and their byte accounting."""
import pytest
import torch

import triton_distributed_amd as tda
from triton_distributed_amd import workloads as wl


def _cpu_inputs(b=2, hq=8, hkv=2, d=128, page=4, pages=8, dtype=torch.bfloat16):
    q = torch.zeros(b, hq, d, dtype=dtype)
    k = torch.zeros(pages, page, hkv, d, dtype=dtype)
    v = torch.zeros(pages, page, hkv, d, dtype=dtype)
    table = torch.zeros(b, 4, dtype=torch.int32)
    lens = torch.ones(b, dtype=torch.int32)
    return q, k, v, table, lens


def test_no_cpu_path():
    q, k, v, table, lens = _cpu_inputs()
    with pytest.raises(ValueError, match="no CPU path"):
        tda.flash_decode(q, k, v, table, lens, 0.1)
    with pytest.raises(ValueError, match="no CPU path"):
        tda.gqa_fwd_batch_decode_intra_rank(q, k, v, None, [1, 1], lens, table, 0.1)
    with pytest.raises(ValueError, match="no CPU path"):
        tda.inter_rank_combine(torch.zeros(2, 2, 8, 129, dtype=torch.bfloat16), torch.ones(2, 2, dtype=torch.int32))


def test_shape_and_dtype_checks_mirror_the_reference_asserts():
    q, k, v, table, lens = _cpu_inputs()
    with pytest.raises(AssertionError):                       # Hq % Hkv, flash_decode.py:860
        tda.get_split_kv_plan(q[:, :7], k, v, table, lens)
    with pytest.raises(AssertionError):                       # page size / kv heads mismatch, :851
        tda.get_split_kv_plan(q, k, v[:, :2], table, lens)
    with pytest.raises(ValueError):
        tda.get_split_kv_plan(q, k, v, table.long(), lens)
    with pytest.raises(ValueError):
        tda.get_split_kv_plan(q, k, v, table[:1], lens)
    with pytest.raises(ValueError):
        tda.get_split_kv_plan(q.float(), k, v, table, lens)
    q2, k2, v2, t2, l2 = _cpu_inputs(d=256)                   # head_dim 256 is in the reference grid
    assert tda.get_split_kv_plan(q2, k2, v2, t2, l2).algo == "mfma"
    with pytest.raises(ValueError):                           # the vector path is built for head_dim 128 only
        tda.get_split_kv_plan(q2, k2, v2, t2, l2, algo="valu")
    with pytest.raises(ValueError):
        q3, k3, v3, t3, l3 = _cpu_inputs(d=96)
        tda.get_split_kv_plan(q3, k3, v3, t3, l3)
    with pytest.raises(ValueError):
        tda.get_split_kv_plan(q.transpose(1, 2).contiguous().transpose(1, 2), k, v, table, lens)


def test_plan_from_tensors():
    inp = wl.make_inputs(wl.scaled_down(wl.CONFIGS["llama3_8b_b32"], batch=2, kv_len=4096))
    p = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, num_cus=256)
    assert p.algo == "mfma" and p.num_splits * p.chunk_tokens >= 4096 and p.workspace_bytes > 0
    p32 = tda.get_split_kv_plan(inp.q, inp.k_cache, inp.v_cache, inp.block_table, inp.kv_lens, kv_split=32, num_cus=256)
    assert p32.num_splits == 32


def test_pack_unpack_layout():
    out = torch.randn(3, 4, 128).to(torch.bfloat16)
    lse = torch.randn(3, 4)
    packed = tda.pack_out_lse(out, lse)
    assert packed.shape == (3, 4, 129) and packed.dtype == torch.bfloat16
    o2, l2 = tda.unpack_out_lse(packed)
    assert torch.equal(o2, out) and torch.equal(l2, lse.to(torch.bfloat16))
    assert tda.pack_out_lse(out, lse, torch.float32).dtype == torch.float32


def test_algorithmic_bytes_match_the_hand_computed_figures():
    # bytes per call of the uniform-length configurations: KV + q + out + lse + table entries used + lengths (+ scales)
    assert wl.make_inputs("tiny").algorithmic_bytes() == 1_060_936

    def bytes_of(name):
        c = wl.CONFIGS[name]
        inp = wl.DecodeInputs(c, None, None, None, None, None, 0.0, kv_lens_host=[c.kv_len] * c.batch)
        return inp.algorithmic_bytes()

    assert bytes_of("llama3_8b_b32") == 537_432_192
    assert bytes_of("long_131k") == 2_147_648_528
    assert bytes_of("fp8_70b_b128") == 2_151_973_440


def test_workload_generator_layout():
    cfg = wl.scaled_down(wl.CONFIGS["ragged_g8"], batch=6, kv_len_range=(1, 300))
    a, b = wl.make_inputs(cfg, poison_tail=True), wl.make_inputs(cfg, poison_tail=True)
    assert torch.equal(a.q, b.q) and torch.equal(a.block_table, b.block_table)       # seeded
    used = []
    for i, n in enumerate(a.kv_lens_host):
        n_pg = (n + 15) // 16
        used += a.block_table[i, :n_pg].tolist()
        tail = a.block_table[i, n_pg:]
        assert ((tail == 2**31 - 1) | (tail == -1)).all()
    assert len(set(used)) == len(used) and max(used) < a.k_cache.shape[0] and min(used) >= 0   # no page shared
    assert a.k_cache.shape[1:] == (16, 1, 128) and a.q.shape == (6, 8, 128)


def test_fp8_workload_quantisation():
    cfg = wl.scaled_down(wl.CONFIGS["fp8_70b_b128"], batch=2, kv_len=64)
    inp = wl.make_inputs(cfg)
    assert inp.k_cache.dtype == torch.float8_e4m3fn and inp.k_scale.shape == (8,) and inp.k_scale.dtype == torch.float32
    assert float(inp.k_cache.float().abs().amax()) == 448.0
    x = torch.randn(5, 16, 8, 128).to(torch.bfloat16)
    x8, s = wl.quantize_kv_fp8(x, chunk_pages=2)
    torch.testing.assert_close(s, x.float().abs().amax(dim=(0, 1, 3)) / 448.0)
    assert torch.equal(x8.view(torch.uint8), (x.float() / s[None, None, :, None]).to(torch.float8_e4m3fn).view(torch.uint8))
