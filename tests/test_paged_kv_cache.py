"""Host-side paged KV cache (the producer of block_table / kv_lens): CPU tests of the bookkeeping, and a GPU test
that runs a short multi-layer decode loop (prefill append, then token-by-token append + decode) against the oracle."""
import pytest
import torch

from triton_distributed_amd.paged_kv_cache import PagedKVCache, alloc_kv_pools


def test_tables_are_one_permutation_and_layers_share_the_pools():
    c = PagedKVCache(PAGE_SIZE=4, num_layers=3, batch_size=5, max_length=30, num_kv_heads=2, head_dim=64,
                     device="cpu", generator=torch.Generator().manual_seed(1))
    blocks = (30 + 3) // 4
    assert c.max_num_blocks_per_seq == blocks
    assert tuple(c.key_cache.shape) == (blocks * 5 * 3, 4, 2, 64) == tuple(c.value_cache.shape)
    assert tuple(c.block_tables.shape) == (3, 5, blocks) and c.block_tables.dtype == torch.int32
    # no page belongs to two sequences or two layers (paged_kv_cache.py:46-49 draws one permutation)
    assert sorted(c.block_tables.flatten().tolist()) == list(range(blocks * 5 * 3))
    k, v, table, lens = c.get_layer_kv_cache(2)
    assert k.data_ptr() == c.key_cache.data_ptr() and v.data_ptr() == c.value_cache.data_ptr()
    assert table.data_ptr() == c.block_tables[2].data_ptr() and lens.data_ptr() == c.kv_lens.data_ptr()
    assert not c.key_cache.any() and not c.value_cache.any()          # zero-filled by default
    assert c.nbytes == 2 * blocks * 5 * 3 * 4 * 2 * 64 * 2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
@pytest.mark.parametrize("shape", [(7, 16, 8, 128), (3, 1, 3, 64), (5, 64, 2, 256)])
def test_pools_share_an_allocation_with_the_v_pool_256_bytes_off_modulo_512(dtype, shape):
    # the placement that lets a workgroup's K and V streams reach different halves of MI355X's memory system
    k, v = alloc_kv_pools(shape, dtype, "cpu")
    assert k.shape == v.shape == torch.Size(shape) and k.dtype == v.dtype == dtype
    assert k.is_contiguous() and v.is_contiguous()
    assert (v.data_ptr() - k.data_ptr()) % 512 == 256
    nbytes = k.numel() * k.element_size()
    assert v.data_ptr() >= k.data_ptr() + nbytes                       # no overlap
    assert k.data_ptr() % 16 == 0 and v.data_ptr() % 16 == 0           # what the decode asks of a cache
    assert k.untyped_storage().data_ptr() == v.untyped_storage().data_ptr()
    assert float(k.float().abs().sum()) == 0.0 and float(v.float().abs().sum()) == 0.0
    cache = PagedKVCache(PAGE_SIZE=16, num_layers=2, batch_size=3, max_length=100, dtype=torch.bfloat16, device="cpu",
                         fill="randn", generator=torch.Generator().manual_seed(1))
    assert (cache.value_cache.data_ptr() - cache.key_cache.data_ptr()) % 512 == 256
    assert float(cache.key_cache.float().std()) > 0.9 and float(cache.value_cache.float().std()) > 0.9


def test_offsets_advance_on_device_and_host_together():
    c = PagedKVCache(PAGE_SIZE=16, num_layers=1, batch_size=3, max_length=40, device="cpu")
    assert c.max_kv_len == 0 and c.kv_lens.tolist() == [0, 0, 0] and c.kv_lens.dtype == torch.int32
    c.inc_offset(17)
    c.inc_offset(1)
    assert c.max_kv_len == 18 and c.kv_lens.tolist() == [18, 18, 18]
    with pytest.raises(ValueError, match="max_length"):
        c.inc_offset(23)
    assert c.max_kv_len == 18                                        # a refused step changes nothing
    c.inc_offset(22)
    c.reset()
    assert c.max_kv_len == 0 and c.kv_lens.tolist() == [0, 0, 0]


def test_a_seed_fixes_tables_and_contents_and_bad_arguments_are_refused():
    mk = lambda s, **kw: PagedKVCache(PAGE_SIZE=2, num_layers=2, batch_size=2, max_length=8, num_kv_heads=1, head_dim=64,
                                      device="cpu", generator=torch.Generator().manual_seed(s), **kw)
    a, b, c = mk(7, fill="randn"), mk(7, fill="randn"), mk(8, fill="randn")
    assert torch.equal(a.block_tables, b.block_tables) and torch.equal(a.key_cache, b.key_cache)
    assert not torch.equal(a.block_tables, c.block_tables)
    assert not torch.equal(a.key_cache, a.value_cache)
    with pytest.raises(ValueError):
        mk(1, fill="ones")
    with pytest.raises(ValueError):
        PagedKVCache(PAGE_SIZE=0, device="cpu")
    with pytest.raises(ValueError, match="k_scale"):
        mk(1, dtype=torch.float8_e4m3fn)
    with pytest.raises(ValueError, match="Hkv"):
        mk(1, dtype=torch.float8_e4m3fn, k_scale=torch.ones(2, 3), v_scale=torch.ones(2, 3))
    f = mk(1, dtype=torch.float8_e4m3fn, k_scale=torch.full((2, 1), 0.5), v_scale=torch.full((2, 1), 0.25))
    assert f.key_cache.dtype == torch.float8_e4m3fn and f.key_cache.element_size() == 1
    ks, vs = f.layer_scales(1)
    assert ks.tolist() == [0.5] and vs.tolist() == [0.25] and mk(1).layer_scales(0) == (None, None)
    with pytest.raises(ValueError, match="inc_offset"):
        mk(1).append(0, torch.zeros(2, 1, 3, 64), None, None, None, None)


@pytest.mark.gpu
@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_decode_loop_over_layers_matches_the_oracle(cuda_device, kv_dtype):
    import triton_distributed_amd as tda
    from oracle import closed_form as cf
    from oracle import fp8 as ofp8
    from oracle import kv_append as okv
    dev = cuda_device
    layers, b, hq, hkv, d, page, prefill, steps = 3, 4, 16, 4, 128, 16, 37, 4
    g = torch.Generator().manual_seed(77)
    fp8 = kv_dtype == torch.float8_e4m3fn
    ks = (0.02 + 0.01 * torch.rand(layers, hkv, generator=g)) if fp8 else None
    vs = (0.02 + 0.01 * torch.rand(layers, hkv, generator=g)) if fp8 else None
    cache = tda.PagedKVCache(PAGE_SIZE=page, num_layers=layers, batch_size=b, max_length=prefill + steps, num_kv_heads=hkv,
                             head_dim=d, dtype=kv_dtype, device=dev, generator=g, k_scale=ks, v_scale=vs)
    # the oracle works on host copies of the same (zeroed) pools and tables
    k_ref, v_ref = cache.key_cache.cpu().clone(), cache.value_cache.cpu().clone()
    tables = cache.block_tables.cpu()
    wq = (1.0 + 0.2 * torch.randn(layers, d, generator=g)).to(torch.bfloat16)
    wk = (1.0 + 0.2 * torch.randn(layers, d, generator=g)).to(torch.bfloat16)
    cos, sin = okv.cos_sin_tables(d, prefill + steps)
    cos_d, sin_d = cos.to(dev), sin.to(dev)
    tab8 = torch.from_numpy(ofp8.e4m3fn_table())
    n = 0
    for step, t in enumerate([prefill] + [1] * steps):
        cache.inc_offset(t)
        n += t
        assert cache.max_kv_len == n
        for layer in range(layers):
            print(f"case loop {kv_dtype} step={step} layer={layer} len={n}", flush=True)
            qkv = torch.randn(b, t, hq + 2 * hkv, d, generator=g).to(torch.bfloat16)
            q_ref = okv.kv_append(qkv, k_ref, v_ref, tables[layer], [n] * b, wq[layer], wk[layer], cos, sin, hq,
                                  k_scale=ks[layer] if fp8 else None, v_scale=vs[layer] if fp8 else None)
            q_out = cache.append(layer, qkv.to(dev), wq[layer].to(dev), wk[layer].to(dev), cos_d, sin_d)
            out, lse = cache.decode(layer, q_out[:, -1], d ** -0.5)
            torch.cuda.synchronize()
            if fp8:
                kf = (tab8[k_ref.view(torch.uint8).long()] * ks[layer].view(1, 1, hkv, 1)).to(torch.bfloat16)
                vf = (tab8[v_ref.view(torch.uint8).long()] * vs[layer].view(1, 1, hkv, 1)).to(torch.bfloat16)
            else:
                kf, vf = k_ref, v_ref
            o64, l64 = cf.attn_fp64(q_ref[:, -1], kf, vf, tables[layer], [n] * b, d ** -0.5)
            tol = 4e-2 if fp8 else 2e-2                      # fp8: a k row one rounding step apart is one e4m3 code apart
            torch.testing.assert_close(out.double().cpu(), o64, atol=tol, rtol=tol)
            torch.testing.assert_close(lse.double().cpu(), l64, atol=tol, rtol=0)
    if not fp8:
        # pages of other layers and unused slots were never written: v rows are bit-exact copies everywhere
        assert torch.equal(cache.value_cache.cpu(), v_ref)
