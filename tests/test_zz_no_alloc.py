"""fdk_decode_static: the decode entry point that allocates nothing (split partials in a static device array).

Checked through the C ABI against fdk_decode with a caller-owned workspace, which the other GPU tests pin to the
oracle: same plan, same kernels, so the results must be bit-identical.  Two calls in a row, the second with a
smaller input, so that stale contents of the shared scratch would show."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(batch, hq, hkv, d, page, lens, seed, dev):
    g = torch.Generator().manual_seed(seed)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 8
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.zeros(batch, max(max(pages), 1), dtype=torch.int32)
    pos = 0
    for b, n_pg in enumerate(pages):
        table[b, :n_pg] = perm[pos:pos + n_pg]
        pos += n_pg
    q = torch.randn(batch, hq, d, generator=g).to(torch.bfloat16)
    k = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16)
    v = torch.randn(pool, page, hkv, d, generator=g).to(torch.bfloat16)
    return (q.to(dev), k.to(dev), v.to(dev), table.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev))


@pytest.mark.parametrize("kv_split", [-1, 32])
def test_static_scratch_entry_matches_fdk_decode(kv_split):
    import triton_distributed_amd as tda
    from triton_distributed_amd import _lib
    from oracle.closed_form import attn_fp64

    dev = torch.device("cuda:0")
    lib = _lib.load()
    # first a larger problem, then a smaller one that reuses the front of the same scratch
    shapes = [(6, 32, 8, 128, 16, [3000, 1711, 64, 2999, 1, 905], 11),
              (2, 16, 2, 128, 16, [700, 333], 12)]
    for batch, hq, hkv, d, page, lens, seed in shapes:
        q, k, v, table, kv_lens = _inputs(batch, hq, hkv, d, page, lens, seed, dev)
        sm_scale = d ** -0.5
        ref_call = tda.prepare_decode(q, k, v, table, kv_lens, sm_scale, kv_split=kv_split, work_queue=False)
        assert ref_call.plan.num_splits > 1, "the case must use the scratch"
        out_ref, lse_ref = ref_call.run()
        torch.cuda.synchronize()
        out_ref, lse_ref = out_ref.clone(), lse_ref.clone()

        call = tda.prepare_decode(q, k, v, table, kv_lens, sm_scale, kv_split=kv_split, static_scratch=True)
        assert call.args.workspace is None and call.args.counters is None
        call.out.fill_(float("nan"))
        call.lse.fill_(float("nan"))
        torch.cuda.synchronize()
        rc = lib.fdk_decode_static(C.byref(call.args), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.fdk_last_error()
        torch.cuda.synchronize()
        assert torch.equal(call.out, out_ref)
        assert torch.equal(call.lse, lse_ref)
        # and the oracle itself, at the usual bars
        o64, l64 = attn_fp64(q.cpu(), k.cpu(), v.cpu(), table.cpu(), lens, sm_scale)
        torch.testing.assert_close(call.out.double().cpu(), o64, atol=8e-3, rtol=1e-2)
        torch.testing.assert_close(call.lse.double().cpu(), l64, atol=1e-3, rtol=0)


def test_static_scratch_rejects_plans_beyond_its_size():
    import triton_distributed_amd as tda
    from triton_distributed_amd import _lib

    dev = torch.device("cuda:0")
    lib = _lib.load()
    # 64 sequences x 64 q heads x 64 forced splits of fp32 partials: 64*64*64*129*4 B = 135 MB > 32 MiB
    q, k, v, table, kv_lens = _inputs(64, 64, 8, 128, 16, [4096] * 64, 13, dev)
    call = tda.prepare_decode(q, k, v, table, kv_lens, 0.1, kv_split=64, static_scratch=True)
    call.out.zero_()
    before = call.out.clone()
    rc = lib.fdk_decode_static(C.byref(call.args), torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.FDK_EWORKSPACE
    assert b"static scratch" in lib.fdk_last_error()
    torch.cuda.synchronize()
    assert torch.equal(call.out, before)          # nothing was launched
