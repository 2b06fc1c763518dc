"""Small seeded decode cases shared by the golden-vector generator and the tests that read the vectors."""
import torch

from triton_distributed_amd.workloads import CONFIGS, make_inputs

# name -> (kv_lens, (Hq, Hkv), page_size, dtype, soft_cap, seed)
EDGE_CASES = {
    "len1_p1": ([1, 1, 1], (8, 2), 1, torch.bfloat16, 0.0, 21),
    "short_p16": ([1, 2, 31, 32, 33, 63, 64, 65], (32, 8), 16, torch.bfloat16, 0.0, 22),
    "ref_grid_a_p16": ([1320, 18, 463], (32, 8), 16, torch.float16, 0.0, 23),
    "ref_grid_b_p1": ([1, 54, 293, 70], (6, 1), 1, torch.float16, 30.0, 24),
    "mha_p16_cap50": ([70, 293], (16, 16), 16, torch.bfloat16, 50.0, 25),
    "g8_p64": ([777, 64, 129], (8, 1), 64, torch.bfloat16, 0.0, 26),
    "g16_p16": ([300, 5], (16, 1), 16, torch.bfloat16, 0.0, 27),
    "odd_page6": ([100, 7, 36], (8, 2), 6, torch.bfloat16, 0.0, 28),
}


def edge_case(name):
    lens, (hq, hkv), page, dtype, cap, seed = EDGE_CASES[name]
    g = torch.Generator().manual_seed(seed)
    d = 128
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 5
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((len(lens), max(pages) + 1), 2**31 - 1, dtype=torch.int32)   # poisoned tail
    pos = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[pos:pos + n]
        pos += n
    q = torch.randn(len(lens), hq, d, generator=g).to(dtype)
    k = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    v = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
    return dict(q=q, k_cache=k, v_cache=v, block_table=table, kv_lens=lens, sm_scale=d ** -0.5, soft_cap=cap)


def tiny_config():
    inp = make_inputs("tiny")
    return dict(q=inp.q, k_cache=inp.k_cache, v_cache=inp.v_cache, block_table=inp.block_table,
                kv_lens=inp.kv_lens_host, sm_scale=inp.sm_scale, soft_cap=0.0)


def all_cases():
    yield "tiny", tiny_config()
    for name in EDGE_CASES:
        yield name, edge_case(name)
