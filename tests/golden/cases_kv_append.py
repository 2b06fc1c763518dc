"""Small seeded cases of the RMSNorm + rotary + paged-append operator, shared by make_golden_kv_append.py, the CPU
test that freezes the oracle and the GPU test that compares the kernel with the same vectors."""
import torch

# name: (kv_lens after the append, new tokens, (Hq, Hkv), head_dim, page, dtype, fp8 cache, seed)
KV_APPEND_CASES = {
    "bf16_d128_p16_t2": ([2, 40, 19], 2, (8, 2), 128, 16, torch.bfloat16, False, 41),
    "fp16_d64_p1_t1": ([1, 33], 1, (4, 4), 64, 1, torch.float16, False, 42),
    "bf16_d256_p6_t3": ([3, 20], 3, (4, 1), 256, 6, torch.bfloat16, False, 43),
    "fp8_d128_p16_t1": ([7, 64, 65], 1, (8, 2), 128, 16, torch.bfloat16, True, 44),
}


def kv_append_case(name):
    lens, t, (hq, hkv), d, page, dtype, fp8, seed = KV_APPEND_CASES[name]
    g = torch.Generator().manual_seed(seed)
    b = len(lens)
    qkv = torch.randn(b, t, hq + 2 * hkv, d, generator=g).to(dtype)
    wq = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    wk = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    pages = [(n + page - 1) // page for n in lens]
    pool = sum(pages) + 2
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.zeros(b, max(pages) + 1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(pages):
        table[i, :n] = perm[at:at + n]
        at += n
    if fp8:
        k = torch.zeros(pool, page, hkv, d, dtype=torch.float8_e4m3fn)
        v = torch.zeros(pool, page, hkv, d, dtype=torch.float8_e4m3fn)
        k_scale = torch.tensor([0.011, 0.017][:hkv], dtype=torch.float32)
        v_scale = torch.tensor([0.013, 0.009][:hkv], dtype=torch.float32)
    else:
        k = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
        v = torch.randn(pool, page, hkv, d, generator=g).to(dtype)
        k_scale = v_scale = None
    return dict(qkv=qkv, wq=wq, wk=wk, table=table, k=k, v=v, lens=lens, hq=hq, k_scale=k_scale, v_scale=v_scale,
                rope_theta=1000000.0, max_positions=max(lens) + 1)


def as_f32(t):
    """16-bit and fp8 tensors as float32 (exact), for storage and comparison."""
    return t.to(torch.float32).numpy()
