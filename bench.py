#!/usr/bin/env python3
"""Benchmark of the flash-decode hot path on one MI355X.

A "step" is one decode call (split-KV kernel + LSE combine) over one batch of synthetic, HBM-resident
inputs.  Default workload: the Llama-3-8B decode shape (batch 32, 32 q heads / 8 kv heads, head_dim 128,
kv_len 4096, page size 16, bf16).  Prints ONE JSON line:

  value          achieved HBM GB/s of the whole call = algorithmic bytes / measured time per call
  us_per_call    the same measurement as a latency
  roofline       the split-KV kernel alone against the 8 TB/s HBM peak, its launches timed with HIP
                 events on the launch stream
  cpu_baseline   the torch restatement of the reference's torch implementation on this box's host cores,
                 timed on a bounded sample of the same inputs (a baseline, not the target)

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--rotate R] [--kv-split S]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=-1,
                    help="untimed warm-up steps; never fewer than 100 calls and 0.1 s of them are run - the GPU clock needs "
                         "some tens of milliseconds of load to come up after the idle time of the input generation (the "
                         "JSON line reports the number run as warmup and the number asked for as warmup_requested)")
    ap.add_argument("--config", default="llama3_8b_b32")
    ap.add_argument("--rotate", type=int, default=2,
                    help="distinct KV pools cycled through, so the working set exceeds the 256 MB memory-side cache "
                         "(raised automatically until the pools together exceed 1 GB)")
    ap.add_argument("--kv-split", type=int, default=-1)
    ap.add_argument("--algo", default="auto", choices=["auto", "valu", "mfma"])
    ap.add_argument("--wavefronts", type=int, default=0, choices=[0, 4, 8],
                    help="measurement aid: wavefronts per workgroup of the matrix-core split kernel (0: the library's choice)")
    ap.add_argument("--shares-per-cu", type=int, default=0, choices=[0, 1, 2, 3, 4],
                    help="measurement aid: workgroups per compute unit of a balanced plan (0: the library's choice, 1)")
    ap.add_argument("--buffers", type=int, default=0, choices=[0, 1, 2],
                    help="measurement aid: register buffers (tiles of loads under way) per wavefront (0: the library's choice)")
    ap.add_argument("--no-hints", action="store_true",
                    help="do not pass the host-known length bounds (max_kv_len / min_kv_len): the plan of a caller that "
                         "knows nothing about the lengths")
    ap.add_argument("--batch", type=int, default=0, help="override the configuration's batch size")
    ap.add_argument("--kv-len", type=int, default=0, help="override the configuration's (uniform) kv_len")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay timing")
    ap.add_argument("--single-launch", action="store_true",
                    help="split plans: let the last workgroup of a (sequence, head block) merge the partials instead "
                         "of launching the combine kernel (FDK_FLAG_SINGLE_LAUNCH; slower on MI355X, for comparison)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="also run a plain device copy of this many MiB three times (a kernel of known traffic, "
                         "for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="budget of the CPU baseline sample")
    ap.add_argument("--kv-placement", default="staggered", choices=["staggered", "separate"],
                    help="where the K pool and the V pool of a call lie: staggered (default) = one allocation, the V pool "
                         "256 bytes off the K pool modulo 512, as this package's PagedKVCache allocates them "
                         "(triton_distributed_amd.alloc_kv_pools); separate = two independent torch allocations")
    ap.add_argument("--fp8-fold", action="store_true",
                    help="fp8 cache: apply the K scale to the logits instead of to every K value "
                         "(FDK_FLAG_FP8_FOLD_K_SCALE; off the dequantise-then-decode definition by the 16-bit rounding of K)")
    ap.add_argument("--fp8-pow2-scales", action="store_true",
                    help="fp8 cache: round the per-kv-head scales up to powers of two (as an unscaled cache has them: 1.0); "
                         "the library then applies the K scale as the exponent operand of the conversion, which is exact")
    ap.add_argument("--kernel-only", action="store_true",
                    help="time the prepared calls only: no legs on other pools, no graph replay, no un-prepared or "
                         "reference-named entry points, no CPU baseline - for profiler runs, so that every dispatch of a "
                         "kernel name in the trace belongs to the one plan and the one algorithm that was asked for")
    ap.add_argument("--batches", type=int, default=5,
                    help="the K timed steps are run this many times, each bracketed by synchronisations; the median "
                         "batch is reported (all of them are listed)")
    ap.add_argument("--no-separate-leg", action="store_true",
                    help="do not also time the calls on independently allocated pools (separate_pools_us_per_call); for "
                         "profiler runs, whose per-kernel averages should cover one placement only")
    ap.add_argument("--probe-loads", action="store_true", help="--op timeline: the load pipeline of the kernel only")
    ap.add_argument("--rotate-heads", type=int, default=0, metavar="R",
                    help="--op timeline: workgroup x of a sequence takes head block (x + R) mod (head blocks) - the same rows "
                         "are then read from other XCDs")
    ap.add_argument("--sweep-max-gb", type=float, default=6.0,
                    help="--op plan-sweep: skip cells whose KV cache exceeds this many GB (they stream for milliseconds and "
                         "every plan is a single pass)")
    ap.add_argument("--sweep-heads", default="32/8,64/8,8/1", help="--op plan-sweep: q/kv head pairs")
    ap.add_argument("--sweep-batches", default="1,4,8,16,24,32,40,64,128")
    ap.add_argument("--sweep-lens", default="1024,4096,16384,65536")
    ap.add_argument("--op", default="decode", choices=["decode", "kv_append", "ceiling", "timeline", "plan-sweep"],
                    help="decode: the hot path (default); kv_append: the step before it (RMSNorm + rotary + "
                         "paged append of one new token per sequence) at the same shape; ceiling: what the memory "
                         "system delivers for this configuration with no arithmetic in the way (a streaming read "
                         "of as many bytes, and the split kernel reduced to its load pipeline) next to the kernel; "
                         "timeline: when the wavefronts of the split kernel start, issue their first loads and finish, by "
                         "XCD and by kv head (needs the measurement build: python -m triton_distributed_amd.build --timeline); "
                         "plan-sweep: the library's plan against the plans it rejects (single pass, forced split counts, "
                         "equal shares) over a grid of batch sizes, lengths and head layouts, as a markdown table")
    return ap.parse_args()


def cpu_baseline(inp, budget_s: float):
    """Time oracle.paged_attn.ref_paged_attn on the host cores for a sample of sequences."""
    import torch
    from oracle.paged_attn import ref_paged_attn

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    lens = inp.kv_lens_host
    batch = len(lens)

    def run(rows):
        t0 = time.perf_counter()
        ref_paged_attn(inp.q[rows], inp.k_cache, inp.v_cache, [lens[i] for i in rows], inp.block_table[rows],
                       inp.sm_scale)
        return time.perf_counter() - t0

    # fp8 cache: the reference behaviour is "dequantise to bf16, then the same decode"; the sample pays
    # for the dequantisation of its own pages only.
    if inp.cfg.kv_dtype == "fp8_e4m3":
        from oracle.fp8 import dequant_per_head

        def run(rows):  # noqa: F811
            t0 = time.perf_counter()
            for i in rows:
                n_pg = (lens[i] + inp.cfg.page_size - 1) // inp.cfg.page_size
                ids = inp.block_table[i, :n_pg].long()
                kd = dequant_per_head(inp.k_cache[ids], inp.k_scale)
                vd = dequant_per_head(inp.v_cache[ids], inp.v_scale)
                tbl = torch.arange(n_pg, dtype=torch.int32)[None]
                ref_paged_attn(inp.q[i:i + 1], kd, vd, [lens[i]], tbl, inp.sm_scale)
            return time.perf_counter() - t0

    run([0])                                   # warm-up
    t_one = run([0])
    n_rows = max(1, min(batch, int(budget_s / 3 / max(t_one, 1e-4))))
    rows = list(range(n_rows))
    best = min(run(rows) for _ in range(3))
    tokens_sample = sum(lens[i] for i in rows)
    tokens_all = sum(lens)
    est_call_s = best * tokens_all / max(tokens_sample, 1)
    return {
        "value": inp.algorithmic_bytes() / est_call_s / 1e9,
        "unit": "GB/s",
        "us_per_call": est_call_s * 1e6,
        "cores": cores,
        "kind": "port",
        "sample": (f"oracle ref_paged_attn (torch CPU, {inp.cfg.q_dtype}) on sequences 0..{n_rows - 1} of {batch}, best of 3, "
                   f"scaled by attended tokens ({tokens_sample}/{tokens_all})" +
                   ("" if n_rows < batch else "; full batch")),
    }


def bench_kv_append(args):
    """One new token per sequence of the configured shape through fdk_kv_append; latency-bound (a few KB per token)."""
    import torch
    import triton_distributed_amd as tda
    from triton_distributed_amd import workloads as wl
    cfg = wl.CONFIGS[args.config]
    dev = torch.device("cuda:0")
    b, hq, hkv, d, page = cfg.batch, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.page_size
    n = cfg.kv_len or cfg.kv_len_range[1]
    g = torch.Generator().manual_seed(cfg.seed)
    pages_per_seq = (n + page - 1) // page
    pool = b * pages_per_seq
    qkv = torch.randn(b, 1, hq + 2 * hkv, d, generator=g).to(torch.bfloat16).to(dev)
    wq = (1.0 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16).to(dev)
    wk = (1.0 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16).to(dev)
    table = torch.randperm(pool, generator=g).to(torch.int32).view(b, pages_per_seq).to(dev)
    lens = torch.full((b,), n, dtype=torch.int32, device=dev)
    fp8 = cfg.kv_dtype == "fp8_e4m3"
    kdt = torch.float8_e4m3fn if fp8 else torch.bfloat16
    k = torch.zeros(pool, page, hkv, d, dtype=kdt, device=dev)
    v = torch.zeros(pool, page, hkv, d, dtype=kdt, device=dev)
    ks = torch.full((hkv,), 0.02, dtype=torch.float32, device=dev) if fp8 else None
    freqs = torch.outer(torch.arange(n + 1, dtype=torch.float32),
                        1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d)))
    cos, sin = torch.cat((freqs, freqs), -1).cos().to(dev), torch.cat((freqs, freqs), -1).sin().to(dev)
    q_out = torch.empty(b, 1, hq, d, dtype=torch.bfloat16, device=dev)

    def step():
        tda.qk_norm_rope_update_kvcache(qkv, k, v, table, lens, wq, wk, cos, sin, q_out, k_scale=ks, v_scale=ks)

    if args.warmup < 0:
        args.warmup = 100
    for _ in range(args.warmup):
        step()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / args.steps
    gpu_us = e0.elapsed_time(e1) * 1e3 / args.steps
    es = 1 if fp8 else 2
    alg = b * (hq + 2 * hkv) * d * 2 + b * hq * d * 2 + 2 * b * hkv * d * es + 2 * b * (d // 2) * 4 + 2 * d * 2 + 8 * b
    print(json.dumps({
        "metric": f"kv-append (RMSNorm + rotary + paged write, 1 new token per sequence) us/call, {args.config} shape",
        "value": round(wall_us, 2), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_us / 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if not fp8 else "bf16 -> fp8_e4m3 cache", "data": "synthetic (seeded N(0,1) bf16)",
        "config": {"workload": f"{args.config}: B{b} {hq}q/{hkv}kv D{d} P{page}, position {n - 1}",
                   "algorithmic_bytes_per_call": alg},
        "roofline": {"bound": "hbm", "kernel": "kv_append_kernel", "achieved": round(alg / gpu_us / 1e3, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(alg / gpu_us / 1e3 / HBM_PEAK_GBPS, 5),
                     "us_per_launch": round(gpu_us, 2), "traffic": None,
                     "note": "latency-bound: less than 1 MB per call"},
    }), flush=True)


def _split_kernel_name(cfg, plan):
    """The kernel family that the library runs this configuration in (the rule of mfma_heads_per_wg and of the dispatch in
    csrc/fdk_splitkv_mfma.hip): the name under which rocprofv3 lists the split kernel."""
    if plan.algo != "mfma":
        return f"splitkv_{plan.algo}_kernel"
    dk, dv, group, fp8 = cfg.head_dim, cfg.dv, cfg.q_heads // cfg.kv_heads, cfg.kv_dtype == "fp8_e4m3"
    if dk + dv > 512 and (not fp8 or group > 16):
        return "splitkv_mfma_shared_kernel"
    if dk != dv or dk == 192 or (dk == 128 and group > 16):
        return "splitkv_mfma_rows2_kernel"
    return "splitkv_mfma_kernel"


def _time_launches(torch, fn, n_iter, warm=10):
    """Average microseconds per call of fn(i), HIP events on the current stream around n_iter back-to-back calls."""
    for i in range(warm):
        fn(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(n_iter):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n_iter


def _placed(args, tda, pools):
    """The (K, V) pools as the run wants them placed: copies into alloc_kv_pools pairs, or the tensors as they are."""
    if args.kv_placement != "staggered":
        return pools
    out = []
    for k, v in pools:
        k2, v2 = tda.alloc_kv_pools(tuple(k.shape), k.dtype, k.device, zero=False, v_shape=tuple(v.shape))
        k2.copy_(k)
        v2.copy_(v)
        out.append((k2, v2))
    return out


def bench_ceiling(args):
    """Load-only figures for one configuration, each timed like the kernel itself (events around back-to-back
    launches that cycle through two KV pools):
      linear_read      a streaming read of as many bytes as the call attends to, with and without the non-temporal hint
      load_pipeline    the split kernel's own pieces, addresses and load instructions without the arithmetic
      kernel           the split kernel"""
    import torch
    import triton_distributed_amd as tda
    from triton_distributed_amd import workloads as wl

    dev = torch.device("cuda:0")
    inp = wl.make_inputs(_config_of(args, wl)).to(dev)
    if inp.cfg.head_dim != 128:
        print("--op ceiling: the load-pipeline probe is built for head_dim 128", file=sys.stderr)
        sys.exit(2)
    fp8 = inp.cfg.kv_dtype == "fp8_e4m3"
    alg_bytes = inp.algorithmic_bytes()
    g = torch.Generator(device=dev).manual_seed(inp.cfg.seed + 100)
    mk = (lambda: torch.randint(0, 120, inp.k_cache.shape, generator=g, device=dev, dtype=torch.uint8).view(
        torch.float8_e4m3fn)) if fp8 else (lambda: torch.randn(inp.k_cache.shape, generator=g, device=dev,
                                                               dtype=inp.k_cache.dtype))
    pools = _placed(args, tda, [(inp.k_cache, inp.v_cache), (mk(), mk())])
    kw = dict(k_scale=inp.k_scale, v_scale=inp.v_scale, kv_split=args.kv_split, always_workspace=True,
              wavefronts=args.wavefronts, buffers=args.buffers, shares_per_cu=args.shares_per_cu,
              fp8_fold_k_scale=args.fp8_fold, **_hints_of(args, inp))
    real = [tda.prepare_decode(inp.q, k, v, inp.block_table, inp.kv_lens, inp.sm_scale, **kw) for k, v in pools]
    probe = [tda.prepare_decode(inp.q, k, v, inp.block_table, inp.kv_lens, inp.sm_scale, probe_loads=True, **kw)
             for k, v in pools]
    plan = real[0].plan
    single_pass = plan.num_splits == 1
    n_iter = args.steps
    kv_bytes = sum(inp.kv_lens_host) * inp.cfg.kv_heads * 2 * inp.cfg.head_dim * (1 if fp8 else 2)
    lin_bytes = max(kv_bytes // 2 // 65536 * 65536, 1 << 20)       # per buffer: the K half, then the V half
    lin = [torch.randint(0, 255, (lin_bytes,), dtype=torch.uint8, device=dev) for _ in range(4)]

    def linear(nt):
        # one "call" = two launches (K-sized and V-sized buffer), four buffers in rotation
        def fn(i):
            tda.probe_linear_read(lin[(2 * i) % 4], nontemporal=nt)
            tda.probe_linear_read(lin[(2 * i + 1) % 4], nontemporal=nt)
        return fn

    res = {}
    res["linear_read_nt_us"] = _time_launches(torch, linear(True), n_iter)
    res["linear_read_plain_us"] = _time_launches(torch, linear(False), n_iter)
    res["load_pipeline_us"] = _time_launches(torch, lambda i: probe[i % 2].run(), n_iter)
    res["kernel_us"] = _time_launches(torch, (lambda i: real[i % 2].run()) if single_pass else
                                      (lambda i: real[i % 2].run_splitkv()), n_iter)
    gb = lambda us, nbytes: round(nbytes / us / 1e3, 1)
    print(json.dumps({
        "metric": f"load-only ceilings of the decode path, {args.config}", "unit": "us per launch (GB/s, % of 8 TB/s)",
        "config": {"workload": f"{args.config}: {inp.cfg.description}", "algorithmic_bytes_per_call": alg_bytes,
                   "num_splits": plan.num_splits, "balanced": plan.balanced, "workgroups": plan.workgroups,
                   "kv_heads_per_wg": plan.kv_heads_per_wg, "forced_kv_split": args.kv_split if args.kv_split > 0 else None},
        "linear_read_bytes": 2 * lin_bytes,
        "linear_read_nontemporal": {"us": round(res["linear_read_nt_us"], 2), "GBps": gb(res["linear_read_nt_us"], 2 * lin_bytes),
                                    "pct_of_peak": round(gb(res["linear_read_nt_us"], 2 * lin_bytes) / 80, 2),
                                    "note": "two launches of 512 workgroups per figure"},
        "linear_read_plain": {"us": round(res["linear_read_plain_us"], 2), "GBps": gb(res["linear_read_plain_us"], 2 * lin_bytes),
                              "pct_of_peak": round(gb(res["linear_read_plain_us"], 2 * lin_bytes) / 80, 2)},
        "load_pipeline_only": {"us": round(res["load_pipeline_us"], 2), "GBps": gb(res["load_pipeline_us"], alg_bytes),
                               "pct_of_peak": round(gb(res["load_pipeline_us"], alg_bytes) / 80, 2)},
        "split_kernel": {"us": round(res["kernel_us"], 2), "GBps": gb(res["kernel_us"], alg_bytes),
                         "pct_of_peak": round(gb(res["kernel_us"], alg_bytes) / 80, 2),
                         "pct_of_load_pipeline": round(100 * res["load_pipeline_us"] / res["kernel_us"], 1)},
        "n_gpus": 1, "steps": n_iter,
    }), flush=True)


def _config_of(args, wl):
    """The named configuration, with --batch / --kv-len applied."""
    cfg = wl.CONFIGS[args.config]
    if args.batch > 0 or args.kv_len > 0:
        import dataclasses
        kw = {}
        if args.batch > 0:
            kw["batch"] = args.batch
        if args.kv_len > 0:
            if cfg.kv_len is None:
                kw["kv_len_range"] = (cfg.kv_len_range[0], args.kv_len)
            else:
                kw["kv_len"] = args.kv_len
        cfg = dataclasses.replace(cfg, **kw, description=cfg.description + " [" + ", ".join(
            f"{k} = {v}" for k, v in kw.items()) + "]")
    return cfg


def _hints_of(args, inp):
    """Host-known length bounds for the planner (none with --no-hints)."""
    return {} if args.no_hints else dict(max_kv_len=max(inp.kv_lens_host), min_kv_len=min(inp.kv_lens_host))


def bench_timeline(args):
    """Per-wavefront clock readings of the matrix-core split kernel, from the library built with -DFDK_TIMELINE:
    medians over the workgroups of each XCD and of each kv head, for ``--steps`` launches (at most 16).  With
    ``--probe-loads`` the kernel is reduced to its load pipeline."""
    import numpy as np
    import torch
    import triton_distributed_amd as tda
    from triton_distributed_amd import workloads as wl

    dev = torch.device("cuda:0")
    inp = wl.make_inputs(_config_of(args, wl)).to(dev)
    kw = dict(k_scale=inp.k_scale, v_scale=inp.v_scale, kv_split=args.kv_split, always_workspace=True,
              wavefronts=args.wavefronts, buffers=args.buffers, shares_per_cu=args.shares_per_cu, **_hints_of(args, inp))
    tl = torch.zeros(8 * 8 * 4096, dtype=torch.int64, device=dev)            # up to 4096 workgroups of 8 wavefronts
    (k_pool, v_pool), = _placed(args, tda, [(inp.k_cache, inp.v_cache)])
    call = tda.prepare_decode(inp.q, k_pool, v_pool, inp.block_table, inp.kv_lens, inp.sm_scale,
                              timeline=tl, probe_loads=args.probe_loads, rotate_heads=args.rotate_heads, **kw)
    plan = call.plan
    launches = []
    for rep in range(max(1, min(args.steps, 16))):
        for _ in range(3):
            call.run_splitkv()
        torch.cuda.synchronize()
        raw = tl.cpu().numpy().reshape(-1, 8)
        raw = raw[raw[:, 0] > 0]                                             # wavefronts that wrote something
        if raw.shape[0] == 0:
            print("--op timeline: nothing was recorded - is FDK_LIBRARY the library built with --timeline?", file=sys.stderr)
            sys.exit(2)
        t0 = raw[:, 0].min()
        us = lambda c: (raw[:, c] - t0) * 0.01                               # 100 MHz clock
        end = np.maximum(us(2), np.where(raw[:, 3] > 0, us(3), 0.0))
        wgs, first = np.unique(raw[:, 7], return_index=True)                 # one entry per workgroup: its last wavefront's end
        es = np.array([end[raw[:, 7] == w].max() for w in wgs])
        xcd, head = raw[first, 4], raw[first, 5] // max(plan.kv_heads_per_wg, 1) * max(plan.kv_heads_per_wg, 1)
        launches.append({
            "first_start_to_last_end_us": round(float(end.max()), 2),
            "start_us_median": round(float(np.median(us(0))), 2),
            "first_loads_issued_us_median": round(float(np.median(us(1)[raw[:, 1] > 0])), 2),
            "end_us_min_median_max": [round(float(v), 2) for v in (es.min(), np.median(es), es.max())],
            "end_us_median_by_xcd": {int(x): round(float(np.median(es[xcd == x])), 2) for x in sorted(set(xcd.tolist()))},
            "end_us_median_by_kv_head": {int(h): round(float(np.median(es[head == h])), 2) for h in sorted(set(head.tolist()))},
        })
    print(json.dumps({"op": "timeline", "config": {"workload": f"{args.config}: {inp.cfg.description}",
                                                     "num_splits": plan.num_splits, "balanced": plan.balanced,
                                                     "workgroups": plan.workgroups, "kv_heads_per_wg": plan.kv_heads_per_wg,
                                                     "load_pipeline_only": bool(args.probe_loads),
                                                     "head_rotation": args.rotate_heads, "kv_placement": args.kv_placement},
                      "clock": "s_memrealtime, 100 MHz; times in us since the first wavefront's start",
                      "launches": launches}))


def bench_plan_sweep(args):
    """The plan the library chooses against the alternatives it rejects, cell by cell: bf16, head_dim 128, page size
    16, batch x length x (q heads / kv heads), in three modes - lengths uniform and known to the host (hinted), uniform
    and unknown (the table is exactly as wide as the sequences, nothing else is said), and ragged (uniform in
    [1, N], unknown).  Every plan is timed as a whole call (split kernel + combine) with HIP events around
    back-to-back launches on one prepared call.  Prints a markdown table and, last, one JSON line with the summary."""
    import torch
    import triton_distributed_amd as tda

    dev = torch.device("cuda:0")
    d, page = 128, 16
    heads = [tuple(int(x) for x in h.split("/")) for h in args.sweep_heads.split(",")]
    batches = [int(x) for x in args.sweep_batches.split(",")]
    lens_list = [int(x) for x in args.sweep_lens.split(",")]
    cap_bytes = args.sweep_max_gb * 1e9
    gen = torch.Generator(device=dev).manual_seed(4711)

    def time_call(calls):
        """(calls: the same plan on distinct regions of the pool, cycled through so that a small cell does not run out
        of the 256 MB memory-side cache)"""
        state = {"i": 0}

        class call:
            @staticmethod
            def run():
                calls[state["i"] % len(calls)].run()
                state["i"] += 1
        for _ in range(3):
            call.run()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):                          # best of three short batches: a cell takes milliseconds
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n = 0
            t0 = time.perf_counter()
            e0.record()
            while n < 5 or (n < 40 and time.perf_counter() - t0 < 1.5e-3):
                call.run()
                n += 1
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / n
            best = us if best is None else min(best, us)
        return best

    print("| heads | batch | kv_len | mode | library's plan | us | best alternative | us | library / best | every plan, us |")
    print("|---|---|---|---|---|---|---|---|---|---|")
    cells = []
    for hq, hkv in heads:
        fits = [(b, n) for b in batches for n in lens_list if b * n * hkv * 2 * d * 2 <= cap_bytes]
        if not fits:
            continue
        max_pages = max(b * n for b, n in fits) // page
        k, v = tda.alloc_kv_pools((max_pages, page, hkv, d), torch.bfloat16, dev, zero=False)
        k.normal_(generator=gen)
        v.normal_(generator=gen)
        q_all = torch.randn(max(batches), hq, d, generator=gen, device=dev, dtype=torch.bfloat16)
        for b, n in fits:
            q = q_all[:b]
            cell_pages = b * n // page
            n_rot = max(1, min(8, max_pages // cell_pages, int(1.5e9 // (cell_pages * page * hkv * 2 * d * 2)) + 1))
            tables = [(torch.randperm(cell_pages, generator=gen, device=dev).to(torch.int32) + r * cell_pages).view(b, n // page)
                      for r in range(n_rot)]
            host_gen = torch.Generator().manual_seed(b * 131 + n)
            modes = [("hinted", torch.full((b,), n, dtype=torch.int32), dict(max_kv_len=n, min_kv_len=n)),
                     ("unhinted", torch.full((b,), n, dtype=torch.int32), {})]
            if b > 1:
                modes.append(("ragged", torch.randint(1, n + 1, (b,), generator=host_gen).to(torch.int32), {}))
            for mode, lens_host, hints in modes:
                lens = lens_host.to(dev)
                alg_bytes = int(lens_host.sum()) * hkv * 2 * d * 2
                variants = [("library", {})]
                variants.append(("single pass", dict(kv_split=1)))
                variants += [(f"{s_} chunks", dict(kv_split=s_)) for s_ in (2, 4, 8, 16, 32) if n // s_ >= 64]
                if b > 1:
                    variants.append(("equal shares", dict(force_balanced=True)))
                prepared = []
                for name, kw in variants:
                    rot = [tda.prepare_decode(q, k, v, t, lens, d ** -0.5, work_queue=False, **hints, **kw) for t in tables]
                    pl = rot[0].plan
                    desc = ("single pass" if pl.num_splits == 1 else
                            f"equal shares, {pl.workgroups} workgroups" if pl.balanced else
                            f"{pl.num_splits} chunks" + (" of own length" if pl.chunk_floor else "")) + f", {pl.kv_heads_per_wg} kv heads/wg"
                    prepared.append((name, desc, rot))
                # two rounds over the plans, the better time of each: whichever plan runs first in a cell also pays for
                # what is new to the cell (its table, its pages' address translations)
                times = [min(t) for t in zip(*[[time_call(rot) for _, _, rot in prepared] for _ in range(2)])]
                res = [(name, desc, t) for (name, desc, _), t in zip(prepared, times)]
                lib = res[0]
                best = min(res[1:], key=lambda r: r[2])
                ratio = lib[2] / best[2]
                cells.append(dict(heads=f"{hq}/{hkv}", batch=b, kv_len=n, mode=mode, library_plan=lib[1], library_us=round(lib[2], 2),
                                  best=best[0], best_plan=best[1], best_us=round(best[2], 2), ratio=round(ratio, 3),
                                  pct_of_peak=round(alg_bytes / lib[2] / 1e3 / HBM_PEAK_GBPS * 100, 1),
                                  all={r[0]: round(r[2], 2) for r in res}))
                print(f"| {hq}/{hkv} | {b} | {n} | {mode} | {lib[1]} | {lib[2]:.1f} | {best[0]} ({best[1]}) | {best[2]:.1f} | "
                      f"{ratio:.3f} | " + ", ".join(f"{r[0]} {r[2]:.1f}" for r in res[1:]) + " |", flush=True)
        del k, v
        torch.cuda.empty_cache()
    worst = sorted(cells, key=lambda c: -c["ratio"])[:12]
    print()
    print(json.dumps({"op": "plan-sweep", "cells": len(cells),
                      "cells_within_5pct_of_best": sum(c["ratio"] <= 1.05 for c in cells),
                      "worst": worst}), flush=True)


def main():
    args = parse_args()
    if args.op == "timeline" and "FDK_LIBRARY" not in os.environ:
        os.environ["FDK_LIBRARY"] = os.path.join(ROOT, "triton_distributed_amd", "lib", "libfdk_timeline.so")
    if args.gpus != 1:
        print(f"bench.py measures one GPU's share of the decode path; --gpus {args.gpus} is not supported "
              "(this build has no multi-GPU leg)", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path for the kernels)", file=sys.stderr)
        sys.exit(2)
    import triton_distributed_amd as tda
    from triton_distributed_amd import workloads as wl

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.op == "kv_append":
        return bench_kv_append(args)
    if args.op == "ceiling":
        return bench_ceiling(args)
    if args.op == "timeline":
        return bench_timeline(args)
    if args.op == "plan-sweep":
        return bench_plan_sweep(args)
    t_gen = time.perf_counter()
    inp_cpu = wl.make_inputs(_config_of(args, wl))
    print(f"[bench] generated {args.config} on CPU in {time.perf_counter() - t_gen:.1f}s", file=sys.stderr, flush=True)
    inp = inp_cpu.to(dev)
    if args.fp8_pow2_scales and inp.cfg.kv_dtype == "fp8_e4m3":      # (timing only: the cache keeps its codes)
        inp.k_scale = torch.exp2(torch.ceil(torch.log2(inp.k_scale)))
        inp.v_scale = torch.exp2(torch.ceil(torch.log2(inp.v_scale)))
    pools = [(inp.k_cache, inp.v_cache)]
    pool_bytes = (inp.k_cache.numel() + inp.v_cache.numel()) * inp.k_cache.element_size()
    rotate = max(1, args.rotate)
    if args.rotate > 1:
        rotate = max(rotate, min(16, -(-(1 << 30) // max(pool_bytes, 1))))       # small pools: more of them
    for r in range(1, rotate):
        # further pools: same pages, different (seeded) contents - the access pattern is identical
        g = torch.Generator(device=dev).manual_seed(inp.cfg.seed + 100 * r)
        if inp.cfg.kv_dtype == "fp8_e4m3":
            mk = lambda like=inp.k_cache: torch.randint(0, 120, like.shape, generator=g, device=dev,
                                                        dtype=torch.uint8).view(torch.float8_e4m3fn)
        else:
            mk = lambda like=inp.k_cache: torch.randn(like.shape, generator=g, device=dev, dtype=like.dtype)
        pools.append((mk(), mk(inp.v_cache)))
    def prepare_all(pp):
        return [tda.prepare_decode(inp.q, k, v, inp.block_table, inp.kv_lens, inp.sm_scale, k_scale=inp.k_scale,
                                   v_scale=inp.v_scale, kv_split=args.kv_split, algo=args.algo, always_workspace=True,
                                   single_launch=args.single_launch, wavefronts=args.wavefronts, buffers=args.buffers,
                                   shares_per_cu=args.shares_per_cu, fp8_fold_k_scale=args.fp8_fold, **_hints_of(args, inp))
                for k, v in pp]

    # ---- the calls on independently allocated pools (the other placement), for the record: timed first, then the
    # pools move into their placed allocations one by one and the originals go back to the driver.  (Freed device
    # memory is wiped in the background, which takes bandwidth for some milliseconds: hence before everything else,
    # followed by a pause, and not in between the timed legs.)
    separate_us = bare_us = None

    def timed_loop(fn, n):
        """Wall-clock microseconds per call of n back-to-back fn(i), after at least 100 calls and 0.1 s of them."""
        n_warm = 0
        t0 = time.perf_counter()
        while n_warm < 100 or time.perf_counter() - t0 < 0.1:
            fn(n_warm)
            n_warm += 1
            if n_warm % 50 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e6 / n

    if args.kernel_only:
        args.no_separate_leg = args.no_graph = args.no_cpu_baseline = True
    if not args.no_separate_leg and not args.kernel_only:
        # the bare signature of the path, flash_decode(q, k_cache, v_cache, block_table, kv_lens, sm_scale) and nothing
        # else - no length bounds, no placement of the pools, outputs and scratch left to the call - on independently
        # allocated pools: what a caller that knows only the reference's interface gets
        kw_bare = dict(k_scale=inp.k_scale, v_scale=inp.v_scale) if inp.cfg.kv_dtype == "fp8_e4m3" else {}
        bare_us = timed_loop(lambda i: tda.flash_decode(inp.q, *pools[i % len(pools)], inp.block_table, inp.kv_lens,
                                                        inp.sm_scale, **kw_bare), args.steps)
    if args.kv_placement == "staggered":
        if not args.no_separate_leg:
            sep = prepare_all(pools)
            separate_us = timed_loop(lambda i: sep[i % len(sep)].run(), args.steps)
            del sep
        placed = []
        while pools:
            placed += _placed(args, tda, [pools.pop(0)])
            if not placed[1:]:
                inp.k_cache, inp.v_cache = placed[0]
        pools = placed
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        time.sleep(0.3)
    calls = prepare_all(pools)
    plan = calls[0].plan
    alg_bytes = inp.algorithmic_bytes()

    # sanity of the timed configuration (parity proper is the job of tests/ and __graft_entry__.smoke())
    out, lse = calls[0].run()
    torch.cuda.synchronize()
    if not (torch.isfinite(out.float()).all() and torch.isfinite(lse).all()):
        raise RuntimeError("non-finite decode output on the benchmark inputs")

    if args.copy_calibration > 0:
        src = torch.full((args.copy_calibration << 20,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def step(i):
        calls[i % len(calls)].run()

    # ---- whole call: W warm-up steps (never fewer than 100 calls and 0.1 s of them: after the idle seconds of the
    # input generation the GPU clock needs some tens of milliseconds of load to come up, and a handful of calls does
    # not give it that), then exactly K timed steps between synchronisations - `--batches` times over, the median
    # batch being the one reported.  HIP events on the launch stream go around the same K steps: for a single-pass
    # plan the call IS one launch of the split kernel, so the events give that kernel's average duration over the very
    # launches the wall clock timed (events sit inside the synchronisations, hence us_per_launch <= us_per_call).
    single_pass = plan.num_splits == 1
    requested_warmup = args.warmup
    n_warm = 0
    t0 = time.perf_counter()
    while n_warm < max(args.warmup, 100) or time.perf_counter() - t0 < 0.1:
        step(n_warm)
        n_warm += 1
        if n_warm % 50 == 0:
            torch.cuda.synchronize()
    args.warmup = n_warm
    batches = []
    for _ in range(max(1, args.batches)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for i in range(args.steps):
            step(i)
        e1.record()
        torch.cuda.synchronize()
        batches.append(((time.perf_counter() - t0), e0.elapsed_time(e1) * 1e-3))
    wall_s, events_s = sorted(batches)[len(batches) // 2]
    ms_per_step = wall_s * 1e3 / args.steps
    gbps = alg_bytes / (wall_s / args.steps) / 1e9

    # ---- dominant kernel alone (split-KV).  Single pass: the events of the timed loop above.  A split plan runs the
    # split kernel and the combine: events go around launches of the split kernel only, warmed up like the call.
    if single_pass:
        split_us = events_s * 1e6 / args.steps
    else:
        kernel_step = lambda i: calls[i % len(calls)].run_splitkv()
        for i in range(100):
            kernel_step(i)
        reps = []
        for _ in range(max(1, args.batches)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for i in range(args.steps):
                kernel_step(i)
            e1.record()
            torch.cuda.synchronize()
            reps.append(e0.elapsed_time(e1) * 1e3 / args.steps)
        split_us = sorted(reps)[len(reps) // 2]
    split_gbps = alg_bytes / (split_us * 1e-6) / 1e9

    # ---- the same calls replayed from one HIP graph (a serving engine replays its decode step from a graph):
    # separates what the host-side launches cost from what the GPU needs
    graph_us = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for c in calls:
                c.run()                            # first use of the stream outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        # a decode step of a served model holds this call once per layer: 32 calls per graph, cycling through the pools
        # (with two calls per graph the cost of launching the graph itself, tens of microseconds, would dominate)
        n_in_graph = max(32, len(calls))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(n_in_graph):
                calls[i % len(calls)].run()
        reps = max(3, args.steps // n_in_graph)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            graph.replay()
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) * 1e6 / (reps * n_in_graph)

    # ---- the un-prepared public entry point: flash_decode() validates, marshals and allocates (out, lse) per call
    kw = dict(k_scale=inp.k_scale, v_scale=inp.v_scale, kv_split=args.kv_split, algo=args.algo, **_hints_of(args, inp))
    n_entry = max(args.steps, 100)
    entry_us = None
    if not args.kernel_only:
        entry_us = timed_loop(lambda i: tda.flash_decode(inp.q, *pools[i % len(pools)], inp.block_table, inp.kv_lens,
                                                         inp.sm_scale, **kw), n_entry)

    # ---- the drop-in for the reference's entry point, called the way the reference's layer calls it: no length bounds,
    # kv_split = 32 (sp_flash_decode_layer.py:62,100-110), output_combine given; fp8 caches are not part of that signature
    ref_entry_us = ref_entry_fb_us = cold_fb_us = None
    if inp.cfg.kv_dtype != "fp8_e4m3" and not args.kernel_only:
        oc = torch.empty((inp.q.shape[0], inp.q.shape[1], inp.v_cache.shape[-1] + 1), dtype=inp.q.dtype, device=dev)
        ref_call = lambda i: tda.gqa_fwd_batch_decode_intra_rank(inp.q, *pools[i % len(pools)], None, None, inp.kv_lens,
                                                                 inp.block_table, inp.sm_scale, output_combine=oc, kv_split=32)
        ref_entry_us = timed_loop(ref_call, n_entry)
        # the same entry point with a LengthFeedback block, as the layer mirror keeps one: each call plans with the
        # bounds of kv_lens that the previous call's last kernel left in pinned host memory
        fb = tda.LengthFeedback()
        fb_call = lambda i: tda.gqa_fwd_batch_decode_intra_rank(inp.q, *pools[i % len(pools)], None, None, inp.kv_lens,
                                                                inp.block_table, inp.sm_scale, output_combine=oc,
                                                                kv_split=32, length_feedback=fb)
        for i in range(5):
            fb_call(i)
            torch.cuda.synchronize()
        ref_entry_fb_us = timed_loop(fb_call, n_entry)
        # ... and what the FIRST call on a feedback block costs (a new batch, a new layer object): every call of this
        # loop is given a block that no call has written yet, so it plans for unknown lengths and only leaves bounds
        cold = [tda.LengthFeedback() for _ in range(n_entry + 128)]
        n_cold = iter(range(len(cold)))
        cold_call = lambda i: tda.gqa_fwd_batch_decode_intra_rank(inp.q, *pools[i % len(pools)], None, None, inp.kv_lens,
                                                                  inp.block_table, inp.sm_scale, output_combine=oc,
                                                                  kv_split=32, length_feedback=cold[next(n_cold)])
        for i in range(100):                       # warm-up on blocks of their own
            cold_call(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_entry):
            cold_call(i)
        torch.cuda.synchronize()
        cold_fb_us = (time.perf_counter() - t0) * 1e6 / n_entry
        assert all(c.read()[2] != 0 for c in cold[:n_entry + 100])        # every block was written exactly by its call
        for c in cold:
            c.close()

    traffic = None
    traffic_source = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    resized = args.batch > 0 or args.kv_len > 0
    if os.path.exists(tpath) and not resized and not args.kv_split > 0 and not args.no_hints:
        with open(tpath) as f:
            traffic = json.load(f).get(args.config, {}).get("bytes_per_launch")
        if traffic is not None:
            traffic_source = "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run, not this one)"

    qd = inp.cfg.q_dtype
    result = {
        "metric": "decode-attn achieved HBM GB/s (algorithmic bytes / time per call; µs/call alongside), "
                  "Llama-3-8B shape b=32" if args.config == "llama3_8b_b32" and not resized else
                  f"decode-attn achieved HBM GB/s, {inp.cfg.name}" + (" (resized)" if resized else ""),
        "value": round(gbps, 1),
        "unit": "GB/s",
        "us_per_call": round(ms_per_step * 1e3, 2),
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "batches_us_per_call": [round(w * 1e6 / args.steps, 2) for w, _ in batches],
        "no_hints_us_per_call": None if bare_us is None else round(bare_us, 2),
        "no_hints_pct_of_hbm_peak": None if bare_us is None else round(alg_bytes / bare_us / 1e3 / HBM_PEAK_GBPS * 100, 2),
        "separate_pools_us_per_call": None if separate_us is None else round(separate_us, 2),
        "graph_replay_us_per_call": None if graph_us is None else round(graph_us, 2),
        "public_entry_us_per_call": None if entry_us is None else round(entry_us, 2),
        "reference_entry_us_per_call": None if ref_entry_us is None else round(ref_entry_us, 2),
        "reference_entry_with_feedback_us_per_call": None if ref_entry_fb_us is None else round(ref_entry_fb_us, 2),
        "first_call_with_cold_feedback_us": None if cold_fb_us is None else round(cold_fb_us, 2),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_requested": requested_warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": qd if inp.cfg.kv_dtype != "fp8_e4m3" else f"fp8_e4m3 KV / {qd} q, fp32 softmax",
        "data": f"synthetic, resident in HBM before timing: seeded N(0,1) {qd} q/K/V generated on the CPU" +
                (f"; the timed calls cycle through {len(pools)} KV pools with the same block_table, pools 2.. filled on "
                 "the GPU (seeded N(0,1), fp8: uniform codes 0..119)" if len(pools) > 1 else ""),
        "config": {
            "workload": f"{args.config}: {inp.cfg.description}",
            "algorithmic_bytes_per_call": alg_bytes,
            "num_splits": plan.num_splits, "chunk_tokens": plan.chunk_tokens, "chunk_floor": plan.chunk_floor,
            "algo": plan.algo,
            "balanced": plan.balanced, "workgroups": plan.workgroups, "kv_heads_per_wg": plan.kv_heads_per_wg,
            "single_launch": bool(args.single_launch and plan.num_splits > 1),
            "fp8_k_scale": None if inp.cfg.kv_dtype != "fp8_e4m3" else
                           ("folded into the logit scale" if args.fp8_fold else
                            "powers of two: the exponent operand of the conversion (exact dequantisation)" if args.fp8_pow2_scales else
                            "applied to every K value (exact dequantisation)"),
            "kv_pool_placement": ("one allocation per (K, V) pair, V 256 bytes off K modulo 512 (alloc_kv_pools, as PagedKVCache "
                                  "allocates)" if args.kv_placement == "staggered" else "two independent torch allocations"),
            "kv_pools_rotated": len(pools), "forced_kv_split": args.kv_split if args.kv_split > 0 else None,
            "host_length_hints": None if args.no_hints else [min(inp.kv_lens_host), max(inp.kv_lens_host)],
            "wavefronts_override": args.wavefronts or None, "buffers_override": args.buffers or None,
            "shares_per_cu_override": args.shares_per_cu or None,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": _split_kernel_name(inp.cfg, plan),
            "variant": "single pass: writes (out, lse) itself" if single_pass else "writes fp32 partials; the combine kernel follows",
            "achieved": round(split_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(split_gbps / HBM_PEAK_GBPS, 4),
            "us_per_launch": round(split_us, 2),
            "timed": "HIP events around the K timed steps of the reported batch" if single_pass else
                     "HIP events around K launches of the split kernel alone (median of the batches)",
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(inp_cpu, args.cpu_seconds)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
