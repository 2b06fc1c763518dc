"""CPU oracle for the paged split-KV GQA decode path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory.  The only callers are
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``, and they use it as the checker / the timed CPU baseline, never as
the thing that is shipped.

Modules
-------
paged_attn      torch restatement of the reference's torch implementation of
                paged decode attention (the function its tests compare
                against) - defines ``out`` to the reference's own tolerance.
closed_form     float64 brute force of ``(out, lse)``, the split/combine
                recurrences of the reference kernels in numpy, and the
                textbook log-sum-exp merge they must reduce to.
fp8             OCP e4m3fn decode table and the per-kv-head dequantisation the
                fp8 KV-cache workload is defined by.
kv_append       the step before the path: per-head RMSNorm, rotary embedding and
                the paged KV-cache append (restates the reference's Triton kernel).

Pinning status (what checks the oracle itself; see tests/test_oracle_*.py):
  * paged_attn.ref_paged_attn      pinned: agrees with closed_form.attn_fp64 within the
                                   reference tests' own 1e-2 tolerance; closed-form special
                                   cases (kv_len=1, q=0, one-hot V).  The reference holds no
                                   golden vectors for this path, so beyond tolerance level the
                                   arithmetic of its Triton kernels (tl.dot order, ex2.approx)
                                   is "parity unpinned".
  * closed_form.attn_fp64          pinned: scipy.special.logsumexp / softmax on tiny dense
                                   cases, brute-force python loops, special cases above.
  * closed_form.split_kv_partials,
    combine_partials, combine_ranks pinned: split invariance (any S gives the S=1 answer),
                                   logsumexp/softmax identity, -inf (empty) entries.
  * fp8.e4m3fn_table               pinned: exhaustive 256-entry comparison with
                                   torch.float8_e4m3fn CPU casts and the OCP bit formula.
  * kv_append.kv_append            pinned at the reference test's 1e-2 tolerance against an independent
                                   float64 route (numpy norm, complex rotation), rotation invariants,
                                   bit-exact copies / untouched rows; the bf16 rounding points of the
                                   reference's Triton kernel beyond that tolerance are "parity unpinned"
                                   (its own oracle, flashinfer, is not available and it stores no vectors).
"""
