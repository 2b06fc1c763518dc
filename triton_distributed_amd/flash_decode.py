"""Host side of the MI355X flash-decode path: split-KV paged GQA decode + LSE combine.

Mirrors the operator interface of the reference's
``python/triton_dist/kernels/nvidia/flash_decode.py`` for this one path:

=====================================  =========================================================
here                                   reference
=====================================  =========================================================
``flash_decode``                       the local step of ``SpGQAFlashDecodeAttention.forward``
                                       (layers/nvidia/sp_flash_decode_layer.py:100-110), returned
                                       as ``(out, lse)`` instead of the packed buffer
``gqa_fwd_batch_decode_intra_rank``    flash_decode.py:847-928  (packed ``[B, Hq, D+1]``)
``gqa_fwd_batch_decode``               flash_decode.py:763-844  (``[B, Hq, D]``)
``*_aot`` variants                     flash_decode.py:979-1092 (explicit stream first)
``inter_rank_combine``                 the final combine of sp_flash_decode_layer.py:143-183 with
                                       kernel flash_decode.py:481-532
``get_split_kv_plan``                  ``get_triton_split_kv_algo_info``, flash_decode.py:103-109
``pack_out_lse`` / ``unpack_out_lse``  the ``[..., :D]`` / ``[..., D]`` layout of :235-239, :441-449
=====================================  =========================================================

Same names, argument order and meaning; the kernels behind them are hand-written gfx950 HIP kernels in
``libfdk.so`` reached through its C ABI (include/fdk.h).  torch only supplies device memory and the
current stream.  There is no fallback path: a missing library raises at import of this module.

Differences that a caller can observe
  * the split count defaults to a value chosen from the shape and the device's compute units
    (reference: fixed 32, :863); ``kv_split`` forces a count in ``flash_decode`` / ``prepare_decode`` and is read as
    an upper bound by the entry points that carry the reference's names (``_reference_kv_split``);
  * the per-split scratch is fp32 and private to the library: a caller-provided ``output_split`` is used
    as scratch only if it is large enough, its contents afterwards are unspecified;
  * ``workspace`` and ``q_lens`` are accepted and ignored, exactly as in the reference (:847, never read);
  * kv_len == 0 gives out = 0, lse = -inf instead of NaN.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple, Union

import torch

from . import _lib
from ._lib import FdkCombineRanksArgs, FdkDecodeArgs, FdkKvAppendArgs, FdkMeasureArgs, FdkPlan

_LIB = _lib.load()          # raises ImportError when libfdk.so is not built - by design

_TORCH_TO_FDK = {torch.bfloat16: _lib.FDK_BF16, torch.float16: _lib.FDK_FP16, torch.float32: _lib.FDK_FP32}
if hasattr(torch, "float8_e4m3fn"):
    _TORCH_TO_FDK[torch.float8_e4m3fn] = _lib.FDK_FP8_E4M3
_ALGOS = {"auto": _lib.FDK_ALGO_AUTO, "valu": _lib.FDK_ALGO_VALU, "mfma": _lib.FDK_ALGO_MFMA}
_ALGO_NAMES = {v: k for k, v in _ALGOS.items()}


def _fdk_dtype(t: torch.dtype, what: str) -> int:
    try:
        return _TORCH_TO_FDK[t]
    except KeyError:
        raise ValueError(f"{what}: unsupported dtype {t}") from None


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# torch's own fast paths to the current stream's handle and its capture state (torch.cuda.current_stream() builds a
# Stream object first: 2.8 us against 0.3 us per call, which a 9 us decode call feels)
_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_CAPTURING = getattr(torch._C, "_cuda_isCurrentStreamCapturing", None)


def _stream_handle(stream) -> int:
    if stream is None:
        if _RAW_STREAM is not None:
            return _RAW_STREAM(torch.cuda.current_device())
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


@dataclass
class SplitKvPlan:
    """Shape-dependent launch constants (the role of the reference's ``algo_info`` dict)."""
    num_splits: int          # partial rows per (sequence, q head) the workspace holds; 1 = single pass
    chunk_tokens: int        # tokens per split (chunk mode; with chunk_floor: at most) / nominal tokens per
                             # workgroup (balanced mode)
    algo: str
    workspace_bytes: int
    kv_heads_per_wg: int = 1
    balanced: bool = False   # the kernel cuts the whole batch's KV ranges into equal shares from kv_lens
    workgroups: int = 0
    chunk_floor: int = 0     # > 0 (chunk mode): the chunks follow each sequence's own length,
                             # clamp(ceil(kv_len / num_splits) rounded up to 16, chunk_floor, chunk_tokens) tokens


class LengthFeedback:
    """Four int32 in pinned host memory that the GPU writes at the end of a decode call: the smallest and the largest
    of the (clamped) ``kv_lens``, a call count and the batch size.  For callers whose lengths exist only on the GPU -
    the reference's entry points take nothing else: ``bounds()`` before a later call gives ``(min_kv_len, max_kv_len)``
    for its plan without a device synchronisation.  The bounds only size the plan: values that are out of date (the
    batch changed since) cost time, never tokens."""

    def __init__(self):
        host, dev = C.c_void_p(), C.c_void_p()
        _lib.check(_LIB.fdk_length_feedback_alloc(C.byref(host), C.byref(dev)))
        self._host = host.value
        self.device_ptr = dev.value
        self._view = (C.c_int32 * 4).from_address(self._host)

    def read(self):
        """``(min, max, epoch, batch)`` as last written (epoch 0: never)."""
        return tuple(self._view)

    def bounds(self, batch: int):
        """``(min_kv_len, max_kv_len)`` for a batch of this size, or ``(None, None)`` if nothing usable is there."""
        lo, hi, epoch, nb = self._view
        if epoch == 0 or nb != batch or lo < 1 or hi < lo:
            return None, None
        return lo, hi

    def close(self):
        """Free the block.  Only when no call that was given it can still be running (the GPU writes to it); a block
        that is never closed stays allocated until the process ends (one page of pinned memory)."""
        host, self._host = self._host, None
        if host:
            self._view = (C.c_int32 * 4)()
            _lib.check(_LIB.fdk_length_feedback_free(host))


def _fill_args(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap, kv_split, max_kv_len,
               k_scale, v_scale, algo, check_device=True, min_kv_len=None) -> FdkDecodeArgs:
    if q.dim() != 3:
        raise ValueError(f"q must be [batch, q_heads, head_dim], got {tuple(q.shape)}")
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise ValueError("k_cache / v_cache must be [num_pages, page_size, kv_heads, head_dim]")
    batch, q_heads, q_head_dim = q.shape
    _, page_size, kv_heads, k_head_dim = k_cache.shape
    # the reference's shape asserts, flash_decode.py:851,860
    assert page_size == v_cache.shape[1] and kv_heads == v_cache.shape[2] and k_head_dim == q_head_dim
    assert q_heads % kv_heads == 0
    v_head_dim = v_cache.shape[-1]       # (the reference: V_DIM next to K_DIM, flash_decode.py:103-109; the library says what is built)
    if k_cache.dtype != v_cache.dtype:
        raise ValueError("k_cache and v_cache must share a dtype")
    if q.stride(-1) != 1 or k_cache.stride(-1) != 1 or v_cache.stride(-1) != 1:
        raise ValueError("the head dimension of q, k_cache and v_cache must be contiguous")
    if block_table.dim() != 2 or block_table.shape[0] != batch:
        raise ValueError(f"block_table must be [batch, max_pages], got {tuple(block_table.shape)}")
    if block_table.dtype != torch.int32 or kv_lens.dtype != torch.int32:
        raise ValueError("block_table and kv_lens must be int32")
    if block_table.stride(-1) != 1 or (kv_lens.dim() != 1 or kv_lens.shape[0] != batch or
                                       (batch > 1 and kv_lens.stride(0) != 1)):
        raise ValueError("block_table rows and kv_lens [batch] must be contiguous")
    if check_device:
        for name, t in (("q", q), ("k_cache", k_cache), ("v_cache", v_cache), ("block_table", block_table),
                        ("kv_lens", kv_lens)):
            if not t.is_cuda:
                raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
            if t.device != q.device:
                raise ValueError(f"{name} is on {t.device}, q on {q.device}")
    a = FdkDecodeArgs()
    a.struct_size = C.sizeof(FdkDecodeArgs)
    a.flags = 0
    a.q = q.data_ptr()
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.q_dtype = _fdk_dtype(q.dtype, "q")
    a.kv_dtype = _fdk_dtype(k_cache.dtype, "k_cache")
    a.k_cache, a.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
    a.k_stride_page, a.k_stride_tok, a.k_stride_head = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    a.v_stride_page, a.v_stride_tok, a.v_stride_head = v_cache.stride(0), v_cache.stride(1), v_cache.stride(2)
    if a.kv_dtype == _lib.FDK_FP8_E4M3:
        for name, s in (("k_scale", k_scale), ("v_scale", v_scale)):
            if s is not None and (s.dtype != torch.float32 or s.numel() != kv_heads or not s.is_contiguous()):
                raise ValueError(f"{name} must be a contiguous fp32 tensor of {kv_heads} per-kv-head scales")
        a.k_scale, a.v_scale = _ptr(k_scale), _ptr(v_scale)
    elif k_scale is not None or v_scale is not None:
        raise ValueError("k_scale / v_scale are only meaningful for an fp8 KV cache")
    a.block_table = block_table.data_ptr()
    a.table_stride_b = block_table.stride(0) if batch > 1 else max(block_table.stride(0), block_table.shape[1])
    a.kv_lens = kv_lens.data_ptr()
    a.batch, a.num_q_heads, a.num_kv_heads, a.head_dim = batch, q_heads, kv_heads, q_head_dim
    a.v_head_dim = v_head_dim if v_head_dim != q_head_dim else 0
    a.page_size = page_size
    a.max_pages = block_table.shape[1]
    a.max_kv_len = int(max_kv_len) if max_kv_len else 0
    a.min_kv_len = int(min_kv_len) if min_kv_len else 0
    a.num_splits = int(kv_split) if kv_split and kv_split > 0 else 0
    a.sm_scale = float(sm_scale)
    a.soft_cap = float(soft_cap) if soft_cap else 0.0
    a.algo = _ALGOS[algo] if isinstance(algo, str) else int(algo)
    return a


_TEMPLATES = {}          # layout key -> [validated argument block without pointers and bounds, {bounds: plan}]


def _args_and_plan(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap, kv_split, max_kv_len, k_scale, v_scale,
                   algo, min_kv_len):
    """``_fill_args`` + ``_plan_of`` with a cache: a serving loop calls with the same layouts over and over, and the
    shape checks depend on shapes, strides, dtypes, devices and scalars only.  A hit copies the validated block and sets
    the pointers (their alignment is checked by the library on every call) and the length bounds; the plan is kept per
    pair of bounds, so a caller whose bounds move with every decode step (``LengthFeedback``) pays one ``fdk_plan``
    call for them, not the checks."""
    def meta(t):
        return None if t is None else (t.shape, t.stride(), t.dtype, t.device)
    key = (meta(q), meta(k_cache), meta(v_cache), meta(block_table), meta(kv_lens), meta(k_scale), meta(v_scale),
           sm_scale, soft_cap, kv_split, algo)
    bounds = (int(max_kv_len) if max_kv_len else 0, int(min_kv_len) if min_kv_len else 0)
    hit = _TEMPLATES.get(key)
    if hit is None:
        a = _fill_args(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap, kv_split, max_kv_len,
                       k_scale, v_scale, algo, min_kv_len=min_kv_len)
        plan = _plan_of(a)
        if len(_TEMPLATES) >= 256:
            _TEMPLATES.clear()
        _TEMPLATES[key] = [bytes(a), {bounds: plan}]
        return a, plan
    a = FdkDecodeArgs.from_buffer_copy(hit[0])
    a.q, a.k_cache, a.v_cache = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr()
    a.block_table, a.kv_lens = block_table.data_ptr(), kv_lens.data_ptr()
    a.max_kv_len, a.min_kv_len = bounds
    if k_scale is not None:
        a.k_scale = k_scale.data_ptr()
    if v_scale is not None:
        a.v_scale = v_scale.data_ptr()
    plan = hit[1].get(bounds)
    if plan is None:
        plan = _plan_of(a)                      # (also where the library refuses the bounds)
        if len(hit[1]) >= 64:
            hit[1].clear()
        hit[1][bounds] = plan
    return a, plan


def _plan_of(a: FdkDecodeArgs, num_cus: int = 0) -> SplitKvPlan:
    plan = FdkPlan()
    _lib.check(_LIB.fdk_plan(C.byref(a), num_cus, C.byref(plan)))
    ws = _LIB.fdk_workspace_bytes(a.batch, a.num_q_heads, a.v_head_dim or a.head_dim, plan.num_splits)
    return SplitKvPlan(plan.num_splits, plan.chunk_tokens, _ALGO_NAMES[plan.algo], int(ws), plan.kv_heads_per_wg,
                       bool(plan.balanced), plan.workgroups, plan.chunk_floor)


def get_split_kv_plan(q, k_cache, v_cache, block_table, kv_lens, sm_scale=1.0, soft_cap=0.0, kv_split=-1,
                      max_kv_len=None, algo="auto", num_cus: int = 0, min_kv_len=None, force_balanced=False) -> SplitKvPlan:
    """The split count / chunk length / algorithm a decode call with these tensors will use (``force_balanced``: the
    plan of ``prepare_decode(..., force_balanced=True)``, a measurement aid)."""
    a = _fill_args(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap, kv_split, max_kv_len,
                   None, None, algo, check_device=False, min_kv_len=min_kv_len)
    if num_cus > 0:
        a.flags |= _lib.FDK_FLAG_DRY_RUN
    if force_balanced:
        measure = FdkMeasureArgs()
        measure.struct_size = C.sizeof(FdkMeasureArgs)
        measure.force_balanced = 1
        a.measure = C.addressof(measure)
    return _plan_of(a, num_cus)


_COUNTER_CACHE = {}
_SCRATCH_CACHE = {}


def _capturing() -> bool:
    if _RAW_CAPTURING is not None and torch.cuda.is_initialized():
        return _RAW_CAPTURING()
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


class _on_stream:
    """Make the stream with this raw handle torch's current stream while a shared per-stream buffer is (re)allocated.

    torch's caching allocator ties a block to the stream that was current when it was allocated: a block that is freed
    can be handed out again at once to later work on that stream, and only there.  The shared buffers are used by kernels
    on the stream whose handle the caller passed, which need not be torch's current one: allocated under the current
    stream, a buffer that is dropped when a larger one takes its place could be reused by the current stream while
    kernels on the caller's stream still write partial rows into it (and a fresh zero-fill would not be ordered before
    its first use).  Allocated under the caller's stream, both the fill and the reuse are ordered with its kernels."""

    def __init__(self, device: torch.device, handle: int):
        self._ctx = None
        current = _RAW_STREAM(device.index) if _RAW_STREAM is not None else torch.cuda.current_stream(device).cuda_stream
        if handle != current:
            self._ctx = torch.cuda.stream(torch.cuda.ExternalStream(handle, device=device))

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


def _stream_counters(device: torch.device, stream, n: int) -> Optional[torch.Tensor]:
    """Zeroed int32 counters shared by the eager calls issued on one stream (they run in order, and every call
    leaves the counters zero), so the convenience entry points need no fill launch per call.  A call made while
    its stream is capturing a HIP graph gets counters of its own instead (None here: ``prepare_decode`` then
    allocates them): a replay may run on another stream and overlap eager calls on this one."""
    if device.type != "cuda" or _capturing():
        return None                                   # CPU tensors: the caller is about to be told there is no CPU path
    handle = _stream_handle(stream)
    key = (device.index, handle)
    t = _COUNTER_CACHE.get(key)
    if t is None or t.numel() < n:
        with _on_stream(device, handle):
            t = torch.zeros(max(n, 1024), dtype=torch.int32, device=device)
        _COUNTER_CACHE[key] = t
    return t


def _stream_scratch(device: torch.device, stream, nbytes: int) -> Optional[torch.Tensor]:
    """fp32 scratch for the split partials of the convenience entry points, kept per (device, stream) and grown on
    demand: calls on one stream run in order, so they can share it.  Not used while capturing (see above)."""
    if device.type != "cuda" or nbytes <= 0 or _capturing():
        return None
    handle = _stream_handle(stream)
    key = (device.index, handle)
    t = _SCRATCH_CACHE.get(key)
    if t is None or t.numel() < nbytes:
        with _on_stream(device, handle):
            t = None                                      # the buffer it replaces goes back to this stream's pool
            _SCRATCH_CACHE.pop(key, None)
            t = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _SCRATCH_CACHE[key] = t
    return t


def _forget_stream_state(device: torch.device, stream) -> None:
    """After a launch that failed the shared counters may not be zero any more: never hand them out again."""
    if device.type == "cuda":
        _COUNTER_CACHE.pop((device.index, _stream_handle(stream)), None)


class PreparedDecode:
    """A fully bound decode call: arguments marshalled once, ``run()`` only enqueues the kernels.

    Keeps references to every tensor it points to.  ``run`` may be called repeatedly (e.g. from a
    serving loop or while capturing a HIP graph): it allocates nothing and does not synchronise."""

    def __init__(self, args: FdkDecodeArgs, plan: SplitKvPlan, keep: tuple, out, lse):
        self.args = args
        self.plan = plan
        self._keep = keep
        self.out = out
        self.lse = lse
        self._ref = C.byref(args)

    def run(self, stream=None):
        rc = _LIB.fdk_decode(self._ref, _stream_handle(stream))
        if rc > 0:                                    # a launch failed (rejected arguments launch nothing)
            _forget_stream_state(self.out.device, stream)
        _lib.check(rc)
        return self.out, self.lse

    def run_static(self, stream=None):
        """The same call with the split partials in the library's static scratch (``fdk_decode_static``): no
        workspace, no allocation of any kind.  Calls that overlap in time on one GPU race on that scratch."""
        _lib.check(_LIB.fdk_decode_static(self._ref, _stream_handle(stream)))
        return self.out, self.lse

    def run_splitkv(self, stream=None):
        _lib.check(_LIB.fdk_decode_splitkv(self._ref, _stream_handle(stream)))

    def run_combine(self, stream=None):
        _lib.check(_LIB.fdk_combine(self._ref, _stream_handle(stream)))
        return self.out, self.lse


def prepare_decode(q, k_cache, v_cache, block_table, kv_lens, sm_scale, *, soft_cap=0.0, kv_split=-1,
                   max_kv_len=None, k_scale=None, v_scale=None, out=None, lse=None, workspace=None,
                   algo="auto", packed_out=None, want_lse=True, always_workspace=False, counters=None,
                   work_queue=True, min_kv_len=None, static_scratch=False, stream_scratch=None,
                   probe_loads=False, single_launch=False, wavefronts=0, buffers=0, shares_per_cu=0,
                   length_feedback: Optional[LengthFeedback] = None, timeline: Optional[torch.Tensor] = None,
                   rotate_heads=0, fp8_fold_k_scale=False, force_balanced=False, _planned=None) -> PreparedDecode:
    """Bind all arguments of one decode call.  See ``flash_decode`` for their meaning.

    ``packed_out``: a ``[B, Hq, D+1]`` tensor that receives out in ``[..., :D]`` and lse (converted to its
    dtype) in ``[..., D]`` - the reference's ``output_combine`` layout - instead of ``out``.
    ``counters``: zeroed int32 tensor (``fdk_counters_len`` elements) for the work-queue form of a split decode (a
    forced split count with more pieces than fit the GPU at once: a fixed set of workgroups pulls the pieces, which
    keeps ragged batches balanced) and for ``single_launch``; by default the call owns a private one (or, with
    ``stream_scratch``, shares the stream's).  Every call leaves the counters zero.
    ``work_queue=False`` launches one workgroup per piece instead.
    ``single_launch=True``: no combine kernel - the workgroup that finishes a (sequence, head block) last merges the
    partials (the reference's persistent kernel does this after a grid barrier, flash_decode.py:719-760).  Slower
    than the two launches on MI355X, whose XCDs do not share an L2: measured, kept for comparison.
    ``stream_scratch``: a stream (handle); scratch that the call has to provide itself is then taken from a buffer
    kept per (device, stream) instead of a fresh allocation - only for calls that are issued on that stream at once.
    ``probe_loads=True`` is a measurement aid: the call runs only the load pipeline of the split kernel (the same
    pieces and addresses, no arithmetic, no combine) and leaves out / lse undefined.
    ``static_scratch=True`` binds no workspace and no counters: the call is then to be issued with
    ``run_static()``, which keeps the split partials in the library's own static scratch.
    ``wavefronts`` (4 or 8) / ``buffers`` (1 or 2) are measurement aids: they override how the matrix-core split
    kernel is shaped (wavefronts per workgroup, tiles of loads under way per wavefront); ``shares_per_cu`` (1..4)
    sets how many workgroups per compute unit a balanced plan gets; 0 lets the library choose.  ``force_balanced``
    makes the plan equal shares of the whole batch wherever the matrix-core path can run them.
    ``length_feedback``: a ``LengthFeedback`` that the call's last kernel fills (see there).
    ``fp8_fold_k_scale=True`` (fp8 cache): the K scale multiplies the logits instead of every K value
    (``FDK_FLAG_FP8_FOLD_K_SCALE``: faster, and off the dequantise-then-decode definition by the 16-bit rounding of K).
    ``timeline``: an int64 GPU tensor, eight values per wavefront of the split kernel; only a library built with
    ``--timeline`` writes it; ``rotate_heads`` moves the head blocks over the workgroups in that build.
    The measurement aids travel in a ``fdk_measure_args`` block (include/fdk_measure.h) that the argument block points
    to; a call that uses none of them passes a null pointer, as a product caller does."""
    if not isinstance(kv_lens, torch.Tensor):
        kv_lens = torch.as_tensor(list(kv_lens), dtype=torch.int32, device=q.device)
    # (_planned: the argument block and plan of exactly these arguments, from a caller that has just computed them)
    a, plan = _planned if _planned is not None else _args_and_plan(
        q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap, kv_split, max_kv_len, k_scale, v_scale, algo,
        min_kv_len)
    batch, q_heads = q.shape[:2]
    d = v_cache.shape[-1]                     # values of an output row: V's head dim (the reference's V_DIM)
    measure = None
    if wavefronts or buffers or shares_per_cu or probe_loads or rotate_heads or force_balanced or timeline is not None:
        measure = FdkMeasureArgs()
        measure.struct_size = C.sizeof(FdkMeasureArgs)
        measure.probe_loads = 1 if probe_loads else 0
        measure.wavefronts, measure.buffers, measure.shares_per_cu = int(wavefronts), int(buffers), int(shares_per_cu)
        measure.rotate_heads = int(rotate_heads)
        measure.force_balanced = 1 if force_balanced else 0
        if timeline is not None:
            if timeline.dtype != torch.int64 or not timeline.is_cuda or not timeline.is_contiguous():
                raise ValueError("timeline must be a contiguous int64 GPU tensor")
            measure.timeline, measure.timeline_len = timeline.data_ptr(), timeline.numel()
        a.measure = C.addressof(measure)
        if shares_per_cu or force_balanced:
            plan = _plan_of(a)                   # these change the plan (workgroups, workspace)
    if length_feedback is not None:
        a.length_feedback = length_feedback.device_ptr
    if packed_out is not None:
        if tuple(packed_out.shape) != (batch, q_heads, d + 1) or packed_out.stride(-1) != 1:
            raise ValueError(f"packed output must be [B, Hq, D+1] = {(batch, q_heads, d + 1)}")
        a.flags |= _lib.FDK_FLAG_PACK_LSE
        target = packed_out
    else:
        if out is None:
            out = torch.empty((batch, q_heads, d), dtype=q.dtype, device=q.device)
        elif tuple(out.shape) != (batch, q_heads, d) or out.stride(-1) != 1:
            raise ValueError(f"out must be [B, Hq, D] = {(batch, q_heads, d)} with contiguous D")
        target = out
    if not target.is_cuda:
        raise ValueError("output tensor must live on the GPU")
    a.out = target.data_ptr()
    a.out_stride_b, a.out_stride_h = target.stride(0), target.stride(1)
    a.out_dtype = _fdk_dtype(target.dtype, "out")
    if lse is None and want_lse:
        lse = torch.empty((batch, q_heads), dtype=torch.float32, device=q.device)
    if lse is not None:
        if lse.dtype != torch.float32 or tuple(lse.shape) != (batch, q_heads) or lse.stride(-1) != 1:
            raise ValueError("lse must be fp32 [B, Hq] with contiguous heads")
        a.lse = lse.data_ptr()
        a.lse_stride_b = lse.stride(0) if batch > 1 else max(lse.stride(0), q_heads)
    need = plan.workspace_bytes if (plan.num_splits > 1 or always_workspace) else 0
    if static_scratch:
        need, work_queue, workspace = 0, False, None
    if need:
        if workspace is not None and (not workspace.is_cuda or not workspace.is_contiguous() or
                                      workspace.numel() * workspace.element_size() < need or
                                      workspace.data_ptr() % 16):
            workspace = None        # too small / unusable: take our own
        if workspace is None and stream_scratch is not None:
            workspace = _stream_scratch(q.device, stream_scratch, need)      # shared by the calls of one stream
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        a.workspace = workspace.data_ptr()
        a.workspace_bytes = workspace.numel() * workspace.element_size()
    if fp8_fold_k_scale:
        a.flags |= _lib.FDK_FLAG_FP8_FOLD_K_SCALE
    if single_launch:
        a.flags |= _lib.FDK_FLAG_SINGLE_LAUNCH
    if plan.num_splits > 1 and plan.algo == "mfma" and ((work_queue and not plan.balanced) or single_launch):
        n_ctr = int(_LIB.fdk_counters_len(C.byref(a)))
        if counters is None and stream_scratch is not None:
            counters = _stream_counters(q.device, stream_scratch, n_ctr)         # None while capturing a graph
        if counters is None:
            counters = torch.zeros(n_ctr, dtype=torch.int32, device=q.device)
        elif counters.dtype != torch.int32 or counters.numel() < n_ctr or not counters.is_cuda or \
                not counters.is_contiguous():
            raise ValueError(f"counters must be a contiguous int32 GPU tensor of at least {n_ctr} zeros")
        a.counters = counters.data_ptr()
        a.counters_len = counters.numel()
    else:
        counters = None
    keep = (q, k_cache, v_cache, block_table, kv_lens, k_scale, v_scale, target, lse, workspace, length_feedback, timeline, measure,
            counters)
    return PreparedDecode(a, plan, keep, target, lse)


def flash_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                 kv_lens: Union[torch.Tensor, Sequence[int]], sm_scale: float, *, soft_cap: float = 0.0,
                 kv_split: int = -1, max_kv_len: Optional[int] = None, k_scale: Optional[torch.Tensor] = None,
                 v_scale: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                 lse: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                 algo: str = "auto", stream=None, min_kv_len: Optional[int] = None,
                 fp8_fold_k_scale: bool = False, force_balanced: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Local (one GPU's share) split-KV GQA decode attention over a paged KV cache.

    q            [B, Hq, D] bf16/fp16, one query token per sequence
    k_cache      [num_pages, P, Hkv, D] in q's dtype or float8_e4m3fn
    v_cache      same shape and dtype as k_cache
    block_table  [B, max_pages] int32: page of token n is ``block_table[b, n // P]``, slot ``n % P``
    kv_lens      [B] int32 (device tensor; never read on the host)
    sm_scale     logit scale
    soft_cap     > 0: logits become ``soft_cap * tanh(logits / soft_cap)``
    kv_split     force this many KV splits (default: chosen from the shape and the CU count)
    max_kv_len   host-known upper bound of kv_lens, used only to size the splits
                 (default ``max_pages * P``)
    min_kv_len   host-known lower bound of kv_lens (default: unknown).  A batch whose bounds lie within 1/32 of
                 each other gets whole sequences per workgroup (a single pass where they fill the GPU, else
                 per-sequence chunks of one size); otherwise long contexts of two or more sequences are cut into
                 equal shares of the tokens on the device (a single pass is as slow as its longest sequence) and
                 per-sequence chunks follow each sequence's own length; results never depend on it
    k_scale/v_scale  [Hkv] fp32 dequantisation scales of an fp8 cache
    fp8_fold_k_scale fp8 cache: apply k_scale to the logits instead of to every K value (see ``prepare_decode``)
    force_balanced   measurement / test aid: equal shares of the whole batch whatever the planner would choose

    Returns ``(out [B,Hq,D] in q's dtype, lse [B,Hq] fp32)``: out is normalised by the local softmax sum
    and lse = ln sum exp(scaled logits) - what the cross-rank combine consumes."""
    if q.is_cuda:
        stream = _stream_handle(stream)               # looked up once: torch.cuda.current_stream() is not free
    call = prepare_decode(q, k_cache, v_cache, block_table, kv_lens, sm_scale, soft_cap=soft_cap,
                          kv_split=kv_split, max_kv_len=max_kv_len, k_scale=k_scale, v_scale=v_scale,
                          out=out, lse=lse, workspace=workspace, algo=algo, min_kv_len=min_kv_len,
                          fp8_fold_k_scale=fp8_fold_k_scale, force_balanced=force_balanced,
                          stream_scratch=stream if q.is_cuda else None,
                          work_queue=kv_split > 0)      # the library's own plans never exceed the resident set
    return call.run(stream)


def _reference_kv_split(kv_split: int, q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap, lo=None, hi=None):
    """How the drop-ins for the reference's entry points read ``kv_split`` (its ``NUM_KV_SPLITS``): as the most splits
    to use, not as a count to force.  The reference's layer passes a fixed 32 (sp_flash_decode_layer.py:62) whatever the
    shape; results do not depend on the count, and a batch that fills the GPU on its own is not to be cut into 32 chunks
    per sequence (the Llama-3-8B shape at batch 32: 89 us as equal shares of the tokens, 135 us in 32 chunks of 128
    tokens).  If the plan the library would choose on its own cuts the batch into equal shares (balanced mode, its answer
    to lengths it does not know) or needs no more partial rows than ``kv_split`` allows, it is used; otherwise the count
    is forced.  Returns the count to pass on (-1: the library's plan) and, if it was computed, that plan with its
    argument block.
    ``flash_decode`` / ``prepare_decode`` always force."""
    if kv_split is None or kv_split <= 0:
        return -1, None
    if not isinstance(kv_lens, torch.Tensor) or not q.is_cuda:
        return kv_split, None
    # the argument block and plan that the call itself uses when the library's own plan is taken: handed on
    planned = _args_and_plan(q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap, -1, hi, None, None, "auto", lo)
    own = planned[1]
    return (-1, planned) if own.balanced or own.num_splits <= kv_split else (kv_split, None)


def _drop_in_bounds(q, kv_lens, fb):
    """Length bounds for the drop-in entry points, whose signature has none: a call that is given a ``LengthFeedback``
    leaves the smallest and the largest of ``kv_lens`` there, and the next call that is given the same block reads
    them on the host - no synchronisation, and one call late at worst, which the plan tolerates (a decode step adds
    one token per sequence; a batch that was recomposed runs its first call on the old bounds, slower but right)."""
    if fb is None or not (q.is_cuda and isinstance(kv_lens, torch.Tensor) and kv_lens.dim() == 1):
        return None, None, None
    if _capturing():
        # A captured call is replayed while kv_lens grows: bounds read now would be baked into the graph, and a plan
        # that trusts them (equal chunks sized for today's length, the last one running to the end) would leave almost
        # all tokens of a much longer replay to one workgroup per sequence.  Plan as for unknown lengths; the block
        # is still written by every replay.
        return fb, None, None
    lo, hi = fb.bounds(kv_lens.numel())
    return fb, lo, hi


def gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                    soft_cap=0.0, output_split=None, output_combine=None, kv_split=-1,
                                    stream=None, length_feedback: Optional[LengthFeedback] = None):
    """Drop-in for the reference function of the same name (flash_decode.py:847-928).

    Returns ``output_combine [B, Hq, D+1]`` in q's dtype: attention output in ``[..., :D]``, lse in
    ``[..., D]``.  ``workspace`` and ``q_lens`` are ignored as in the reference.
    ``length_feedback`` (not in the reference): a ``LengthFeedback`` that the caller keeps for this batch; the call
    plans with the bounds the previous call left there and leaves its own (see ``LengthFeedback``).  Without it the
    call knows nothing about the lengths and every call plans alike."""
    batch, q_heads = q.shape[:2]
    d = v_cache.shape[-1]
    if output_combine is None:
        output_combine = torch.empty((batch, q_heads, d + 1), dtype=q.dtype, device=q.device)
    if q.is_cuda:
        stream = _stream_handle(stream)
    fb, lo, hi = _drop_in_bounds(q, kv_lens, length_feedback)
    kv_split, planned = _reference_kv_split(kv_split, q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap, lo, hi)
    call = prepare_decode(q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap=soft_cap,
                          kv_split=kv_split, workspace=_as_scratch(output_split), packed_out=output_combine,
                          want_lse=False, stream_scratch=stream if q.is_cuda else None, work_queue=kv_split > 0,
                          max_kv_len=hi, min_kv_len=lo, length_feedback=fb, _planned=planned)
    call.run(stream)
    return output_combine


def gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0.0,
                         output_split=None, output_combine=None, kv_split=-1, stream=None,
                         length_feedback: Optional[LengthFeedback] = None):
    """Drop-in for the reference function of the same name (flash_decode.py:763-844): ``[B, Hq, D]``."""
    if q.is_cuda:
        stream = _stream_handle(stream)
    fb, lo, hi = _drop_in_bounds(q, kv_lens, length_feedback)
    kv_split, planned = _reference_kv_split(kv_split, q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap, lo, hi)
    call = prepare_decode(q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap=soft_cap,
                          kv_split=kv_split, workspace=_as_scratch(output_split), out=output_combine,
                          want_lse=False, stream_scratch=stream if q.is_cuda else None, work_queue=kv_split > 0,
                          max_kv_len=hi, min_kv_len=lo, length_feedback=fb, _planned=planned)
    return call.run(stream)[0]


def gqa_fwd_batch_decode_intra_rank_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table,
                                        scale, soft_cap=0, output_split=None, output_combine=None, kv_split=-1):
    """Stream-first form (flash_decode.py:1037-1092)."""
    return gqa_fwd_batch_decode_intra_rank(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                           soft_cap, output_split, output_combine, kv_split, stream=stream)


def gqa_fwd_batch_decode_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                             soft_cap=0, output_split=None, output_combine=None, kv_split=-1):
    """Stream-first form (flash_decode.py:979-1034)."""
    return gqa_fwd_batch_decode(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap,
                                output_split, output_combine, kv_split, stream=stream)


def gqa_fwd_batch_decode_persistent(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap=0,
                                    output_split=None, output_combine=None, kv_split=-1, stream=None):
    """Drop-in for the reference function of the same name (flash_decode.py:931-976): ``[B, Hq, D]``.

    The reference runs a fixed grid of 132 programs that loop over (sequence, head, split) items and merge after a
    grid barrier on the int32 ``workspace``.  Here the same split count (32 unless ``kv_split`` says otherwise) runs
    as the work-queue form of the split kernel - two workgroups per compute unit pulling items - followed by the
    combine kernel (``prepare_decode(..., single_launch=True)`` is the one-launch form; it is slower on MI355X).  ``workspace`` is ignored: the reference's barrier works with any initial contents of it
    (common_ops.py:57-81), whereas the queue's counters must be zero on entry, so the library always uses counters
    of its own (per stream, left at zero by every call).  The result is in q's dtype (the reference allocates
    float16 whatever q is)."""
    splits, planned = _reference_kv_split(32 if kv_split == -1 else kv_split, q, k_cache, v_cache, block_table, kv_lens,
                                          scale, soft_cap)
    if q.is_cuda:
        stream = _stream_handle(stream)
    call = prepare_decode(q, k_cache, v_cache, block_table, kv_lens, scale, soft_cap=soft_cap, kv_split=splits,
                          workspace=_as_scratch(output_split), out=output_combine, want_lse=False,
                          stream_scratch=stream if q.is_cuda else None, _planned=planned)
    return call.run(stream)[0]


def gqa_fwd_batch_decode_persistent_aot(stream, q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale,
                                        soft_cap=0, output_split=None, output_combine=None, kv_split=-1):
    """Stream-first form (flash_decode.py:1095-1150)."""
    return gqa_fwd_batch_decode_persistent(q, k_cache, v_cache, workspace, q_lens, kv_lens, block_table, scale, soft_cap,
                                           output_split, output_combine, kv_split, stream=stream)


def _as_scratch(output_split: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if output_split is None or not output_split.is_contiguous():
        return None
    return output_split.view(-1).view(torch.uint8)


def pack_out_lse(out: torch.Tensor, lse: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``(out [B,Hq,D], lse [B,Hq]) -> [B,Hq,D+1]`` with lse in the last column (flash_decode.py:235-239)."""
    dtype = dtype or out.dtype
    packed = torch.empty(out.shape[:-1] + (out.shape[-1] + 1,), dtype=dtype, device=out.device)
    packed[..., :-1] = out
    packed[..., -1] = lse
    return packed


def unpack_out_lse(packed: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Inverse of ``pack_out_lse`` (views, no copy)."""
    return packed[..., :-1], packed[..., -1]


def inter_rank_combine(all_ranks_output: torch.Tensor, global_kv_lens: torch.Tensor,
                       final_output: Optional[torch.Tensor] = None, *, all_ranks_lse: Optional[torch.Tensor] = None,
                       lse_out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """Merge per-rank local results into the global attention output.

    all_ranks_output  ``[R, B, Hq, D+1]`` packed (the all-gathered buffer of
                      sp_flash_decode_layer.py:143-145) or ``[R, B, Hq, D]`` together with
                      ``all_ranks_lse [R, B, Hq]`` fp32
    global_kv_lens    ``[R, B]`` int32; rank r takes part for sequence b iff ``> 0`` (flash_decode.py:513-515)
    Returns ``final_output [B, Hq, D]`` in the input dtype."""
    if all_ranks_output.dim() != 4:
        raise ValueError("all_ranks_output must be [R, B, Hq, D(+1)]")
    n_ranks, batch, q_heads, last = all_ranks_output.shape
    packed = all_ranks_lse is None
    d = last - 1 if packed else last
    if all_ranks_output.stride(-1) != 1:
        raise ValueError("last dimension must be contiguous")
    if global_kv_lens.dtype != torch.int32 or tuple(global_kv_lens.shape) != (n_ranks, batch) or \
            not global_kv_lens.is_contiguous():
        raise ValueError("global_kv_lens must be contiguous int32 [R, B]")
    if not all_ranks_output.is_cuda or not global_kv_lens.is_cuda:
        raise ValueError("inputs must live on the GPU; there is no CPU path")
    if final_output is None:
        final_output = torch.empty((batch, q_heads, d), dtype=all_ranks_output.dtype, device=all_ranks_output.device)
    elif tuple(final_output.shape) != (batch, q_heads, d) or final_output.stride(-1) != 1 or \
            final_output.device != all_ranks_output.device:
        raise ValueError(f"final_output must be a GPU tensor [B, Hq, D] = {(batch, q_heads, d)} with contiguous D")
    a = FdkCombineRanksArgs()
    a.struct_size = C.sizeof(FdkCombineRanksArgs)
    a.flags = _lib.FDK_FLAG_PACK_LSE if packed else 0
    a.partial = all_ranks_output.data_ptr()
    a.stride_r, a.stride_b, a.stride_h = all_ranks_output.stride(0), all_ranks_output.stride(1), all_ranks_output.stride(2)
    a.partial_dtype = _fdk_dtype(all_ranks_output.dtype, "all_ranks_output")
    a.out_dtype = _fdk_dtype(final_output.dtype, "final_output")
    if not packed:
        if all_ranks_lse.dtype != torch.float32 or tuple(all_ranks_lse.shape) != (n_ranks, batch, q_heads) or \
                all_ranks_lse.stride(-1) != 1:
            raise ValueError("all_ranks_lse must be fp32 [R, B, Hq]")
        a.partial_lse = all_ranks_lse.data_ptr()
        a.lse_stride_r, a.lse_stride_b = all_ranks_lse.stride(0), all_ranks_lse.stride(1)
    a.kv_lens = global_kv_lens.data_ptr()
    a.num_ranks, a.batch, a.num_q_heads, a.head_dim = n_ranks, batch, q_heads, d
    a.out = final_output.data_ptr()
    a.out_stride_b, a.out_stride_h = final_output.stride(0), final_output.stride(1)
    if lse_out is not None:
        if lse_out.dtype != torch.float32 or tuple(lse_out.shape) != (batch, q_heads) or lse_out.stride(-1) != 1 or \
                lse_out.device != all_ranks_output.device:
            raise ValueError(f"lse_out must be an fp32 GPU tensor [B, Hq] = {(batch, q_heads)} with contiguous heads")
        a.lse = lse_out.data_ptr()
        a.lse_stride_b_out = lse_out.stride(0) if batch > 1 else max(lse_out.stride(0), q_heads)
    _lib.check(_LIB.fdk_combine_ranks(C.byref(a), _stream_handle(stream)))
    return final_output


def flash_decode_bsnh(query: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                      block_tables: torch.Tensor, kv_lens: torch.Tensor, output: Optional[torch.Tensor] = None,
                      sm_scale: Optional[float] = None, soft_cap: float = 0.0, stream=None) -> torch.Tensor:
    """Decode in the layout of the reference's mega-kernel builder: argument order of
    ``ModelBuilder.make_flash_decode`` (mega_triton_kernel/models/model_builder.py:248-286), which records an
    ``attn_split`` + ``attn_combine`` task pair; this runs at once.

    query / output ``[B, 1, Hq, D]`` (one new token per sequence, :274), caches ``[num_pages, P, Hkv, D]``,
    ``sm_scale`` defaults to ``D ** -0.5`` (:275-276).  ``soft_cap`` is honoured (the builder zeroes it, :277)."""
    if query.dim() != 4 or query.shape[1] != 1:
        raise ValueError("query must be [B, 1, Hq, D]: flash decoding takes one query token per sequence")
    batch, _, q_heads, d = query.shape
    if output is None:
        output = torch.empty((batch, 1, q_heads, d), dtype=query.dtype, device=query.device)
    elif tuple(output.shape) != (batch, 1, q_heads, d):
        raise ValueError(f"output must be [B, 1, Hq, D] = {(batch, 1, q_heads, d)}")
    if sm_scale is None:
        sm_scale = d ** -0.5
    if query.is_cuda:
        stream = _stream_handle(stream)
    call = prepare_decode(query[:, 0], key_cache, value_cache, block_tables, kv_lens, sm_scale, soft_cap=soft_cap,
                          out=output[:, 0], want_lse=False, stream_scratch=stream, work_queue=False)
    call.run(stream)
    return output


_KV_APPEND_TEMPLATES = {}      # layout key -> (validated argument block, shape of q_norm_rope, fp8 cache)


def qk_norm_rope_update_kvcache(qkv: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                                block_tables: torch.Tensor, kv_lens: torch.Tensor, q_rms_weight: torch.Tensor,
                                k_rms_weight: torch.Tensor, cos_cache: torch.Tensor, sin_cache: torch.Tensor,
                                q_norm_rope: Optional[torch.Tensor] = None, q_rms_eps: float = 1e-6,
                                k_rms_eps: float = 1e-6, *, k_scale: Optional[torch.Tensor] = None,
                                v_scale: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """The step before the decode: per-head RMSNorm and rotary embedding of the new tokens' q and k rows, and the
    append of their K / V rows to the paged cache.  Argument order of the reference's
    ``ModelBuilder.make_qk_norm_rope_update_kvcache`` (mega_triton_kernel/models/model_builder.py:341-345).

    qkv          [B, T, Hq + 2 Hkv, D] bf16/fp16: q heads, k heads, v heads of the T new tokens
    key_cache    [num_pages, P, Hkv, D] in qkv's dtype or float8_e4m3fn (then with k_scale / v_scale [Hkv] fp32);
    value_cache  updated in place at positions ``kv_lens[b] - T + t``
    block_tables [B, max_pages] int32;  kv_lens [B] int32, ALREADY counting the new tokens (model_builder.py:347)
    q/k_rms_weight [D] in qkv's dtype;  cos_cache / sin_cache [S, D], [1, S, D] or [B, S, D] fp32, row = position
    Returns ``q_norm_rope [B, T, Hq, D]`` - the query the decode takes (reshape to [B, Hq, D] for T = 1)."""
    # A decode loop calls this once per layer and step with the same layouts: the checks and the argument block depend
    # on shapes, strides, dtypes and devices only, so a call whose layouts were seen before copies the validated block
    # and sets the pointers (11 us -> 6 us per call on the host; the kernel takes 3.5 us).
    def meta(t):
        return None if t is None else (t.shape, t.stride(), t.dtype, t.device)
    key = (meta(qkv), meta(key_cache), meta(value_cache), meta(block_tables), meta(kv_lens), meta(q_rms_weight),
           meta(k_rms_weight), meta(cos_cache), meta(sin_cache), meta(q_norm_rope), meta(k_scale), meta(v_scale),
           q_rms_eps, k_rms_eps)
    hit = _KV_APPEND_TEMPLATES.get(key)
    if hit is not None:
        a = FdkKvAppendArgs.from_buffer_copy(hit[0])
        if q_norm_rope is None:
            q_norm_rope = torch.empty(hit[1], dtype=qkv.dtype, device=qkv.device)
        a.qkv, a.q_out = qkv.data_ptr(), q_norm_rope.data_ptr()
        a.q_weight, a.k_weight = q_rms_weight.data_ptr(), k_rms_weight.data_ptr()
        a.cos, a.sin = cos_cache.data_ptr(), sin_cache.data_ptr()
        a.block_table, a.kv_lens = block_tables.data_ptr(), kv_lens.data_ptr()
        a.k_cache, a.v_cache = key_cache.data_ptr(), value_cache.data_ptr()
        if k_scale is not None and v_scale is not None and hit[2]:
            a.k_scale, a.v_scale = k_scale.data_ptr(), v_scale.data_ptr()
        _lib.check(_LIB.fdk_kv_append(C.byref(a), _stream_handle(stream)))
        return q_norm_rope
    q_given = q_norm_rope is not None
    if qkv.dim() != 4 or key_cache.dim() != 4 or value_cache.dim() != 4:
        raise ValueError("qkv must be [B, T, heads, D]; caches [num_pages, P, Hkv, D]")
    batch, new_tokens, heads, d = qkv.shape
    num_pages, page_size, kv_heads, dk = key_cache.shape
    if dk != d or tuple(value_cache.shape) != tuple(key_cache.shape) or key_cache.dtype != value_cache.dtype:
        raise ValueError("caches must share shape and dtype, with qkv's head_dim")
    q_heads = heads - 2 * kv_heads
    if q_heads < 0:
        raise ValueError(f"qkv has {heads} heads, fewer than 2 * {kv_heads} kv heads")
    fp8 = key_cache.dtype == torch.float8_e4m3fn
    if not fp8 and key_cache.dtype != qkv.dtype:
        raise ValueError("a 16-bit cache must have qkv's dtype")
    if fp8 and (k_scale is None or v_scale is None):
        raise ValueError("k_scale / v_scale are required for an fp8 cache")
    for name, tns in (("qkv", qkv), ("key_cache", key_cache), ("value_cache", value_cache)):
        if tns.stride(-1) != 1:
            raise ValueError(f"{name}: the head dimension must be contiguous")
        if not tns.is_cuda:
            raise ValueError(f"{name} must live on the GPU; there is no CPU path")
    for name, w in (("q_rms_weight", q_rms_weight), ("k_rms_weight", k_rms_weight)):
        if w.dtype != qkv.dtype or tuple(w.shape) != (d,) or not w.is_contiguous() or not w.is_cuda:
            raise ValueError(f"{name} must be a contiguous [{d}] GPU tensor of qkv's dtype")
    if cos_cache.shape != sin_cache.shape or cos_cache.dtype != torch.float32 or sin_cache.dtype != torch.float32 or \
            cos_cache.stride() != sin_cache.stride() or not cos_cache.is_cuda or not sin_cache.is_cuda:
        raise ValueError("cos_cache and sin_cache must be fp32 GPU tensors of one shape and layout")
    cs = cos_cache if cos_cache.dim() == 3 else cos_cache[None]
    if cs.dim() != 3 or cs.shape[0] not in (1, batch) or cs.shape[-1] < d // 2 or cs.stride(-1) != 1:
        raise ValueError("cos_cache / sin_cache must be [S, D], [1, S, D] or [B, S, D]")
    if block_tables.dtype != torch.int32 or kv_lens.dtype != torch.int32 or block_tables.dim() != 2 or \
            block_tables.shape[0] != batch or block_tables.stride(-1) != 1 or tuple(kv_lens.shape) != (batch,) or \
            not kv_lens.is_contiguous() or not block_tables.is_cuda or not kv_lens.is_cuda:
        raise ValueError("block_tables [B, max_pages] and kv_lens [B] must be contiguous int32 GPU tensors")
    if q_norm_rope is None:
        q_norm_rope = torch.empty((batch, new_tokens, q_heads, d), dtype=qkv.dtype, device=qkv.device)
    elif tuple(q_norm_rope.shape) != (batch, new_tokens, q_heads, d) or q_norm_rope.dtype != qkv.dtype or \
            q_norm_rope.stride(-1) != 1 or not q_norm_rope.is_cuda:
        raise ValueError(f"q_norm_rope must be a GPU tensor [{batch}, {new_tokens}, {q_heads}, {d}] of qkv's dtype")
    a = FdkKvAppendArgs()
    a.struct_size = C.sizeof(FdkKvAppendArgs)
    a.qkv = qkv.data_ptr()
    a.qkv_stride_b, a.qkv_stride_t, a.qkv_stride_h = qkv.stride(0), qkv.stride(1), qkv.stride(2)
    a.qkv_dtype = _fdk_dtype(qkv.dtype, "qkv")
    a.kv_dtype = _fdk_dtype(key_cache.dtype, "key_cache")
    a.q_weight, a.k_weight = q_rms_weight.data_ptr(), k_rms_weight.data_ptr()
    a.q_eps, a.k_eps = float(q_rms_eps), float(k_rms_eps)
    a.cos, a.sin = cos_cache.data_ptr(), sin_cache.data_ptr()
    a.cs_stride_b = cs.stride(0) if cs.shape[0] > 1 else 0
    a.cs_stride_pos, a.max_positions = cs.stride(1), cs.shape[1]
    a.batch, a.new_tokens, a.num_q_heads, a.num_kv_heads, a.head_dim = batch, new_tokens, q_heads, kv_heads, d
    a.block_table, a.table_stride_b, a.kv_lens = block_tables.data_ptr(), block_tables.stride(0), kv_lens.data_ptr()
    a.page_size, a.max_pages, a.num_pages = page_size, block_tables.shape[1], num_pages
    a.k_cache, a.v_cache = key_cache.data_ptr(), value_cache.data_ptr()
    a.k_stride_page, a.k_stride_tok, a.k_stride_head = key_cache.stride(0), key_cache.stride(1), key_cache.stride(2)
    a.v_stride_page, a.v_stride_tok, a.v_stride_head = value_cache.stride(0), value_cache.stride(1), value_cache.stride(2)
    if fp8:
        for name, sc in (("k_scale", k_scale), ("v_scale", v_scale)):
            if sc.dtype != torch.float32 or tuple(sc.shape) != (kv_heads,) or not sc.is_contiguous() or not sc.is_cuda:
                raise ValueError(f"{name} must be a contiguous fp32 GPU tensor [{kv_heads}]")
        a.k_scale, a.v_scale = k_scale.data_ptr(), v_scale.data_ptr()
    a.q_out = q_norm_rope.data_ptr()
    a.q_out_stride_b, a.q_out_stride_t, a.q_out_stride_h = q_norm_rope.stride(0), q_norm_rope.stride(1), q_norm_rope.stride(2)
    _lib.check(_LIB.fdk_kv_append(C.byref(a), _stream_handle(stream)))
    # (only after the library has accepted the block; a result tensor of the call's own has the contiguous layout)
    if q_given or q_norm_rope.is_contiguous():
        if len(_KV_APPEND_TEMPLATES) >= 256:
            _KV_APPEND_TEMPLATES.clear()
        _KV_APPEND_TEMPLATES[key] = (bytes(a), tuple(q_norm_rope.shape), fp8)
    return q_norm_rope


def probe_linear_read(buf: torch.Tensor, nontemporal: bool = True, workgroups: int = 512, stream=None) -> None:
    """Measurement aid: stream ``buf`` (a contiguous GPU tensor) through ``workgroups`` workgroups once, with
    16-byte loads that carry the non-temporal hint or not; nothing is written (``fdk_probe_linear_read``)."""
    if not buf.is_cuda or not buf.is_contiguous():
        raise ValueError("buf must be a contiguous GPU tensor")
    _lib.check(_LIB.fdk_probe_linear_read(buf.data_ptr(), buf.numel() * buf.element_size(), int(bool(nontemporal)),
                                          int(workgroups), _stream_handle(stream)))
