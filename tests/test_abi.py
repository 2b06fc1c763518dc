"""C-ABI checks that need no GPU: the library loads, exports what include/fdk.h declares, the ctypes
mirror has the C layout, and argument validation / planning work on fake pointers (dry run)."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fdk.h")
MEASURE_HEADER = os.path.join(ROOT, "include", "fdk_measure.h")
FROZEN_HEADER = os.path.join(ROOT, "tests", "c_abi", "fdk_abi8_rev0.h")      # include/fdk.h as first released (ABI 8)

from triton_distributed_amd import _lib  # noqa: E402
from triton_distributed_amd._lib import (FdkCombineRanksArgs, FdkDecodeArgs, FdkKvAppendArgs, FdkMeasureArgs,  # noqa: E402
                                         FdkPlan)


def _declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fdk_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS), names
    measure = _declared_functions(MEASURE_HEADER)
    assert set(measure) == set(_lib.MEASURE_EXPORTS), measure
    # a caller compiled against the first release of this ABI version finds every function it was promised
    for n in names + measure + _declared_functions(FROZEN_HEADER):
        assert hasattr(lib, n), n
    assert lib.fdk_abi_version() == _lib.FDK_ABI_VERSION
    assert lib.fdk_abi_revision() >= _lib.FDK_ABI_REVISION
    # the product header names no measurement aid
    product = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for word in ("tune_", "timeline", "probe", "PROBE"):
        assert word not in product, word


def test_ctypes_structs_match_the_c_layout(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "fdk_measure.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(fdk_decode_args), offsetof(fdk_decode_args, kv_dtype),
         offsetof(fdk_decode_args, block_table), offsetof(fdk_decode_args, sm_scale),
         offsetof(fdk_decode_args, out), offsetof(fdk_decode_args, lse), offsetof(fdk_decode_args, workspace_bytes),
         offsetof(fdk_decode_args, length_feedback), offsetof(fdk_decode_args, measure),
         sizeof(fdk_measure_args), offsetof(fdk_measure_args, rotate_heads), offsetof(fdk_measure_args, timeline_len));
  printf("%zu %zu %zu %zu\n", sizeof(fdk_combine_ranks_args), offsetof(fdk_combine_ranks_args, partial_lse),
         offsetof(fdk_combine_ranks_args, kv_lens), offsetof(fdk_combine_ranks_args, lse_stride_b_out));
  printf("%zu %zu %zu\n", sizeof(fdk_plan_t), offsetof(fdk_plan_t, balanced), offsetof(fdk_plan_t, workgroups));
  printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(fdk_kv_append_args), offsetof(fdk_kv_append_args, q_weight),
         offsetof(fdk_kv_append_args, cos), offsetof(fdk_kv_append_args, max_positions),
         offsetof(fdk_kv_append_args, block_table), offsetof(fdk_kv_append_args, k_cache),
         offsetof(fdk_kv_append_args, k_scale), offsetof(fdk_kv_append_args, q_out_stride_h));
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True)
    lines = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    got = [int(x) for x in lines[0].split()]
    want = [C.sizeof(FdkDecodeArgs)] + [getattr(FdkDecodeArgs, f).offset for f in
                                       ("kv_dtype", "block_table", "sm_scale", "out", "lse", "workspace_bytes",
                                        "length_feedback", "measure")] + \
           [C.sizeof(FdkMeasureArgs), FdkMeasureArgs.rotate_heads.offset, FdkMeasureArgs.timeline_len.offset]
    assert got == want
    got = [int(x) for x in lines[1].split()]
    want = [C.sizeof(FdkCombineRanksArgs)] + [getattr(FdkCombineRanksArgs, f).offset for f in
                                             ("partial_lse", "kv_lens", "lse_stride_b_out")]
    assert got == want
    assert [int(x) for x in lines[2].split()] == [C.sizeof(FdkPlan), FdkPlan.balanced.offset, FdkPlan.workgroups.offset]
    got = [int(x) for x in lines[3].split()]
    want = [C.sizeof(FdkKvAppendArgs)] + [getattr(FdkKvAppendArgs, f).offset for f in
                                         ("q_weight", "cos", "max_positions", "block_table", "k_cache", "k_scale",
                                          "q_out_stride_h")]
    assert got == want


def _args(**kw):
    """A valid dry-run argument block on fake (never dereferenced) pointers: B32 32q/8kv P16 N4096."""
    a = FdkDecodeArgs()
    a.struct_size = C.sizeof(FdkDecodeArgs)
    a.flags = _lib.FDK_FLAG_DRY_RUN
    a.q, a.k_cache, a.v_cache = 0x10000, 0x20000, 0x30000
    a.block_table, a.kv_lens, a.out, a.lse = 0x40000, 0x50000, 0x60000, 0x70000
    a.q_dtype = a.kv_dtype = a.out_dtype = _lib.FDK_BF16
    a.batch, a.num_q_heads, a.num_kv_heads, a.head_dim = 32, 32, 8, 128
    a.page_size, a.max_pages = 16, 256
    a.q_stride_b, a.q_stride_h = 32 * 128, 128
    a.k_stride_page, a.k_stride_tok, a.k_stride_head = 16 * 8 * 128, 8 * 128, 128
    a.v_stride_page, a.v_stride_tok, a.v_stride_head = 16 * 8 * 128, 8 * 128, 128
    a.table_stride_b = 256
    a.out_stride_b, a.out_stride_h = 32 * 128, 128
    a.lse_stride_b = 32
    a.sm_scale = 128 ** -0.5
    a.workspace, a.workspace_bytes = 0x80000, 1 << 30
    for k, v in kw.items():
        setattr(a, k, v)
    return a


def _decode_rc(a):
    return _lib.load().fdk_decode(C.byref(a), None)


def test_valid_arguments_pass_dry_run():
    assert _decode_rc(_args()) == 0
    assert _lib.load().fdk_last_error() == b""


@pytest.mark.parametrize("field,value,code", [
    ("struct_size", 8, _lib.FDK_EABI),
    ("q", None, _lib.FDK_ENULL),
    ("kv_lens", None, _lib.FDK_ENULL),
    ("out", None, _lib.FDK_ENULL),
    ("q", 0x10008, _lib.FDK_EALIGN),
    ("k_cache", 0x20004, _lib.FDK_EALIGN),
    ("k_stride_tok", 8 * 128 + 4, _lib.FDK_EALIGN),
    ("q_stride_h", 132, _lib.FDK_EALIGN),
    ("num_kv_heads", 5, _lib.FDK_ESHAPE),
    ("num_q_heads", 0, _lib.FDK_ESHAPE),
    ("batch", -1, _lib.FDK_ESHAPE),
    ("page_size", 0, _lib.FDK_ESHAPE),
    ("max_pages", 0, _lib.FDK_ESHAPE),
    ("table_stride_b", 255, _lib.FDK_ESHAPE),
    ("out_stride_h", 127, _lib.FDK_ESHAPE),
    ("num_splits", 5000, _lib.FDK_ESHAPE),
    ("head_dim", 96, _lib.FDK_EUNSUPPORTED),
    ("head_dim", 512, _lib.FDK_EUNSUPPORTED),
    ("q_dtype", _lib.FDK_FP32, _lib.FDK_EUNSUPPORTED),
    ("kv_dtype", _lib.FDK_FP16, _lib.FDK_EUNSUPPORTED),
    ("out_dtype", _lib.FDK_FP8_E4M3, _lib.FDK_EUNSUPPORTED),
    ("algo", 7, _lib.FDK_EUNSUPPORTED),
    ("sm_scale", float("nan"), _lib.FDK_ESHAPE),
    ("sm_scale", float("inf"), _lib.FDK_ESHAPE),
    ("sm_scale", float("-inf"), _lib.FDK_ESHAPE),
    ("soft_cap", float("nan"), _lib.FDK_ESHAPE),
    ("soft_cap", float("inf"), _lib.FDK_ESHAPE),
    ("k_stride_tok", 1 << 27, _lib.FDK_ESHAPE),             # 16 rows of 2^28 bytes: offsets would not fit 32 bits
    ("v_stride_tok", 1 << 27, _lib.FDK_ESHAPE),
])
def test_bad_arguments_are_rejected_without_a_launch(field, value, code):
    rc = _decode_rc(_args(**{field: value}))
    assert rc == code, (_lib.load().fdk_last_error(), rc)
    assert len(_lib.load().fdk_last_error()) > 0
    with pytest.raises((ValueError, _lib.FdkError)):
        _lib.check(rc)


def test_fp8_scale_pointers_must_be_aligned():
    ok = dict(kv_dtype=_lib.FDK_FP8_E4M3, k_scale=0x90000, v_scale=0x90100)
    assert _decode_rc(_args(**ok)) == 0
    assert _decode_rc(_args(**{**ok, "k_scale": 0x90002})) == _lib.FDK_EALIGN
    assert _decode_rc(_args(**{**ok, "v_scale": 0x90101})) == _lib.FDK_EALIGN


def test_static_scratch_entry_validates_like_fdk_decode():
    lib = _lib.load()
    # needs neither workspace nor counters, whatever the plan
    assert lib.fdk_decode_static(C.byref(_args(workspace=None, workspace_bytes=0)), None) == 0
    assert lib.fdk_decode_static(C.byref(_args(batch=4, workspace=None, workspace_bytes=0)), None) == 0, lib.fdk_last_error()
    assert lib.fdk_decode_static(C.byref(_args(num_splits=8, workspace=None, workspace_bytes=0)), None) == 0
    # partials beyond the static scratch: 512 sequences x 32 heads x 64 splits x 129 fp32 = 541 MB
    big = _args(batch=512, num_splits=64, workspace=None, workspace_bytes=0)
    assert lib.fdk_workspace_bytes(512, 32, 128, 64) > _lib.FDK_STATIC_SCRATCH_BYTES
    assert lib.fdk_decode_static(C.byref(big), None) == _lib.FDK_EWORKSPACE
    assert b"static scratch" in lib.fdk_last_error()
    # and the usual rejections
    assert lib.fdk_decode_static(None, None) == _lib.FDK_ENULL
    assert lib.fdk_decode_static(C.byref(_args(out=None)), None) == _lib.FDK_ENULL
    assert lib.fdk_decode_static(C.byref(_args(head_dim=96)), None) == _lib.FDK_EUNSUPPORTED


def test_workspace_is_required_only_when_the_plan_splits():
    # 32 sequences x 8 kv heads, all known to be 4096 tokens long, fill 256 compute units on their own: one pass,
    # no scratch.  Without the lower bound the lengths may differ: equal shares, partial rows, scratch.
    assert _decode_rc(_args(workspace=None, workspace_bytes=0, max_kv_len=4096, min_kv_len=4096)) == 0
    assert _decode_rc(_args(workspace=None, workspace_bytes=0)) == _lib.FDK_EWORKSPACE
    # 4 sequences do not: the KV range is split and the partials need scratch
    assert _decode_rc(_args(batch=4, workspace=None)) == _lib.FDK_EWORKSPACE
    assert _decode_rc(_args(batch=4, workspace_bytes=1024)) == _lib.FDK_EWORKSPACE
    assert _decode_rc(_args(batch=4)) == 0
    # a forced split count needs it as well
    assert _decode_rc(_args(num_splits=4, workspace=None)) == _lib.FDK_EWORKSPACE


def test_counters_of_the_work_queue_form():
    lib = _lib.load()
    a = _args(batch=4)
    n = lib.fdk_counters_len(C.byref(a))
    assert n == 2 + 4 * 8          # queue head, finished workgroups, a ticket per (sequence, kv head, head tile)
    assert lib.fdk_counters_len(None) == 0
    a.counters, a.counters_len = 0x90000, n
    assert _decode_rc(a) == 0
    # the work-queue form exists for forced split counts (chunk mode): there a short or misaligned array is refused,
    # in a dry run as in a real call, before anything is launched
    assert _decode_rc(_args(batch=4, num_splits=8, counters=0x90000, counters_len=n)) == 0
    assert _decode_rc(_args(batch=4, num_splits=8, counters=0x90000, counters_len=1)) == _lib.FDK_EWORKSPACE
    assert _decode_rc(_args(batch=4, num_splits=8, counters=0x90002, counters_len=n)) == _lib.FDK_EALIGN


def test_dry_run_refuses_what_a_real_call_would_refuse():
    lib = _lib.load()
    # a block_table row addresses at most 2^30 tokens (32-bit token arithmetic in the kernels)
    assert _decode_rc(_args(page_size=1 << 20, max_pages=1 << 10, table_stride_b=1 << 10,
                            k_stride_page=(1 << 20) * 1024, v_stride_page=(1 << 20) * 1024)) == 0
    rc = _decode_rc(_args(page_size=1 << 20, max_pages=(1 << 10) + 1, table_stride_b=(1 << 10) + 1,
                          k_stride_page=(1 << 20) * 1024, v_stride_page=(1 << 20) * 1024))
    assert rc == _lib.FDK_ESHAPE and b"2^30" in lib.fdk_last_error()
    # more workgroups than a grid holds
    big = dict(batch=1 << 22, num_splits=1024, workspace_bytes=1 << 62, q_stride_b=32 * 128, out_stride_b=32 * 128)
    rc = _decode_rc(_args(**big))
    assert rc == _lib.FDK_ESHAPE and b"grid" in lib.fdk_last_error()
    a = _args(**big)
    assert lib.fdk_decode_splitkv(C.byref(a), None) == _lib.FDK_ESHAPE
    # a misaligned workspace
    assert _decode_rc(_args(batch=4, workspace=0x80004)) == _lib.FDK_EALIGN


def _measured(measure_kw, **kw):
    """An argument block that points to a measurement block (include/fdk_measure.h); the block is kept alive on it."""
    m = FdkMeasureArgs()
    m.struct_size = C.sizeof(FdkMeasureArgs)
    for k, v in measure_kw.items():
        setattr(m, k, v)
    a = _args(**kw)
    a.measure = C.addressof(m)
    a._measure_block = m
    return a


def test_tuning_overrides_are_validated():
    # measurement aids: 0 (the library's choice), 4 or 8 wavefronts, 1 or 2 buffers; anything else is refused
    for wf, nb, rc in [(0, 0, 0), (4, 1, 0), (8, 2, 0), (8, 0, 0), (2, 0, _lib.FDK_ESHAPE), (16, 0, _lib.FDK_ESHAPE),
                       (0, 3, _lib.FDK_ESHAPE), (0, -1, _lib.FDK_ESHAPE)]:
        assert _decode_rc(_measured(dict(wavefronts=wf, buffers=nb))) == rc, (wf, nb)
    # they never change the plan
    p0, p1 = _plan(_args()), _plan(_measured(dict(wavefronts=8, buffers=1)))
    assert (p0.num_splits, p0.balanced, p0.workgroups, p0.kv_heads_per_wg) == (p1.num_splits, p1.balanced, p1.workgroups,
                                                                                p1.kv_heads_per_wg)
    # workgroups per compute unit of a balanced plan: 0 (one, the library's choice) .. 4; this one is part of the plan
    assert p0.balanced == 1 and p0.workgroups == 256
    p2 = _plan(_measured(dict(shares_per_cu=2)))
    assert p2.balanced == 1 and p2.workgroups == 512 and p2.num_splits > p0.num_splits
    assert _plan(_measured(dict(shares_per_cu=1))).workgroups == 256
    assert _decode_rc(_measured(dict(shares_per_cu=5))) == _lib.FDK_ESHAPE
    assert _decode_rc(_measured(dict(shares_per_cu=-1))) == _lib.FDK_ESHAPE
    # a measurement block of another size than this library's is refused
    bad = _measured({})
    bad._measure_block.struct_size = 8
    assert _decode_rc(bad) == _lib.FDK_EABI


def test_argument_blocks_of_older_and_newer_callers():
    """The structs only grow at the end: a caller compiled against the first release passes a smaller struct_size and
    is served (the fields it lacks read as zero, whatever lies behind its block); what that release kept where the
    reserved fields are now - measurement overrides - is ignored; a block larger than the library's is refused."""
    lib = _lib.load()
    first = FdkDecodeArgs.measure.offset                   # sizeof(fdk_decode_args) of the first release
    a = _args(struct_size=first)
    a.measure = 0xdeadbeef0                                # not part of the caller's block: must not be looked at
    assert _decode_rc(a) == 0, lib.fdk_last_error()
    assert _plan(a).num_splits == _plan(_args()).num_splits
    old = _args(struct_size=first)
    old.reserved0[0], old.reserved0[1], old.reserved0[2] = 16, 3, 7    # were tune_wavefronts / tune_buffers / tune_shares_per_cu
    old.reserved1, old.reserved2 = 0x20004, -5                          # were timeline / timeline_len
    old.flags |= 4                                                      # was the load-probe flag
    assert _decode_rc(old) == 0, lib.fdk_last_error()
    p_old, p_new = _plan(old), _plan(_args())
    assert (p_old.num_splits, p_old.workgroups, p_old.balanced) == (p_new.num_splits, p_new.workgroups, p_new.balanced)
    for size, rc in [(first - 8, _lib.FDK_EABI), (C.sizeof(FdkDecodeArgs) + 8, _lib.FDK_EABI), (0, _lib.FDK_EABI),
                     (first + 4, 0)]:
        assert _decode_rc(_args(struct_size=size)) == rc, size
    assert b"struct_size" in lib.fdk_last_error() or lib.fdk_last_error() == b""


def test_frozen_header_is_a_prefix_of_the_current_one(tmp_path):
    """tests/c_abi/fdk_abi8_rev0.h is include/fdk.h as first released.  Every field of its structs keeps its offset
    (or became a reserved field of the same size), its enums keep their values, and its struct sizes are the
    smallest struct_size the library accepts."""
    prog = r'''
#include <stdio.h>
#include <stddef.h>
#include HEADER
#define O(f) (unsigned)offsetof(fdk_decode_args, f)
int main(void) {
  printf("%u %u %u %u %u %u %u %u %u %u %u\n", (unsigned)sizeof(fdk_decode_args), O(flags), O(q), O(kv_lens), O(num_splits),
         O(sm_scale), O(out), O(workspace), O(counters_len), O(length_feedback), (unsigned)sizeof(fdk_plan_t));
  printf("%u %u %d %d %d %d %u %u\n", (unsigned)sizeof(fdk_combine_ranks_args), (unsigned)sizeof(fdk_kv_append_args),
         FDK_EABI, FDK_FP32, FDK_ALGO_MFMA, FDK_ABI_VERSION, FDK_FLAG_SINGLE_LAUNCH, FDK_STATIC_SCRATCH_BYTES);
  return 0;
}'''
    outs = []
    for name, header in (("old", FROZEN_HEADER), ("new", HEADER)):
        src = tmp_path / f"{name}.c"
        src.write_text(prog.replace("HEADER", f'"{header}"'))
        exe = tmp_path / name
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True)
        outs.append([x.split() for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()])
    old, new = outs
    assert old[0][1:] == new[0][1:] and old[1] == new[1]
    assert int(old[0][0]) == FdkDecodeArgs.measure.offset and int(new[0][0]) == C.sizeof(FdkDecodeArgs)


def test_length_feedback_pointer_is_validated():
    assert _decode_rc(_args(length_feedback=0x20000)) == 0
    assert _decode_rc(_args(length_feedback=0x20008)) == _lib.FDK_EALIGN
    assert _decode_rc(_measured(dict(timeline=0x20008, timeline_len=64))) == 0
    assert _decode_rc(_measured(dict(timeline=0x20004, timeline_len=64))) == _lib.FDK_EALIGN
    lib = _lib.load()
    assert lib.fdk_length_feedback_alloc(None, None) == _lib.FDK_ENULL
    assert lib.fdk_length_feedback_free(None) == 0


def test_packed_output_needs_a_wider_row():
    a = _args(flags=_lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE)
    assert _decode_rc(a) == _lib.FDK_ESHAPE
    a = _args(flags=_lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE, out_stride_h=129, out_stride_b=32 * 129)
    assert _decode_rc(a) == 0


def test_null_args_and_empty_batch():
    lib = _lib.load()
    assert lib.fdk_decode(None, None) == _lib.FDK_ENULL
    # an empty batch is a successful no-op even without the dry-run flag and with null tensors
    a = _args(batch=0, flags=0, q=None, k_cache=None, out=None)
    assert lib.fdk_decode(C.byref(a), None) == 0


def _plan(a, cus=256):
    p = FdkPlan()
    rc = _lib.load().fdk_plan(C.byref(a), cus, C.byref(p))
    assert rc == 0, _lib.load().fdk_last_error()
    return p


def test_plan_scales_splits_with_occupancy():
    p = _plan(_args(max_kv_len=4096, min_kv_len=4096))    # 256 (sequence, kv head) units of equal length on 256 CUs
    assert p.num_splits == 1 and p.chunk_tokens >= 4096   # they fill the device: one pass, no combine
    assert p.algo == _lib.FDK_ALGO_MFMA and p.kv_heads_per_wg == 1
    # the same batch with lengths the host does not vouch for: a single pass would be as slow as its longest
    # sequence, so the tokens are cut into equal shares (one workgroup per compute unit, two kv heads each)
    p = _plan(_args())
    assert p.balanced == 1 and p.workgroups == 256 and p.kv_heads_per_wg == 2 and p.num_splits > 1
    assert _plan(_args(max_kv_len=4096, min_kv_len=2000)).balanced == 1
    # short contexts keep the single pass (nothing to gain from cutting them), and so do batches with four or more
    # workgroups per compute unit, which even out by themselves
    assert _plan(_args(max_kv_len=1024)).num_splits == 1
    p = _plan(_args(batch=1024, q_stride_b=32 * 128, out_stride_b=32 * 128))
    assert p.num_splits == 1 and p.balanced == 0 and p.kv_heads_per_wg == 8
    # equal lengths that fill the compute units unevenly (40 x 8 units on 256: a quarter of them carry two) are
    # cut into equal shares as well; 60 x 8 fill them well enough
    assert _plan(_args(batch=40, max_kv_len=4096, min_kv_len=4096)).balanced == 1
    p = _plan(_args(batch=60, max_kv_len=4096, min_kv_len=4096))
    assert p.balanced == 0 and p.num_splits == 1
    # fewer sequences, short context: chunk mode - chunks are multiples of 64 tokens and cover the range
    p4 = _plan(_args(batch=4))
    assert p4.balanced == 0 and p4.num_splits > 1 and p4.chunk_tokens % 64 == 0
    assert p4.num_splits * p4.chunk_tokens >= 4096 > (p4.num_splits - 1) * p4.chunk_tokens
    # chunk mode aims at one workgroup per compute unit and never launches more than there are compute units
    assert p4.kv_heads_per_wg == 2 and p4.num_splits == 256 // (4 * 4)
    # chunks end on tile boundaries (16 tokens), not coarser: 6 head blocks x 42 chunks of 208 tokens use 252 of the
    # 256 compute units for the reference's benchmark shape at 8K (rounded to 64 tokens it would be 32 x 256 on 192)
    p_ref = _plan(_args(batch=1, num_q_heads=96, num_kv_heads=12, page_size=1, max_pages=8192, table_stride_b=8192,
                        k_stride_page=12 * 128, k_stride_tok=12 * 128, v_stride_page=12 * 128, v_stride_tok=12 * 128,
                        q_stride_b=96 * 128, out_stride_b=96 * 128, lse_stride_b=96))
    assert p_ref.balanced == 0 and p_ref.chunk_tokens % 16 == 0 and p_ref.kv_heads_per_wg == 2
    assert 6 * p_ref.num_splits <= 256 < 6 * (p_ref.num_splits + 3)
    # 96 units, 1024 tokens: one workgroup per compute unit where the host vouches for the lengths; lengths it knows
    # nothing about get two (finer chunks of the long sequences, should the batch be ragged) once the cache streams for
    # more than a dozen microseconds
    p24 = _plan(_args(batch=24, max_pages=64, table_stride_b=64, max_kv_len=1024, min_kv_len=1024))
    assert p24.balanced == 0 and p24.num_splits == 2 and p24.chunk_tokens == 512 and p24.chunk_floor == 0
    p24u = _plan(_args(batch=24, max_pages=64, table_stride_b=64))
    assert p24u.balanced == 0 and p24u.num_splits == 4 and p24u.chunk_tokens == 256 and p24u.chunk_floor == 64
    p8u = _plan(_args(batch=8, max_pages=64, table_stride_b=64))        # 5 us of streaming: one per compute unit
    assert p8u.balanced == 0 and p8u.num_splits == 8 and p8u.chunk_floor == 64
    # few units, long context: balanced mode - one workgroup per compute unit, they share the KV ranges of the whole
    # batch, each gets a long share, and the workspace holds (shares + batch) slots per head block
    p_long = _plan(_args(batch=4, num_q_heads=64, page_size=64, max_pages=2048, table_stride_b=2048,
                         q_stride_b=64 * 128, out_stride_b=64 * 128, lse_stride_b=64))
    assert p_long.balanced == 1 and p_long.workgroups == 256 and p_long.chunk_tokens >= 512
    units = 8 // p_long.kv_heads_per_wg
    shares = p_long.workgroups // units
    rows = (shares + 4) * units * p_long.kv_heads_per_wg * 8           # group = 8 heads per tile
    assert p_long.num_splits * 4 * 64 >= rows > (p_long.num_splits - 1) * 4 * 64
    assert shares * p_long.chunk_tokens >= 4 * 131072                   # the shares cover every sequence
    # ... but only where streaming the cache at its bound takes some tens of microseconds: a batch of the same kind with
    # 8192-token tables (4 x 8192 x 8 heads x 512 B = 134 MB, about 20 us) is cut into chunks of each sequence's own
    # length, two workgroups per compute unit (lengths unknown); equal shares can still be forced for measurements
    short_kw = dict(batch=4, num_q_heads=64, page_size=64, max_pages=128, table_stride_b=128, q_stride_b=64 * 128,
                    out_stride_b=64 * 128, lse_stride_b=64)
    p_mid = _plan(_args(**short_kw))
    assert p_mid.balanced == 0 and p_mid.chunk_floor == 64 and p_mid.num_splits * 4 * (8 // p_mid.kv_heads_per_wg) == 512
    assert _plan(_measured(dict(force_balanced=1), **short_kw)).balanced == 1
    assert _decode_rc(_measured(dict(force_balanced=2), **short_kw)) == _lib.FDK_ESHAPE
    # a single sequence has nothing to balance: per-sequence chunks that follow its own length
    p_one = _plan(_args(batch=1, num_q_heads=64, page_size=64, max_pages=2048, table_stride_b=2048,
                        q_stride_b=64 * 128, out_stride_b=64 * 128, lse_stride_b=64))
    assert p_one.balanced == 0 and p_one.chunk_floor == 64 and p_one.num_splits * (8 // p_one.kv_heads_per_wg) == 256
    assert p_one.chunk_tokens % 16 == 0 and p_one.num_splits * p_one.chunk_tokens >= 131072
    assert p_long.chunk_floor == 0
    # the same shape with a host-known lower bound close to the upper one: the batch is uniform, so per-sequence
    # chunks (one workgroup per compute unit) replace the balanced shares; a looser bound changes nothing
    long_kw = dict(batch=4, num_q_heads=64, page_size=64, max_pages=2048, table_stride_b=2048, q_stride_b=64 * 128,
                   out_stride_b=64 * 128, lse_stride_b=64)
    p_uni = _plan(_args(min_kv_len=131072, **long_kw))
    assert p_uni.balanced == 0 and p_uni.num_splits * (4 * 8 // p_uni.kv_heads_per_wg) == 256
    assert p_uni.num_splits * p_uni.chunk_tokens == 131072 and p_uni.chunk_floor == 0
    assert _plan(_args(min_kv_len=131072 * 31 // 32, **long_kw)).balanced == 0
    assert _plan(_args(min_kv_len=131072 * 31 // 32 - 1, **long_kw)).balanced == 1
    # alike lengths whose per-sequence chunks would leave compute units idle (22 x 4 head blocks x 2 chunks = 176
    # workgroups on 256) get equal shares where the context is long enough to pay for them; fuller grids keep chunks
    wide = dict(max_pages=1024, table_stride_b=1024, max_kv_len=16384, min_kv_len=16384)
    assert _plan(_args(batch=22, **wide)).balanced == 1
    p26 = _plan(_args(batch=26, **wide))
    assert p26.balanced == 0 and p26.num_splits == 2 and p26.chunk_floor == 0
    assert _plan(_args(batch=22, max_kv_len=1024, min_kv_len=1024)).balanced == 0
    assert _decode_rc(_args(min_kv_len=-1)) == _lib.FDK_ESHAPE
    assert _decode_rc(_args(max_kv_len=4096, min_kv_len=4097)) == _lib.FDK_ESHAPE
    assert _decode_rc(_args(max_kv_len=4096, min_kv_len=4096)) == 0
    # a short context is latency-bound: chunk mode, split down to chunks of 64 tokens, never finer
    p_short = _plan(_args(batch=1, max_pages=8, table_stride_b=8))
    assert p_short.balanced == 0 and p_short.num_splits == 2 and p_short.chunk_tokens == 64
    p_one = _plan(_args(batch=1, max_pages=4, table_stride_b=4))      # 64 tokens: nothing to split
    assert p_one.num_splits == 1 and p_one.balanced == 0
    # the host's bound on kv_len drives the plan, not the table width
    p_hint = _plan(_args(batch=4, max_pages=2048, table_stride_b=2048, max_kv_len=4096))
    assert (p_hint.num_splits, p_hint.workgroups, p_hint.chunk_tokens) == (p4.num_splits, p4.workgroups, p4.chunk_tokens)
    # a forced split count is honoured in chunk mode: chunks are multiples of 64 tokens and cover the range
    p_forced = _plan(_args(num_splits=32))
    assert p_forced.balanced == 0 and p_forced.num_splits == 32 and p_forced.chunk_tokens * 32 >= 4096
    assert p_forced.chunk_floor == 64                       # lengths unknown: the chunks follow each sequence's length
    assert _plan(_args(num_splits=32, max_kv_len=4096, min_kv_len=4096)).chunk_floor == 0
    p_f4 = _plan(_args(batch=4, num_splits=5))
    assert p_f4.balanced == 0 and p_f4.chunk_tokens % 64 == 0
    assert 5 * p_f4.chunk_tokens >= 4096 > 4 * p_f4.chunk_tokens
    # the vector path splits in chunk mode
    p_v = _plan(_args(batch=4, algo=_lib.FDK_ALGO_VALU))
    assert p_v.balanced == 0 and p_v.num_splits > 1 and p_v.chunk_floor == 0
    assert p_v.num_splits * p_v.chunk_tokens >= 4096 > (p_v.num_splits - 1) * p_v.chunk_tokens
    # fewer compute units -> no more splits / workgroups than with many
    assert _plan(_args(batch=4), cus=64).num_splits <= p4.num_splits
    assert _plan(_args(batch=4, num_q_heads=64, page_size=64, max_pages=2048, table_stride_b=2048, q_stride_b=64 * 128,
                       out_stride_b=64 * 128, lse_stride_b=64), cus=64).workgroups <= p_long.workgroups
    # very large batches stay in chunk mode (every wavefront would have to scan kv_lens)
    assert _plan(_args(batch=600, num_q_heads=1, num_kv_heads=1, q_stride_b=128, out_stride_b=128, lse_stride_b=1,
                       max_pages=4096, table_stride_b=4096), cus=1024).balanced == 0
    assert _plan(_args(batch=500, num_q_heads=1, num_kv_heads=1, q_stride_b=128, out_stride_b=128, lse_stride_b=1,
                       max_pages=4096, table_stride_b=4096), cus=1024).balanced == 1
    # the vector path can be forced
    assert _plan(_args(algo=_lib.FDK_ALGO_VALU)).algo == _lib.FDK_ALGO_VALU


def test_workspace_bytes_formula():
    lib = _lib.load()
    assert lib.fdk_workspace_bytes(32, 32, 128, 4) >= 32 * 32 * 4 * 129 * 4
    assert lib.fdk_workspace_bytes(32, 32, 128, 4) % 256 == 0
    assert lib.fdk_workspace_bytes(0, 32, 128, 4) == 0
    assert lib.fdk_workspace_bytes(32, 32, 128, 0) == 0
    # a product that does not fit size_t saturates instead of wrapping to a small number
    assert lib.fdk_workspace_bytes(2**31 - 1, 2**31 - 1, 2**31 - 1, 2**31 - 1) == 2**64 - 1


def test_combine_ranks_validation():
    lib = _lib.load()
    a = FdkCombineRanksArgs()
    a.struct_size = C.sizeof(FdkCombineRanksArgs)
    a.flags = _lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE
    a.partial, a.kv_lens, a.out = 0x1000, 0x2000, 0x3000
    a.partial_dtype = a.out_dtype = _lib.FDK_BF16
    a.num_ranks, a.batch, a.num_q_heads, a.head_dim = 8, 4, 32, 128
    a.stride_r, a.stride_b, a.stride_h = 4 * 32 * 129, 32 * 129, 129
    a.out_stride_b, a.out_stride_h = 32 * 128, 128
    assert lib.fdk_combine_ranks(C.byref(a), None) == 0
    a.stride_h = 128
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_ESHAPE
    a.stride_h = 129
    a.flags = _lib.FDK_FLAG_DRY_RUN        # unpacked but no lse tensor
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_ENULL
    a.num_ranks = 0
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_ESHAPE
    assert lib.fdk_combine_ranks(None, None) == _lib.FDK_ENULL
    # the merged-lse output: aligned fp32 rows of at least Hq elements
    a.num_ranks, a.flags = 8, _lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE
    a.lse, a.lse_stride_b_out = 0x4000, 32
    assert lib.fdk_combine_ranks(C.byref(a), None) == 0
    a.lse_stride_b_out = 31
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_ESHAPE
    a.lse, a.lse_stride_b_out = 0x4002, 32
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_EALIGN
    # unpacked: the per-rank lse rows must hold Hq elements too
    a.lse, a.flags, a.partial_lse = 0x4000, _lib.FDK_FLAG_DRY_RUN, 0x5000
    a.lse_stride_r, a.lse_stride_b = 4 * 32, 16
    assert lib.fdk_combine_ranks(C.byref(a), None) == _lib.FDK_ESHAPE
    a.lse_stride_b = 32
    assert lib.fdk_combine_ranks(C.byref(a), None) == 0


def _append_args(**kw):
    """A valid dry-run fdk_kv_append block on fake pointers: B32, 1 new token, 32q/8kv, D128, P16."""
    a = FdkKvAppendArgs()
    a.struct_size = C.sizeof(FdkKvAppendArgs)
    a.flags = _lib.FDK_FLAG_DRY_RUN
    a.qkv, a.q_weight, a.k_weight, a.cos, a.sin = 0x10000, 0x20000, 0x30000, 0x40000, 0x50000
    a.qkv_stride_b, a.qkv_stride_t, a.qkv_stride_h = 48 * 128, 48 * 128, 128
    a.qkv_dtype = a.kv_dtype = _lib.FDK_BF16
    a.q_eps = a.k_eps = 1e-6
    a.cs_stride_b, a.cs_stride_pos, a.max_positions = 0, 128, 8192
    a.batch, a.new_tokens, a.num_q_heads, a.num_kv_heads, a.head_dim = 32, 1, 32, 8, 128
    a.block_table, a.table_stride_b, a.kv_lens = 0x60000, 256, 0x70000
    a.page_size, a.max_pages, a.num_pages = 16, 256, 9000
    a.k_cache, a.v_cache = 0x80000, 0x90000
    a.k_stride_page = a.v_stride_page = 16 * 8 * 128
    a.k_stride_tok = a.v_stride_tok = 8 * 128
    a.k_stride_head = a.v_stride_head = 128
    a.q_out, a.q_out_stride_b, a.q_out_stride_t, a.q_out_stride_h = 0xA0000, 32 * 128, 32 * 128, 128
    for k, v in kw.items():
        setattr(a, k, v)
    return a


def test_kv_append_accepts_valid_arguments_and_rejects_bad_ones():
    lib = _lib.load()
    assert lib.fdk_kv_append(C.byref(_append_args()), None) == 0, lib.fdk_last_error()
    assert lib.fdk_kv_append(C.byref(_append_args(kv_dtype=_lib.FDK_FP8_E4M3, k_scale=0xB0000, v_scale=0xC0000)), None) == 0
    assert lib.fdk_kv_append(C.byref(_append_args(batch=0, qkv=None)), None) == 0         # nothing to do
    assert lib.fdk_kv_append(None, None) == _lib.FDK_ENULL
    for field, value, code in [
        ("struct_size", 8, _lib.FDK_EABI),
        ("head_dim", 96, _lib.FDK_EUNSUPPORTED),
        ("qkv_dtype", _lib.FDK_FP32, _lib.FDK_EUNSUPPORTED),
        ("kv_dtype", _lib.FDK_FP16, _lib.FDK_EUNSUPPORTED),
        ("kv_dtype", _lib.FDK_FP8_E4M3, _lib.FDK_ENULL),              # fp8 cache without scales
        ("qkv", None, _lib.FDK_ENULL),
        ("cos", None, _lib.FDK_ENULL),
        ("q_out", None, _lib.FDK_ENULL),
        ("k_cache", None, _lib.FDK_ENULL),
        ("num_kv_heads", 0, _lib.FDK_ESHAPE),
        ("new_tokens", -1, _lib.FDK_ESHAPE),
        ("page_size", 0, _lib.FDK_ESHAPE),
        ("num_pages", 0, _lib.FDK_ESHAPE),
        ("max_positions", 0, _lib.FDK_ESHAPE),
        ("qkv_stride_h", 64, _lib.FDK_ESHAPE),
        ("q_out_stride_h", 127, _lib.FDK_ESHAPE),
        ("cs_stride_pos", 32, _lib.FDK_ESHAPE),
        ("table_stride_b", 255, _lib.FDK_ESHAPE),
        ("new_tokens", 2 ** 31 - 1, _lib.FDK_ESHAPE),                 # batch * tokens * head rows beyond a grid
        ("k_stride_head", 64, _lib.FDK_ESHAPE),
        ("v_stride_tok", -8, _lib.FDK_ESHAPE),
        ("q_eps", float("nan"), _lib.FDK_ESHAPE),
        ("k_eps", -1.0, _lib.FDK_ESHAPE),
    ]:
        rc = lib.fdk_kv_append(C.byref(_append_args(**{field: value})), None)
        assert rc == code, (field, value, rc, lib.fdk_last_error())
        assert lib.fdk_last_error() != b""


def test_linear_read_probe_rejects_bad_arguments():
    lib = _lib.load()
    assert lib.fdk_probe_linear_read(None, 1 << 20, 1, 512, None) == _lib.FDK_ENULL
    assert lib.fdk_probe_linear_read(0x10008, 1 << 20, 1, 512, None) == _lib.FDK_EALIGN
    assert lib.fdk_probe_linear_read(0x10000, 1024, 1, 512, None) == _lib.FDK_ESHAPE
    assert lib.fdk_probe_linear_read(0x10000, 1 << 20, 1, 0, None) == _lib.FDK_ESHAPE
    assert lib.fdk_probe_linear_read(0x10000, 1 << 20, 1, 1 << 21, None) == _lib.FDK_ESHAPE


def test_load_probe_flag_is_limited_to_what_is_built():
    # the load-only variant of the split kernel exists for the matrix-core path and head_dim 128
    ok = _measured(dict(probe_loads=1))
    assert _decode_rc(ok) == 0
    assert _decode_rc(_measured(dict(probe_loads=1), algo=_lib.FDK_ALGO_VALU)) == _lib.FDK_EUNSUPPORTED
    assert _decode_rc(_measured(dict(probe_loads=2))) == _lib.FDK_ESHAPE
    wide = _measured(dict(probe_loads=1), head_dim=256, q_stride_b=32 * 256, q_stride_h=256,
                 k_stride_page=16 * 8 * 256, k_stride_tok=8 * 256, k_stride_head=256, v_stride_page=16 * 8 * 256,
                 v_stride_tok=8 * 256, v_stride_head=256, out_stride_b=32 * 256, out_stride_h=256)
    assert _decode_rc(wide) == _lib.FDK_EUNSUPPORTED


def test_single_launch_flag_needs_counters_to_take_effect():
    # without counters the flag is ignored (split + combine); with them the usual checks on the counters apply
    lib = _lib.load()
    fl = _lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_SINGLE_LAUNCH
    assert _decode_rc(_args(batch=4, flags=fl)) == 0
    n = lib.fdk_counters_len(C.byref(_args(batch=4)))
    assert _decode_rc(_args(batch=4, flags=fl, counters=0x90000, counters_len=n)) == 0
    assert _decode_rc(_args(batch=4, flags=fl, counters=0x90000, counters_len=n - 1)) == _lib.FDK_EWORKSPACE


def _dims(dk, dv, **kw):
    """The block of _args with q / K rows of dk values and V / output rows of dv (v_head_dim; 0 where they are alike)."""
    base = dict(head_dim=dk, v_head_dim=0 if dv == dk else dv, q_stride_b=32 * dk, q_stride_h=dk,
                k_stride_page=16 * 8 * dk, k_stride_tok=8 * dk, k_stride_head=dk,
                v_stride_page=16 * 8 * dv, v_stride_tok=8 * dv, v_stride_head=dv,
                out_stride_b=32 * dv, out_stride_h=dv, sm_scale=dk ** -0.5)
    base.update(kw)
    return _args(**base)


def test_head_dims_of_two_segments_and_v_rows_of_their_own_length():
    # the reference's BLOCK_HEAD_DIM + BLOCK_DPE and V_DIM (flash_decode.py:103-109): 192 = 128 + 64, 576 = 512 + 64
    lib = _lib.load()
    for dk, dv in ((192, 192), (192, 128), (576, 512), (128, 128), (64, 64), (256, 256)):
        assert _decode_rc(_dims(dk, dv)) == 0, (dk, dv, lib.fdk_last_error())
    assert _decode_rc(_args(v_head_dim=128)) == 0                       # spelled out, equal to head_dim
    for dk, dv in ((192, 64), (128, 64), (576, 576), (256, 128), (96, 96), (512, 512), (576, 192)):
        assert _decode_rc(_dims(dk, dv)) == _lib.FDK_EUNSUPPORTED, (dk, dv)
    assert _decode_rc(_args(v_head_dim=-1)) == _lib.FDK_ESHAPE
    # what follows v_head_dim: the output row (and the packed row), the V head stride, the workspace
    assert _decode_rc(_dims(192, 128, out_stride_h=127)) == _lib.FDK_ESHAPE
    assert _decode_rc(_dims(192, 128, flags=_lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE)) == _lib.FDK_ESHAPE
    assert _decode_rc(_dims(192, 128, flags=_lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_PACK_LSE, out_stride_h=129,
                            out_stride_b=32 * 129)) == 0
    assert _decode_rc(_dims(192, 128, v_stride_head=64)) == _lib.FDK_ESHAPE
    a = _dims(576, 512, batch=4, max_kv_len=8192)
    p = _plan(a)
    assert p.num_splits > 1
    need = lib.fdk_workspace_bytes(4, 32, 512, p.num_splits)
    a.workspace_bytes = need
    assert _decode_rc(a) == 0
    a.workspace_bytes = need - 1
    assert _decode_rc(a) == _lib.FDK_EWORKSPACE
    # built on the matrix-core path, without the single-launch form
    assert _decode_rc(_dims(192, 192, kv_dtype=_lib.FDK_FP8_E4M3, k_stride_page=16 * 8 * 192, v_stride_page=16 * 8 * 192)) == 0   # fp8 caches are built
    assert _decode_rc(_dims(192, 192, algo=_lib.FDK_ALGO_VALU)) == _lib.FDK_EUNSUPPORTED
    assert _decode_rc(_dims(192, 192, flags=_lib.FDK_FLAG_DRY_RUN | _lib.FDK_FLAG_SINGLE_LAUNCH)) == _lib.FDK_EUNSUPPORTED
    assert _plan(_dims(192, 128)).algo == _lib.FDK_ALGO_MFMA
    # a caller of the revision before v_head_dim existed: the field reads as zero
    old = _dims(192, 128)
    old.struct_size = FdkDecodeArgs.v_head_dim.offset
    assert _decode_rc(old) == _lib.FDK_ESHAPE              # V strides of 128-value rows are too short for 192-value rows
    old = _args()
    old.struct_size = FdkDecodeArgs.v_head_dim.offset
    assert _decode_rc(old) == 0


def test_plans_of_wide_rows_keep_to_what_a_compute_unit_holds():
    # blocks of 4 or 8 kv heads are eight wavefronts; rows of more than 512 values per token and kv head (K and V
    # together): 16-bit caches run in the kernels whose wavefronts share the staged tiles, one kv head per workgroup
    # whatever the group; e4m3 caches with at most 16 q heads per kv head in the 16-head kernels, whose registers and
    # LDS hold four wavefronts, i.e. at most two heads per workgroup
    big = dict(batch=512, max_kv_len=2048, min_kv_len=2048)
    assert _plan(_dims(192, 192, **big)).kv_heads_per_wg == 8
    assert _plan(_dims(192, 128, **big)).kv_heads_per_wg == 8
    p = _plan(_dims(576, 512, **big))
    assert p.kv_heads_per_wg == 1 and p.num_splits == 1
    p = _plan(_dims(576, 512, kv_dtype=_lib.FDK_FP8_E4M3, **big))
    assert p.kv_heads_per_wg == 2 and p.num_splits == 1
    # large q-head groups on one kv head of 576 + 512 values: one kv head and 64 q heads per workgroup (the kernels whose
    # wavefronts share the staged tiles), so 32 sequences x 128 q heads are 64 units and split four ways on 256 compute units
    mla = _dims(576, 512, batch=32, num_q_heads=128, num_kv_heads=1, max_kv_len=4096, min_kv_len=4096, q_stride_b=128 * 576,
                k_stride_page=16 * 576, k_stride_tok=576, v_stride_page=16 * 512, v_stride_tok=512, out_stride_b=128 * 512,
                lse_stride_b=128)
    p = _plan(mla)
    assert p.kv_heads_per_wg == 1 and p.num_splits == 4 and not p.balanced
    # streaming estimates count the K and the V row: a (192, 128) cache streams 5/6 of what a (192, 192) cache does
    a, b = _plan(_dims(192, 192, batch=8, max_kv_len=4096)), _plan(_dims(192, 128, batch=8, max_kv_len=4096))
    assert a.num_splits >= 1 and b.num_splits >= 1
