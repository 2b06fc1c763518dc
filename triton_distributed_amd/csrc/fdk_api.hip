// C ABI of the flash-decode kernels: argument validation, launch planning, dispatch.
// Declarations and the reference interfaces they replace: include/fdk.h.
#include <float.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "../../include/fdk_measure.h"
#include "fdk_device.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int elem_size(int dt) {
    switch (dt) {
        case FDK_BF16:
        case FDK_FP16: return 2;
        case FDK_FP8_E4M3: return 1;
        case FDK_FP32: return 4;
        default: return 0;
    }
}

int ilog2_exact(int x) {
    if (x <= 0 || (x & (x - 1)) != 0) return -1;
    int s = 0;
    while ((1 << s) < x) ++s;
    return s;
}

int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Compute units of the current device; 256 (MI355X) when no device answers.
int query_cus() {
    static int cached[64] = {0};     // idempotent per-device cache; a race only repeats the query
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 256;
    }
    if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return 256;
    }
    if (dev >= 0 && dev < 64) cached[dev] = n;
    return n;
}

constexpr int kChunkAlign = 64;     // granularity of the shortest chunk and of balanced shares
constexpr int kTileAlign = 16;      // chunk boundaries fall on multiples of a 16-token tile (a tile never leaves its page)
constexpr int kMinChunk = 64;       // shortest chunk (short contexts: latency matters more than the partials)
constexpr double kBalancedExtraUs = 4.5;   // a balanced call against per-sequence chunks of the same batch, lengths alike
constexpr int kMaxMinChunk = 512;   // long contexts are never split finer than this
constexpr int kMaxSplits = 1024;
constexpr int64_t kMaxTableTokens = (int64_t)1 << 30;
constexpr int kDryRunCus = 256;           // a dry run plans for an MI355X and never asks the runtime
constexpr int kMaxBalancedBatch = 512;   // balanced mode: every wavefront scans kv_lens, keep that short
constexpr int kMinBalancedShare = 512;   // balanced mode only if a workgroup's share has this many tokens
constexpr int kMinRaggedLen = 2048;      // shorter contexts: a single pass that fills the compute units stays
constexpr double kFinerChunksStreamUs = 12.0;   // see make_plan
constexpr double kBalancedMinStreamUs = 40.0;   // batches that do not fill the compute units, lengths unknown: equal shares
                                                // only if streaming the cache at its bound takes this long (below, chunks of
                                                // each sequence's own length are 1-4 us faster whether the lengths turn out
                                                // ragged or alike; above, equal shares win by 2-14 % on ragged batches and
                                                // lose 2-5 % on uniform ones: bench.py --op plan-sweep)
constexpr int64_t kPieceOverheadBytes = 128 << 10;  // balanced mode: see piece_cost_granules
constexpr double kStreamBytesPerUs = 6.5e6;   // what a well-filled split kernel streams (plan estimates only)
constexpr double kSplitOverheadUs = 7.0;      // partial rows + combine launch of a split plan (plan estimates only)

// Scratch of fdk_decode_static: one copy per GPU, part of the loaded code object, never allocated or freed.
constexpr size_t kStaticScratchBytes = FDK_STATIC_SCRATCH_BYTES;
// (256 more bytes behind it: where the streaming-read probe's checksum would go)
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes + 256];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};      // device address of g_static_scratch on each GPU

// Device address of the static scratch on the current device, resolved once per device.
int static_scratch_of_current_device(void** ptr) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(FDK_EUNSUPPORTED, "device index %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess || !sym)
            return fail(e != hipSuccess ? (int)e : FDK_EWORKSPACE, "hipGetSymbolAddress(static scratch) failed on device %d: %s",
                        dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = sym;
    }
    *ptr = g_scratch_ptr[dev];
    return FDK_OK;
}

// The argument structs only grow at the end.  A caller's block is copied into one of this library's layout: the
// fields it does not have read as zero.  Blocks smaller than the first revision's or larger than this library's
// are refused.
template <typename T>
int adopt(const void* src, uint32_t struct_size, size_t first_revision_size, const char* what, T* dst) {
    if (struct_size < first_revision_size || struct_size > sizeof(T))
        return fail(FDK_EABI, "%s.struct_size %u outside [%zu, %zu]: built against another ABI line", what, struct_size,
                    first_revision_size, sizeof(T));
    memset(static_cast<void*>(dst), 0, sizeof(T));
    memcpy(static_cast<void*>(dst), src, struct_size);
    dst->struct_size = (uint32_t)sizeof(T);
    return FDK_OK;
}

// A decode call's arguments in this library's layout, with the measurement block (all zero unless the caller
// passed one) beside them; a.measure points at m or is null.
struct Call {
    fdk_decode_args a;
    fdk_measure_args m;
};

constexpr size_t kDecodeArgsFirstRevision = offsetof(fdk_decode_args, measure);
constexpr size_t kMeasureArgsFirstRevision = sizeof(fdk_measure_args);

int adopt_call(const fdk_decode_args* args, Call* c) {
    if (!args) return fail(FDK_ENULL, "args is null");
    int rc = adopt(args, args->struct_size, kDecodeArgsFirstRevision, "fdk_decode_args", &c->a);
    if (rc) return rc;
    memset(&c->m, 0, sizeof(c->m));
    if (c->a.measure) {
        rc = adopt(c->a.measure, c->a.measure->struct_size, kMeasureArgsFirstRevision, "fdk_measure_args", &c->m);
        if (rc) return rc;
        c->a.measure = &c->m;
    }
    return FDK_OK;
}

// values per V row / output row
inline int v_dim(const fdk_decode_args* a) { return a->v_head_dim > 0 ? a->v_head_dim : a->head_dim; }
// rows of one power-of-two segment, K and V alike: every path and option is built for them
inline bool plain_dims(int dk, int dv) { return dk == dv && (dk == 64 || dk == 128 || dk == 256); }
// rows of two segments (the reference's BLOCK_HEAD_DIM + BLOCK_DPE) and V rows shorter than K rows: matrix-core path,
// 16-bit caches
inline bool two_segment_dims(int dk, int dv) { return (dk == 192 && (dv == 192 || dv == 128)) || (dk == 576 && dv == 512); }

// (a: a block in this library's layout, from adopt_call)
int validate(const fdk_decode_args* a, bool need_out, bool need_workspace_only) {
    if (a->batch < 0) return fail(FDK_ESHAPE, "batch %d < 0", a->batch);
    if (a->num_q_heads <= 0 || a->num_kv_heads <= 0)
        return fail(FDK_ESHAPE, "head counts must be positive (Hq=%d, Hkv=%d)", a->num_q_heads, a->num_kv_heads);
    if (a->num_q_heads % a->num_kv_heads != 0)
        return fail(FDK_ESHAPE, "Hq=%d not a multiple of Hkv=%d", a->num_q_heads, a->num_kv_heads);
    if (a->v_head_dim < 0) return fail(FDK_ESHAPE, "v_head_dim %d < 0", a->v_head_dim);
    const int dv = v_dim(a);
    if (!plain_dims(a->head_dim, dv) && !two_segment_dims(a->head_dim, dv))
        return fail(FDK_EUNSUPPORTED, "head_dim %d / v_head_dim %d not built (64, 128, 256; 192 with 192 or 128; 576 with 512)",
                    a->head_dim, dv);
    if (two_segment_dims(a->head_dim, dv)) {
        if (a->algo == FDK_ALGO_VALU)
            return fail(FDK_EUNSUPPORTED, "head_dim %d / v_head_dim %d: built on the matrix-core path", a->head_dim, dv);
        if (a->flags & FDK_FLAG_SINGLE_LAUNCH)
            return fail(FDK_EUNSUPPORTED, "head_dim %d / v_head_dim %d: the single-launch form is not built", a->head_dim, dv);
    }
    if (a->page_size <= 0) return fail(FDK_ESHAPE, "page_size %d <= 0", a->page_size);
    if (a->max_pages <= 0) return fail(FDK_ESHAPE, "max_pages %d <= 0", a->max_pages);
    // token positions, chunk bounds (start + chunk) and granule counts are 32-bit in the kernels
    if ((int64_t)a->max_pages * a->page_size > kMaxTableTokens)
        return fail(FDK_ESHAPE, "max_pages*page_size = %lld: a block_table row may address at most 2^30 tokens",
                    (long long)((int64_t)a->max_pages * a->page_size));
    if (a->max_kv_len < 0) return fail(FDK_ESHAPE, "max_kv_len %d < 0", a->max_kv_len);
    if (a->min_kv_len < 0 || (a->max_kv_len > 0 && a->min_kv_len > a->max_kv_len))
        return fail(FDK_ESHAPE, "min_kv_len %d outside [0, max_kv_len = %d]", a->min_kv_len, a->max_kv_len);
    if (a->num_splits < 0 || a->num_splits > kMaxSplits)
        return fail(FDK_ESHAPE, "num_splits %d outside [0, %d]", a->num_splits, kMaxSplits);
    if (a->q_dtype != FDK_BF16 && a->q_dtype != FDK_FP16)
        return fail(FDK_EUNSUPPORTED, "q_dtype %d (bf16 or fp16 only)", a->q_dtype);
    if (a->kv_dtype != a->q_dtype && a->kv_dtype != FDK_FP8_E4M3)
        return fail(FDK_EUNSUPPORTED, "kv_dtype %d must equal q_dtype or be fp8_e4m3", a->kv_dtype);
    if (a->algo < FDK_ALGO_AUTO || a->algo > FDK_ALGO_MFMA) return fail(FDK_EUNSUPPORTED, "algo %d", a->algo);
    if (a->length_feedback && (reinterpret_cast<uintptr_t>(a->length_feedback) & 15u))
        return fail(FDK_EALIGN, "length_feedback must be 16-byte aligned");
    if (const fdk_measure_args* m = a->measure) {
        if ((m->wavefronts != 0 && m->wavefronts != 4 && m->wavefronts != 8) || m->buffers < 0 || m->buffers > 2)
            return fail(FDK_ESHAPE, "measure: wavefronts %d (0, 4, 8) / buffers %d (0, 1, 2)", m->wavefronts, m->buffers);
        if (m->shares_per_cu < 0 || m->shares_per_cu > 4)
            return fail(FDK_ESHAPE, "measure: shares_per_cu %d (0 .. 4)", m->shares_per_cu);
        if (m->probe_loads > 1) return fail(FDK_ESHAPE, "measure: probe_loads %u (0, 1)", m->probe_loads);
        if (m->force_balanced < 0 || m->force_balanced > 1)
            return fail(FDK_ESHAPE, "measure: force_balanced %d (0, 1)", m->force_balanced);
        if (m->timeline && ((reinterpret_cast<uintptr_t>(m->timeline) & 7u) || m->timeline_len < 0))
            return fail(FDK_EALIGN, "measure: timeline must be 8-byte aligned, timeline_len >= 0");
    }
    if (!(fabsf(a->sm_scale) <= FLT_MAX)) return fail(FDK_ESHAPE, "sm_scale is not finite");
    if (!(a->soft_cap <= FLT_MAX)) return fail(FDK_ESHAPE, "soft_cap is not a finite number (<= 0 switches it off)");
    if (a->batch == 0) return FDK_OK;

    if (!a->q || !a->k_cache || !a->v_cache || !a->block_table || !a->kv_lens)
        return fail(FDK_ENULL, "q / k_cache / v_cache / block_table / kv_lens must be non-null");
    if (!aligned16(a->q) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
        return fail(FDK_EALIGN, "q, k_cache and v_cache must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(a->block_table) & 3u) || (reinterpret_cast<uintptr_t>(a->kv_lens) & 3u))
        return fail(FDK_EALIGN, "block_table / kv_lens must be 4-byte aligned");
    const int kes = elem_size(a->kv_dtype);
    if ((a->q_stride_b * 2) % 16 || (a->q_stride_h * 2) % 16)
        return fail(FDK_EALIGN, "q strides must be multiples of 16 bytes");
    const int64_t ks[6] = {a->k_stride_page, a->k_stride_tok, a->k_stride_head,
                           a->v_stride_page, a->v_stride_tok, a->v_stride_head};
    for (int i = 0; i < 6; ++i) {
        if (ks[i] < 0) return fail(FDK_ESHAPE, "negative cache stride");
        if ((ks[i] * kes) % 16) return fail(FDK_EALIGN, "cache strides must be multiples of 16 bytes");
    }
    // the kernels keep the byte offsets of a tile's 16 token rows relative to its first row in 32 bits
    if (a->k_stride_tok * kes * 16 >= ((int64_t)1 << 32) || a->v_stride_tok * kes * 16 >= ((int64_t)1 << 32))
        return fail(FDK_ESHAPE, "cache token stride too large: 16 rows must span less than 4 GiB");
    // page number x page stride is a 32 x 32 -> 64 bit product in the kernels; token-in-page offsets are 32 bit
    if (a->k_stride_page * kes >= ((int64_t)1 << 32) || a->v_stride_page * kes >= ((int64_t)1 << 32))
        return fail(FDK_ESHAPE, "cache page stride too large: a page must span less than 4 GiB");
    if ((int64_t)a->page_size * a->k_stride_tok * kes >= ((int64_t)1 << 32) ||
        (int64_t)a->page_size * a->v_stride_tok * kes >= ((int64_t)1 << 32))
        return fail(FDK_ESHAPE, "page_size x token stride must be less than 4 GiB");
    if (a->kv_dtype == FDK_FP8_E4M3 &&
        ((reinterpret_cast<uintptr_t>(a->k_scale) & 3u) || (reinterpret_cast<uintptr_t>(a->v_scale) & 3u)))
        return fail(FDK_EALIGN, "k_scale / v_scale must be 4-byte aligned");
    if ((a->k_stride_head < a->head_dim || a->v_stride_head < dv) && a->num_kv_heads > 1)
        return fail(FDK_ESHAPE, "cache head stride < head_dim (k %lld, v %lld)", (long long)a->k_stride_head,
                    (long long)a->v_stride_head);
    if (a->table_stride_b < a->max_pages)
        return fail(FDK_ESHAPE, "table_stride_b %lld < max_pages %d", (long long)a->table_stride_b, a->max_pages);

    if (need_out) {
        if (!a->out) return fail(FDK_ENULL, "out is null");
        const int oes = elem_size(a->out_dtype);
        if (a->out_dtype != FDK_BF16 && a->out_dtype != FDK_FP16 && a->out_dtype != FDK_FP32)
            return fail(FDK_EUNSUPPORTED, "out_dtype %d", a->out_dtype);
        if (reinterpret_cast<uintptr_t>(a->out) % oes) return fail(FDK_EALIGN, "out not element aligned");
        const int row = dv + ((a->flags & FDK_FLAG_PACK_LSE) ? 1 : 0);
        if (a->out_stride_h < row) return fail(FDK_ESHAPE, "out_stride_h %lld < %d", (long long)a->out_stride_h, row);
        if (a->lse && (reinterpret_cast<uintptr_t>(a->lse) & 3u)) return fail(FDK_EALIGN, "lse not 4-byte aligned");
        if (a->lse && a->lse_stride_b < a->num_q_heads)
            return fail(FDK_ESHAPE, "lse_stride_b %lld < Hq", (long long)a->lse_stride_b);
    }
    (void)need_workspace_only;
    return FDK_OK;
}

int make_plan(const fdk_decode_args* a, int num_cus, fdk_plan_t* plan) {
    const int group = a->num_q_heads / a->num_kv_heads;
    int algo = a->algo;
    if (algo == FDK_ALGO_AUTO) {
        // The matrix-core path is the default for every group size: on MI355X it is at least as fast as the
        // vector path even for small groups, because it needs an order of magnitude fewer issue slots per KV byte.
        algo = fdk::mfma_supported(a->q_dtype, a->kv_dtype, group, a->head_dim, v_dim(a)) ? FDK_ALGO_MFMA : FDK_ALGO_VALU;
    }
    if (algo == FDK_ALGO_MFMA && !fdk::mfma_supported(a->q_dtype, a->kv_dtype, group, a->head_dim, v_dim(a)))
        return fail(FDK_EUNSUPPORTED, "MFMA path not built for q_dtype=%d kv_dtype=%d head_dim=%d", a->q_dtype,
                    a->kv_dtype, a->head_dim);
    if (algo == FDK_ALGO_VALU && (v_dim(a) != a->head_dim || !fdk::valu_supported(a->q_dtype, a->kv_dtype, group, a->head_dim)))
        return fail(FDK_EUNSUPPORTED, "VALU path not built for q_dtype=%d kv_dtype=%d head_dim=%d (128 only)", a->q_dtype,
                    a->kv_dtype, a->head_dim);

    int64_t max_len = a->max_kv_len > 0 ? a->max_kv_len : (int64_t)a->max_pages * a->page_size;
    const int64_t table_cap = (int64_t)a->max_pages * a->page_size;
    if (max_len > table_cap) max_len = table_cap;
    if (max_len < 1) max_len = 1;

    if (num_cus <= 0) num_cus = query_cus();
    const int batch = a->batch > 0 ? a->batch : 1;
    const bool heads_contiguous = a->k_stride_head == a->head_dim && a->v_stride_head == a->head_dim;
    int kv_heads_per_wg = 1;
    int units_per_seq;
    const int tile_heads = algo == FDK_ALGO_MFMA ? fdk::mfma_heads_per_wg(group, a->head_dim + v_dim(a), a->kv_dtype) : 16;   // q heads of a kv head per workgroup
    if (algo == FDK_ALGO_MFMA) {
        kv_heads_per_wg = fdk::mfma_kv_heads_per_wg(batch, a->num_kv_heads, group, num_cus, a->head_dim + v_dim(a), a->kv_dtype);
        units_per_seq = fdk::mfma_units_per_seq(a->num_kv_heads, group, kv_heads_per_wg, tile_heads);
    } else {
        units_per_seq = fdk::valu_units_per_seq(a->num_kv_heads, group, heads_contiguous, a->kv_dtype);
    }
    const int64_t units = (int64_t)batch * units_per_seq;
    const int single_pass_heads_per_wg = kv_heads_per_wg;

    // A single pass gives every workgroup whole sequences, which is only as good as the sequences are alike and
    // as evenly as the workgroups fill the compute units.  It is replaced by balanced mode (equal shares of the
    // tokens that kv_lens holds, narrow head blocks, a combine launch) when
    //  - the host has not said that the lengths are alike (min_kv_len) and there are fewer than four workgroups
    //    per compute unit to even things out (batch 64 x 8 kv heads, lengths uniform in [1, 8192]: 223 us as a
    //    single pass, the longest sequence decides) and the sequences can be long (max_len >= kMinRaggedLen); or
    //  - the lengths are alike but the workgroups do not fill the compute units evenly - 1.25 per compute unit:
    //    a quarter of the compute units carry two and finish long after the rest - and the estimate says that
    //    pays for the combine launch.  Measured for batch 40 / 48 / 60 x 8 kv heads x 4096 tokens: the single
    //    pass runs at (fill + 1) / 2 of the even rate, fill = units / (rounds x compute units): 131 / 139 /
    //    159 us against 103 / 124 / 155 us of streaming time.
    const bool alike = a->min_kv_len > 0 && (int64_t)a->min_kv_len * 32 >= max_len * 31;
    // what streaming the batch's cache takes (the shared-tile kernels are bound by the 16-bit tile they stage, not by
    // the bytes they read: a one-byte cache takes them as long as a 16-bit one, and is planned like one)
    const int stream_elem = tile_heads > 16 ? 2 : elem_size(a->kv_dtype);
    const double stream_us = (double)batch * (double)max_len * a->num_kv_heads * (double)(a->head_dim + v_dim(a)) *
                             stream_elem / kStreamBytesPerUs;
    bool rebalance = false;
    // (measurement aid: equal shares wherever they can run, to time them against the plan chosen here)
    const bool force_balanced = a->measure && a->measure->force_balanced && algo == FDK_ALGO_MFMA && a->num_splits <= 0 &&
                                batch > 1 && batch <= kMaxBalancedBatch;
    if (algo == FDK_ALGO_MFMA && a->num_splits <= 0 && units >= num_cus && batch <= kMaxBalancedBatch) {
        if (force_balanced) {
            rebalance = true;
        } else if (!alike) {
            rebalance = units < 4 * (int64_t)num_cus && max_len >= kMinRaggedLen;
        } else if (units > num_cus) {
            const int64_t rounds = cdiv64(units, num_cus);
            const double fill = (double)units / (double)(rounds * num_cus);
            rebalance = stream_us * 2.0 / (fill + 1.0) > 1.05 * (stream_us * 1.03 + kSplitOverheadUs);
        }
        if (rebalance) {
            kv_heads_per_wg = a->num_kv_heads % 2 ? 1 : 2;
            if (tile_heads > 16) kv_heads_per_wg = 1;
            units_per_seq = fdk::mfma_units_per_seq(a->num_kv_heads, group, kv_heads_per_wg, tile_heads);
        }
    }

    // Split count: none when the (sequence, head block) units alone fill the compute units - a single pass
    // then writes the final result and no combine runs.  Otherwise the per-sequence chunks aim at one workgroup
    // per compute unit and never more: on MI355X 256 workgroups finish 2-7 % sooner than 512 with the same
    // total work, and a grid a little larger than what is resident at once runs in two rounds.
    // The shortest chunk grows with the context (max_len / 64, between kMinChunk and kMaxMinChunk tokens):
    // a short context is latency-bound and gains from every extra split, a long one pays for each partial
    // row it writes and re-reads.
    int64_t min_chunk = cdiv64(cdiv64(max_len, 64), kChunkAlign) * kChunkAlign;
    if (min_chunk < kMinChunk) min_chunk = kMinChunk;
    if (min_chunk > kMaxMinChunk) min_chunk = kMaxMinChunk;
    const int64_t most_chunks = cdiv64(max_len, min_chunk);
    const bool may_split = a->num_splits <= 0 && (units < num_cus || rebalance) && (most_chunks > 1 || force_balanced);
    int64_t splits = 1;
    if (a->num_splits > 0) {
        splits = a->num_splits;
    } else if (may_split && !rebalance) {
        splits = (int64_t)num_cus / units;
        // Lengths the host does not vouch for, and enough to stream that the start of a workgroup is not what counts
        // (kFinerChunksStreamUs): two workgroups per compute unit.  If the batch turns out ragged, the chunks of its long
        // sequences are what the call waits for, and finer ones end up to 10 % sooner; if it turns out uniform, the
        // second workgroup per unit costs 1-3 %.
        if (!alike && algo == FDK_ALGO_MFMA && batch > 1 && stream_us >= kFinerChunksStreamUs) splits *= 2;
        if (splits > most_chunks) splits = most_chunks;
    }
    memset(plan, 0, sizeof(*plan));
    plan->algo = algo;
    plan->kv_heads_per_wg = kv_heads_per_wg;

    // Balanced mode replaces the per-sequence chunks whenever the matrix-core path would split on its own
    // account: the kernel cuts the KV ranges of the whole batch, as kv_lens gives them, into equal shares, so
    // that a ragged batch loads every workgroup alike.  A batch the host knows to be of (nearly) uniform length
    // needs none of that: per-sequence chunks, one workgroup per compute unit, are 2-7 % faster there.  The
    // workspace then holds (shares + batch) slots of partial rows per (head block, head tile) unit; it is reported
    // as rows per (sequence, q head).
    const int64_t columns = (int64_t)batch * cdiv64(max_len, fdk::kBalanceGranule);   // granules of all sequences, at most
    // Lengths that are alike, but per-sequence chunks that leave compute units idle (units x splits well below the
    // compute units: batch 22 x 4 head blocks x 2 chunks = 176 workgroups on 256): the busy units do not make up for
    // the idle ones - measured against equal shares of the same batch, 16384 tokens: 9 % slower at a fill of 0.69,
    // 1 % at 0.81, level from 0.86 on - while equal shares cost about kBalancedExtraUs more per call (the pass over
    // kv_lens before the first load, a combine that has to find its rows).
    bool underfilled = false;
    if (alike && may_split && !rebalance && batch > 1) {
        const double fill = (double)(units * splits) / (double)num_cus;
        const double slower = 0.75 * (0.82 - fill);
        underfilled = slower > 0.0 && stream_us * slower > 1.2 * kBalancedExtraUs;
    }
    const bool uniform = alike && !rebalance && !underfilled && !force_balanced;
    // (a single sequence has nothing to balance: its own length in equal chunks, below, does the same without the
    // pass over kv_lens and with a combine that knows where its rows are - 27 us against 34 us for 32768 tokens)
    const bool long_enough = alike || rebalance || force_balanced || stream_us >= kBalancedMinStreamUs;
    if (algo == FDK_ALGO_MFMA && may_split && !uniform && long_enough && batch > 1 && batch <= kMaxBalancedBatch &&
        columns < (1 << 30)) {                                            // the kernel counts granules in int32
        const int64_t gran = fdk::kBalanceGranule;
        int64_t shares = columns / (min_chunk / gran);
        // one workgroup per compute unit: the kernel sizes such a workgroup to keep the unit's memory pipeline
        // full by itself, and a second one only queues up behind it (measured 0.6-1.8 % slower, with twice the
        // partial rows to merge)
        const int shares_per_cu = a->measure && a->measure->shares_per_cu > 0 ? a->measure->shares_per_cu : 1;
        const int64_t most = shares_per_cu * (int64_t)num_cus / units_per_seq;
        if (shares > most) shares = most;
        if (shares < 1) shares = 1;
        const int64_t share_tokens = cdiv64(columns, shares) * gran;
        // Deriving the partition costs every workgroup a pass over kv_lens before its first load: worth it
        // only when a share is long enough to hide that.
        if (share_tokens >= kMinBalancedShare || force_balanced) {
            const int64_t rows_per_slot = (int64_t)kv_heads_per_wg * (group < tile_heads ? group : tile_heads);
            const int64_t rows = (shares + batch) * units_per_seq * rows_per_slot;
            plan->balanced = 1;
            plan->workgroups = (int32_t)(shares * units_per_seq);
            plan->num_splits = (int32_t)cdiv64(rows, (int64_t)batch * a->num_q_heads);
            plan->chunk_tokens = (int32_t)(cdiv64(share_tokens, kChunkAlign) * kChunkAlign);
            return FDK_OK;
        }
    }
    if (rebalance) plan->kv_heads_per_wg = single_pass_heads_per_wg;     // no equal shares after all: the single pass
    // (rounded up to tiles, not further: rounding to 64 tokens cost the reference's shape at 8K a quarter of its
    // workgroups - 32 chunks of 256 tokens instead of 40 of 208 on 6 head blocks x 256 compute units)
    const int64_t align = a->num_splits > 0 ? kChunkAlign : kTileAlign;
    int64_t chunk = cdiv64(cdiv64(max_len, splits), align) * align;
    if (a->num_splits <= 0) splits = cdiv64(max_len, chunk);   // drop splits that would always be empty
    if (splits > kMaxSplits) {
        splits = kMaxSplits;
        chunk = cdiv64(cdiv64(max_len, splits), kChunkAlign) * kChunkAlign;
    }
    plan->num_splits = (int32_t)splits;
    plan->chunk_tokens = (int32_t)chunk;
    // Lengths the host does not vouch for: the chunks follow each sequence's own length, so that a sequence far
    // below the bound (the capacity of the table, if the host gave none) still uses every workgroup it was given.
    // A forced split count is cut the same way - it is the reference's NUM_KV_SPLITS, and the reference cuts every
    // sequence into that many parts of its own length (flash_decode.py:151-153).  Not for lengths known to be alike:
    // the kernel then requests kv_lens and its first page numbers together.
    if (algo == FDK_ALGO_MFMA && splits > 1 && !alike)
        plan->chunk_floor = (int32_t)(chunk < kMinChunk ? chunk : kMinChunk);
    return FDK_OK;
}

// Balanced mode: what a sequence boundary inside a share costs its workgroup, in granules of the partition.  The
// fixed time of a piece (table and q loads before its first rows, the merge of the wavefronts after its last) is
// what a workgroup needs to stream about kPieceOverheadBytes (measured on ragged batches of 16 and 64 sequences with
// one and eight kv heads: 0 / 48 / 96 / 144 / 192 KB give 90.7 / 88.3 / 88.3 / 87.4 / 88.9, 165.7 / 164.0 / 162.3 /
// 162.5 / 163.6 and 30.8 / 30.4 / 28.8 / 28.3 / 28.4 us per call).
int piece_cost_granules(const fdk_decode_args* a, int kv_heads_per_wg) {
    const int64_t granule_bytes = (int64_t)fdk::kBalanceGranule * kv_heads_per_wg * (a->head_dim + v_dim(a)) * elem_size(a->kv_dtype);
    // an even number: the kernel puts half of it in front of a sequence's tokens and half behind
    const int64_t c = 2 * ((kPieceOverheadBytes + granule_bytes) / (2 * granule_bytes));
    return (int)(c > 64 ? 64 : c);
}

// q-head tiles per kv head, as the resolved algorithm's kernel counts them
int head_tiles_of(const fdk_decode_args* a, int algo) {
    const int group = a->num_q_heads / a->num_kv_heads;
    const int hpw = algo == FDK_ALGO_MFMA ? fdk::mfma_heads_per_wg(group, a->head_dim + v_dim(a), a->kv_dtype) : fdk::valu_heads_per_wg(group);
    return (group + hpw - 1) / hpw;
}

struct Resolved {
    fdk_plan_t plan;
    fdk::SplitParams sp;
    fdk::CombineParams cp;
};

int resolve(const fdk_decode_args* a, bool direct_ok, int num_cus, Resolved* r) {
    if (num_cus <= 0) num_cus = query_cus();
    int rc = make_plan(a, num_cus, &r->plan);
    if (rc) return rc;
    const int S = r->plan.num_splits;
    const bool direct = direct_ok && S == 1;
    const int64_t rows = (int64_t)a->batch * a->num_q_heads;
    if ((int64_t)a->batch * S * a->num_kv_heads * head_tiles_of(a, r->plan.algo) > INT32_MAX || a->batch > 65535)
        return fail(FDK_ESHAPE, "grid too large (batch x splits x heads; at most 65535 sequences)");
    float* part_o = nullptr;
    float* part_lse = nullptr;
    int2* slot_desc = nullptr;           // one per (sequence, unit), behind the partial rows
    if (!direct && a->batch > 0) {
        const size_t need = fdk_workspace_bytes(a->batch, a->num_q_heads, v_dim(a), S);
        if (!a->workspace) return fail(FDK_EWORKSPACE, "workspace is null; %zu bytes needed", need);
        if (!aligned16(a->workspace)) return fail(FDK_EALIGN, "workspace must be 16-byte aligned");
        if (a->workspace_bytes < need)
            return fail(FDK_EWORKSPACE, "workspace has %zu bytes; %zu needed for %d splits", a->workspace_bytes, need, S);
        part_o = reinterpret_cast<float*>(a->workspace);
        part_lse = part_o + rows * S * v_dim(a);
        slot_desc = reinterpret_cast<int2*>((reinterpret_cast<uintptr_t>(part_lse + rows * S) + 7) & ~uintptr_t(7));
    }
    fdk::SplitParams& sp = r->sp;
    memset(&sp, 0, sizeof(sp));
    sp.q = a->q; sp.k = a->k_cache; sp.v = a->v_cache;
    sp.block_table = a->block_table; sp.kv_lens = a->kv_lens;
    sp.k_scale = a->kv_dtype == FDK_FP8_E4M3 ? a->k_scale : nullptr;
    sp.v_scale = a->kv_dtype == FDK_FP8_E4M3 ? a->v_scale : nullptr;
    sp.part_o = part_o; sp.part_lse = part_lse; sp.slot_desc = slot_desc;
    sp.out = a->out; sp.lse = a->lse;
    sp.counters = nullptr;
    sp.num_cus = num_cus;
    sp.q_sb = a->q_stride_b; sp.q_sh = a->q_stride_h;
    sp.k_sp = a->k_stride_page; sp.k_st = a->k_stride_tok; sp.k_sh = a->k_stride_head;
    sp.v_sp = a->v_stride_page; sp.v_st = a->v_stride_tok; sp.v_sh = a->v_stride_head;
    sp.tbl_sb = a->table_stride_b;
    sp.out_sb = a->out_stride_b; sp.out_sh = a->out_stride_h; sp.lse_sb = a->lse_stride_b;
    sp.batch = a->batch; sp.hq = a->num_q_heads; sp.hkv = a->num_kv_heads;
    sp.group = a->num_q_heads / a->num_kv_heads;
    sp.head_dim = a->head_dim; sp.v_head_dim = v_dim(a);
    sp.page_size = a->page_size; sp.page_shift = ilog2_exact(a->page_size);
    sp.num_splits = S; sp.chunk = r->plan.chunk_tokens; sp.chunk_floor = r->plan.chunk_floor;
    sp.max_tokens = (int32_t)((int64_t)a->max_pages * a->page_size);
    sp.head_tiles = head_tiles_of(a, r->plan.algo);
    sp.hg_per_wg = r->plan.kv_heads_per_wg;
    sp.balanced = r->plan.balanced;
    sp.workgroups = r->plan.workgroups;
    sp.tile_heads = r->plan.algo == FDK_ALGO_MFMA ? fdk::mfma_heads_per_wg(sp.group, a->head_dim + v_dim(a), a->kv_dtype) : 16;
    sp.heads_per_tile = sp.group < sp.tile_heads ? sp.group : sp.tile_heads;
    sp.rows_per_slot = sp.hg_per_wg * sp.heads_per_tile;
    sp.piece_cost = sp.balanced ? piece_cost_granules(a, sp.hg_per_wg) : 0;
    const fdk_measure_args* const ms = a->measure;
    sp.tune_wavefronts = ms ? ms->wavefronts : 0;
    sp.tune_buffers = ms ? ms->buffers : 0;
    sp.out_dtype = a->out_dtype;
    sp.pack_lse = (a->flags & FDK_FLAG_PACK_LSE) ? 1 : 0;
    sp.direct = direct ? 1 : 0;
    sp.fp8_fold = (a->flags & FDK_FLAG_FP8_FOLD_K_SCALE) && a->kv_dtype == FDK_FP8_E4M3 ? 1 : 0;
    // length feedback: stored by the last kernel of the call - a single pass (or the single-launch form) itself,
    // else the combine kernel
    static std::atomic<int32_t> epoch{0};
    int32_t this_epoch = 0;
    if (a->length_feedback) {
        this_epoch = epoch.fetch_add(1) + 1;
        if (this_epoch <= 0) { epoch.store(1); this_epoch = 1; }
    }
    sp.length_feedback = direct ? a->length_feedback : nullptr;
    sp.feedback_epoch = this_epoch;
    sp.timeline = ms ? reinterpret_cast<long long*>(ms->timeline) : nullptr;
    sp.timeline_len = ms && ms->timeline ? ms->timeline_len : 0;
    sp.timeline_rotate = ms ? ms->rotate_heads & 1023 : 0;
    sp.probe = ms && ms->probe_loads ? 1 : 0;
    if (sp.probe && (r->plan.algo != FDK_ALGO_MFMA || a->head_dim != 128 || v_dim(a) != 128))
        return fail(FDK_EUNSUPPORTED, "measure: probe_loads is built for the matrix-core path and head_dim 128");
    sp.scale_log2 = a->sm_scale * fdk::kLog2e;
    sp.soft_cap = a->soft_cap > 0.f ? a->soft_cap : 0.f;
    sp.sm_scale = a->sm_scale;

    fdk::CombineParams& cp = r->cp;
    memset(&cp, 0, sizeof(cp));
    cp.part_o = part_o; cp.part_lse = part_lse; cp.slot_desc = slot_desc; cp.kv_lens = a->kv_lens;
    cp.out = a->out; cp.lse = a->lse;
    cp.out_sb = a->out_stride_b; cp.out_sh = a->out_stride_h; cp.lse_sb = a->lse_stride_b;
    cp.batch = a->batch; cp.hq = a->num_q_heads; cp.head_dim = v_dim(a);
    cp.num_splits = S; cp.chunk = r->plan.chunk_tokens; cp.chunk_floor = r->plan.chunk_floor;
    cp.max_tokens = sp.max_tokens;
    cp.out_dtype = a->out_dtype; cp.pack_lse = sp.pack_lse;
    cp.balanced = sp.balanced; cp.workgroups = sp.workgroups;
    cp.group = sp.group; cp.kv_heads_per_wg = sp.hg_per_wg; cp.head_tiles = sp.head_tiles;
    cp.hg_blocks = a->num_kv_heads / (sp.hg_per_wg > 0 ? sp.hg_per_wg : 1);
    cp.rows_per_slot = sp.rows_per_slot; cp.heads_per_tile = sp.heads_per_tile; cp.tile_heads = sp.tile_heads;
    cp.piece_cost = sp.piece_cost;
    cp.length_feedback = a->length_feedback;
    cp.feedback_epoch = this_epoch;
    return FDK_OK;
}

int launch_split(const fdk_decode_args* a, const Resolved& r, hipStream_t stream) {
    int rc = r.plan.algo == FDK_ALGO_MFMA ? fdk::launch_splitkv_mfma(r.sp, a->q_dtype, a->kv_dtype, stream)
                                          : fdk::launch_splitkv_valu(r.sp, a->q_dtype, a->kv_dtype, stream);
    if (rc) return fail(rc, "split kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return FDK_OK;
}

// Split launch + combine launch (a single launch for a one-split plan); the body of fdk_decode and fdk_decode_static.
int decode_impl(const fdk_decode_args* args, void* hip_stream) {
    int rc = validate(args, true, false);
    if (rc) return rc;
    if (args->batch == 0) return FDK_OK;
    // A dry run goes through everything the host decides (plan, workspace, counters) and stops before the launch.
    const bool dry = (args->flags & FDK_FLAG_DRY_RUN) != 0;
    Resolved r;
    rc = resolve(args, true, dry ? kDryRunCus : 0, &r);
    if (rc) return rc;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    // With counters (matrix-core path only): a forced split count with more items than are resident at once runs
    // as a work queue; and with FDK_FLAG_SINGLE_LAUNCH the workgroup that finishes a (sequence, head block,
    // head tile) last merges its pieces, so no combine launch follows.
    const bool with_counters = !r.sp.direct && !r.sp.probe && args->counters != nullptr && r.plan.algo == FDK_ALGO_MFMA;
    if (with_counters) {
        if (reinterpret_cast<uintptr_t>(args->counters) & 3u) return fail(FDK_EALIGN, "counters not 4-byte aligned");
        if (args->counters_len < fdk_counters_len(args))
            return fail(FDK_EWORKSPACE, "counters_len %lld < %lld", (long long)args->counters_len,
                        (long long)fdk_counters_len(args));
        r.sp.counters = args->counters;
        // the merging workgroup addresses the partials with 32-bit offsets
        const size_t ws_need = fdk_workspace_bytes(args->batch, args->num_q_heads, v_dim(args), r.plan.num_splits);
        if ((args->flags & FDK_FLAG_SINGLE_LAUNCH) && ws_need < ((size_t)1 << 32)) {
            r.sp.fused = 1;
            r.sp.ws_bytes = (uint32_t)ws_need;
            r.sp.length_feedback = args->length_feedback;        // no combine follows: the split kernel stores it
        }
    }
    if (dry) return FDK_OK;
    rc = launch_split(args, r, stream);
    if (rc) return rc;
    if (!r.sp.direct && !r.sp.probe && !r.sp.fused) {
        rc = fdk::launch_combine(r.cp, stream);
        if (rc) return fail(rc, "combine kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    }
    return FDK_OK;
}

}  // namespace

extern "C" {

int fdk_abi_version(void) { return FDK_ABI_VERSION; }

int fdk_abi_revision(void) { return FDK_ABI_REVISION; }

const char* fdk_last_error(void) { return g_err; }

int fdk_device_cus(void) { return query_cus(); }

int64_t fdk_counters_len(const fdk_decode_args* a) {
    // (reads fields of the first revision only: no need to adopt the block)
    if (!a || a->struct_size < kDecodeArgsFirstRevision || a->batch <= 0 || a->num_q_heads <= 0 || a->num_kv_heads <= 0 || a->num_q_heads % a->num_kv_heads) return 0;
    // queue head, finished-workgroup count, then one ticket per (sequence, kv head, tile of 16 q heads): an upper
    // bound of the (sequence, head block, head tile) units of any plan
    const int64_t group = a->num_q_heads / a->num_kv_heads;
    return 2 + (int64_t)a->batch * a->num_kv_heads * ((group + 15) / 16);
}

size_t fdk_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t head_dim, int32_t num_splits) {
    if (batch <= 0 || num_q_heads <= 0 || head_dim <= 0 || num_splits <= 0) return 0;
    // batch * heads * splits < 2^93 would overflow: saturate instead, so that no buffer ever passes the size check
    const unsigned __int128 rows = (unsigned __int128)batch * (unsigned __int128)num_q_heads * (unsigned __int128)num_splits;
    // partial rows and their lse, then (balanced plans) eight bytes per (sequence, unit) that say where a sequence's
    // pieces are; there are at most batch x q heads units
    const unsigned __int128 desc = (unsigned __int128)batch * (unsigned __int128)num_q_heads * 8 + 8;
    const unsigned __int128 bytes = rows * ((unsigned __int128)head_dim + 1) * sizeof(float) + desc + 255;
    if (bytes > (unsigned __int128)SIZE_MAX) return SIZE_MAX;
    return (size_t)bytes & ~(size_t)255;
}

int fdk_plan(const fdk_decode_args* caller_args, int num_cus, fdk_plan_t* plan) {
    g_err[0] = 0;
    if (!plan) return fail(FDK_ENULL, "plan is null");
    Call call;
    int rc = adopt_call(caller_args, &call);
    if (rc) return rc;
    const fdk_decode_args* args = &call.a;
    rc = validate(args, false, false);
    if (rc) return rc;
    if (num_cus <= 0 && (args->flags & FDK_FLAG_DRY_RUN)) num_cus = kDryRunCus;
    return make_plan(args, num_cus, plan);
}

int fdk_decode(const fdk_decode_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    Call call;
    const int rc = adopt_call(caller_args, &call);
    if (rc) return rc;
    return decode_impl(&call.a, hip_stream);
}

int fdk_decode_static(const fdk_decode_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    Call call;
    int rc = adopt_call(caller_args, &call);
    if (rc) return rc;
    const fdk_decode_args* args = &call.a;
    rc = validate(args, true, false);
    if (rc) return rc;
    if (args->batch == 0) return FDK_OK;
    const bool dry = (args->flags & FDK_FLAG_DRY_RUN) != 0;
    fdk_plan_t plan;
    rc = make_plan(args, dry ? kDryRunCus : 0, &plan);
    if (rc) return rc;
    fdk_decode_args a = *args;
    a.workspace = nullptr;
    a.workspace_bytes = 0;
    a.counters = nullptr;          // one workgroup per item: nothing in the scratch has to start at zero
    a.counters_len = 0;
    if (plan.num_splits > 1) {
        const size_t need = fdk_workspace_bytes(a.batch, a.num_q_heads, v_dim(&a), plan.num_splits);
        if (need > kStaticScratchBytes)
            return fail(FDK_EWORKSPACE,
                        "fdk_decode_static: the partials of %d splits need %zu bytes, the static scratch holds %zu; "
                        "use fdk_decode with a caller-owned workspace", plan.num_splits, need, kStaticScratchBytes);
        if (dry) {
            a.workspace = reinterpret_cast<void*>(uintptr_t(256));      // never dereferenced in a dry run
        } else {
            rc = static_scratch_of_current_device(&a.workspace);
            if (rc) return rc;
        }
        a.workspace_bytes = kStaticScratchBytes;
    }
    return decode_impl(&a, hip_stream);
}

int fdk_decode_splitkv(const fdk_decode_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    Call call;
    int rc = adopt_call(caller_args, &call);
    if (rc) return rc;
    const fdk_decode_args* args = &call.a;
    rc = validate(args, false, true);
    if (rc) return rc;
    if (args->batch == 0) return FDK_OK;
    const bool dry = (args->flags & FDK_FLAG_DRY_RUN) != 0;
    Resolved r;
    rc = resolve(args, false, dry ? kDryRunCus : 0, &r);
    if (rc || dry) return rc;
    return launch_split(args, r, reinterpret_cast<hipStream_t>(hip_stream));
}

int fdk_combine(const fdk_decode_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    Call call;
    int rc = adopt_call(caller_args, &call);
    if (rc) return rc;
    const fdk_decode_args* args = &call.a;
    rc = validate(args, true, true);
    if (rc) return rc;
    if (args->batch == 0) return FDK_OK;
    const bool dry = (args->flags & FDK_FLAG_DRY_RUN) != 0;
    Resolved r;
    rc = resolve(args, false, dry ? kDryRunCus : 0, &r);
    if (rc || dry) return rc;
    rc = fdk::launch_combine(r.cp, reinterpret_cast<hipStream_t>(hip_stream));
    if (rc) return fail(rc, "combine kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return FDK_OK;
}

int fdk_combine_ranks(const fdk_combine_ranks_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    if (!caller_args) return fail(FDK_ENULL, "args is null");
    fdk_combine_ranks_args local;
    if (int rc = adopt(caller_args, caller_args->struct_size, sizeof(fdk_combine_ranks_args), "fdk_combine_ranks_args", &local))
        return rc;
    const fdk_combine_ranks_args* a = &local;
    if (a->num_ranks <= 0 || a->batch < 0 || a->num_q_heads <= 0)
        return fail(FDK_ESHAPE, "bad dims R=%d B=%d Hq=%d", a->num_ranks, a->batch, a->num_q_heads);
    if (a->head_dim != 64 && a->head_dim != 128 && a->head_dim != 192 && a->head_dim != 256 && a->head_dim != 512)
        return fail(FDK_EUNSUPPORTED, "head_dim %d not built (values of an output row: 64, 128, 192, 256 or 512)", a->head_dim);
    const bool packed = (a->flags & FDK_FLAG_PACK_LSE) != 0;
    if (elem_size(a->partial_dtype) < 2) return fail(FDK_EUNSUPPORTED, "partial_dtype %d", a->partial_dtype);
    if (elem_size(a->out_dtype) < 2) return fail(FDK_EUNSUPPORTED, "out_dtype %d", a->out_dtype);
    if (a->batch == 0) return FDK_OK;
    if (!a->partial || !a->kv_lens || !a->out) return fail(FDK_ENULL, "partial / kv_lens / out must be non-null");
    if (!packed && !a->partial_lse) return fail(FDK_ENULL, "partial_lse is null and FDK_FLAG_PACK_LSE is not set");
    if (a->stride_h < a->head_dim + (packed ? 1 : 0)) return fail(FDK_ESHAPE, "stride_h too small");
    if (a->out_stride_h < a->head_dim) return fail(FDK_ESHAPE, "out_stride_h too small");
    if (a->lse && (reinterpret_cast<uintptr_t>(a->lse) & 3u)) return fail(FDK_EALIGN, "lse not 4-byte aligned");
    if (a->lse && a->lse_stride_b_out < a->num_q_heads)
        return fail(FDK_ESHAPE, "lse_stride_b_out %lld < Hq %d", (long long)a->lse_stride_b_out, a->num_q_heads);
    if (!packed && a->lse_stride_b < a->num_q_heads)
        return fail(FDK_ESHAPE, "lse_stride_b %lld < Hq %d", (long long)a->lse_stride_b, a->num_q_heads);
    if (a->flags & FDK_FLAG_DRY_RUN) return FDK_OK;
    fdk::CombineRanksParams p;
    memset(&p, 0, sizeof(p));
    p.partial = a->partial; p.partial_lse = a->partial_lse; p.kv_lens = a->kv_lens;
    p.out = a->out; p.lse = a->lse;
    p.stride_r = a->stride_r; p.stride_b = a->stride_b; p.stride_h = a->stride_h;
    p.lse_stride_r = a->lse_stride_r; p.lse_stride_b = a->lse_stride_b;
    p.out_sb = a->out_stride_b; p.out_sh = a->out_stride_h; p.lse_sb_out = a->lse_stride_b_out;
    p.num_ranks = a->num_ranks; p.batch = a->batch; p.hq = a->num_q_heads; p.head_dim = a->head_dim;
    p.partial_dtype = a->partial_dtype; p.out_dtype = a->out_dtype; p.packed = packed ? 1 : 0;
    int rc = fdk::launch_combine_ranks(p, reinterpret_cast<hipStream_t>(hip_stream));
    if (rc) return fail(rc, "rank combine launch failed: %s", hipGetErrorString((hipError_t)rc));
    return FDK_OK;
}

int fdk_length_feedback_alloc(int32_t** host, int32_t** device) {
    if (!host || !device) return fail(FDK_ENULL, "host / device is null");
    *host = *device = nullptr;
    void* h = nullptr;
    hipError_t e = hipHostMalloc(&h, 4 * sizeof(int32_t), hipHostMallocMapped);
    if (e != hipSuccess) return fail((int)e, "hipHostMalloc: %s", hipGetErrorString(e));
    void* d = nullptr;
    e = hipHostGetDevicePointer(&d, h, 0);
    if (e != hipSuccess || !d || (reinterpret_cast<uintptr_t>(d) & 15u)) {
        (void)hipHostFree(h);
        return fail(e != hipSuccess ? (int)e : FDK_EALIGN, "hipHostGetDevicePointer: %s", hipGetErrorString(e));
    }
    memset(h, 0, 4 * sizeof(int32_t));
    *host = static_cast<int32_t*>(h);
    *device = static_cast<int32_t*>(d);
    return FDK_OK;
}

int fdk_length_feedback_free(int32_t* host) {
    if (!host) return FDK_OK;
    const hipError_t e = hipHostFree(host);
    if (e != hipSuccess) return fail((int)e, "hipHostFree: %s", hipGetErrorString(e));
    return FDK_OK;
}

int fdk_probe_linear_read(const void* buf, size_t bytes, int nontemporal, int workgroups, void* hip_stream) {
    g_err[0] = 0;
    if (!buf) return fail(FDK_ENULL, "buf is null");
    if (!aligned16(buf)) return fail(FDK_EALIGN, "buf must be 16-byte aligned");
    if (bytes < 65536) return fail(FDK_ESHAPE, "bytes %zu: at least 64 KB", bytes);
    if (workgroups <= 0 || workgroups > (1 << 20)) return fail(FDK_ESHAPE, "workgroups %d outside [1, 2^20]", workgroups);
    // the checksum's (practically never taken) store goes to the library's own scratch, not to the caller's buffer
    void* sink = nullptr;
    int rc = static_scratch_of_current_device(&sink);
    if (rc) return rc;
    sink = static_cast<unsigned char*>(sink) + kStaticScratchBytes;
    rc = fdk::launch_linear_read(buf, bytes, nontemporal, workgroups, static_cast<uint32_t*>(sink),
                                 reinterpret_cast<hipStream_t>(hip_stream));
    if (rc) return fail(rc, "linear read launch failed: %s", hipGetErrorString((hipError_t)rc));
    return FDK_OK;
}

int fdk_kv_append(const fdk_kv_append_args* caller_args, void* hip_stream) {
    g_err[0] = 0;
    if (!caller_args) return fail(FDK_ENULL, "args is null");
    fdk_kv_append_args local;
    if (int rc = adopt(caller_args, caller_args->struct_size, sizeof(fdk_kv_append_args), "fdk_kv_append_args", &local))
        return rc;
    const fdk_kv_append_args* a = &local;
    if (a->batch < 0 || a->new_tokens < 0) return fail(FDK_ESHAPE, "batch %d / new_tokens %d < 0", a->batch, a->new_tokens);
    if (a->num_q_heads < 0 || a->num_kv_heads <= 0)
        return fail(FDK_ESHAPE, "bad head counts Hq=%d Hkv=%d", a->num_q_heads, a->num_kv_heads);
    if (a->head_dim != 64 && a->head_dim != 128 && a->head_dim != 256)
        return fail(FDK_EUNSUPPORTED, "head_dim %d not built (64, 128 or 256)", a->head_dim);
    if (a->qkv_dtype != FDK_BF16 && a->qkv_dtype != FDK_FP16)
        return fail(FDK_EUNSUPPORTED, "qkv_dtype %d (bf16 or fp16 only)", a->qkv_dtype);
    if (a->kv_dtype != a->qkv_dtype && a->kv_dtype != FDK_FP8_E4M3)
        return fail(FDK_EUNSUPPORTED, "kv_dtype %d must equal qkv_dtype or be fp8_e4m3", a->kv_dtype);
    if (a->page_size <= 0 || a->max_pages <= 0 || a->num_pages <= 0)
        return fail(FDK_ESHAPE, "page_size %d, max_pages %d, num_pages %d must be positive", a->page_size, a->max_pages,
                    a->num_pages);
    if ((int64_t)a->max_pages * a->page_size > INT32_MAX) return fail(FDK_ESHAPE, "max_pages*page_size overflows int32");
    if (a->max_positions <= 0) return fail(FDK_ESHAPE, "max_positions %d <= 0", a->max_positions);
    if (!(a->q_eps == a->q_eps) || !(a->k_eps == a->k_eps) || a->q_eps < 0.f || a->k_eps < 0.f)
        return fail(FDK_ESHAPE, "eps must be non-negative numbers");
    if (a->batch == 0 || a->new_tokens == 0) return FDK_OK;
    const int64_t head_rows = (int64_t)a->num_q_heads + 2 * (int64_t)a->num_kv_heads;
    if ((int64_t)a->batch * a->new_tokens > (int64_t)INT32_MAX * 4 / head_rows)       // one wavefront per head row
        return fail(FDK_ESHAPE, "grid too large");
    if (!a->qkv || !a->k_weight || !a->cos || !a->sin || !a->block_table || !a->kv_lens || !a->k_cache || !a->v_cache)
        return fail(FDK_ENULL, "qkv / k_weight / cos / sin / block_table / kv_lens / k_cache / v_cache must be non-null");
    if (a->num_q_heads > 0 && (!a->q_weight || !a->q_out)) return fail(FDK_ENULL, "q_weight / q_out is null");
    if (a->kv_dtype == FDK_FP8_E4M3 && (!a->k_scale || !a->v_scale))
        return fail(FDK_ENULL, "k_scale / v_scale are required for an fp8 cache");
    if (a->qkv_stride_h < a->head_dim) return fail(FDK_ESHAPE, "qkv_stride_h %lld < head_dim", (long long)a->qkv_stride_h);
    if (a->num_q_heads > 0 && a->q_out_stride_h < a->head_dim)
        return fail(FDK_ESHAPE, "q_out_stride_h %lld < head_dim", (long long)a->q_out_stride_h);
    if (a->cs_stride_pos < a->head_dim / 2) return fail(FDK_ESHAPE, "cos/sin rows shorter than head_dim/2");
    if (a->table_stride_b < a->max_pages)
        return fail(FDK_ESHAPE, "table_stride_b %lld < max_pages %d", (long long)a->table_stride_b, a->max_pages);
    const int64_t st[6] = {a->k_stride_page, a->k_stride_tok, a->k_stride_head,
                           a->v_stride_page, a->v_stride_tok, a->v_stride_head};
    for (int i = 0; i < 6; ++i)
        if (st[i] < 0) return fail(FDK_ESHAPE, "negative cache stride");
    if (a->num_kv_heads > 1 && (a->k_stride_head < a->head_dim || a->v_stride_head < a->head_dim))
        return fail(FDK_ESHAPE, "cache head stride < head_dim");
    if (a->flags & FDK_FLAG_DRY_RUN) return FDK_OK;
    fdk::KvAppendParams p;
    memset(&p, 0, sizeof(p));
    p.qkv = a->qkv; p.q_weight = a->q_weight; p.k_weight = a->k_weight; p.cos = a->cos; p.sin = a->sin;
    p.block_table = a->block_table; p.kv_lens = a->kv_lens; p.k_scale = a->k_scale; p.v_scale = a->v_scale;
    p.k_cache = a->k_cache; p.v_cache = a->v_cache; p.q_out = a->q_out;
    p.qkv_sb = a->qkv_stride_b; p.qkv_st = a->qkv_stride_t; p.qkv_sh = a->qkv_stride_h;
    p.cs_sb = a->cs_stride_b; p.cs_sp = a->cs_stride_pos; p.tbl_sb = a->table_stride_b;
    p.k_sp = a->k_stride_page; p.k_st = a->k_stride_tok; p.k_sh = a->k_stride_head;
    p.v_sp = a->v_stride_page; p.v_st = a->v_stride_tok; p.v_sh = a->v_stride_head;
    p.qo_sb = a->q_out_stride_b; p.qo_st = a->q_out_stride_t; p.qo_sh = a->q_out_stride_h;
    p.batch = a->batch; p.new_tokens = a->new_tokens; p.hq = a->num_q_heads; p.hkv = a->num_kv_heads;
    p.head_dim = a->head_dim; p.page_size = a->page_size; p.max_pages = a->max_pages; p.num_pages = a->num_pages;
    p.max_positions = a->max_positions; p.q_eps = a->q_eps; p.k_eps = a->k_eps;
    int rc = fdk::launch_kv_append(p, a->qkv_dtype, a->kv_dtype, reinterpret_cast<hipStream_t>(hip_stream));
    if (rc) return fail(rc, "kv append launch failed: %s", hipGetErrorString((hipError_t)rc));
    return FDK_OK;
}

}  // extern "C"
