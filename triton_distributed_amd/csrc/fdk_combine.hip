// Log-sum-exp merges: per-split partials -> (out, lse), and per-rank results -> out.  gfx950.
//
// Counterparts in the reference (python/triton_dist/kernels/nvidia/flash_decode.py):
//   combine_kernel        kernel_intra_rank_gqa_fwd_batch_decode_combine_kv, :392-449
//                         (and kernel_gqa_fwd_batch_decode_combine_kv, :307-360, which stores no lse)
//   combine_ranks_kernel  kernel_inter_rank_gqa_fwd_batch_decode_combine_kv, :481-532
// Same recurrence (running max, rescale, weighted sum) but evaluated 64 splits at a time: one lane
// per split loads its lse, the wavefront reduces max and sum with cross-lane ops, and the weighted
// accumulation over the partial rows then runs with independent loads.  One wavefront per
// (sequence, q head); each lane owns head_dim/64 adjacent output columns.
//   combine_slots_kernel  the same merge for balanced plans (equal shares of the whole batch), whose pieces are whole
//                         slots of adjacent rows: one workgroup per (sequence, unit) with 16-byte loads
#include "fdk_device.h"

namespace fdk {

namespace {

constexpr int kRowsPerWg = 4;  // (b, h) rows per 256-thread workgroup

// value of lane `i` (the same i in every lane) in all lanes
__device__ __forceinline__ float bcast_lane(float x, int i) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), i));
}

// EPL adjacent fp32 values (EPL = values of an output row / 64) with as few loads as their alignment allows
template <int EPL> struct Vec;
template <> struct Vec<1> {
    static __device__ __forceinline__ void load(const float* p, float (&o)[1]) { o[0] = *p; }
};
template <> struct Vec<2> {
    static __device__ __forceinline__ void load(const float* p, float (&o)[2]) {
        const float2 v = *reinterpret_cast<const float2*>(p);
        o[0] = v.x; o[1] = v.y;
    }
};
template <> struct Vec<4> {
    static __device__ __forceinline__ void load(const float* p, float (&o)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec<3> {                       // rows of 192 values: 12 bytes per lane
    static __device__ __forceinline__ void load(const float* p, float (&o)[3]) { o[0] = p[0]; o[1] = p[1]; o[2] = p[2]; }
};
template <> struct Vec<8> {                       // rows of 512 values
    static __device__ __forceinline__ void load(const float* p, float (&o)[8]) {
        const float4 v = *reinterpret_cast<const float4*>(p), w = *reinterpret_cast<const float4*>(p + 4);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; o[4] = w.x; o[5] = w.y; o[6] = w.z; o[7] = w.w;
    }
};

// Where the partial rows of output row (b, h) are: `live` rows, the s-th at o[s * o_step] / lse[s * lse_step].
struct PartRows {
    const float* o;
    const float* lse;
    int64_t o_step;
    int lse_step;
    int live;
};

// chunk mode: split c holds tokens [c*chunk, ...) - the split kernel wrote exactly the live ones
template <int D>
__device__ __forceinline__ PartRows locate_rows(const CombineParams& p, int b, int h) {
    PartRows r;
    const int kv_len = min(p.kv_lens[b], p.max_tokens);
    const int64_t row = (int64_t)b * p.hq + h;
    const int chunk = chunk_tokens_of(kv_len, p.num_splits, p.chunk, p.chunk_floor);
    r.live = min(p.num_splits, (kv_len + chunk - 1) / chunk);
    r.o = p.part_o + row * p.num_splits * D;
    r.lse = p.part_lse + row * p.num_splits;
    r.o_step = D;
    r.lse_step = 1;
    return r;
}

template <int D>
__global__ __launch_bounds__(256) void combine_kernel(const CombineParams p) {
    constexpr int EPL = D / 64;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + wave;   // b * Hq + h
    if (row >= (int64_t)p.batch * p.hq) return;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);
    // The first kPre partial rows are requested before anything that depends on kv_lens is known (chunk mode:
    // their addresses follow from (b, h) alone; rows past the live ones hold stale but readable workspace and
    // are never used) - the kernel is a chain of dependent memory round trips, this removes one or two.
    constexpr int kPre = 8;
    float pre[kPre][EPL];
    float lse_early = 0.f;                       // lse of split `lane`, requested just as early
    {
        const float* o_early = p.part_o + row * p.num_splits * D + EPL * lane;
#pragma unroll
        for (int j = 0; j < kPre; ++j)
            if (j < p.num_splits) Vec<EPL>::load(o_early + (int64_t)j * D, pre[j]);
        if (lane < p.num_splits) lse_early = p.part_lse[row * p.num_splits + lane];
    }
    const PartRows pr = locate_rows<D>(p, b, h);
    const int live = pr.live;
    const float* lse_row = pr.lse;
    const float* o_row = pr.o + EPL * lane;

    float m_run = -INFINITY, l_run = 0.f;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
    for (int s0 = 0; s0 < live; s0 += 64) {
        const int n = min(64, live - s0);
        const float my = lane < n ? (s0 == 0 ? lse_early : lse_row[(s0 + lane) * pr.lse_step]) * kLog2e
                                  : -INFINITY;   // log2 units
        const float m_blk = wave_max(my);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float w = fast_exp2(my - m_safe);                                 // 0 for idle lanes
        const float alpha = fast_exp2(m_run - m_safe);
        l_run = l_run * alpha + wave_sum(w);
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] *= alpha;
        int s = 0;
        if (s0 == 0) {
#pragma unroll
            for (int j = 0; j < kPre; ++j) {
                if (j < n) {
                    const float ws = bcast_lane(w, j);
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[e] += ws * pre[j][e];
                }
            }
            s = kPre;
        }
#pragma unroll 4
        for (; s < n; ++s) {
            const float ws = bcast_lane(w, s);
            float o[EPL];
            Vec<EPL>::load(o_row + (s0 + s) * pr.o_step, o);
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += ws * o[e];
        }
        m_run = m_new;
    }
    float inv = 0.f, lse = -INFINITY;                 // no live split: out = 0, lse = -inf
    if (live > 0) {
        inv = 1.0f / l_run;
        lse = (m_run + fast_log2(l_run)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
#pragma unroll
    for (int e = 0; e < EPL; ++e) store_out(p.out, ob + EPL * lane + e, acc[e] * inv, p.out_dtype);
    if (lane == 0) {
        if (p.lse) p.lse[(int64_t)b * p.lse_sb + h] = lse;
        if (p.pack_lse) store_out(p.out, ob + D, lse, p.out_dtype);
    }
    if (p.length_feedback && row == 0)
        store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
}

// Many splits: one workgroup per (sequence, head) row.  Every wavefront finds the global maximum and the sum
// of weights (a few lse loads), then the four wavefronts share the partial rows (s = wave, wave+4, ...) with
// eight independent loads in flight each, and the four sums meet in LDS.  Same result as combine_kernel.
template <int D>
__global__ __launch_bounds__(256) void combine_wide_kernel(const CombineParams p) {
    constexpr int EPL = D / 64;
    __shared__ float sm[kRowsPerWg][D];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row = blockIdx.x;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);
    // as in combine_kernel: the first kPre rows of this wavefront (s = wave, wave + 4, ...: all of them up to 64
    // splits) and the lse values are requested before the number of live splits is known
    constexpr int kPre = 16;
    float pre[kPre][EPL];
    float lse_early = 0.f;
    {
        const float* o_early = p.part_o + row * p.num_splits * D + EPL * lane;
#pragma unroll
        for (int j = 0; j < kPre; ++j)
            if (wave + kRowsPerWg * j < p.num_splits) Vec<EPL>::load(o_early + (int64_t)(wave + kRowsPerWg * j) * D, pre[j]);
        if (lane < p.num_splits) lse_early = p.part_lse[row * p.num_splits + lane];
    }
    const PartRows pr = locate_rows<D>(p, b, h);
    const int live = pr.live;
    const float* lse_row = pr.lse;
    const float* o_row = pr.o + EPL * lane;

    float m = -INFINITY;
    float my_first = -INFINITY;                    // lse of split `lane`, kept for the second pass
    for (int s0 = 0; s0 < live; s0 += 64) {
        const float my = s0 + lane < live ? (s0 == 0 ? lse_early : lse_row[(s0 + lane) * pr.lse_step])
                                          : -INFINITY;
        if (s0 == 0) my_first = my;
        m = fmaxf(m, wave_max(my));
    }
    m *= kLog2e;
    float l = 0.f;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
    for (int s0 = 0; s0 < live; s0 += 64) {
        const int n = min(64, live - s0);
        const float lse_s = s0 == 0 ? my_first : (lane < n ? lse_row[(s0 + lane) * pr.lse_step] : -INFINITY);
        const float w = lane < n ? fast_exp2(lse_s * kLog2e - m) : 0.f;
        l += wave_sum(w);
        int s = wave;
        if (s0 == 0) {
#pragma unroll
            for (int j = 0; j < kPre; ++j) {
                if (wave + kRowsPerWg * j < n) {
                    const float ws = bcast_lane(w, wave + kRowsPerWg * j);
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[e] += ws * pre[j][e];
                }
            }
            s = wave + kRowsPerWg * kPre;
        }
#pragma unroll 8
        for (; s < n; s += kRowsPerWg) {
            const float ws = bcast_lane(w, s);
            float o[EPL];
            Vec<EPL>::load(o_row + (s0 + s) * pr.o_step, o);
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += ws * o[e];
        }
    }
#pragma unroll
    for (int e = 0; e < EPL; ++e) sm[wave][EPL * lane + e] = acc[e];
    __syncthreads();
    if (wave != 0) return;
    float inv = 0.f, lse = -INFINITY;
    if (live > 0) {
        inv = 1.0f / l;
        lse = (m + fast_log2(l)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        const int d = EPL * lane + e;
        store_out(p.out, ob + d, (sm[0][d] + sm[1][d] + sm[2][d] + sm[3][d]) * inv, p.out_dtype);
    }
    if (lane == 0) {
        if (p.lse) p.lse[(int64_t)b * p.lse_sb + h] = lse;
        if (p.pack_lse) store_out(p.out, ob + D, lse, p.out_dtype);
    }
    if (p.length_feedback && row == 0)
        store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
}

// Balanced plans.  The pieces of a (sequence, unit) are whole slots - rows_per_slot adjacent partial rows, one per
// (kv head of the block, q head of the tile) - in consecutive shares, and the split kernel has left {first share,
// live pieces} for every (sequence, unit) that holds tokens.  One workgroup per (sequence, unit); a thread owns four
// adjacent columns of one row, requests that row's lse values and its 16 bytes of up to eight pieces at once, and
// merges them by itself: no cross-lane traffic, no pass over kv_lens, one dependent round trip after the descriptor.
template <int D>
__global__ __launch_bounds__(1024) void combine_slots_kernel(const CombineParams p) {
    constexpr int LPR = D / 4;                    // threads per row
    constexpr int NB = 8;                         // pieces per batch of loads
    const int units = p.hg_blocks * p.head_tiles;
    const int b = blockIdx.x / units, u = blockIdx.x % units;
    const int2 desc = p.slot_desc[blockIdx.x];                  // (garbage for a sequence without tokens: not used)
    const int kv_len = p.kv_lens[b];
    const int hgb = u / p.head_tiles, ht = u % p.head_tiles;
    const int heads_here = min(p.tile_heads, p.group - ht * p.tile_heads);
    const int c4 = threadIdx.x % LPR;
    const int64_t piece_step = (int64_t)units * p.rows_per_slot;                 // rows from one piece to the next
    for (int r = threadIdx.x / LPR; r < p.rows_per_slot; r += p.rows_per_pass) {
        const int hl = r / p.heads_per_tile, g = r % p.heads_per_tile;
        if (g >= heads_here) continue;                                       // the last tile of a group may be short
        const int hq = (hgb * p.kv_heads_per_wg + hl) * p.group + ht * p.tile_heads + g;
        const int64_t ob = (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        float inv = 0.f, lse = -INFINITY;                                    // no tokens: out = 0, lse = -inf
        if (kv_len > 0) {
            const int64_t row0 = ((int64_t)(desc.x + b) * units + u) * p.rows_per_slot + r;
            const float* lse_p = p.part_lse + row0;
            const float* o_p = p.part_o + row0 * D + 4 * c4;
            float m_run = -INFINITY, l_run = 0.f;
            for (int s0 = 0; s0 < desc.y; s0 += NB) {
                float ls[NB];
                float4 o[NB];
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    ls[j] = -INFINITY;
                    o[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (s0 + j < desc.y) {
                        ls[j] = lse_p[(s0 + j) * piece_step];
                        o[j] = *reinterpret_cast<const float4*>(o_p + (s0 + j) * piece_step * D);
                    }
                }
                float m_new = m_run;
#pragma unroll
                for (int j = 0; j < NB; ++j) m_new = fmaxf(m_new, ls[j] * kLog2e);     // finite: a live piece holds a token
                const float alpha = fast_exp2(m_run - m_new);
                l_run *= alpha;
                acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha;
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const float w = fast_exp2(ls[j] * kLog2e - m_new);                  // 0 past the last piece
                    l_run += w;
                    acc.x += w * o[j].x; acc.y += w * o[j].y; acc.z += w * o[j].z; acc.w += w * o[j].w;
                }
                m_run = m_new;
            }
            inv = 1.0f / l_run;
            lse = (m_run + fast_log2(l_run)) * kLn2;
        }
        store_out4(p.out, ob + 4 * c4, make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv), p.out_dtype);
        if (c4 == 0) {
            if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse;
            if (p.pack_lse) store_out(p.out, ob + D, lse, p.out_dtype);
        }
    }
    if (p.length_feedback && blockIdx.x == 0 && threadIdx.x < 64)
        store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, threadIdx.x);
}

__device__ __forceinline__ float load_any(const void* base, int64_t idx, int dtype) {
    if (dtype == FDK_BF16) return (float)reinterpret_cast<const __bf16*>(base)[idx];
    if (dtype == FDK_FP16) return (float)reinterpret_cast<const _Float16*>(base)[idx];
    return reinterpret_cast<const float*>(base)[idx];
}

template <int D>
__global__ __launch_bounds__(256) void combine_ranks_kernel(const CombineRanksParams p) {
    constexpr int EPL = D / 64;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + wave;
    if (row >= (int64_t)p.batch * p.hq) return;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);

    float m_run = -INFINITY, l_run = 0.f;
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
    for (int r0 = 0; r0 < p.num_ranks; r0 += 64) {
        const int n = min(64, p.num_ranks - r0);
        float my = -INFINITY;
        if (lane < n) {
            const int r = r0 + lane;
            if (p.kv_lens[(int64_t)r * p.batch + b] > 0) {      // skip rule of :513-515
                my = p.packed ? load_any(p.partial, r * p.stride_r + b * p.stride_b + h * p.stride_h + D,
                                         p.partial_dtype)
                              : p.partial_lse[r * p.lse_stride_r + b * p.lse_stride_b + h];
                my *= kLog2e;
            }
        }
        const float m_blk = wave_max(my);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float w = fast_exp2(my - m_safe);
        const float alpha = fast_exp2(m_run - m_safe);
        l_run = l_run * alpha + wave_sum(w);
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] *= alpha;
        for (int s = 0; s < n; ++s) {
            const float ws = bcast_lane(w, s);
            if (ws != 0.f) {   // wave-uniform; ranks without tokens may hold garbage rows
                const int64_t base = (int64_t)(r0 + s) * p.stride_r + b * p.stride_b + h * p.stride_h + EPL * lane;
#pragma unroll
                for (int e = 0; e < EPL; ++e) acc[e] += ws * load_any(p.partial, base + e, p.partial_dtype);
            }
        }
        m_run = m_new;
    }
    float inv = 0.f, lse = -INFINITY;
    if (l_run > 0.f) {
        inv = 1.0f / l_run;
        lse = (m_run + fast_log2(l_run)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
#pragma unroll
    for (int e = 0; e < EPL; ++e) store_out(p.out, ob + EPL * lane + e, acc[e] * inv, p.out_dtype);
    if (lane == 0 && p.lse) p.lse[(int64_t)b * p.lse_sb_out + h] = lse;
}

}  // namespace

int launch_combine(const CombineParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.hq;
    if (rows == 0) return 0;
    if (p.balanced) {
        const int units = p.hg_blocks * p.head_tiles;
        const dim3 grid((unsigned)(p.batch * units));
        const int lpr = p.head_dim / 4;
        // whole rows only: a row's threads must not start over on another row (48 threads per row of 192 values)
        const int rows_per_pass = p.rows_per_slot * lpr > 1024 ? 1024 / lpr : p.rows_per_slot;
        const dim3 block((unsigned)(rows_per_pass * lpr < 64 ? 64 : rows_per_pass * lpr));
        CombineParams q = p;
        q.rows_per_pass = rows_per_pass;
        switch (p.head_dim) {
            case 64: hipLaunchKernelGGL(combine_slots_kernel<64>, grid, block, 0, stream, q); break;
            case 128: hipLaunchKernelGGL(combine_slots_kernel<128>, grid, block, 0, stream, q); break;
            case 256: hipLaunchKernelGGL(combine_slots_kernel<256>, grid, block, 0, stream, q); break;
            case 192: hipLaunchKernelGGL(combine_slots_kernel<192>, grid, block, 0, stream, q); break;
            case 512: hipLaunchKernelGGL(combine_slots_kernel<512>, grid, block, 0, stream, q); break;
            default: return (int)hipErrorInvalidValue;
        }
        return (int)hipGetLastError();
    }
    const bool wide = p.num_splits > 8;
    const dim3 grid((unsigned)(wide ? rows : (rows + kRowsPerWg - 1) / kRowsPerWg));
#define FDK_COMBINE_LAUNCH(DV)                                                                     \
    do {                                                                                           \
        if (wide) hipLaunchKernelGGL(combine_wide_kernel<DV>, grid, dim3(256), 0, stream, p);      \
        else hipLaunchKernelGGL(combine_kernel<DV>, grid, dim3(256), 0, stream, p);                \
    } while (0)
    switch (p.head_dim) {
        case 64: FDK_COMBINE_LAUNCH(64); break;
        case 128: FDK_COMBINE_LAUNCH(128); break;
        case 256: FDK_COMBINE_LAUNCH(256); break;
        case 192: FDK_COMBINE_LAUNCH(192); break;
        case 512: FDK_COMBINE_LAUNCH(512); break;
        default: return (int)hipErrorInvalidValue;
    }
#undef FDK_COMBINE_LAUNCH
    return (int)hipGetLastError();
}

int launch_combine_ranks(const CombineRanksParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.hq;
    if (rows == 0) return 0;
    const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
    switch (p.head_dim) {
        case 64: hipLaunchKernelGGL(combine_ranks_kernel<64>, grid, dim3(256), 0, stream, p); break;
        case 128: hipLaunchKernelGGL(combine_ranks_kernel<128>, grid, dim3(256), 0, stream, p); break;
        case 256: hipLaunchKernelGGL(combine_ranks_kernel<256>, grid, dim3(256), 0, stream, p); break;
        case 192: hipLaunchKernelGGL(combine_ranks_kernel<192>, grid, dim3(256), 0, stream, p); break;
        case 512: hipLaunchKernelGGL(combine_ranks_kernel<512>, grid, dim3(256), 0, stream, p); break;
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

}  // namespace fdk
