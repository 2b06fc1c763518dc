// Log-sum-exp merges: per-split partials -> (out, lse), and per-rank results -> out.  gfx950.
//
// Counterparts in the reference (python/triton_dist/kernels/nvidia/flash_decode.py):
//   combine_kernel        kernel_intra_rank_gqa_fwd_batch_decode_combine_kv, :392-449
//                         (and kernel_gqa_fwd_batch_decode_combine_kv, :307-360, which stores no lse)
//   combine_ranks_kernel  kernel_inter_rank_gqa_fwd_batch_decode_combine_kv, :481-532
// Same recurrence (running max, rescale, weighted sum) but evaluated 64 splits at a time: one lane
// per split loads its lse, the wavefront reduces max and sum with cross-lane ops, and the weighted
// accumulation over the partial rows then runs with independent loads.  One wavefront per
// (sequence, q head); each lane owns two of the 128 output columns.
#include "fdk_device.h"

namespace fdk {

namespace {

constexpr int kRowsPerWg = 4;  // (b, h) rows per 256-thread workgroup

__global__ __launch_bounds__(256) void combine_kernel(const CombineParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + wave;   // b * Hq + h
    if (row >= (int64_t)p.batch * p.hq) return;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);
    const int kv_len = min(p.kv_lens[b], p.max_tokens);
    // live splits: chunk c holds tokens [c*chunk, ...) - the split kernel wrote exactly these
    const int live = min(p.num_splits, (kv_len + p.chunk - 1) / p.chunk);

    const float* lse_row = p.part_lse + row * p.num_splits;
    const float* o_row = p.part_o + row * p.num_splits * kHeadDim;

    float m_run = -INFINITY, l_run = 0.f, acc0 = 0.f, acc1 = 0.f;
    for (int s0 = 0; s0 < live; s0 += 64) {
        const int n = min(64, live - s0);
        const float my = lane < n ? lse_row[s0 + lane] * kLog2e : -INFINITY;   // log2 units
        const float m_blk = wave_max(my);
        const float m_new = fmaxf(m_run, m_blk);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float w = fast_exp2(my - m_safe);                                 // 0 for idle lanes
        const float alpha = fast_exp2(m_run - m_safe);
        l_run = l_run * alpha + wave_sum(w);
        acc0 *= alpha;
        acc1 *= alpha;
#pragma unroll 4
        for (int s = 0; s < n; ++s) {
            const float ws = __shfl(w, s, 64);
            const float2 o = *reinterpret_cast<const float2*>(o_row + (int64_t)(s0 + s) * kHeadDim + 2 * lane);
            acc0 += ws * o.x;
            acc1 += ws * o.y;
        }
        m_run = m_new;
    }
    float r0 = 0.f, r1 = 0.f, lse = -INFINITY;
    if (live > 0) {
        const float inv = 1.0f / l_run;
        r0 = acc0 * inv;
        r1 = acc1 * inv;
        lse = (m_run + fast_log2(l_run)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
    store_out(p.out, ob + 2 * lane, r0, p.out_dtype);
    store_out(p.out, ob + 2 * lane + 1, r1, p.out_dtype);
    if (lane == 0) {
        if (p.lse) p.lse[(int64_t)b * p.lse_sb + h] = lse;
        if (p.pack_lse) store_out(p.out, ob + kHeadDim, lse, p.out_dtype);
    }
}

// Many splits: one workgroup per (sequence, head) row.  Every wavefront finds the global maximum and the sum
// of weights (a few lse loads), then the four wavefronts share the partial rows (s = wave, wave+4, ...) with
// eight independent loads in flight each, and the four sums meet in LDS.  Same result as combine_kernel.
__global__ __launch_bounds__(256) void combine_wide_kernel(const CombineParams p) {
    __shared__ float sm[kRowsPerWg][kHeadDim];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);
    const int kv_len = min(p.kv_lens[b], p.max_tokens);
    const int live = min(p.num_splits, (kv_len + p.chunk - 1) / p.chunk);
    const float* lse_row = p.part_lse + row * p.num_splits;
    const float* o_row = p.part_o + row * p.num_splits * kHeadDim;

    float m = -INFINITY;
    for (int s0 = 0; s0 < live; s0 += 64) {
        const float my = s0 + lane < live ? lse_row[s0 + lane] : -INFINITY;
        m = fmaxf(m, wave_max(my));
    }
    m *= kLog2e;
    float l = 0.f, acc0 = 0.f, acc1 = 0.f;
    for (int s0 = 0; s0 < live; s0 += 64) {
        const int n = min(64, live - s0);
        const float w = lane < n ? fast_exp2(lse_row[s0 + lane] * kLog2e - m) : 0.f;
        l += wave_sum(w);
#pragma unroll 8
        for (int s = wave; s < n; s += kRowsPerWg) {
            const float ws = __shfl(w, s, 64);
            const float2 o = *reinterpret_cast<const float2*>(o_row + (int64_t)(s0 + s) * kHeadDim + 2 * lane);
            acc0 += ws * o.x;
            acc1 += ws * o.y;
        }
    }
    sm[wave][2 * lane] = acc0;
    sm[wave][2 * lane + 1] = acc1;
    __syncthreads();
    if (wave != 0) return;
    float r0 = 0.f, r1 = 0.f, lse = -INFINITY;
    if (live > 0) {
        const float inv = 1.0f / l;
        r0 = (sm[0][2 * lane] + sm[1][2 * lane] + sm[2][2 * lane] + sm[3][2 * lane]) * inv;
        r1 = (sm[0][2 * lane + 1] + sm[1][2 * lane + 1] + sm[2][2 * lane + 1] + sm[3][2 * lane + 1]) * inv;
        lse = (m + fast_log2(l)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
    store_out(p.out, ob + 2 * lane, r0, p.out_dtype);
    store_out(p.out, ob + 2 * lane + 1, r1, p.out_dtype);
    if (lane == 0) {
        if (p.lse) p.lse[(int64_t)b * p.lse_sb + h] = lse;
        if (p.pack_lse) store_out(p.out, ob + kHeadDim, lse, p.out_dtype);
    }
}

__device__ __forceinline__ float load_any(const void* base, int64_t idx, int dtype) {
    if (dtype == FDK_BF16) return (float)reinterpret_cast<const __bf16*>(base)[idx];
    if (dtype == FDK_FP16) return (float)reinterpret_cast<const _Float16*>(base)[idx];
    return reinterpret_cast<const float*>(base)[idx];
}

__global__ __launch_bounds__(256) void combine_ranks_kernel(const CombineRanksParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + wave;
    if (row >= (int64_t)p.batch * p.hq) return;
    const int b = (int)(row / p.hq), h = (int)(row % p.hq);

    float m_run = -INFINITY, l_run = 0.f, acc0 = 0.f, acc1 = 0.f;
    for (int r0 = 0; r0 < p.num_ranks; r0 += 64) {
        const int n = min(64, p.num_ranks - r0);
        float my = -INFINITY;
        if (lane < n) {
            const int r = r0 + lane;
            if (p.kv_lens[(int64_t)r * p.batch + b] > 0) {      // skip rule of :513-515
                my = p.packed ? load_any(p.partial, r * p.stride_r + b * p.stride_b + h * p.stride_h + kHeadDim,
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
        acc0 *= alpha;
        acc1 *= alpha;
        for (int s = 0; s < n; ++s) {
            const float ws = __shfl(w, s, 64);
            if (ws != 0.f) {   // wave-uniform; ranks without tokens may hold garbage rows
                const int64_t base = (int64_t)(r0 + s) * p.stride_r + b * p.stride_b + h * p.stride_h + 2 * lane;
                acc0 += ws * load_any(p.partial, base, p.partial_dtype);
                acc1 += ws * load_any(p.partial, base + 1, p.partial_dtype);
            }
        }
        m_run = m_new;
    }
    float o0 = 0.f, o1 = 0.f, lse = -INFINITY;
    if (l_run > 0.f) {
        const float inv = 1.0f / l_run;
        o0 = acc0 * inv;
        o1 = acc1 * inv;
        lse = (m_run + fast_log2(l_run)) * kLn2;
    }
    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)h * p.out_sh;
    store_out(p.out, ob + 2 * lane, o0, p.out_dtype);
    store_out(p.out, ob + 2 * lane + 1, o1, p.out_dtype);
    if (lane == 0 && p.lse) p.lse[(int64_t)b * p.lse_sb_out + h] = lse;
}

}  // namespace

int launch_combine(const CombineParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.hq;
    if (rows == 0) return 0;
    if (p.num_splits > 8) {
        hipLaunchKernelGGL(combine_wide_kernel, dim3((unsigned)rows), dim3(256), 0, stream, p);
    } else {
        const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
        hipLaunchKernelGGL(combine_kernel, grid, dim3(256), 0, stream, p);
    }
    return (int)hipGetLastError();
}

int launch_combine_ranks(const CombineRanksParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.hq;
    if (rows == 0) return 0;
    const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
    hipLaunchKernelGGL(combine_ranks_kernel, grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace fdk
