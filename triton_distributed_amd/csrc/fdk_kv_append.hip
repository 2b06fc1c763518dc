// Per-head RMSNorm + rotary embedding of the new tokens and their append to the paged KV cache.  gfx950.
//
// Counterpart in the reference: rmsnorm_rope_update_kv_cache_task_compute,
// python/triton_dist/mega_triton_kernel/kernels/norm.py:32-190 (one tile per q / k head row, the k tile also
// copies the token's v heads).  Here: one wavefront per head row of qkv (q, k and v rows alike; two or four rows for
// grids that would not be resident at once), four wavefronts per workgroup.  A lane owns the rotary pairs (i, i + D/2), i = lane + 64 j, so that the rotation needs no
// cross-lane traffic; the only reduction is the sum of squares of the row.  The work is a few kilobytes per
// token: the kernel is bound by launch and memory latency, not by bandwidth.
#include "fdk_device.h"

namespace fdk {

namespace {

template <int QDT> struct Elem;
template <> struct Elem<FDK_BF16> {
    using T = __bf16;
};
template <> struct Elem<FDK_FP16> {
    using T = _Float16;
};

// one e4m3 byte: saturating, round to nearest even
__device__ __forceinline__ uint8_t to_e4m3(float x) {
    x = __builtin_fminf(__builtin_fmaxf(x, -448.0f), 448.0f);      // NaN stays NaN
    return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false) & 0xFF);
}

// R head rows per wavefront: a grid that would not be resident at once (more than 8192 wavefronts on MI355X) runs its
// latency chain - kv_lens, then the table entry and the rotary row, then the stores - once per round; with R rows per
// wavefront, their loads requested together, it stays one round.
template <int QDT, bool FP8, int D, int R>
__global__ __launch_bounds__(256) void kv_append_kernel(const KvAppendParams p) {
    using T = typename Elem<QDT>::T;
    constexpr int HALF = D / 2;
    constexpr int PPL = HALF > 64 ? HALF / 64 : 1;      // rotary pairs per lane
    const int lane = threadIdx.x & 63;
    const int heads = p.hq + 2 * p.hkv;
    const int64_t total = (int64_t)p.batch * p.new_tokens * heads;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
    if (row0 >= total) return;
    const bool active = HALF >= 64 || lane < HALF;

    int h_[R], t_[R], b_[R], pos_[R];
    bool live_[R];
    float x0[R][PPL], x1[R][PPL];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t row = row0 + r;
        live_[r] = row < total;
        const int64_t rr = live_[r] ? row : row0;
        h_[r] = (int)(rr % heads);
        t_[r] = (int)((rr / heads) % p.new_tokens);
        b_[r] = (int)(rr / ((int64_t)heads * p.new_tokens));
        pos_[r] = p.kv_lens[b_[r]] - p.new_tokens + t_[r];
        const T* x = reinterpret_cast<const T*>(p.qkv) + b_[r] * p.qkv_sb + t_[r] * p.qkv_st + h_[r] * p.qkv_sh;
#pragma unroll
        for (int j = 0; j < PPL; ++j) {
            const int i = lane + 64 * j;
            x0[r][j] = active ? (float)x[i] : 0.f;
            x1[r][j] = active ? (float)x[i + HALF] : 0.f;
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!live_[r]) continue;
        const int h = h_[r], t = t_[r], b = b_[r], pos = pos_[r];
        // where the row goes: q_out, or a cache row (k and v heads)
        const bool is_q = h < p.hq;
        const bool is_k = !is_q && h < p.hq + p.hkv;
        const int kvh = is_q ? 0 : (is_k ? h - p.hq : h - p.hq - p.hkv);
        bool writable = true;
        int64_t cache_row = 0;            // element offset of the row inside its cache
        if (!is_q) {
            writable = pos >= 0 && pos < (int64_t)p.max_pages * p.page_size;
            if (writable) {
                const int page = p.block_table[b * p.tbl_sb + pos / p.page_size];
                writable = page >= 0 && page < p.num_pages;
                const int slot = pos % p.page_size;
                cache_row = is_k ? page * p.k_sp + slot * p.k_st + kvh * p.k_sh : page * p.v_sp + slot * p.v_st + kvh * p.v_sh;
            }
            if (!writable) continue;      // wave-uniform
        }

        float o0[PPL], o1[PPL];
        if (is_q || is_k) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < PPL; ++j) ss += x0[r][j] * x0[r][j] + x1[r][j] * x1[r][j];
            ss = wave_sum(ss);
            const float rms = 1.0f / sqrtf(ss / (float)D + (is_q ? p.q_eps : p.k_eps));
            const T* w = reinterpret_cast<const T*>(is_q ? p.q_weight : p.k_weight);
            const int cpos = min(max(pos, 0), p.max_positions - 1);
            const float* cr = p.cos + b * p.cs_sb + cpos * p.cs_sp;
            const float* sr = p.sin + b * p.cs_sb + cpos * p.cs_sp;
#pragma unroll
            for (int j = 0; j < PPL; ++j) {
                const int i = lane + 64 * j;
                if (!active) continue;
                // halves rounded to the 16-bit dtype before the rotation, as the reference does (norm.py:168-171)
                const float y0 = (float)(T)((float)w[i] * (x0[r][j] * rms));
                const float y1 = (float)(T)((float)w[i + HALF] * (x1[r][j] * rms));
                const float c = cr[i], sn = sr[i];
                o0[j] = y0 * c - y1 * sn;
                o1[j] = y1 * c + y0 * sn;
            }
        } else {
#pragma unroll
            for (int j = 0; j < PPL; ++j) {
                o0[j] = x0[r][j];
                o1[j] = x1[r][j];
            }
        }

        if (!active) continue;
        if (is_q) {
            T* q = reinterpret_cast<T*>(p.q_out) + b * p.qo_sb + t * p.qo_st + h * p.qo_sh;
#pragma unroll
            for (int j = 0; j < PPL; ++j) {
                q[lane + 64 * j] = (T)o0[j];
                q[lane + 64 * j + HALF] = (T)o1[j];
            }
        } else if (FP8) {
            uint8_t* c = reinterpret_cast<uint8_t*>(is_k ? p.k_cache : p.v_cache) + cache_row;
            const float scale = is_k ? p.k_scale[kvh] : p.v_scale[kvh];
#pragma unroll
            for (int j = 0; j < PPL; ++j) {
                c[lane + 64 * j] = to_e4m3((float)(T)o0[j] / scale);
                c[lane + 64 * j + HALF] = to_e4m3((float)(T)o1[j] / scale);
            }
        } else {
            T* c = reinterpret_cast<T*>(is_k ? p.k_cache : p.v_cache) + cache_row;
#pragma unroll
            for (int j = 0; j < PPL; ++j) {
                c[lane + 64 * j] = (T)o0[j];
                c[lane + 64 * j + HALF] = (T)o1[j];
            }
        }
    }
}

template <int QDT, bool FP8, int R>
int launch_r(const KvAppendParams& p, int64_t rows, hipStream_t stream) {
    const int64_t waves = (rows + R - 1) / R;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    switch (p.head_dim) {
        case 64: hipLaunchKernelGGL((kv_append_kernel<QDT, FP8, 64, R>), grid, block, 0, stream, p); break;
        case 128: hipLaunchKernelGGL((kv_append_kernel<QDT, FP8, 128, R>), grid, block, 0, stream, p); break;
        case 256: hipLaunchKernelGGL((kv_append_kernel<QDT, FP8, 256, R>), grid, block, 0, stream, p); break;
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

template <int QDT, bool FP8>
int launch_d(const KvAppendParams& p, hipStream_t stream) {
    const int64_t rows = (int64_t)p.batch * p.new_tokens * (p.hq + 2 * p.hkv);
    if (rows == 0) return 0;
    // rows per wavefront: as few as keep the grid within the wavefronts a GPU of 256 compute units holds at once
    constexpr int64_t kResidentWaves = 256 * 32;
    if (rows <= kResidentWaves) return launch_r<QDT, FP8, 1>(p, rows, stream);
    if (rows <= 2 * kResidentWaves) return launch_r<QDT, FP8, 2>(p, rows, stream);
    return launch_r<QDT, FP8, 4>(p, rows, stream);
}

}  // namespace

int launch_kv_append(const KvAppendParams& p, int qkv_dtype, int kv_dtype, hipStream_t stream) {
    const bool fp8 = kv_dtype == FDK_FP8_E4M3;
    if (qkv_dtype == FDK_BF16) return fp8 ? launch_d<FDK_BF16, true>(p, stream) : launch_d<FDK_BF16, false>(p, stream);
    return fp8 ? launch_d<FDK_FP16, true>(p, stream) : launch_d<FDK_FP16, false>(p, stream);
}

}  // namespace fdk
