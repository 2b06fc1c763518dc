// Split-KV paged GQA decode, vector-ALU path (v_dot2 + FMA), gfx950.
//
// Counterpart of kernel_gqa_fwd_batch_decode_split_kv in the reference
// (python/triton_dist/kernels/nvidia/flash_decode.py:129-239): one workgroup per
// (sequence, kv head [x head tile], split); online softmax in fp32; per-split normalised
// partial output and lse = m + ln(l).  Differences by design: splits are fixed-length token
// chunks (so ragged batches give equally sized work items), the page lookup is 64-bit, an
// empty chunk writes nothing (the combine derives the live split count from kv_len), and with
// a single split the final (out, lse) is written directly.
//
// Data flow per wavefront: a 16-byte load per lane covers 64/LPR whole token rows (LPR lanes per
// 256-byte bf16 row or 128-byte fp8 row), so every global load instruction reads whole,
// contiguous rows.  Four K loads and four V loads make one tile (16 bf16 / 32 fp8 tokens); the
// next tile's loads are issued before the current tile is consumed and the page ids one tile
// further ahead.  Each group of LPR lanes keeps its own running (m, l, acc) for the rows it sees;
// the groups and the four wavefronts are merged once at the end through DPP/shuffles and LDS.
#include "fdk_device.h"

namespace fdk {

namespace {

template <bool FP8>
struct Geo {
    static constexpr int EPL = FP8 ? 16 : 8;        // cache elements per lane per 16-byte load
    static constexpr int LPR = kHeadDim / EPL;      // lanes per token row
    static constexpr int TPL = kWaveSize / LPR;     // token rows per wave load
    static constexpr int NJ = 4;                    // loads per tile and tensor
    static constexpr int TILE = TPL * NJ;           // tokens per tile
    static constexpr int QW = EPL / 2;              // q dwords per lane and head
    static constexpr int ES = FP8 ? 1 : 2;          // cache element size
};

template <bool FP8>
struct KvTile {
    uint32_t k[Geo<FP8>::NJ][4];
    uint32_t v[Geo<FP8>::NJ][4];
};

__device__ __forceinline__ void put(uint32_t (&dst)[4], const uint4 x) {
    dst[0] = x.x;
    dst[1] = x.y;
    dst[2] = x.z;
    dst[3] = x.w;
}

struct PageIds {          // page of each of the tile's four loads (wave-uniform or per lane)
    int32_t pg[4];
};

template <int QDT, bool FP8, int GT, bool PUNIF, bool PVDOT>
__global__ __launch_bounds__(256) void splitkv_valu_kernel(const SplitParams p) {
    using G_ = Geo<FP8>;
    using P2 = Pack2<QDT>;
    constexpr int EPL = G_::EPL, LPR = G_::LPR, TPL = G_::TPL, NJ = G_::NJ, TILE = G_::TILE, QW = G_::QW,
                  ES = G_::ES;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int piece = lane % LPR;
    const int rgrp = lane / LPR;

    // workgroup -> (sequence, split, kv head, head tile); kv heads vary fastest so neighbouring
    // workgroups read neighbouring 256-byte pieces of the same token rows.
    int wg = blockIdx.x;
    const int units = p.hkv * p.head_tiles;
    const int unit = wg % units;
    wg /= units;
    const int split = wg % p.num_splits;
    const int b = wg / p.num_splits;
    const int kvh = unit / p.head_tiles;
    const int ht = unit % p.head_tiles;
    const int head0 = kvh * p.group + ht * GT;       // first q head of this workgroup
    const int heads_here = min(GT, p.group - ht * GT);

    const int kv_len = min(p.kv_lens[b], p.max_tokens);
    const int c_start = split * p.chunk;
    if (c_start >= kv_len) {
        if (p.direct) {   // kv_len == 0 with a single split: defined result, no combine follows
            for (int idx = threadIdx.x; idx < heads_here * kHeadDim; idx += 256) {
                const int g = idx / kHeadDim, d = idx % kHeadDim;
                store_out(p.out, (int64_t)b * p.out_sb + (int64_t)(head0 + g) * p.out_sh + d, 0.f, p.out_dtype);
            }
            if (threadIdx.x < heads_here) {
                const int hq = head0 + threadIdx.x;
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = -INFINITY;
                if (p.pack_lse)
                    store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + kHeadDim, -INFINITY,
                              p.out_dtype);
            }
        }
        return;
    }
    const int c_end = min(c_start + p.chunk, kv_len);
    const int n_tiles = (c_end - c_start + TILE - 1) / TILE;

    // ---- q: each lane keeps, for every head, the EPL elements matching its piece of the row -----
    uint32_t qreg[GT][QW];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        const bool valid = g < heads_here;
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)b * p.q_sb +
                             (int64_t)(head0 + (valid ? g : 0)) * p.q_sh + piece * EPL;
#pragma unroll
        for (int w4 = 0; w4 < QW / 4; ++w4) {
            uint4 t = reinterpret_cast<const uint4*>(qp)[w4];
            if (!valid) t = make_uint4(0, 0, 0, 0);
            qreg[g][4 * w4 + 0] = t.x;
            qreg[g][4 * w4 + 1] = t.y;
            qreg[g][4 * w4 + 2] = t.z;
            qreg[g][4 * w4 + 3] = t.w;
        }
    }

    float kscale = 1.f, vscale = 1.f;
    if (FP8) {
        if (p.k_scale) kscale = p.k_scale[kvh];
        if (p.v_scale) vscale = p.v_scale[kvh];
    }
    const float scale_log2 = p.scale_log2;               // raw dot -> log2-unit logit
    const float scale_nat = p.sm_scale;                   // raw dot -> natural-unit logit (soft cap)
    const bool softcap = p.soft_cap > 0.f;
    const float inv_cap = softcap ? 1.0f / p.soft_cap : 0.f;

    const char* kbase = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES + piece * 16;
    const char* vbase = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES + piece * 16;
    const int32_t* tbl = p.block_table + (int64_t)b * p.tbl_sb;

    // Pages of tile t.  With PUNIF (page_size % TPL == 0) all rows of one load share a page and the
    // lookup is wave-uniform; otherwise every lane looks up the page of its own row.
    auto pages_of = [&](int t, PageIds& pi) {
        const int tok0 = c_start + t * TILE;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            int n = tok0 + j * TPL;
            if (!PUNIF) n += rgrp;
            n = min(n, c_end - 1);              // rows past the chunk are never loaded; keep the lookup in range
            const int pg_idx = (p.page_shift >= 0) ? (n >> p.page_shift) : (n / p.page_size);
            pi.pg[j] = tbl[pg_idx];
        }
    };
    const int64_t lane_row_k = PUNIF ? (int64_t)rgrp * p.k_st : 0;
    const int64_t lane_row_v = PUNIF ? (int64_t)rgrp * p.v_st : 0;
    auto issue = [&](int t, const PageIds& pi, KvTile<FP8>& kt) {
        const int tok0 = c_start + t * TILE;
        const bool full = tok0 + TILE <= c_end;
        const char* kp[NJ];
        const char* vp[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            int n = tok0 + j * TPL;
            if (!PUNIF) n += rgrp;
            const int slot = (p.page_shift >= 0) ? (n & (p.page_size - 1)) : (n % p.page_size);
            kp[j] = kbase + ((int64_t)pi.pg[j] * p.k_sp + (int64_t)slot * p.k_st + lane_row_k) * ES;
            vp[j] = vbase + ((int64_t)pi.pg[j] * p.v_sp + (int64_t)slot * p.v_st + lane_row_v) * ES;
        }
        if (full) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) put(kt.k[j], *reinterpret_cast<const uint4*>(kp[j]));
#pragma unroll
            for (int j = 0; j < NJ; ++j) put(kt.v[j], *reinterpret_cast<const uint4*>(vp[j]));
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const bool ok = tok0 + j * TPL + rgrp < c_end;
                uint4 kk = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
                if (ok) {
                    kk = *reinterpret_cast<const uint4*>(kp[j]);
                    vv = *reinterpret_cast<const uint4*>(vp[j]);
                }
                put(kt.k[j], kk);
                put(kt.v[j], vv);
            }
        }
    };

    // ---- running state of this lane's row group ------------------------------------------------
    float m_run[GT], l_run[GT], acc[GT][EPL];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        m_run[g] = -INFINITY;
        l_run[g] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
    }

    auto consume = [&](int t, const KvTile<FP8>& kt) {
        const int tok0 = c_start + t * TILE;
        const bool full = tok0 + TILE <= c_end;
        float s[GT][NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint32_t kk[QW];
            if (FP8) {
                // dequantise exactly as "(k8 * scale) rounded to the q dtype": the logits, and with them
                // lse, then equal those of a decode over the dequantised cache
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const f32x2_t f01 = __builtin_amdgcn_cvt_pk_f32_fp8(kt.k[j][w], false);
                    const f32x2_t f23 = __builtin_amdgcn_cvt_pk_f32_fp8(kt.k[j][w], true);
                    kk[2 * w] = P2::pack(f01.x * kscale, f01.y * kscale);
                    kk[2 * w + 1] = P2::pack(f23.x * kscale, f23.y * kscale);
                }
            } else {
#pragma unroll
                for (int w = 0; w < 4; ++w) kk[w] = kt.k[j][w];
            }
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                float d = 0.f;
#pragma unroll
                for (int w = 0; w < QW; ++w) d = P2::dot2(qreg[g][w], kk[w], d);
                s[g][j] = group_sum<LPR>(d);
            }
        }
        if (softcap) {   // wave-uniform
#pragma unroll
            for (int g = 0; g < GT; ++g)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    s[g][j] = soft_cap_fn(s[g][j] * scale_nat, p.soft_cap, inv_cap) * kLog2e;
        } else {
#pragma unroll
            for (int g = 0; g < GT; ++g)
#pragma unroll
                for (int j = 0; j < NJ; ++j) s[g][j] *= scale_log2;
        }
        if (!full) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (tok0 + j * TPL + rgrp >= c_end) {
#pragma unroll
                    for (int g = 0; g < GT; ++g) s[g][j] = -INFINITY;
                }
            }
        }
        float alpha[GT];
        bool grew = false;
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            float mx = s[g][0];
#pragma unroll
            for (int j = 1; j < NJ; ++j) mx = fmaxf(mx, s[g][j]);
            const float m_new = fmaxf(m_run[g], mx);
            grew |= m_new > m_run[g];
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            alpha[g] = fast_exp2(m_run[g] - m_safe);
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                s[g][j] = fast_exp2(s[g][j] - m_safe);
                psum += s[g][j];
            }
            l_run[g] = l_run[g] * alpha[g] + psum;
            m_run[g] = m_new;
        }
        if (__builtin_amdgcn_ballot_w64(grew) != 0) {   // rescale only when some lane's maximum moved
#pragma unroll
            for (int g = 0; g < GT; ++g)
#pragma unroll
                for (int e = 0; e < EPL; ++e) acc[g][e] *= alpha[g];
        }
        if (FP8) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const f32x2_t f01 = __builtin_amdgcn_cvt_pk_f32_fp8(kt.v[j][w], false);
                    const f32x2_t f23 = __builtin_amdgcn_cvt_pk_f32_fp8(kt.v[j][w], true);
#pragma unroll
                    for (int g = 0; g < GT; ++g) {
                        acc[g][4 * w + 0] += s[g][j] * f01.x;
                        acc[g][4 * w + 1] += s[g][j] * f01.y;
                        acc[g][4 * w + 2] += s[g][j] * f23.x;
                        acc[g][4 * w + 3] += s[g][j] * f23.y;
                    }
                }
        } else if (PVDOT) {
            // pair rows (j, j+1): one v_dot2 does two tokens; p is rounded to the cache dtype first,
            // as the reference does before its second dot (flash_decode.py:230).
#pragma unroll
            for (int j = 0; j < NJ; j += 2) {
                uint32_t pp[GT];
#pragma unroll
                for (int g = 0; g < GT; ++g) pp[g] = P2::pack(s[g][j], s[g][j + 1]);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t a = kt.v[j][w], c = kt.v[j + 1][w];
                    const uint32_t lo2 = __builtin_amdgcn_perm(c, a, 0x05040100u);
                    const uint32_t hi2 = __builtin_amdgcn_perm(c, a, 0x07060302u);
#pragma unroll
                    for (int g = 0; g < GT; ++g) {
                        acc[g][2 * w] = P2::dot2(lo2, pp[g], acc[g][2 * w]);
                        acc[g][2 * w + 1] = P2::dot2(hi2, pp[g], acc[g][2 * w + 1]);
                    }
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float lo = P2::lo(kt.v[j][w]), hi = P2::hi(kt.v[j][w]);
#pragma unroll
                    for (int g = 0; g < GT; ++g) {
                        acc[g][2 * w] += s[g][j] * lo;
                        acc[g][2 * w + 1] += s[g][j] * hi;
                    }
                }
        }
    };

    // ---- software pipeline: loads one tile ahead, page ids two tiles ahead ----------------------
    {
        KvTile<FP8> ta, tb;
        PageIds ra, rb;
        int t = wave;
        if (t < n_tiles) {
            pages_of(t, ra);
            issue(t, ra, ta);
        }
        if (t + kWavesPerWg < n_tiles) pages_of(t + kWavesPerWg, rb);
        while (t < n_tiles) {
            if (t + kWavesPerWg < n_tiles) issue(t + kWavesPerWg, rb, tb);
            if (t + 2 * kWavesPerWg < n_tiles) pages_of(t + 2 * kWavesPerWg, ra);
            consume(t, ta);
            t += kWavesPerWg;
            if (t >= n_tiles) break;
            if (t + kWavesPerWg < n_tiles) issue(t + kWavesPerWg, ra, ta);
            if (t + 2 * kWavesPerWg < n_tiles) pages_of(t + 2 * kWavesPerWg, rb);
            consume(t, tb);
            t += kWavesPerWg;
        }
    }

    // ---- merge the row groups of this wave -------------------------------------------------------
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        float mw = m_run[g];
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) mw = fmaxf(mw, __shfl_xor(mw, o, 64));
        const float mw_safe = (mw == -INFINITY) ? 0.f : mw;
        const float sc = fast_exp2(m_run[g] - mw_safe);
        float lw = l_run[g] * sc;
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) lw += __shfl_xor(lw, o, 64);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            float a = acc[g][e] * sc;
#pragma unroll
            for (int o = LPR; o < 64; o <<= 1) a += __shfl_xor(a, o, 64);
            acc[g][e] = a;
        }
        m_run[g] = mw;
        l_run[g] = lw;
    }

    // ---- merge the four waves through LDS ---------------------------------------------------------
    __shared__ float sm_o[kWavesPerWg][GT][kHeadDim];
    __shared__ float sm_m[kWavesPerWg][GT];
    __shared__ float sm_l[kWavesPerWg][GT];
    if (rgrp == 0) {
#pragma unroll
        for (int g = 0; g < GT; ++g)
#pragma unroll
            for (int e = 0; e < EPL; ++e) sm_o[wave][g][piece * EPL + e] = acc[g][e];
        if (piece == 0) {
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                sm_m[wave][g] = m_run[g];
                sm_l[wave][g] = l_run[g];
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < heads_here * kHeadDim; idx += 256) {
        const int g = idx / kHeadDim, d = idx % kHeadDim;
        float mx = sm_m[0][g];
#pragma unroll
        for (int w = 1; w < kWavesPerWg; ++w) mx = fmaxf(mx, sm_m[w][g]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < kWavesPerWg; ++w) {
            const float sc = fast_exp2(sm_m[w][g] - mx);   // mx is finite: the chunk holds >= 1 token
            o += sm_o[w][g][d] * sc;
            l += sm_l[w][g] * sc;
        }
        const float res = o * vscale / l;
        const int hq = head0 + g;
        const float lse_nat = (mx + fast_log2(l)) * kLn2;
        if (p.direct) {
            store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + d, res, p.out_dtype);
            if (d == 0) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse_nat;
                if (p.pack_lse)
                    store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + kHeadDim, lse_nat,
                              p.out_dtype);
            }
        } else {
            const int64_t row = ((int64_t)b * p.hq + hq) * p.num_splits + split;
            p.part_o[row * kHeadDim + d] = res;
            if (d == 0) p.part_lse[row] = lse_nat;
        }
    }
}

template <int QDT, bool FP8, int GT>
int launch_gt(const SplitParams& p, hipStream_t stream) {
    using G_ = Geo<FP8>;
    const bool punif = (p.page_size % G_::TPL) == 0;
    const dim3 grid((unsigned)((int64_t)p.batch * p.num_splits * p.hkv * p.head_tiles));
    const dim3 block(256);
    if (punif) {
        hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, true, true>), grid, block, 0, stream, p);
    } else {
        hipLaunchKernelGGL((splitkv_valu_kernel<QDT, FP8, GT, false, true>), grid, block, 0, stream, p);
    }
    return (int)hipGetLastError();
}

template <int QDT, bool FP8>
int launch_dt(const SplitParams& p, hipStream_t stream) {
    switch (valu_heads_per_wg(p.group)) {
        case 1: return launch_gt<QDT, FP8, 1>(p, stream);
        case 2: return launch_gt<QDT, FP8, 2>(p, stream);
        case 4: return launch_gt<QDT, FP8, 4>(p, stream);
        default: return launch_gt<QDT, FP8, 8>(p, stream);
    }
}

}  // namespace

int valu_heads_per_wg(int group) {
    if (group <= 1) return 1;
    if (group <= 2) return 2;
    if (group <= 4) return 4;
    return 8;
}

bool valu_supported(int q_dtype, int kv_dtype, int /*group*/) {
    if (q_dtype != FDK_BF16 && q_dtype != FDK_FP16) return false;
    return kv_dtype == q_dtype || kv_dtype == FDK_FP8_E4M3;
}

int launch_splitkv_valu(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    const bool fp8 = kv_dtype == FDK_FP8_E4M3;
    if (q_dtype == FDK_BF16) return fp8 ? launch_dt<FDK_BF16, true>(p, stream) : launch_dt<FDK_BF16, false>(p, stream);
    return fp8 ? launch_dt<FDK_FP16, true>(p, stream) : launch_dt<FDK_FP16, false>(p, stream);
}

}  // namespace fdk
