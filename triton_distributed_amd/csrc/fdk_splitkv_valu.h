// Split-KV paged GQA decode, vector-ALU path (v_dot2 + FMA), gfx950: kernel template.
//
// Counterpart of kernel_gqa_fwd_batch_decode_split_kv in the reference
// (python/triton_dist/kernels/nvidia/flash_decode.py:129-239): online softmax in fp32 over one
// split of the KV range, per-split normalised partial output and lse = m + ln(l).  Differences by
// design: splits are fixed-length token chunks (ragged batches give equal work items), page
// arithmetic is 64-bit, an empty chunk writes nothing (the combine derives the live split count
// from kv_len), and with a single split the final (out, lse) is written directly.
//
// Work decomposition.  A 16-byte load per lane covers 1 KB per wavefront: NG = 64/LPR groups of
// LPR lanes, one group per 256-byte (bf16) or 128-byte (fp8) row of one kv head.  A load spans HS
// adjacent kv heads of TPL = NG/HS consecutive tokens, i.e. 1 KB of contiguous cache memory when
// the heads of a token are contiguous.  The wavefronts of a workgroup split the kv heads into
// head groups of HS heads and, where head groups are fewer than wavefronts, interleave tokens, so
// that a workgroup as a whole streams whole token rows (all kv heads) in address order - the
// pattern that keeps DRAM pages open.  HS = 1 is the layout-agnostic fallback: one kv head per
// workgroup, wavefronts interleave 4-token loads.
//
// Each lane group keeps its own running (m, l, acc) for the rows it sees; lane groups of the same
// kv head and the wavefronts that share a head group are merged once at the end (shuffles, LDS).
// Loads run one tile ahead of the arithmetic; page ids one tile further.
#pragma once

#include "fdk_device.h"

namespace fdk {
namespace valu {

enum PageMode {
    PM_TILE = 0,      // page_size is a power of two and a multiple of the workgroup tile: one lookup per tile
    PM_LOAD = 1,      // power of two, multiple of TPL: one (wave-uniform) lookup per load
    PM_LANE = 2,      // power of two: every lane looks up its own row
    PM_LANE_DIV = 3   // any page size: per-lane lookup with an integer division
};

template <bool FP8>
struct Geo {
    static constexpr int EPL = FP8 ? 16 : 8;        // cache elements per lane per 16-byte load
    static constexpr int LPR = kHeadDim / EPL;      // lanes per row
    static constexpr int NG = kWaveSize / LPR;      // rows per wave load
    static constexpr int QW = EPL / 2;              // q dwords per lane and head
    static constexpr int ES = FP8 ? 1 : 2;          // cache element size
};

constexpr int NJ = 4;                               // loads per tile and tensor

struct KvTile {
    uint32_t k[NJ][4];
    uint32_t v[NJ][4];
};

__device__ __forceinline__ void put(uint32_t (&dst)[4], const uint4 x) {
    dst[0] = x.x;
    dst[1] = x.y;
    dst[2] = x.z;
    dst[3] = x.w;
}

template <bool B> struct BoolTag { static constexpr bool value = B; };

template <int QDT, bool FP8, int GT, int HS, int PM>
__global__ __launch_bounds__(512) void splitkv_valu_kernel(const SplitParams p) {
    using G_ = Geo<FP8>;
    using P2 = Pack2<QDT>;
    constexpr int EPL = G_::EPL, LPR = G_::LPR, NG = G_::NG, QW = G_::QW, ES = G_::ES;
    constexpr int TPL = NG / HS;                    // tokens per wave load
    static_assert(NG % HS == 0, "HS must divide the rows of a load");

    extern __shared__ float smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = p.wavefronts;                    // (= blockDim.x / 64; see SplitParams)
    const int piece = lane % LPR;
    const int lgrp = lane / LPR;
    const int hh = lgrp % HS;                       // kv head within the head group
    const int a = lgrp / HS;                        // token within the load
    const int nhg = p.hg_per_wg;                    // head groups per workgroup (1, 2 or 4 .. nw)
    const int ti_n = nw / nhg;                      // wavefronts interleaving tokens of one head group
    const int hgl = wave % nhg;
    const int ti = wave / nhg;

    // workgroup -> (sequence, split, head-group block, q-head tile); innermost indices vary fastest
    int wg = blockIdx.x;
    const int ht = wg % p.head_tiles;
    wg /= p.head_tiles;
    const int hgb = wg % p.hg_blocks;
    wg /= p.hg_blocks;
    const int split = wg % p.num_splits;
    const int b = wg / p.num_splits;
    const int kvh = (hgb * nhg + hgl) * HS + hh;    // this lane's kv head
    const int head0 = kvh * p.group + ht * GT;      // first q head of this lane
    const int heads_here = min(GT, p.group - ht * GT);

    // Length feedback (set only where this kernel is the last of the call: a single pass), stored where the first
    // workgroup LEAVES the kernel: a store in front of the loop would make the compiler assume that block_table and
    // kv_lens may have changed, and read them with vector loads in the loop (measured: 83 -> 103 us per launch).
    auto store_feedback = [&]() {
        if (p.length_feedback && blockIdx.x == 0 && wave == 0)
            store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
    };

    const int kv_len = min(p.kv_lens[b], p.max_tokens);
    const int c_start = split * p.chunk;
    if (c_start >= kv_len) {
        if (p.direct) {   // kv_len == 0 with a single split: defined result, no combine follows
            const int kv_heads_here = nhg * HS;
            for (int idx = threadIdx.x; idx < kv_heads_here * heads_here * kHeadDim; idx += 64 * nw) {
                const int d = idx % kHeadDim, g = (idx / kHeadDim) % heads_here, kh = idx / (kHeadDim * heads_here);
                const int hq = (hgb * kv_heads_here + kh) * p.group + ht * GT + g;
                store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + d, 0.f, p.out_dtype);
                if (d == 0) {
                    if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = -INFINITY;
                    if (p.pack_lse)
                        store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + kHeadDim, -INFINITY,
                                  p.out_dtype);
                }
            }
        }
        store_feedback();
        return;
    }
    // the last split runs to the end of the sequence (see the matrix-core kernel)
    const int c_end = split == p.num_splits - 1 ? kv_len : min(c_start + p.chunk, kv_len);
    const int tile_tokens = NJ * ti_n * TPL;        // tokens one workgroup tile covers
    const int n_full = (c_end - c_start) / tile_tokens;
    const bool has_tail = (c_end - c_start) % tile_tokens != 0;

    // ---- q: per head, the EPL elements that match this lane's piece of the row ------------------
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
    const bool softcap = p.soft_cap > 0.f;
    const float inv_cap = softcap ? 1.0f / p.soft_cap : 0.f;

    // per-lane row bases: kv head, piece of the row, and this lane's token offset inside a tile
    const int tok_in_tile0 = ti * TPL + a;          // token offset of load j=0; load j adds j*ti_n*TPL
    const char* kbase = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES + piece * 16;
    const char* vbase = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES + piece * 16;
    const int32_t* tbl = p.block_table + (int64_t)b * p.tbl_sb;
    const int pmask = p.page_size - 1;

    struct PageIds { int32_t pg[PM == PM_TILE ? 1 : NJ]; };

    // page ids of tile T (tokens past the chunk are never loaded; the lookup is clamped into range)
    auto pages_of = [&](int T, PageIds& pi) {
        const int tok0 = c_start + T * tile_tokens;
        if (PM == PM_TILE) {
            pi.pg[0] = tbl[tok0 >> p.page_shift];
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * ti_n * TPL + ti * TPL;
                if (PM >= PM_LANE) n += a;
                n = min(n, c_end - 1);
                pi.pg[PM == PM_TILE ? 0 : j] = tbl[PM == PM_LANE_DIV ? n / p.page_size : n >> p.page_shift];
            }
        }
    };
    auto row_ptrs = [&](int T, const PageIds& pi, const char* (&kp)[NJ], const char* (&vp)[NJ]) {
        const int tok0 = c_start + T * tile_tokens;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int n = tok0 + j * ti_n * TPL + tok_in_tile0;
            const int slot = PM == PM_LANE_DIV ? n % p.page_size : (n & pmask);
            const int64_t pg = pi.pg[PM == PM_TILE ? 0 : j];
            kp[j] = kbase + (pg * p.k_sp + (int64_t)slot * p.k_st) * ES;
            vp[j] = vbase + (pg * p.v_sp + (int64_t)slot * p.v_st) * ES;
        }
    };
    auto issue = [&](int T, const PageIds& pi, KvTile& kt) {
        const char* kp[NJ];
        const char* vp[NJ];
        row_ptrs(T, pi, kp, vp);
#pragma unroll
        for (int j = 0; j < NJ; ++j) put(kt.k[j], load_stream16(kp[j]));
#pragma unroll
        for (int j = 0; j < NJ; ++j) put(kt.v[j], load_stream16(vp[j]));
    };
    auto issue_masked = [&](int T, const PageIds& pi, KvTile& kt) {
        const char* kp[NJ];
        const char* vp[NJ];
        row_ptrs(T, pi, kp, vp);
        const int tok0 = c_start + T * tile_tokens;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint4 kk = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
            if (tok0 + j * ti_n * TPL + tok_in_tile0 < c_end) {
                kk = load_stream16(kp[j]);
                vv = load_stream16(vp[j]);
            }
            put(kt.k[j], kk);
            put(kt.v[j], vv);
        }
    };

    // ---- running state of this lane group ----------------------------------------------------------
    float m_run[GT], l_run[GT], acc[GT][EPL];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        m_run[g] = -INFINITY;
        l_run[g] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
    }

    auto consume = [&](int T, const KvTile& kt, auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
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
                    kk[(2 * w) % QW] = P2::pack(f01.x * kscale, f01.y * kscale);
                    kk[(2 * w + 1) % QW] = P2::pack(f23.x * kscale, f23.y * kscale);
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
                    s[g][j] = soft_cap_fn(s[g][j] * p.sm_scale, p.soft_cap, inv_cap) * kLog2e;
        } else {
#pragma unroll
            for (int g = 0; g < GT; ++g)
#pragma unroll
                for (int j = 0; j < NJ; ++j) s[g][j] *= p.scale_log2;
        }
        if (MASKED) {
            const int tok0 = c_start + T * tile_tokens;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if (tok0 + j * ti_n * TPL + tok_in_tile0 >= c_end) {
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
            const float m_safe = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
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
                        acc[g][(4 * w + 0) % EPL] += s[g][j] * f01.x;
                        acc[g][(4 * w + 1) % EPL] += s[g][j] * f01.y;
                        acc[g][(4 * w + 2) % EPL] += s[g][j] * f23.x;
                        acc[g][(4 * w + 3) % EPL] += s[g][j] * f23.y;
                    }
                }
        } else {
            // pair rows (j, j+1): one v_dot2 does two tokens; p is rounded to the cache dtype first,
            // as the reference does before its second dot (flash_decode.py:230).
#pragma unroll
            for (int j = 0; j < NJ; j += 2) {
                uint32_t pp[GT];
#pragma unroll
                for (int g = 0; g < GT; ++g) pp[g] = P2::pack(s[g][j], s[g][j + 1]);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t x = kt.v[j][w], y = kt.v[j + 1][w];
                    const uint32_t lo2 = __builtin_amdgcn_perm(y, x, 0x05040100u);
                    const uint32_t hi2 = __builtin_amdgcn_perm(y, x, 0x07060302u);
#pragma unroll
                    for (int g = 0; g < GT; ++g) {
                        acc[g][(2 * w) % EPL] = P2::dot2(lo2, pp[g], acc[g][(2 * w) % EPL]);
                        acc[g][(2 * w + 1) % EPL] = P2::dot2(hi2, pp[g], acc[g][(2 * w + 1) % EPL]);
                    }
                }
            }
        }
    };

    // ---- software pipeline over the full tiles: loads one tile ahead, page ids one more ------------
    // The steady-state loop always issues before it consumes, and the last one or two tiles are
    // straight-line code: every consume then sees a fixed number of loads in flight behind its own,
    // so its waits can be partial (a conditional issue would force a wait for the prefetch as well).
    {
        KvTile ta, tb;
        PageIds pid;
        int T = 0;
        if (n_full > 0) {
            pages_of(0, pid);
            issue(0, pid, ta);
            if (n_full > 1) pages_of(1, pid);
        }
        while (T + 2 < n_full) {
            issue(T + 1, pid, tb);
            pages_of(T + 2, pid);
            consume(T, ta, BoolTag<false>());
            issue(T + 2, pid, ta);
            if (T + 3 < n_full) pages_of(T + 3, pid);
            consume(T + 1, tb, BoolTag<false>());
            T += 2;
        }
        if (n_full - T == 2) {
            issue(T + 1, pid, tb);
            consume(T, ta, BoolTag<false>());
            consume(T + 1, tb, BoolTag<false>());
        } else if (n_full - T == 1) {
            consume(T, ta, BoolTag<false>());
        }
        if (has_tail) {
            pages_of(n_full, pid);
            issue_masked(n_full, pid, ta);
            consume(n_full, ta, BoolTag<true>());
        }
    }

    // ---- merge the lane groups of this wave that share a kv head (TPL > 1) -------------------------
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        float mw = m_run[g];
#pragma unroll
        for (int o = LPR * HS; o < 64; o <<= 1) mw = fmaxf(mw, __shfl_xor(mw, o, 64));
        const float mw_safe = (mw == -INFINITY) ? 0.f : mw;
        const float sc = fast_exp2(m_run[g] - mw_safe);
        float lw = l_run[g] * sc;
#pragma unroll
        for (int o = LPR * HS; o < 64; o <<= 1) lw += __shfl_xor(lw, o, 64);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            float x = acc[g][e] * sc;
#pragma unroll
            for (int o = LPR * HS; o < 64; o <<= 1) x += __shfl_xor(x, o, 64);
            acc[g][e] = x;
        }
        m_run[g] = mw;
        l_run[g] = lw;
    }

    // ---- merge the wavefronts that share a head group (ti_n of them, a power of two) -----------------
    // 1. publish (m, l); every wave rescales its accumulators to the common maximum; 2. tree-sum the
    // accumulators through LDS, halving the number of live waves per round (fixed order: deterministic).
    float* sm_m = smem;                                  // [nw][HS][GT]
    float* sm_l = smem + nw * HS * GT;                   // [nw][HS][GT]
    float* sm_o = smem + 2 * nw * HS * GT;               // [nw/2][HS][GT][128]
    float l_tot[GT];
    if (ti_n > 1) {
        if (a == 0 && piece == 0) {
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                sm_m[(wave * HS + hh) * GT + g] = m_run[g];
                sm_l[(wave * HS + hh) * GT + g] = l_run[g];
            }
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            float mx = -INFINITY;
            for (int t = 0; t < ti_n; ++t) mx = fmaxf(mx, sm_m[((hgl + nhg * t) * HS + hh) * GT + g]);
            float l = 0.f;                               // mx is finite: the chunk holds >= 1 token
            for (int t = 0; t < ti_n; ++t) {
                const int w = hgl + nhg * t;
                l += sm_l[(w * HS + hh) * GT + g] * fast_exp2(sm_m[(w * HS + hh) * GT + g] - mx);
            }
            const float sc = fast_exp2(m_run[g] - mx);
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[g][e] *= sc;
            m_run[g] = mx;
            l_tot[g] = l;
        }
        for (int half = ti_n >> 1; half >= 1; half >>= 1) {
            if (ti >= half && ti < 2 * half && a == 0) {
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    float* dst = sm_o + ((((ti - half) * nhg + hgl) * HS + hh) * GT + g) * kHeadDim + piece * EPL;
#pragma unroll
                    for (int e4 = 0; e4 < EPL / 4; ++e4)
                        *reinterpret_cast<float4*>(dst + 4 * e4) =
                            make_float4(acc[g][4 * e4], acc[g][4 * e4 + 1], acc[g][4 * e4 + 2], acc[g][4 * e4 + 3]);
                }
            }
            __syncthreads();
            if (ti < half && a == 0) {
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    const float* src = sm_o + (((ti * nhg + hgl) * HS + hh) * GT + g) * kHeadDim + piece * EPL;
#pragma unroll
                    for (int e4 = 0; e4 < EPL / 4; ++e4) {
                        const float4 x = *reinterpret_cast<const float4*>(src + 4 * e4);
                        acc[g][4 * e4] += x.x;
                        acc[g][4 * e4 + 1] += x.y;
                        acc[g][4 * e4 + 2] += x.z;
                        acc[g][4 * e4 + 3] += x.w;
                    }
                }
            }
            __syncthreads();
        }
    } else {
#pragma unroll
        for (int g = 0; g < GT; ++g) l_tot[g] = l_run[g];
    }

    // ---- the first wave of every head group writes its rows: lane (hh, piece) holds EPL columns ----
    if (ti == 0 && a == 0) {
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            if (g < heads_here) {
                const int hq = head0 + g;
                const float inv = vscale / l_tot[g];
                const float lse_nat = (m_run[g] + fast_log2(l_tot[g])) * kLn2;
                if (p.direct) {
                    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) store_out(p.out, ob + piece * EPL + e, acc[g][e] * inv, p.out_dtype);
                    if (piece == 0) {
                        if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse_nat;
                        if (p.pack_lse) store_out(p.out, ob + kHeadDim, lse_nat, p.out_dtype);
                    }
                } else {
                    const int64_t row = ((int64_t)b * p.hq + hq) * p.num_splits + split;
                    float* dst = p.part_o + row * kHeadDim + piece * EPL;
#pragma unroll
                    for (int e4 = 0; e4 < EPL / 4; ++e4)
                        *reinterpret_cast<float4*>(dst + 4 * e4) =
                            make_float4(acc[g][4 * e4] * inv, acc[g][4 * e4 + 1] * inv, acc[g][4 * e4 + 2] * inv,
                                        acc[g][4 * e4 + 3] * inv);
                    if (piece == 0) p.part_lse[row] = lse_nat;
                }
            }
        }
    }
    store_feedback();
}

// Kernel geometry chosen on the host for one launch.
struct ValuGeometry {
    int hs;          // kv heads per wave load (template HS)
    int hg_per_wg;   // head groups per workgroup
    int hg_blocks;   // workgroups along the kv-head axis
    int nwaves;      // wavefronts per workgroup
    int gt;          // q heads per kv head handled by one workgroup (template GT)
    int head_tiles;
};

ValuGeometry choose_geometry(const SplitParams& p, int kv_dtype);

template <int QDT, bool FP8>
int launch_typed(const SplitParams& p, const ValuGeometry& geo, hipStream_t stream);

}  // namespace valu
}  // namespace fdk
