// Split-KV paged GQA decode, matrix-core path, gfx950: the kernel template (one translation unit per head
// dimension instantiates it).
//
// Same contract as the vector-ALU kernel (fdk_splitkv_valu.h) and the same counterpart in the reference
// (kernel_gqa_fwd_batch_decode_split_kv, python/triton_dist/kernels/nvidia/flash_decode.py:129-239, which
// pads the q-head group to a 16-row tile for its tl.dot, :170-176).  A workgroup of four or eight wavefronts
// works on pieces: a token range of one sequence for a block of 1, 2, 4 or 8 adjacent kv heads and a tile of 16
// q heads.  Each wavefront owns one kv head; the wavefronts of a workgroup together stream runs of adjacent
// heads of every token (all heads of a token are adjacent in the cache), which is worth ~8% of bandwidth over
// workgroups reading one head each.  With fewer kv heads than wavefronts, the wavefronts of a head interleave
// 16-token tiles and are merged through LDS at the end.  How pieces are handed out (one per workgroup, from a
// queue, or as equal shares of the whole batch) is described at the end of the kernel.
//
// Per tile and wavefront:
//   global -> registers   coalesced 16-byte loads, each instruction reads whole cache rows (head_dim 128: four
//                          256-byte bf16 rows or eight 128-byte fp8 rows); a tile's loads are in flight while
//                          the previous tile is computed.  Rows
//                          past the end of the chunk are clamped to the last valid row, so every load is in
//                          bounds and finite.
//   registers -> LDS       a private scratch per wavefront (64 x head_dim bytes), XOR-swizzled in 16-byte chunks; fp8 is
//                          dequantised to the q dtype on the way (K as round(k8*scale), V exactly)
//   S^T = K Q^T            head_dim/32 x v_mfma_f32_16x16x32 (A = K rows read back as ds_read_b128, B = Q^T kept in
//                          registers); lane (h, a) then holds the logits of head h for tokens 4a..4a+3
//   online softmax         fp32, running max shared by the four lane groups of a head
//   O^T += V^T P^T         head_dim/16 x v_mfma_f32_16x16x16 (A = V^T through the LDS transpose read
//                          ds_read_b64_tr_b16, B = P^T taken straight from the softmax registers)
#pragma once

#include "fdk_device.h"

namespace fdk {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// Timeline build (-DFDK_TIMELINE, a second library for measurements only; the product library has none of this): every
// wavefront leaves eight int64 at p.timeline[8 * (linear workgroup * wavefronts + wavefront)] - the 100 MHz constant
// clock at kernel entry, before the first K/V loads of its last piece, after that piece's last tile and after its
// merge and stores (0 if the wavefront left earlier), then the XCD it ran on, the kv head, the sequence and the
// linear workgroup index.  In that build p.timeline_rotate = r makes workgroup x of a sequence take head block
// (x + r) mod (head blocks) instead of x (chunk mode and single pass, one q-head tile): which XCD reads which head's
// rows then changes, the rows themselves do not.
#ifdef FDK_TIMELINE
#define FDK_STAMP(i) ts[i] = (long long)__builtin_amdgcn_s_memrealtime()
#else
#define FDK_STAMP(i) ((void)0)
#endif
typedef const __attribute__((address_space(4))) int32_t* ConstI32;     // read-only for the whole kernel
__device__ __forceinline__ ConstI32 as_const(const int32_t* p) { return (ConstI32)(uintptr_t)p; }

enum PageMode { PM_TILE = 0, PM_LOAD = 1, PM_LANE = 2, PM_LANE_DIV = 3 };
template <bool B> struct BoolTag { static constexpr bool value = B; };
template <int N> struct IntTag { static constexpr int value = N; };

constexpr int kTile = 16;                 // tokens per tile
constexpr int kGranule = kBalanceGranule; // balanced mode: tokens per unit of the partition

template <int QDT> struct Mma;
template <> struct Mma<FDK_BF16> {
    static __device__ __forceinline__ f32x4_t qk(uint4 a, uint4 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t pv(uint2 a, uint2 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint2 read_tr(const char* p) {
        return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4_t, p)));
    }
};
template <> struct Mma<FDK_FP16> {
    static __device__ __forceinline__ f32x4_t qk(uint4 a, uint4 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t pv(uint2 a, uint2 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint2 read_tr(const char* p) {
        return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4_t, p)));
    }
};

// byte offset of 16-byte chunk `c` of row `r` inside a staged tile of 16 rows x RB bytes (RB = 2 D >= 128)
template <int RB> __device__ __forceinline__ int k_off(int r, int c) { return r * RB + ((c ^ (r & 7)) << 4); }
template <int RB> __device__ __forceinline__ int v_off(int r, int c) { return r * RB + ((c ^ ((r & 3) << 1)) << 4); }

template <bool FP8, int D>
struct Regs {                                  // one tile in registers, as loaded
    static constexpr int LPR = D * (FP8 ? 1 : 2) / 16;   // lanes (16-byte pieces) per cache row
    static constexpr int RPL = 64 / LPR;                 // rows per load instruction
    static constexpr int NJ = kTile / RPL;               // load instructions per tensor and tile
    uint32_t k[NJ][4];
    uint32_t v[NJ][4];
};

__device__ __forceinline__ void put(uint32_t (&dst)[4], const uint4 x) {
    dst[0] = x.x;
    dst[1] = x.y;
    dst[2] = x.z;
    dst[3] = x.w;
}
__device__ __forceinline__ uint4 get(const uint32_t (&src)[4]) { return make_uint4(src[0], src[1], src[2], src[3]); }

// ---- partial rows that another workgroup of the same launch merges (fused combine) ----------------------------
// The L2 caches of the eight XCDs are not coherent with each other.  Rows that cross workgroups are therefore
// written and read with relaxed atomic accesses of agent scope (write-through stores, loads that do not hit
// stale lines), which need no cache write-back or invalidation; the order "rows, then ticket" is enforced by
// waiting for the stores before the ticket is drawn (ticket_arrive).
__device__ __forceinline__ void st_agent2(float* p, float a, float b) {
    const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, a) | ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent1(float* p, float a) {
    __hip_atomic_store(p, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Where the pieces of an output row are: piece s of (kv head hl of the block, head g of the tile) is partial row
// base + s * piece_step + hl * hl_step + g * g_step; `live` pieces exist (each holds at least one token).
struct MergeRows {
    int64_t base, piece_step, hl_step, g_step;
    int live;
};

// Log-sum-exp merge of the live pieces of up to NR output rows by one wavefront.  The rows go together so that
// their loads are under way at the same time: a lane per piece loads the lse values, D / 4 lanes load a piece's row
// 16 bytes each (64 / (D / 4) pieces per instruction), and the first batch of rows is requested before the
// weights are known.  The loads bypass this XCD's L2 (sc1): the rows were written by workgroups on any XCD.
template <int D, int NR>
__device__ __forceinline__ void merge_rows(const SplitParams& p, const int64_t (&row0)[NR], const int (&hq)[NR], const int nrows,
                                           const int64_t piece_step, const int live, const int b, const int lane) {
    constexpr int LPR = D / 4;              // lanes per partial row
    constexpr int PPI = 64 / LPR;           // pieces per load instruction
    constexpr int NB = 8;                   // load instructions per row and batch
    constexpr int kSc1 = 16;                // cache policy of the buffer loads: agent scope
    const int sub = lane / LPR, col = lane % LPR;
    const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(p.part_o, 0, (int)p.ws_bytes, 0x00020000);
    const uint32_t lse_base = (uint32_t)((p.part_lse - p.part_o) * 4);
    const uint32_t o_step = (uint32_t)(piece_step * D * 4), l_step = (uint32_t)(piece_step * 4);
    f32x4_t acc[NR];
    float m_run[NR], l_run[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        acc[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
    }
    for (int s0 = 0; s0 < live; s0 += 64) {             // blocks of 64 pieces: a lane per piece for the weights
        const int n = min(64, live - s0);
        float my[NR];
        f32x4_t o[NR][NB];
        auto request = [&](int t0) {                     // rows of pieces s0 + t0 + j * PPI + sub, j < NB
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                if (r < nrows) {
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const int t = t0 + j * PPI + sub;
                        o[r][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                        if (t < n)
                            o[r][j] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                ws, (uint32_t)(s0 + t) * o_step + col * 16, (uint32_t)(row0[r] * D * 4), kSc1));
                    }
                }
            }
        };
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            my[r] = -INFINITY;
            if (r < nrows && lane < n)
                my[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                            ws, (uint32_t)(s0 + lane) * l_step, lse_base + (uint32_t)(row0[r] * 4), kSc1)) * kLog2e;
        }
        request(0);
        float w[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            w[r] = 0.f;
            if (r < nrows) {
                const float m_new = fmaxf(m_run[r], wave_max(my[r]));      // finite: a live piece holds a token
                w[r] = fast_exp2(my[r] - m_new);                           // 0 for idle lanes
                const float alpha = fast_exp2(m_run[r] - m_new);
                l_run[r] = l_run[r] * alpha + wave_sum(w[r]);
                acc[r] *= alpha;
                m_run[r] = m_new;
            }
        }
        for (int t0 = 0; t0 < n; t0 += NB * PPI) {
            if (t0 > 0) request(t0);
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                if (r < nrows) {
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const int t = min(t0 + j * PPI + sub, 63);
                        acc[r] += __shfl(w[r], t, 64) * o[r][j];           // rows past the end were set to zero
                    }
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        if (r < nrows) {
            f32x4_t a = acc[r];
            if (PPI >= 2) {
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] += __shfl_xor(a[i], 32, 64);
            }
            if (PPI >= 4) {
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] += __shfl_xor(a[i], 16, 64);
            }
            const float inv = fast_rcp(l_run[r]);
            const float lse = (m_run[r] + fast_log2(l_run[r])) * kLn2;
            const int64_t ob = (int64_t)b * p.out_sb + (int64_t)hq[r] * p.out_sh;
            if (sub == 0) store_out4(p.out, ob + 4 * col, make_float4(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv), p.out_dtype);
            if (lane == 0) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq[r]] = lse;
                if (p.pack_lse) store_out(p.out, ob + D, lse, p.out_dtype);
            }
        }
    }
}

// PROBE: the load pipeline alone - the same pieces, addresses and load instructions in the same order, but what
// arrives is only folded into a checksum: how fast the memory system serves this call's access pattern.
// MODE: how pieces are handed out - a kernel for each, see "work distribution" below.
enum WorkMode { WM_ONE = 0,     // one piece per workgroup: single pass, per-sequence chunks
                WM_QUEUE = 1,   // chunk mode, a fixed set of workgroups pulls the pieces from a queue
                WM_SHARES = 2 };// balanced mode: equal shares of the whole batch
template <int QDT, bool FP8, int PM, int NBUF, int D, bool PROBE = false, int MODE = WM_ONE>
__global__ __launch_bounds__(512) void splitkv_mfma_kernel(const SplitParams p) {
    constexpr bool BAL = MODE == WM_SHARES;
    using M = Mma<QDT>;
    using P2 = Pack2<QDT>;
    using R = Regs<FP8, D>;
    constexpr int NJ = R::NJ;
    constexpr int LPR = R::LPR;                // lanes per cache row
    constexpr int RPL = R::RPL;                // rows per load instruction
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int RB = 2 * D;                  // bytes of a staged (16-bit) row
    constexpr int KS = D / 32;                 // k-steps of the QK product
    constexpr int DB = D / 16;                 // 16-column blocks of the output
    constexpr int kScratch = 2 * kTile * RB;   // LDS bytes per wavefront: K tile + V tile; also 16 fp32 output rows

#ifdef FDK_TIMELINE
    long long ts[4] = {0, 0, 0, 0};
#endif
    FDK_STAMP(0);
    extern __shared__ __attribute__((aligned(16))) char lds[];      // [nw][kScratch] then m[nw][16], l[nw][16]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int a = lane >> 4;                   // lane group: MFMA k-group / token group
    const int c = lane & 15;                   // MFMA row/column index
    const int lrow = lane / LPR;               // row of this lane within a load
    const int lpiece = lane % LPR;             // 16-byte piece of the row

    const int nw = p.wavefronts;               // (= blockDim.x / 64; see SplitParams)
    const int nh = p.hg_per_wg;                // kv heads per workgroup
    const int ti_n = nw / nh;                  // wavefronts interleaving the tiles of one kv head
    const int hl = wave % nh;
    const int tix = wave / nh;
    float* sm_m = reinterpret_cast<float*>(lds + nw * kScratch);
    float* sm_l = sm_m + nw * 16;

    int* const s_next = reinterpret_cast<int*>(sm_l + nw * 16);     // next work item (persistent mode)

    // ---- one piece of work: tokens [c_start, min(c_limit, kv_len)) of sequence b for kv-head block hgb and q-head
    // tile ht.  Partial results of head g of the tile go to row prow0 + g * prow_step of the workspace.
    // out = 0, lse = -inf for the q heads [head0, head0 + heads_here) of an empty sequence; one wavefront
    auto write_empty_rows = [&](const int b, const int head0, const int heads_here) {
        for (int idx = lane; idx < heads_here * D; idx += 64) {
            const int g = idx / D, d = idx % D;
            const int64_t ob = (int64_t)b * p.out_sb + (int64_t)(head0 + g) * p.out_sh;
            store_out(p.out, ob + d, 0.f, p.out_dtype);
            if (d == 0) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + head0 + g] = -INFINITY;
                if (p.pack_lse) store_out(p.out, ob + D, -INFINITY, p.out_dtype);
            }
        }
    };

    // With p.fused the workgroup that completes a (sequence, head block, head tile) - the last of its mr.live pieces
    // to draw a ticket - merges the pieces into the final rows; no combine launch follows.
    auto run_piece = [&](const int b, const int hgb, const int ht, const int c_start, const int c_limit,
                         const int64_t prow0, const int prow_step, MergeRows mr) {
    const int kvh = hgb * nh + hl;
    const int head0 = kvh * p.group + ht * 16;
    const int heads_here = min(16, p.group - ht * 16);
#ifdef FDK_TIMELINE
    auto timeline_out = [&]() {
        const int64_t w = ((int64_t)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * nw + wave) * 8;
        if (p.timeline && lane == 0 && w + 8 <= p.timeline_len) {
            long long* o = p.timeline + w;
            o[0] = ts[0]; o[1] = ts[1]; o[2] = ts[2]; o[3] = ts[3];
            o[4] = (long long)(__builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15);        // XCC_ID
            o[5] = kvh; o[6] = b; o[7] = (long long)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));
        }
    };
#endif

    // Issue everything that does not depend on kv_len first, so that the dependent chain before the first K/V
    // load is as short as possible: Q^T (the B operand of S^T = K Q^T: lane (h = c, a) holds
    // q[h][32 ks + 8 a .. +7]; columns past the group repeat its last head - their results are never stored,
    // and nothing waits for a select) and, speculatively, the page of this wave's first tile (any table column
    // may be read; the value is used only if the tile exists).
    uint4 qb[KS];
    {
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)b * p.q_sb +
                             (int64_t)(head0 + min(c, heads_here - 1)) * p.q_sh + 8 * a;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qb[ks] = *reinterpret_cast<const uint4*>(qp + 32 * ks);
    }
    // block_table and kv_lens are never written by this kernel: read through the constant address space, so that
    // wave-uniform reads stay scalar loads on every code path.  (Where a piece follows another in a loop, the
    // compiler otherwise assumes that the previous piece's stores may have changed them and falls back to vector
    // loads, which complete in order with the K/V loads: waiting for a page number then waits for the tile of rows
    // requested before it, and the loop of an fp8 cache ran 20 % slower.)
    const ConstI32 tbl = as_const(p.block_table + (int64_t)b * p.tbl_sb);
    const int pmask = p.page_size - 1;
    struct PageIds { int32_t pg[PM == PM_TILE ? 1 : NJ]; };
    // Page numbers of tile t, for any t: positions are clamped to the table only, not to the sequence, so that
    // nothing here waits for kv_len.  The numbers of positions past the end are never used (a full tile has
    // none; the partial last tile asks again, clamped to its last token).
    auto pages_ahead = [&](int t, PageIds& pi) {
        const int tok0 = c_start + t * kTile;
        if (PM == PM_TILE) {
            pi.pg[0] = tbl[min(tok0, p.max_tokens - 1) >> p.page_shift];
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * RPL;
                if (PM >= PM_LANE) n += lrow;
                n = min(n, p.max_tokens - 1);
                pi.pg[PM == PM_TILE ? 0 : j] = tbl[PM == PM_LANE_DIV ? n / p.page_size : n >> p.page_shift];
            }
        }
    };
    PageIds pa, pb;                        // page numbers of the tiles that go to rg / rb
    pages_ahead(tix, pa);
    pages_ahead(tix + ti_n, pb);
    const int kv_len = min(as_const(p.kv_lens)[b], p.max_tokens);
    if (c_start >= kv_len) {
        // kv_len == 0: a defined result where no combine follows (the first piece writes it)
        if ((p.direct || (p.fused && c_start == 0)) && tix == 0) write_empty_rows(b, head0, heads_here);
        return;
    }
    const int c_end = min(c_limit, kv_len);
    if (!BAL && p.fused) {                                                              // chunks that hold tokens
        const int chunk = chunk_tokens_of(kv_len, p.num_splits, p.chunk, p.chunk_floor);
        mr.live = min(p.num_splits, (kv_len + chunk - 1) / chunk);
    }

    float kscale = 1.f, vscale = 1.f;
    if (FP8) {
        if (p.k_scale) kscale = __builtin_bit_cast(float, as_const(reinterpret_cast<const int32_t*>(p.k_scale))[kvh]);
        if (p.v_scale) vscale = __builtin_bit_cast(float, as_const(reinterpret_cast<const int32_t*>(p.v_scale))[kvh]);
    }
    const bool softcap = p.soft_cap > 0.f;
    const float inv_cap = softcap ? 1.0f / p.soft_cap : 0.f;
    // fp8 K, two forms.  Exact (default): every value becomes round_to_q_dtype(k8 * scale) before the product, i.e. the
    // logits of a decode over the dequantised cache, at two conversions, four multiplications and two packings per
    // four values.  Folded (p.fp8_fold): the values are converted exactly (two instructions per four values) and the
    // head's scale multiplies the logits - (q . k8) * scale instead of q . round(k8 * scale), which differs by the
    // rounding of K to the 16-bit type (relative 2^-9 per element).
    const bool fold = FP8 && p.fp8_fold;
    const float logit_scale_log2 = fold ? p.scale_log2 * kscale : p.scale_log2;
    const float logit_scale = fold ? p.sm_scale * kscale : p.sm_scale;

    const char* kbase = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES + lpiece * 16;
    const char* vbase = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES + lpiece * 16;
    const uint32_t ksp_bytes = (uint32_t)(p.k_sp * ES), vsp_bytes = (uint32_t)(p.v_sp * ES);
    const uint32_t kst_bytes = (uint32_t)(p.k_st * ES), vst_bytes = (uint32_t)(p.v_st * ES);
    char* my_lds = lds + wave * kScratch;
    char* lds_k = my_lds;
    char* lds_v = my_lds + kScratch / 2;

    auto pages_of = [&](int t, PageIds& pi) {        // clamped to the sequence: for the partial last tile
        const int tok0 = c_start + t * kTile;
        if (PM == PM_TILE) {
            pi.pg[0] = tbl[min(tok0, c_end - 1) >> p.page_shift];      // clamped: any tile index may be asked for
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * RPL;
                if (PM >= PM_LANE) n += lrow;
                n = min(n, c_end - 1);
                pi.pg[PM == PM_TILE ? 0 : j] = tbl[PM == PM_LANE_DIV ? n / p.page_size : n >> p.page_shift];
            }
        }
    };
    auto issue = [&](int t, const PageIds& pi, R& rg, auto clamp_tag) {
        const int tok0 = c_start + t * kTile;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            int n = tok0 + j * RPL + lrow;
            if (decltype(clamp_tag)::value) n = min(n, c_end - 1);     // partial tile: always a valid, finite row
            const uint32_t slot = PM == PM_LANE_DIV ? n % p.page_size : (n & pmask);
            // page number x page stride: one 32 x 32 -> 64 bit multiply-add per address (the strides, in bytes, fit
            // 32 bits; a page number is never negative where it is used)
            const uint32_t pg = (uint32_t)pi.pg[PM == PM_TILE ? 0 : j];
            put(rg.k[j], load_stream16(kbase + ((uint64_t)pg * ksp_bytes + (uint64_t)(slot * kst_bytes))));
            put(rg.v[j], load_stream16(vbase + ((uint64_t)pg * vsp_bytes + (uint64_t)(slot * vst_bytes))));
        }
    };

    // PM_TILE: a tile never leaves its page, so a load address is (page base + first slot of the tile), which
    // is wave-uniform, plus a per-lane byte offset that is the same for every full tile.
    // Per-lane byte offsets of the NJ loads.  Up to head_dim 128 they are kept in registers; the widest rows need
    // the registers elsewhere and add a wave-uniform step per load instead (slightly slower).
    constexpr bool kOffsetsInRegs = D <= 128;
    uint32_t koff[kOffsetsInRegs ? NJ : 1], voff[kOffsetsInRegs ? NJ : 1];
#pragma unroll
    for (int j = 0; j < (kOffsetsInRegs ? NJ : 1); ++j) {
        koff[j] = (uint32_t)(((int64_t)(j * RPL + lrow) * p.k_st) * ES + lpiece * 16);
        voff[j] = (uint32_t)(((int64_t)(j * RPL + lrow) * p.v_st) * ES + lpiece * 16);
    }
    const int64_t kstep = (int64_t)RPL * p.k_st * ES;                                 // per load, wave-uniform
    const int64_t vstep = (int64_t)RPL * p.v_st * ES;
    const char* kplane = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES;   // wave-uniform
    const char* vplane = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES;
    auto issue_full = [&](int t, const PageIds& pi, R& rg) {
        if (PM == PM_TILE) {
            const int tok0 = c_start + t * kTile;
            const int64_t pg = pi.pg[0];
            const int slot0 = tok0 & pmask;
            const char* kp = kplane + (pg * p.k_sp + (int64_t)slot0 * p.k_st) * ES;
            const char* vp = vplane + (pg * p.v_sp + (int64_t)slot0 * p.v_st) * ES;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                put(rg.k[j], load_stream16(kOffsetsInRegs ? kp + koff[j] : kp + j * kstep + koff[0]));
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                put(rg.v[j], load_stream16(kOffsetsInRegs ? vp + voff[j] : vp + j * vstep + voff[0]));
        } else {
            issue(t, pi, rg, BoolTag<false>());
        }
    };

    uint32_t sink = 0;                           // PROBE: checksum of everything loaded
    float m_run = -INFINITY, l_run = 0.f;       // for head c; l_run is this lane group's share of the sum
    f32x4_t acc[DB];                             // acc[db][i] = O[h = c][16 db + 4 a + i]
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // registers -> LDS (16-bit elements, swizzled).  Once staged, the registers are free for the next tile's loads.
    auto stage = [&](const R& rg) {
        if (PROBE) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int w = 0; w < 4; ++w) sink ^= rg.k[j][w] ^ rg.v[j][w];
        } else if (FP8) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int r = j * RPL + lrow;
                uint32_t ko[8], vo[8];
                if (fold) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        ko[2 * w] = P2::from_fp8(rg.k[j][w], false);
                        ko[2 * w + 1] = P2::from_fp8(rg.k[j][w], true);
                    }
                } else {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        // K: (k8 * scale) rounded to the q dtype, i.e. the dequantised cache the reference decodes
                        const f32x2_t k01 = __builtin_amdgcn_cvt_pk_f32_fp8(rg.k[j][w], false);
                        const f32x2_t k23 = __builtin_amdgcn_cvt_pk_f32_fp8(rg.k[j][w], true);
                        ko[2 * w] = P2::pack(k01.x * kscale, k01.y * kscale);
                        ko[2 * w + 1] = P2::pack(k23.x * kscale, k23.y * kscale);
                    }
                }
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    // V: exact conversion; its scale multiplies the output once at the end
                    vo[2 * w] = P2::from_fp8(rg.v[j][w], false);
                    vo[2 * w + 1] = P2::from_fp8(rg.v[j][w], true);
                }
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int ch = 2 * lpiece + half;
                    *reinterpret_cast<uint4*>(lds_k + k_off<RB>(r, ch)) =
                        make_uint4(ko[4 * half], ko[4 * half + 1], ko[4 * half + 2], ko[4 * half + 3]);
                    *reinterpret_cast<uint4*>(lds_v + v_off<RB>(r, ch)) =
                        make_uint4(vo[4 * half], vo[4 * half + 1], vo[4 * half + 2], vo[4 * half + 3]);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int r = j * RPL + lrow;
                *reinterpret_cast<uint4*>(lds_k + k_off<RB>(r, lpiece)) = get(rg.k[j]);
                *reinterpret_cast<uint4*>(lds_v + v_off<RB>(r, lpiece)) = get(rg.v[j]);
            }
        }
    };

    auto compute = [&](int t, auto masked_tag) {
        if (PROBE) return;
        constexpr bool MASKED = decltype(masked_tag)::value;
        const int tok0 = c_start + t * kTile;
        // ---- S^T[token][head] = K Q^T ----
        // All LDS reads of the tile are requested up front (K rows, then the transposed V blocks, which do not
        // depend on the softmax): a wavefront is alone on its SIMD in the single-pass plans, so a read that is
        // requested only when its MFMA is due costs its full latency every time (worth 0.5-1 % on 16-bit caches).
        f32x4_t s = {0.f, 0.f, 0.f, 0.f};
        uint4 ka[KS];
        // Not for the widest rows (no registers to spare) nor for fp8 caches (two wavefronts per SIMD already
        // overlap, and the longer register lifetimes cost more than they gain: measured 1 % slower).
        constexpr bool kReadVEarly = D <= 128 && !FP8;
        const int k4 = c >> 2, cc = c & 3;
        const int vrow = 4 * a + k4;
        uint2 va[DB];
        if (kReadVEarly) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) ka[ks] = *reinterpret_cast<const uint4*>(lds_k + k_off<RB>(c, 4 * ks + a));
#pragma unroll
            for (int db = 0; db < DB; ++db) va[db] = M::read_tr(lds_v + v_off<RB>(vrow, 2 * db + (cc >> 1)) + (cc & 1) * 8);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (!kReadVEarly) ka[ks] = *reinterpret_cast<const uint4*>(lds_k + k_off<RB>(c, 4 * ks + a));
            s = M::qk(ka[ks], qb[ks], s);
        }
        // ---- online softmax for head c over tokens 4a .. 4a+3 of this tile ----
        float sv[4] = {s.x, s.y, s.z, s.w};
        if (softcap) {
#pragma unroll
            for (int i = 0; i < 4; ++i) sv[i] = soft_cap_fn(sv[i] * logit_scale, p.soft_cap, inv_cap) * kLog2e;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) sv[i] *= logit_scale_log2;
        }
        if (MASKED) {                         // the partial last tile of the chunk
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (tok0 + 4 * a + i >= c_end) sv[i] = -INFINITY;
        }
        float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));          // finite: token tok0 is valid
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2(m_run - m_new);
        float pr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) pr[i] = fast_exp2(sv[i] - m_new);
        l_run = l_run * alpha + (pr[0] + pr[1]) + (pr[2] + pr[3]);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[db] *= alpha;
        }
        m_run = m_new;
        // P^T as B operand: lane (h = c, a) supplies p for tokens 4a..4a+3, rounded to the cache dtype as the
        // reference does before its second dot (flash_decode.py:230)
        const uint2 pb = make_uint2(P2::pack(pr[0], pr[1]), P2::pack(pr[2], pr[3]));
        // ---- O^T[d][head] += V^T P^T ----
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            if (!kReadVEarly) va[db] = M::read_tr(lds_v + v_off<RB>(vrow, 2 * db + (cc >> 1)) + (cc & 1) * 8);
            acc[db] = M::pv(va[db], pb, acc[db]);
        }
    };

    // ---- pipeline over the full tiles: a tile is copied to LDS as soon as it has arrived, the next tile's
    // loads are issued into the same registers, and the arithmetic on the staged tile overlaps them.  The
    // partial last tile of the chunk goes to the wave whose turn it is.
    // Page numbers run two tiles ahead of the arithmetic.  Per-lane page numbers (vector loads) are requested
    // BEFORE the K/V loads of the tile in between: vector loads complete in order, so a page number requested
    // after a tile's rows could only be used once those rows had arrived, and the tile after them could not be
    // requested while they are under way.  Wave-uniform page numbers (scalar loads) are requested AFTER them:
    // scalar loads complete in any order, so waiting for the older number also waits for the newest request.
    constexpr bool kIdsFirst = PM >= PM_LANE;
    const int n_full = (c_end - c_start) / kTile;
    {
        R rg;
        int t = tix;
        const int st = ti_n;
        FDK_STAMP(1);
        if (t < n_full) issue_full(t, pa, rg);
        if (NBUF == 1) {
            // one register buffer: the next tile's loads go into the registers just staged
            while (t < n_full) {
                if (kIdsFirst) pages_ahead(t + 2 * st, pa);
                stage(rg);
                const int tn = t + st;
                if (tn < n_full) issue_full(tn, pb, rg);
                if (!kIdsFirst) pages_ahead(t + 2 * st, pa);
                compute(t, BoolTag<false>());
                pb = pa;
                t = tn;
            }
        } else {
            // two register buffers: a second tile is requested before the first is staged.  The steady state
            // always issues before it stages, so the waits on the older tile can be partial.
            R rb;
            while (t + 2 * st < n_full) {
                if (kIdsFirst) pages_ahead(t + 2 * st, pa);
                issue_full(t + st, pb, rb);
                if (!kIdsFirst) pages_ahead(t + 2 * st, pa);
                stage(rg);
                compute(t, BoolTag<false>());
                if (kIdsFirst) pages_ahead(t + 3 * st, pb);
                issue_full(t + 2 * st, pa, rg);
                if (!kIdsFirst) pages_ahead(t + 3 * st, pb);
                stage(rb);
                compute(t + st, BoolTag<false>());
                t += 2 * st;
            }
            if (t + st < n_full) {
                issue_full(t + st, pb, rb);
                stage(rg);
                compute(t, BoolTag<false>());
                stage(rb);
                compute(t + st, BoolTag<false>());
            } else if (t < n_full) {
                stage(rg);
                compute(t, BoolTag<false>());
            }
        }
        if (n_full * kTile < c_end - c_start && (n_full % ti_n) == tix) {
            pages_of(n_full, pa);
            issue(n_full, pa, rg, BoolTag<true>());
            stage(rg);
            compute(n_full, BoolTag<true>());
        }
    }

    FDK_STAMP(2);
#ifdef FDK_TIMELINE
    timeline_out();
#endif
    // ---- merge: lane groups (sum of l), then the wavefronts that share a kv head through LDS --------------
    // A wave leaves its accumulators in its own scratch as [column block][lane] float4, i.e. exactly as its lanes
    // hold them: every LDS instruction then touches one contiguous kilobyte.  The waves of a head share the
    // column blocks; lane (h = c, a) of the merging wave reads the same lane slot of every wave's scratch and
    // owns output columns 16 db + 4 a .. + 3 of head h.  Lanes of the padding heads neither write nor read.
    if (PROBE) {                                             // never true for real data; keeps the loads alive
        if (sink == 0x9e3779b9u) *reinterpret_cast<volatile uint32_t*>(p.out ? p.out : (void*)p.part_o) = sink;
        return;
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    const bool live = c < heads_here;
    float4* my_o = reinterpret_cast<float4*>(my_lds);
    if (live) {
#pragma unroll
        for (int db = 0; db < DB; ++db) my_o[db * 64 + lane] = make_float4(acc[db].x, acc[db].y, acc[db].z, acc[db].w);
        if (a == 0) {
            sm_m[wave * 16 + c] = m_run;
            sm_l[wave * 16 + c] = l_run;
        }
    }
    if (ti_n > 1) __syncthreads();                           // ti_n == 1: a wave reads back only its own rows
    if (live) {
        // The merge is written out for each number of wavefronts that share a kv head (1, 2, 4; 8 where tiles
        // are small, see launch_pm): straight-line code keeps all LDS reads of a column block under way together.
        const int hq = head0 + c;
        float lse_nat = 0.f;
        auto merge = [&](auto share_tag) {
            constexpr int TI = decltype(share_tag)::value;
            float mw[TI], lw[TI];
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < TI; ++t) {
                mw[t] = sm_m[(hl + nh * t) * 16 + c];
                lw[t] = sm_l[(hl + nh * t) * 16 + c];
                mx = fmaxf(mx, mw[t]);
            }
            float sc[TI], l = 0.f;
#pragma unroll
            for (int t = 0; t < TI; ++t) {
                sc[t] = fast_exp2(mw[t] - mx);                   // mx is finite: the chunk holds >= 1 token
                l += lw[t] * sc[t];
            }
            const float norm = vscale * fast_rcp(l);
            lse_nat = (mx + fast_log2(l)) * kLn2;
#pragma unroll
            for (int t = 0; t < TI; ++t) sc[t] *= norm;
            for (int db = tix; db < DB; db += TI) {
                float4 x[TI];
#pragma unroll
                for (int t = 0; t < TI; ++t) x[t] = reinterpret_cast<const float4*>(lds + (hl + nh * t) * kScratch)[db * 64 + lane];
                float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int t = 0; t < TI; ++t) {
                    o.x += x[t].x * sc[t];
                    o.y += x[t].y * sc[t];
                    o.z += x[t].z * sc[t];
                    o.w += x[t].w * sc[t];
                }
                const int d0 = 16 * db + 4 * a;
                if (p.direct) {
                    const int64_t ob = (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + d0;
                    store_out4(p.out, ob, o, p.out_dtype);
                } else {
                    float* dst = p.part_o + (prow0 + (int64_t)c * prow_step) * D + d0;
                    if (p.fused) {
                        st_agent2(dst, o.x, o.y);
                        st_agent2(dst + 2, o.z, o.w);
                    } else {
                        *reinterpret_cast<float4*>(dst) = o;
                    }
                }
            }
        };
        constexpr bool kSmallTiles = 2 * kTile * D * (FP8 ? 1 : 2) <= 4096;
        if (ti_n == 1) merge(IntTag<1>());
        else if (ti_n == 2) merge(IntTag<2>());
        else if (ti_n == 4 || !kSmallTiles) merge(IntTag<4>());
        else merge(IntTag<kSmallTiles ? 8 : 4>());
        if (tix == 0 && a == 0) {
            if (p.direct) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse_nat;
                if (p.pack_lse) store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + D, lse_nat, p.out_dtype);
            } else if (p.fused) {
                st_agent1(p.part_lse + prow0 + (int64_t)c * prow_step, lse_nat);
            } else {
                p.part_lse[prow0 + (int64_t)c * prow_step] = lse_nat;
            }
        }
    }
    if (p.fused && !p.direct) {
        // rows first, then the ticket: every wave waits until its stores are done, the barrier collects the
        // waves, one thread draws.  The last piece of the unit to arrive finds live - 1 and merges.
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        int* ticket = p.counters + 2 + (b * p.hg_blocks + hgb) * p.head_tiles + ht;
        if (threadIdx.x == 0)
            s_next[1] = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_next[1] == mr.live - 1) {
            if (threadIdx.x == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            constexpr int NR = 2;                                     // rows a wavefront merges together
            const int n_rows = nh * heads_here;
            for (int r0 = wave * NR; r0 < n_rows; r0 += nw * NR) {
                int64_t row0[NR];
                int hq_of[NR];
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    const int r = min(r0 + i, n_rows - 1);
                    const int rh = r / heads_here, g = r % heads_here;
                    row0[i] = mr.base + rh * mr.hl_step + g * mr.g_step;
                    hq_of[i] = (hgb * nh + rh) * p.group + ht * 16 + g;
                }
                merge_rows<D, NR>(p, row0, hq_of, min(NR, n_rows - r0), mr.piece_step, mr.live, b, lane);
            }
        }
    }
    FDK_STAMP(3);
#ifdef FDK_TIMELINE
    timeline_out();
#endif

    };   // run_piece

    // ---- work distribution --------------------------------------------------------------------------------------
    // Chunk mode: item -> (sequence, split, kv-head block, q-head tile), partial row (b, head, split); one item per
    // workgroup, or (persistent) a fixed set of workgroups that pull items from a queue: counters[0] is its head,
    // counters[1] counts finished workgroups, and the last one to finish puts both back to zero.  The first item
    // of every workgroup is its own index.
    // Balanced mode: the sequences, counted in granules of kGranule tokens and laid end to end, are cut into
    // p.shares (= gridDim.y) equal shares (fewer if there are fewer granules), units = (kv-head block, q-head tile)
    // pairs of a sequence; workgroup (share wc, unit u) = (blockIdx.y, blockIdx.x) works its share off for its unit, sequence
    // by sequence.  Its partial rows for sequence b go to slot (wc + b) * units + u: pieces are ordered by
    // (wc, b) with at least one of the two growing from one piece to the next, so the slot is unique, and the
    // pieces of a sequence occupy consecutive wc.  Neighbouring workgroups read the same tokens of neighbouring
    // heads.  Every wavefront derives the same partition from kv_lens.
    //
    // The modes are kernels of their own (template parameter MODE): the code of one does not get in the way of the
    // others' registers and schedule.  In all of them the FIRST piece of a workgroup - in chunk mode without a queue
    // its only one - runs through straight-line code: that lets the compiler put the piece's first loads ahead of everything that
    // does not feed them.  A loop for the pieces after it is entered only by workgroups that have more (a share that
    // holds the end of one sequence and the beginning of the next; the work queue): what the compiler computes once in
    // front of a loop - several hundred instructions here - would otherwise stand between every workgroup and its
    // first loads (measured in balanced mode: first loads 2.7 us after the start of the kernel instead of 1.9 us).
    if constexpr (MODE == WM_ONE) {
        {
            // grid = (head blocks x head tiles, splits, sequences): the piece follows from the block index without a
            // division, so the table and q loads of the piece can be requested as soon as the arguments are there.
            // (Workgroups are handed out in x-major order: neighbours still read neighbouring heads of the same tokens.)
            const int split = blockIdx.y, pb = blockIdx.z;
            int ht = 0, hgb = blockIdx.x;
#ifdef FDK_TIMELINE
            if (p.head_tiles == 1) hgb = (int)((blockIdx.x + (unsigned)p.timeline_rotate) % (unsigned)p.grid_x);
#endif
            if (p.head_tiles > 1) {
                ht = blockIdx.x % p.head_tiles;
                hgb = blockIdx.x / p.head_tiles;
            }
            // the last split runs to the end of the sequence: a max_kv_len hint that was too small costs balance, not tokens
            const int64_t unit_row0 = ((int64_t)pb * p.hq + hgb * nh * p.group + ht * 16) * p.num_splits;
            // (chunks that follow the sequence's own length: the first table read then waits for kv_lens, one more
            // round trip before the first rows - the price of not needing a length bound from the host)
            int chunk = p.chunk;
            if (p.chunk_floor) chunk = chunk_tokens_of(min(as_const(p.kv_lens)[pb], p.max_tokens), p.num_splits, p.chunk, p.chunk_floor);
            run_piece(pb, hgb, ht, split * chunk, split == p.num_splits - 1 ? p.max_tokens : split * chunk + chunk,
                      unit_row0 + (int64_t)hl * p.group * p.num_splits + split, p.num_splits,
                      MergeRows{unit_row0, 1, (int64_t)p.group * p.num_splits, p.num_splits, 0});
            if (p.length_feedback && (blockIdx.x | blockIdx.y | blockIdx.z) == 0 && wave == 0)
                store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
            return;
        }
    } else if constexpr (MODE == WM_QUEUE) {
        // work queue (single-launch form with a forced split count: it ends the call, so it reports the lengths)
        if (p.length_feedback && blockIdx.x == 0 && wave == 0)
            store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
        int item = blockIdx.x;
        if (item >= p.total_items) return;
        for (;;) {
            int wg = item;
            int ht = wg % p.head_tiles;
            wg /= p.head_tiles;
            int hgb = wg % p.hg_blocks;
            wg /= p.hg_blocks;
            const int split = wg % p.num_splits;
            int pb = wg / p.num_splits;
            int chunk = p.chunk;
            if (p.chunk_floor) chunk = chunk_tokens_of(min(as_const(p.kv_lens)[pb], p.max_tokens), p.num_splits, p.chunk, p.chunk_floor);
            int c_start = split * chunk;
            int c_limit = split == p.num_splits - 1 ? p.max_tokens : c_start + chunk;
            int64_t prow0 = ((int64_t)pb * p.hq + (hgb * nh + hl) * p.group + ht * 16) * p.num_splits + split;
            MergeRows mr;
            mr.live = 0;                                              // from kv_len, inside run_piece
            mr.base = ((int64_t)pb * p.hq + hgb * nh * p.group + ht * 16) * p.num_splits;
            mr.piece_step = 1;
            mr.hl_step = (int64_t)p.group * p.num_splits;
            mr.g_step = p.num_splits;
            // everything that describes the piece is wave-uniform: keep it in scalar registers
            pb = __builtin_amdgcn_readfirstlane(pb);
            hgb = __builtin_amdgcn_readfirstlane(hgb);
            ht = __builtin_amdgcn_readfirstlane(ht);
            c_start = __builtin_amdgcn_readfirstlane(c_start);
            c_limit = __builtin_amdgcn_readfirstlane(c_limit);
            prow0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(prow0 >> 32)) << 32) |
                    (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)prow0);
            run_piece(pb, hgb, ht, c_start, c_limit, prow0, p.num_splits, mr);
            __syncthreads();                                          // the LDS scratch is reused by the next piece
            if (threadIdx.x == 0) s_next[0] = p.grid_x + atomicAdd(p.counters, 1);
            __syncthreads();
            item = s_next[0];
            // unsigned: a queue head that was not zero on entry ends the queue instead of yielding a negative item
            if ((unsigned)item >= (unsigned)p.total_items) break;
        }
        if (threadIdx.x == 0) {                       // leave the counters at zero
            const int done = atomicAdd(p.counters + 1, 1);
            if (done == p.grid_x - 1) {
                atomicExch(p.counters, 0);
                atomicExch(p.counters + 1, 0);
            }
        }
    } else {
        struct Piece {
            int pb, hgb, ht, c_start, c_limit;
            int64_t prow0;
            MergeRows mr;
        };
        const int units = p.hg_blocks * p.head_tiles;
        // A sequence counts for its granules plus p.piece_cost more (none if it is empty), half of them in front of its
        // tokens and half behind: every sequence boundary inside a share costs its workgroup a fixed time (the merge of
        // the wavefronts after the last rows of one piece, table and q loads before the first rows of the next), and a
        // share that holds several boundaries gets fewer tokens for it.  (Half and half: a boundary that coincides
        // with the edge of a share costs nothing extra, and split like this it is at least charged to both neighbours
        // alike - all in front, uniform batches gave every other share 2-4 % more tokens than the shares between.)
        const int pc = p.piece_cost, pcf = p.piece_cost >> 1;
        auto granules_of = [&](int bb) {
            const int g = (max(min(as_const(p.kv_lens)[bb], p.max_tokens), 0) + kGranule - 1) / kGranule;
            return g > 0 ? g + pc : 0;
        };
        int x = 0, hi = 0;                            // next granule, end of this workgroup's share
        int b = 0, before = 0, gb = 1;                // sequence of x, granules of the sequences before it, its granules
        const int wc = blockIdx.y, bu = blockIdx.x;   // grid = (units, shares)
        int share_q = 1, share_r = 0;                 // granules per share, shares with one more
        // the piece of sequence b in this workgroup's share, and where the share's part of the sequence ends
        auto piece_of = [&](int& piece_end) {
            Piece pp;
            piece_end = min(before + gb, hi);
            pp.pb = b;
            pp.hgb = bu;
            pp.ht = 0;
            if (p.head_tiles > 1) {
                pp.hgb = bu / p.head_tiles;
                pp.ht = bu % p.head_tiles;
            }
            pp.c_start = max(x - before - pcf, 0) * kGranule;               // the first pcf positions hold no tokens,
            pp.c_limit = min(piece_end - before - pcf, gb - pc) * kGranule; // nor do the last pc - pcf; <= c_start:
                                                                            // nothing of this sequence in the share
            const int64_t slot = (int64_t)(wc + b) * units + bu;
            pp.prow0 = slot * p.rows_per_slot + hl * p.heads_per_tile;
            // the shares that hold granules [before, before + gb) of this sequence (the first share_r shares
            // have share_q + 1 granules)
            auto share_of = [&](int g) {
                const int big = share_r * (share_q + 1);
                return g < big ? g / (share_q + 1) : share_r + (g - big) / share_q;
            };
            pp.mr = MergeRows{0, 0, 0, 0, 0};
            if (p.fused) {                       // (two integer divisions each: not on the way to the first loads)
                const int wc_first = share_of(before + pcf);
                pp.mr.live = share_of(before + pcf + (gb - pc) - 1) - wc_first + 1;
                pp.mr.base = ((int64_t)(wc_first + b) * units + bu) * p.rows_per_slot;
                pp.mr.piece_step = (int64_t)units * p.rows_per_slot;
                pp.mr.hl_step = p.heads_per_tile;
                pp.mr.g_step = 1;
            }
            // everything that describes the piece is wave-uniform: keep it in scalar registers
            pp.pb = __builtin_amdgcn_readfirstlane(pp.pb);
            pp.hgb = __builtin_amdgcn_readfirstlane(pp.hgb);
            pp.ht = __builtin_amdgcn_readfirstlane(pp.ht);
            pp.c_start = __builtin_amdgcn_readfirstlane(pp.c_start);
            pp.c_limit = __builtin_amdgcn_readfirstlane(pp.c_limit);
            pp.prow0 = ((int64_t)__builtin_amdgcn_readfirstlane((int)(pp.prow0 >> 32)) << 32) |
                       (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)pp.prow0);
            return pp;
        };
        // After a piece: the piece that holds the first token of its sequence says where the combine finds the
        // sequence's pieces for this unit - its own share and the number of shares up to the one with the last token
        // (after the piece, so that the divisions are not on the way to its loads); then on to the next sequence that
        // has tokens.  False: the share is worked off.
        auto next_piece = [&](const Piece& pp, int piece_end) {
            if (!p.fused && pp.c_start == 0 && pp.c_limit > 0 && threadIdx.x == 0) {
                const int big = share_r * (share_q + 1);
                const int g_last = before + pcf + (gb - pc) - 1;          // the granule of the last token
                const int wc_last = g_last < big ? g_last / (share_q + 1) : share_r + (g_last - big) / share_q;
                p.slot_desc[b * units + bu] = make_int2(wc, wc_last - wc + 1);
            }
            x = piece_end;
            if (x >= hi) return false;
            before += gb;
            do {                                                          // one exists: granule x < hi is somewhere
                b = min(b + 1, p.batch - 1);
                gb = granules_of(b);
            } while (gb == 0 && b + 1 < p.batch);
            return gb != 0;
        };
        // every wavefront derives the partition: a prefix sum over the sequences' granules, 64 at a time
        const int g_first = lane < p.batch ? granules_of(lane) : 0;          // sequences 0..63
        const int incl_first = wave_scan_i32(g_first);
        int total = __builtin_amdgcn_readlane(incl_first, 63);
        for (int b0 = 64; b0 < p.batch; b0 += 64) total += wave_sum_i32(b0 + lane < p.batch ? granules_of(b0 + lane) : 0);
        const int shares = min(p.shares, total);
        if (p.fused && wc == 0 && tix == 0) {
            // no piece, hence no merge, ever touches a sequence without tokens: the first share writes those rows
            for (int b0 = 0; b0 < p.batch; b0 += 64) {
                const int g = b0 == 0 ? g_first : (b0 + lane < p.batch ? granules_of(b0 + lane) : 0);
                uint64_t empty = __builtin_amdgcn_ballot_w64(b0 + lane < p.batch && g == 0);
                for (; empty; empty &= empty - 1) {
                    const int ht_e = bu % p.head_tiles;
                    write_empty_rows(b0 + __builtin_ctzll(empty), ((bu / p.head_tiles) * nh + hl) * p.group + ht_e * 16,
                                     min(16, p.group - ht_e * 16));
                }
            }
        }
        if (p.length_feedback && (bu | wc) == 0 && wave == 0)          // single-launch form: no combine follows
            store_length_bounds(p.length_feedback, p.kv_lens, p.batch, p.max_tokens, p.feedback_epoch, lane);
        if (wc >= shares) return;                                            // also total == 0
        const int q = total / shares, r = total % shares;
        share_q = q;
        share_r = r;
        x = wc * q + min(wc, r);
        hi = x + q + (wc < r ? 1 : 0);
        for (int b0 = 0, run = 0; b0 < p.batch; b0 += 64) {
            const int g = b0 == 0 ? g_first : (b0 + lane < p.batch ? granules_of(b0 + lane) : 0);
            const int incl = b0 == 0 ? incl_first : wave_scan_i32(g);
            const int excl = run + incl - g;
            const uint64_t mask = __builtin_amdgcn_ballot_w64(g > 0 && excl <= x && x < excl + g);
            if (mask) {
                const int src = __builtin_ctzll(mask);
                b = b0 + src;
                before = __builtin_amdgcn_readlane(excl, src);
                gb = __builtin_amdgcn_readlane(g, src);
                break;
            }
            run += __builtin_amdgcn_readlane(incl, 63);
        }
        int piece_end = 0;
        const Piece first = piece_of(piece_end);
        if (first.c_limit > first.c_start) run_piece(first.pb, first.hgb, first.ht, first.c_start, first.c_limit, first.prow0, 1, first.mr);
        if (!next_piece(first, piece_end)) return;
        for (;;) {
            __syncthreads();                                          // the LDS scratch is reused by the next piece
            const Piece pp = piece_of(piece_end);
            if (pp.c_limit > pp.c_start) run_piece(pp.pb, pp.hgb, pp.ht, pp.c_start, pp.c_limit, pp.prow0, 1, pp.mr);
            if (!next_piece(pp, piece_end)) return;
        }
    }
}

// Whether the call runs as a work queue: whenever the KV range is split into per-sequence chunks, the caller provided
// counters and there are more pieces than are resident at once - pieces of a ragged batch differ in length, and a
// queue keeps every compute unit busy until the end.
inline bool mfma_runs_as_queue(const SplitParams& p) {
    const int hg_per_wg = (p.hg_per_wg < 1 || p.hkv % p.hg_per_wg) ? 1 : p.hg_per_wg;
    const int64_t items = (int64_t)p.batch * p.num_splits * (p.hkv / hg_per_wg) * ((p.group + 15) / 16);
    const int resident = 2 * (p.num_cus > 0 ? p.num_cus : 256);     // two 4-wave workgroups fit a compute unit
    return p.counters != nullptr && !p.direct && !p.balanced && items > resident;
}
inline int mfma_work_mode(const SplitParams& p) { return p.balanced ? WM_SHARES : mfma_runs_as_queue(p) ? WM_QUEUE : WM_ONE; }

// (MODE must be mfma_work_mode(p_in): the translation units of the modes instantiate one each, see launch_mfma_d)
template <int QDT, bool FP8, int D, bool PROBE = false, int MODE = WM_ONE>
int launch_pm(const SplitParams& p_in, hipStream_t stream) {
    if (mfma_work_mode(p_in) != MODE) return (int)hipErrorInvalidValue;
    constexpr int kScratch = 4 * kTile * D;
    SplitParams p = p_in;
    p.head_tiles = (p.group + 15) / 16;
    if (p.hg_per_wg < 1 || p.hkv % p.hg_per_wg) p.hg_per_wg = 1;
    p.hg_blocks = p.hkv / p.hg_per_wg;
    // How much a compute unit keeps under way decides how well the memory system runs, and about 32 KB is the
    // optimum on MI355X (a tile of 16 tokens is kTileBytes per wavefront): less leaves it idle, more only queues
    // up and costs 3-5 %.  A single pass (one workgroup per compute unit) is shaped for that: wavefronts per
    // workgroup and register buffers per wavefront (below) follow from the tile size; blocks of 4 or 8 kv heads
    // always take 8 wavefronts.  Measured, batch 32 x 8 kv heads x 4096 tokens: 16-bit cache 85.3 us with two
    // buffers, 81.7 us with one; fp8 cache 52.3 us with 4 wavefronts x 2 buffers, 47.1 us with 8 x 1.
    constexpr int kTileBytes = 2 * kTile * D * (FP8 ? 1 : 2);                    // K and V rows of one tile
    const int64_t items = (int64_t)p.batch * p.num_splits * p.hg_blocks * p.head_tiles;
    const bool single_pass = p.num_splits == 1 && !p.balanced;
    // small tiles: also per-sequence chunks that give each compute unit at most one workgroup (one-byte-per-value
    // caches cut like that measure 13-16 % faster with 8 wavefronts x 1 buffer than with 4 x 2)
    const bool shaped = single_pass || (kTileBytes <= 4096 && !p.balanced && items <= (p.num_cus > 0 ? p.num_cus : 256));
    // (equal shares of the whole batch also come one workgroup to a compute unit)
    int nw = (p.hg_per_wg >= 4 || ((shaped || p.balanced) && kTileBytes <= 4096)) ? 8 : 4;   // wavefronts per workgroup
    // a caller's override (measurements), if the kernel can run it: every kv head of the block needs a wavefront,
    // and at most four (small tiles: eight) wavefronts share a head
    if (p.tune_wavefronts >= p.hg_per_wg && p.tune_wavefronts / p.hg_per_wg <= (kTileBytes <= 4096 ? 8 : 4))
        nw = p.tune_wavefronts;
    const size_t lds_bytes = (size_t)nw * (kScratch + 2 * 16 * sizeof(float)) + 16;
    constexpr int RPL = Regs<FP8, D>::RPL;
    int pm;
    if (p.page_shift < 0) pm = PM_LANE_DIV;
    else if (p.page_size % kTile == 0) pm = PM_TILE;
    else if (p.page_size % RPL == 0) pm = PM_LOAD;
    else pm = PM_LANE;
    p.total_items = (int32_t)((int64_t)p.batch * p.num_splits * p.hg_blocks * p.head_tiles);
    const int resident = 2 * (p.num_cus > 0 ? p.num_cus : 256);     // two 4-wave workgroups fit a compute unit
    p.persistent = MODE == WM_QUEUE ? 1 : 0;
    const unsigned units = (unsigned)(p.hg_blocks * p.head_tiles);
    const dim3 grid = p.balanced ? dim3(units, (unsigned)p.workgroups / units)
                    : p.persistent ? dim3((unsigned)resident)
                                   : dim3(units, (unsigned)p.num_splits, (unsigned)p.batch);
    const dim3 block(64 * nw);
    p.shares = (int32_t)grid.y;
    p.grid_x = (int32_t)grid.x;
    p.wavefronts = nw;
    // Register buffers per wavefront (tiles of loads that can be under way while a tile is worked on): two, or
    // one for the widest rows (two would not leave room for two workgroups per compute unit), in a single pass
    // whose wavefronts together hold 32 KB with one, and for long pieces with wave-uniform page numbers (equal
    // shares come one workgroup to a compute unit and hold 32 KB with one buffer, chunks of a forced split come
    // several to a unit and hold more: 0.6-1.4 % faster either way).  Short pieces, and page sizes
    // whose page numbers come by vector loads (in order with the rows), are up to 7 % faster with two.
    const bool long_pieces = pm == PM_TILE && !single_pass && p.chunk >= 512;
    // (a block of 4 or 8 kv heads of a one-byte cache is the exception: its eight wavefronts hold 32 KB with one
    // buffer as well, but measure 1-1.5 % faster with two - batch 128 / 256 x 8 kv heads x 8192 tokens: 329.7 -> 324.7
    // and 667.8 -> 661.5 us)
    const bool wide_fp8 = FP8 && p.hg_per_wg >= 4;
    const bool one_buffer = D > 128 || (p.tune_buffers ? p.tune_buffers == 1
                                                       : ((shaped && kTileBytes * nw >= 32768 && !wide_fp8) || long_pieces));
#define FDK_MFMA_LAUNCH(PMV, NB) \
    hipLaunchKernelGGL((splitkv_mfma_kernel<QDT, FP8, PMV, NB, D, PROBE, MODE>), grid, block, lds_bytes, stream, p)
#define FDK_MFMA_LAUNCH_PM(NB)                                    \
    switch (pm) {                                                 \
        case PM_TILE: FDK_MFMA_LAUNCH(PM_TILE, NB); break;        \
        case PM_LOAD: FDK_MFMA_LAUNCH(PM_LOAD, NB); break;        \
        case PM_LANE: FDK_MFMA_LAUNCH(PM_LANE, NB); break;        \
        default: FDK_MFMA_LAUNCH(PM_LANE_DIV, NB); break;         \
    }
    if (one_buffer) {
        FDK_MFMA_LAUNCH_PM(1)
    } else {
        FDK_MFMA_LAUNCH_PM((D > 128 ? 1 : 2))
    }
#undef FDK_MFMA_LAUNCH_PM
#undef FDK_MFMA_LAUNCH
    return (int)hipGetLastError();
}


template <int D, int MODE>
int launch_mfma_d(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    const bool fp8 = kv_dtype == FDK_FP8_E4M3;
    if (q_dtype == FDK_BF16)
        return fp8 ? launch_pm<FDK_BF16, true, D, false, MODE>(p, stream) : launch_pm<FDK_BF16, false, D, false, MODE>(p, stream);
    return fp8 ? launch_pm<FDK_FP16, true, D, false, MODE>(p, stream) : launch_pm<FDK_FP16, false, D, false, MODE>(p, stream);
}

}  // namespace

}  // namespace fdk
