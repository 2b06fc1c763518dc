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

// Where the page numbers of a tile's rows come from: one per tile (a tile never leaves its page), one per load
// instruction, one per lane (shift or division by the page size), or - rows of two segments, any page size - one per row,
// fetched by the lane of that number and passed to the lanes that load the row.
enum PageMode { PM_TILE = 0, PM_LOAD = 1, PM_LANE = 2, PM_LANE_DIV = 3, PM_ROW = 4 };
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

// How the load instructions of a tile (16 rows of D values) cover its rows.  A row is a power-of-two segment of D0
// values and, for head dims like 192 = 128 + 64 or 576 = 512 + 64, a second one of D1 values behind it (the reference's
// BLOCK_HEAD_DIM and BLOCK_DPE, flash_decode.py:103-109,187-191,210-214); a load instruction reads one segment of RPL
// whole rows, a lane 16 bytes of it.
template <bool FP8, int D>
struct Rows {
    static constexpr int ES = FP8 ? 1 : 2;
    static constexpr int D0 = D >= 512 ? 512 : D >= 256 ? 256 : D >= 128 ? 128 : 64;
    static constexpr int D1 = D - D0;
    static constexpr int LPR0 = D0 * ES / 16, RPL0 = 64 / LPR0, NJ0 = kTile / RPL0;
    static constexpr int LPR1 = D1 ? D1 * ES / 16 : 64, RPL1 = 64 / LPR1, NJ1 = D1 ? kTile / RPL1 : 0;
    static constexpr int NJ = NJ0 + NJ1;                 // load instructions per tile
    static_assert(D1 == 0 || ((D1 & (D1 - 1)) == 0 && LPR1 >= 4), "second segment: a power of two, at most 16 rows per load");
    static_assert(LPR0 >= 4 && LPR0 <= 64, "first segment: 4 to 64 lanes per row");
    // load instruction j (a constant after unrolling): lanes per row, first row, byte offset of its segment in a cache row
    static constexpr int lpr(int j) { return j < NJ0 ? LPR0 : LPR1; }
    static constexpr int rpl(int j) { return j < NJ0 ? RPL0 : RPL1; }
    static constexpr int row0(int j) { return j < NJ0 ? j * RPL0 : (j - NJ0) * RPL1; }
    static constexpr int seg_byte(int j) { return j < NJ0 ? 0 : D0 * ES; }
};

template <bool FP8, int DK, int DV>
struct Regs {                                  // one tile in registers, as loaded
    using K = Rows<FP8, DK>;
    using V = Rows<FP8, DV>;
    static constexpr int LPR = K::LPR0;                  // one segment, K and V rows alike: lanes (16-byte pieces) per cache row,
    static constexpr int RPL = K::RPL0;                  // rows per load instruction,
    static constexpr int NJ = K::NJ0;                    // load instructions per tensor and tile
    uint32_t k[K::NJ][4];
    uint32_t v[V::NJ][4];
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
// Several q-head tiles per kv head (groups of more than 16 heads) read the same K / V rows.  Workgroups go to the eight
// XCDs round-robin in linear order and every XCD has an L2 of its own: with the tile index running fastest, the tiles of
// a row of work (a kv-head block of a sequence's piece) land on different XCDs and each of them fetches the rows from
// memory.  This maps the linear workgroup id so that the T tiles of a row sit on ONE XCD, within 8 T consecutive ids
// (they run at the same time and share what the first of them brought into the L2):
// id = block * 8 T + tile * 8 + slot  ->  row = block * 8 + slot.  Rows past the last full block of eight keep the plain order.
__device__ __forceinline__ void tiles_on_one_xcd(int id, int rows, int T, int& row, int& tile) {
    const int full_rows = rows & ~7;
    if (id < full_rows * T) {
        const int blk = id / (8 * T), in = id - blk * 8 * T;
        tile = in >> 3;
        row = blk * 8 + (in & 7);
    } else {
        const int rest = id - full_rows * T;
        row = full_rows + rest / T;
        tile = rest % T;
    }
}

// max over the four lanes l, l ^ 16, l ^ 32, l ^ 48 without the LDS crossbar: v_permlane16_swap exchanges the odd rows (16
// lanes) of its first operand with the even rows of its second, v_permlane32_swap the upper half of the first with the lower
// half of the second; applied to two copies of x they leave (x[l & ~16], x[l | 16]) resp. (x[l & 31], x[l | 32]) in lane l.
// (From inline asm: given the same value twice, the compiler folds the builtins' two results into one.)
__device__ __forceinline__ float max_across_rows(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    a = fmaxf(a, b);
    b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}

// Eight wavefronts may share a kv head where a tile is small: one-byte caches with rows of 192 values (6 KB a tile;
// four wavefronts would keep 24 KB of a compute unit under way, eight keep 48 KB).
constexpr bool rows2_eight_share(bool fp8, int dk, int dv) { return fp8 && dk + dv <= 384; }

// head_dim 64, 128, 256 (K and V rows alike, one segment)
template <int QDT, bool FP8, int PM, int NBUF, int D, bool PROBE = false, int MODE = WM_ONE>
__global__ __launch_bounds__(512) void splitkv_mfma_kernel(const SplitParams p) {
    constexpr int DK = D, DV = D;
    constexpr bool REUSE = false;
    constexpr bool kPairedRows = true;
#include "fdk_splitkv_mfma_body.h"
#include "fdk_splitkv_mfma_work.h"
}
// Rows of two segments and V rows shorter than K rows (q / K rows of DK values, V / output rows of DV): 16-bit and fp8
// caches, one register buffer.  Also rows of 128 values where a kv head has more than 16 q heads (DK = DV = 128): the
// q-head tiles of a kv head then run on one XCD and load with plain loads (REUSE), which the kernels above do not.  Beyond 512 values per token and kv head a workgroup has four wavefronts, each alone on its
// SIMD with the whole register file.
constexpr int rows2_max_threads(int dk, int dv) { return dk + dv > 512 ? 256 : 512; }
// REUSE: several workgroups read the same K / V rows (more than one q-head tile per kv head).
template <int QDT, int PM, int DK, int DV, int MODE, bool REUSE, bool FP8 = false>
__global__ __launch_bounds__(rows2_max_threads(DK, DV)) void splitkv_mfma_rows2_kernel(const SplitParams p) {
    constexpr bool PROBE = false;
    constexpr int NBUF = 1;
    constexpr bool kPairedRows = false;
#include "fdk_splitkv_mfma_body.h"
#include "fdk_splitkv_mfma_work.h"
}

// Whether the call runs as a work queue: whenever the KV range is split into per-sequence chunks, the caller provided
// counters and there are more pieces than are resident at once - pieces of a ragged batch differ in length, and a
// queue keeps every compute unit busy until the end.
inline bool mfma_runs_as_queue(const SplitParams& p) {
    const int hg_per_wg = (p.hg_per_wg < 1 || p.hkv % p.hg_per_wg) ? 1 : p.hg_per_wg;
    const int tile_heads = p.tile_heads > 16 ? p.tile_heads : 16;       // q heads of a kv head per workgroup
    const int64_t items = (int64_t)p.batch * p.num_splits * (p.hkv / hg_per_wg) * ((p.group + tile_heads - 1) / tile_heads);
    // two 4-wave workgroups fit a compute unit; of the kernels that cover 64 q heads per workgroup, one
    const int resident = (tile_heads > 16 ? 1 : 2) * (p.num_cus > 0 ? p.num_cus : 256);
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
    constexpr int RPL = Regs<FP8, D, D>::RPL;
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

// The kernels for rows of two segments / V rows shorter than K rows (splitkv_mfma_rows2_kernel): no single-launch form,
// no load-only probe.  The plan keeps the kv heads per workgroup within what the kernel's workgroup
// size and the LDS allow (mfma_kv_heads_per_wg).
template <int QDT, int DK, int DV, int MODE, bool FP8>
int launch_rows2(const SplitParams& p_in, hipStream_t stream) {
    if (mfma_work_mode(p_in) != MODE || p_in.fused || p_in.probe) return (int)hipErrorInvalidValue;
    constexpr int kScratch = 2 * kTile * (DK + DV);
    constexpr size_t kLdsPerCu = 160 * 1024;
    SplitParams p = p_in;
    p.head_tiles = (p.group + 15) / 16;
    if (p.hg_per_wg < 1 || p.hkv % p.hg_per_wg) p.hg_per_wg = 1;
    p.hg_blocks = p.hkv / p.hg_per_wg;
    // (one workgroup per compute unit - a single pass, equal shares - takes eight wavefronts where the tiles are small)
    const bool one_per_cu = p.balanced || p.num_splits == 1;
    const int nw = (p.hg_per_wg >= 4 || (rows2_eight_share(FP8, DK, DV) && one_per_cu)) ? 8 : 4;
    const size_t lds_bytes = (size_t)nw * (kScratch + 2 * 16 * sizeof(float)) + 16;
    if (64 * nw > rows2_max_threads(DK, DV) || lds_bytes > kLdsPerCu) return (int)hipErrorInvalidValue;
    const int pm = (p.page_shift >= 0 && p.page_size % kTile == 0) ? PM_TILE : PM_ROW;
    p.total_items = (int32_t)((int64_t)p.batch * p.num_splits * p.hg_blocks * p.head_tiles);
    const int resident = 2 * (p.num_cus > 0 ? p.num_cus : 256);
    p.persistent = MODE == WM_QUEUE ? 1 : 0;
    const unsigned units = (unsigned)(p.hg_blocks * p.head_tiles);
    const dim3 grid = p.balanced ? dim3(units, (unsigned)p.workgroups / units)
                    : p.persistent ? dim3((unsigned)resident)
                                   : dim3(units, (unsigned)p.num_splits, (unsigned)p.batch);
    const dim3 block(64 * nw);
    p.shares = (int32_t)grid.y;
    p.grid_x = (int32_t)grid.x;
    p.wavefronts = nw;
    // plain loads (rows stay in the L2 for the workgroup that needs them next) where several q-head tiles read the same
    // rows, and where the rows of neighbouring kv heads share 128-byte lines and belong to different workgroups (one-byte
    // rows of 192 values, an odd number of kv heads per workgroup; measured, batch 32 x 8 kv heads x 4096 tokens in a single
    // pass: 88.3 -> 72.9 us, memory traffic 1.29 -> 1.00 of the bytes attended to; with two heads per workgroup plain loads
    // are 3 % slower than streaming ones)
    const bool reuse = p.head_tiles > 1 || (FP8 && (DK % 128 != 0 || DV % 128 != 0) && (p.hg_per_wg & 1) && p.hg_blocks > 1);
#define FDK_ROWS2_LAUNCH(PMV, RU)                                                                                          \
    do {                                                                                                                   \
        if (lds_bytes > 64 * 1024) {                                                                                       \
            const hipError_t e = hipFuncSetAttribute(                                                                      \
                reinterpret_cast<const void*>(&splitkv_mfma_rows2_kernel<QDT, PMV, DK, DV, MODE, RU, FP8>),                \
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);                                               \
            if (e != hipSuccess) return (int)e;                                                                            \
        }                                                                                                                  \
        hipLaunchKernelGGL((splitkv_mfma_rows2_kernel<QDT, PMV, DK, DV, MODE, RU, FP8>), grid, block, lds_bytes, stream, p); \
    } while (0)
    if (pm == PM_TILE) {
        if (reuse) FDK_ROWS2_LAUNCH(PM_TILE, true);
        else FDK_ROWS2_LAUNCH(PM_TILE, false);
    } else {
        if (reuse) FDK_ROWS2_LAUNCH(PM_ROW, true);
        else FDK_ROWS2_LAUNCH(PM_ROW, false);
    }
#undef FDK_ROWS2_LAUNCH
    return (int)hipGetLastError();
}

template <int DK, int DV, int MODE>
int launch_mfma_rows2(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    if (kv_dtype == FDK_FP8_E4M3)
        return q_dtype == FDK_BF16 ? launch_rows2<FDK_BF16, DK, DV, MODE, true>(p, stream) : launch_rows2<FDK_FP16, DK, DV, MODE, true>(p, stream);
    if (kv_dtype != q_dtype) return (int)hipErrorInvalidValue;
    // (16-bit caches with rows of more than 512 values run in the shared-tile kernels whatever the group: mfma_heads_per_wg)
    if constexpr (DK + DV > 512) return (int)hipErrorInvalidValue;
    else return q_dtype == FDK_BF16 ? launch_rows2<FDK_BF16, DK, DV, MODE, false>(p, stream) : launch_rows2<FDK_FP16, DK, DV, MODE, false>(p, stream);
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
