// Split-KV paged decode for LARGE q-head groups on one kv head, matrix-core path, gfx950: the shape of latent
// attention, where 128 q heads share one kv head whose rows hold 576 (K) and 512 (V) values.
//
// The kernels of fdk_splitkv_mfma.h give a wavefront one kv head and 16 q heads (the reference's BLOCK_H,
// python/triton_dist/kernels/nvidia/flash_decode.py:103-109,170-176): with G q heads per kv head the K / V rows are
// read G / 16 times, and every tile of 16 tokens is copied to LDS once per 16 q heads.  That is the right shape while
// the memory system is the limit (G <= 16: every row is read once).  At G = 128 it is not: the rows cross the L2 eight
// times and the matrix cores idle.  Here the wavefronts of a workgroup take DIFFERENT q-head tiles of the SAME kv head
// and the same tokens: a tile of K / V rows is loaded once by the workgroup (each wavefront loads its share of the
// rows), staged once in LDS, and every wavefront multiplies it with its own 16 q heads.
//
// A workgroup covers kSharedTileHeads = 64 q heads with eight wavefronts: two per tile of 16 q heads, each of which
// forms the tile's softmax for itself and accumulates one half of the output columns (64 accumulation registers per
// lane at 512 values), two wavefronts per SIMD.  A group of 128 q heads is two such workgroups, which the launch places
// on one XCD (tiles_on_one_xcd).  Same arithmetic per (q head, token) as the other kernels (fdk_splitkv_mfma_body.h):
// S^T = K Q^T with 16x16x32 MFMA, online softmax in fp32, O^T += V^T P^T with 16x16x16 MFMA and P rounded to the cache
// dtype; the running maximum of the softmax is a reference that moves rarely, so that the tile loop holds no rescale of
// the output tile (see move_reference).  Page numbers per tile or per row (PM_TILE, PM_ROW).  How pieces are handed out
// is shared with the other kernels (fdk_splitkv_mfma_work.h) with a head tile of 64 q heads.
//
// The rows never pass through registers.  global_load_lds_dwordx4 writes the 16 bytes of lane i to LDS byte M0 + 16 i, so
// a load instruction fills 1 KB of LDS directly.  The compiler would put "wait for every load under way" in front of each
// LDS read that follows such a load, so the loads are issued from inline asm and the tile loop waits by count itself
// (loads return in order, every wavefront issues the same number per tile).
// 16-bit caches: the loads fill the staged tile itself; the swizzle of the staged rows is applied on the memory side (the
// lane whose bytes land in chunk x of row r fetches chunk x ^ swizzle(r) of that row).  Four staged tiles: tile t is
// worked on while tiles t + 1 ... t + 3 land.
// e4m3 caches (kRaw): the loads fill one of two raw tiles, and the wavefront that requested them converts its own share
// from there into one of three staged tiles (16-bit values either way).
// The two wavefronts of a head tile split the q . k products - even and odd k-steps, nine each, 36 registers of Q^T each -
// and exchange their halves through LDS; a step of the loop holds the half dot products of tile t + 1 next to the softmax
// and the PV product of tile t, which do not depend on each other, and ONE barrier.
#pragma once

#include "fdk_splitkv_mfma.h"

namespace fdk {

namespace {

constexpr int kSharedWaves = 8;                        // wavefronts per workgroup
constexpr int kSharedColSplit = 2;                     // wavefronts that share a tile of 16 q heads, each with 1 / kSharedColSplit
                                                       // of the output columns (both form the tile's logits and softmax)
constexpr int kSharedTileHeads = 16 * kSharedWaves / kSharedColSplit;    // q heads of one kv head that a workgroup covers

// REUSE: another workgroup reads the same K / V rows (a group of more than 64 q heads): plain loads, so that the rows
// stay in the XCD's L2 for it; otherwise the rows are read once and come with the non-temporal hint.
// FP8: an e4m3 cache; the rows are dequantised on their way into the staged tile, which holds 16-bit values either way.
template <int QDT, int PM, int DK, int DV, int MODE, bool REUSE, bool FP8 = false>
__global__ __launch_bounds__(64 * kSharedWaves) void splitkv_mfma_shared_kernel(const SplitParams p) {
    using M = Mma<QDT>;
    using P2 = Pack2<QDT>;
    using RK = Rows<FP8, DK>;
    using RV = Rows<FP8, DV>;
    static_assert(PM == PM_TILE || PM == PM_ROW, "page numbers per tile or per row");
    static_assert(DK % 64 == 0 && DV % 64 == 0, "the LDS swizzle acts on groups of eight 16-byte chunks");
    constexpr bool kOneSegment = false;        // (fdk_splitkv_mfma_work.h: several head tiles of a kv head go to one XCD)
    constexpr bool kRowsShareLines = false;    // (16-bit rows: whole 128-byte lines per kv head)
    constexpr int kTileHeads = kSharedTileHeads;
    constexpr bool kFirstPieceStraight = true;  // (fdk_splitkv_mfma_work.h)
    constexpr int NW = kSharedWaves;
    constexpr int ES = FP8 ? 1 : 2;            // bytes per cache value
    constexpr int RBK = 2 * DK, RBV = 2 * DV;  // bytes of a staged row
    constexpr int KS = DK / 32;                // k-steps of the QK product
    constexpr int CS = kSharedColSplit;
    constexpr int DB = DV / 16 / CS;           // 16-column blocks of the output that this wavefront holds
    constexpr int kTileBytes = kTile * (RBK + RBV);
    // 16-bit caches: the rows go from memory straight into the staged tile (global_load_lds_dwordx4: lane i of a load
    // instruction writes its 16 bytes at M0 + 16 i, no registers in between and nothing to store), four staged tiles.
    // A load instruction then fills 1 KB of consecutive LDS, so the second K segment of the 16 rows lies behind their
    // first segments instead of behind each row, and the swizzle is applied on the memory side: the lane whose bytes
    // land in chunk x of row r fetches chunk x ^ swizzle(r) (the same 128-byte line either way).
    // e4m3 caches (kRaw): the bytes take the same road into one of two raw tiles in LDS, and the wavefront that requested
    // them converts them from there into a staged tile (its own share only: no other wavefront has to know when they
    // landed); three staged tiles.
    constexpr bool kRaw = FP8;
    constexpr int kStaged = kRaw ? 3 : 4;      // staged tiles in LDS
    static_assert(kRaw || (RK::LPR0 == 64 && RV::LPR0 == 64 && RV::D1 == 0 && (RK::D1 == 0 || RK::LPR1 == 8)),
                  "direct loads: a first segment of 1 KB per row, a second K segment of 128 bytes");
    static_assert(!kRaw || (RK::NJ0 == NW && RV::NJ0 == NW && RK::NJ1 == 1 && RV::D1 == 0), "raw tiles: rows of 512 (+ 64) one-byte values");
    constexpr int kK0Row = RK::D0 * 2;         // bytes from one staged row's first K segment to the next row's
    constexpr int kK1Base = kTile * RK::D0 * 2; // where row 0's second K segment starts, and
    constexpr int kK1Row = RK::D1 * 2;         // the step to the next row's
    // load instructions of a tile that one wavefront issues, per segment of the rows (Rows<>)
    constexpr int KS0 = (RK::NJ0 + NW - 1) / NW, KS1 = (RK::NJ1 + NW - 1) / NW;
    constexpr int VS0 = (RV::NJ0 + NW - 1) / NW, VS1 = (RV::NJ1 + NW - 1) / NW;

    extern __shared__ __attribute__((aligned(16))) char lds[];      // the staged tiles, the next work item, the exchange area, ...

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int a = lane >> 4;                   // lane group: MFMA k-group / token group
    const int c = lane & 15;                   // MFMA row/column index
    const int nh = 1, hl = 0, tix = 0;         // one kv head per workgroup; every wavefront sees every tile
    const int wtile = wave / CS;               // this wavefront's tile of 16 q heads within the workgroup's
    const int whalf = wave % CS;               // ... and its part of the output columns
    int* const s_next = reinterpret_cast<int*>(lds + kStaged * kTileBytes);

    auto write_empty_rows = [&](const int b, const int head0, const int heads_here) {
        for (int idx = lane; idx < heads_here * DV; idx += 64) {
            const int g = idx / DV, d = idx % DV;
            const int64_t ob = (int64_t)b * p.out_sb + (int64_t)(head0 + g) * p.out_sh;
            store_out(p.out, ob + d, 0.f, p.out_dtype);
            if (d == 0) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + head0 + g] = -INFINITY;
                if (p.pack_lse) store_out(p.out, ob + DV, -INFINITY, p.out_dtype);
            }
        }
    };

    // One piece: tokens [c_start, min(c_limit, kv_len)) of sequence b for kv head hgb and the q heads
    // [ht * 64, ht * 64 + 64) of its group; this wavefront's are the 16 from ht * 64 + 16 * wave on.  The partial
    // results of head g of the 64 go to row prow0 + g * prow_step of the workspace.  (mr: the single-launch form is not
    // built for this kernel.)
    auto run_piece = [&](const int b, const int hgb, const int ht, const int c_start, const int c_limit,
                         const int64_t prow0, const int prow_step, MergeRows /*mr*/) {
        const int kvh = hgb;
        const int head_w = ht * kTileHeads + 16 * wtile;            // this wavefront's first q head within the group
        const int heads_here = min(16, p.group - head_w);           // <= 0: the wavefront only helps to load
        const bool active = heads_here > 0;
        const int head0 = kvh * p.group + head_w;

        // Q^T, the B operand of S^T = K Q^T: lane (h = c, a) supplies q[h][32 ks + 8 a .. + 7] in k-step ks; 72 registers per
        // lane at 576 values, kept for the whole piece (read from LDS per tile instead, they doubled the LDS traffic of
        // the QK product, which is what bounds it).  Columns past the group repeat its last head; their results are
        // never stored.
        // (Direct loads: the two wavefronts of a tile of 16 q heads share the dot products as well - the one with the even
        // k-steps, the other with the odd ones, KQ = KS / 2 each - and exchange their halves through LDS: half the reads of
        // the staged K rows, half the Q^T registers.)
        constexpr int KQ = KS / CS;                                 // k-steps of this wavefront: ks = kq_step * i + kq_first
        constexpr int kq_step = CS;
        const int kq_first = whalf;
        static_assert(KS % CS == 0 && CS == 2, "the k-steps split by parity");
        uint4 qreg[KQ];
#pragma unroll
        for (int i = 0; i < KQ; ++i) qreg[i] = make_uint4(0, 0, 0, 0);
        auto load_q = [&]() {
            if (active) {
                const uint16_t* qp = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)b * p.q_sb +
                                     (int64_t)(head0 + min(c, heads_here - 1)) * p.q_sh + 8 * a + 32 * kq_first;
#pragma unroll
                for (int i = 0; i < KQ; ++i) qreg[i] = *reinterpret_cast<const uint4*>(qp + 32 * kq_step * i);
            }
        };
        const ConstI32 tbl = as_const(p.block_table + (int64_t)b * p.tbl_sb);
        const int pmask = p.page_size - 1;
        const int kv_len = min(as_const(p.kv_lens)[b], p.max_tokens);
        if (c_start >= kv_len) {                                    // (the same for every wavefront of the workgroup)
            if (p.direct && active && whalf == 0) write_empty_rows(b, head0, heads_here);
            return;
        }
        const int c_end = min(c_limit, kv_len);
        const int n_tiles = (c_end - c_start + kTile - 1) / kTile;
        // the page number of tile t (PM_TILE), or of its row c in every lane (c, any a) (PM_ROW); any t may be asked for
        auto page_id = [&](int t) {
            const int tok0 = c_start + t * kTile;
            if (PM == PM_TILE) return tbl[min(tok0, c_end - 1) >> p.page_shift];
            const int n = min(tok0 + c, c_end - 1);
            return tbl[p.page_shift < 0 ? n / p.page_size : n >> p.page_shift];
        };

        const bool softcap = p.soft_cap > 0.f;
        const float inv_cap = softcap ? 1.0f / p.soft_cap : 0.f;
        // e4m3 caches, as in the other kernels: K becomes (k8 * k_scale) rounded to the q dtype on its way into LDS - the
        // dequantised cache that the reference would decode - or, folded, the exact k8 with k_scale in the logit scale;
        // V is converted exactly and v_scale multiplies the output rows once at the end
        float kscale = 1.f, vscale = 1.f;
        if (FP8) {
            if (p.k_scale) kscale = __builtin_bit_cast(float, as_const(reinterpret_cast<const int32_t*>(p.k_scale))[kvh]);
            if (p.v_scale) vscale = __builtin_bit_cast(float, as_const(reinterpret_cast<const int32_t*>(p.v_scale))[kvh]);
        }
        // (A scale that is a power of two needs neither: the conversion instruction applies it as an exponent, which is the
        // exact k8 * scale - the code of the folded form with the scale in the conversion instead of in the logit scale.)
        const bool by_exponent = FP8 && !p.fp8_fold && is_pow2_scale(kscale);
        const bool fold = FP8 && (p.fp8_fold || by_exponent);
        const float kconv = by_exponent ? kscale : 1.0f;      // the scale operand of the K conversions of the folded form
        const float logit_scale_log2 = fold && !by_exponent ? p.scale_log2 * kscale : p.scale_log2;
        const float logit_scale = fold && !by_exponent ? p.sm_scale * kscale : p.sm_scale;
        const char* kplane = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES;
        const char* vplane = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES;
        const uint32_t ksp_bytes = (uint32_t)(p.k_sp * ES), vsp_bytes = (uint32_t)(p.v_sp * ES);
        const uint32_t kst_bytes = (uint32_t)(p.k_st * ES), vst_bytes = (uint32_t)(p.v_st * ES);
        // Load instruction j of a segment covers rows j * RPL .. + RPL - 1 (a lane: row j * RPL + lane / LPR, 16 bytes
        // from byte seg + (lane % LPR) * 16 of the cache row); wavefront w issues the instructions j = w, w + 4, ...
        // This lane's place within the rows of a load instruction, as a byte offset from the first row (one value per
        // segment and tensor; everything else about an address of a full tile is wave-uniform or a few lane operations).
        const uint32_t k_lane0 = (uint32_t)(lane / RK::LPR0) * kst_bytes + (uint32_t)(lane % RK::LPR0) * 16;
        const uint32_t k_lane1 = (uint32_t)(lane / RK::LPR1) * kst_bytes + (uint32_t)(RK::D0 * ES + (lane % RK::LPR1) * 16);
        const uint32_t v_lane0 = (uint32_t)(lane / RV::LPR0) * vst_bytes + (uint32_t)(lane % RV::LPR0) * 16;
        const uint32_t v_lane1 = (uint32_t)(lane / RV::LPR1) * vst_bytes + (uint32_t)(RV::D0 * ES + (lane % RV::LPR1) * 16);
        // One load: rows first_row .. of the tile at token tok0, this lane's 16 bytes.  CLAMP (the partial last tile of
        // a piece): rows past the end repeat the last one, which is masked later.
        // The load instruction of a segment (it has n of them per tile) that this wavefront issues in its slot s.  Where
        // the wavefronts outnumber the instructions left for the last slot, the surplus wavefronts repeat instructions
        // of the others (same rows, same place in LDS): every wavefront then runs the same straight-line sequence of
        // loads and stores, and the waits the compiler puts in front of the stores can count the loads they follow
        // instead of waiting for all of them.
        auto slot_instr = [&](int s, int n) {
            const int j = NW * s + wave;
            return j < n ? j : j % n;
        };
        auto row_ptr = [&](auto clamp_tag, int tok0, int32_t pg_id, int first_row, int lane_row, uint32_t lane_off,
                           uint32_t lane_byte, const char* plane, uint32_t sp_bytes, uint32_t st_bytes) {
            constexpr bool CLAMP = decltype(clamp_tag)::value;
            if (PM == PM_TILE && !CLAMP) {
                // the tile lies in one page: a wave-uniform base plus the lane's offset
                const int n0 = tok0 + first_row;
                return plane + ((uint64_t)(uint32_t)pg_id * sp_bytes + (uint64_t)((uint32_t)(n0 & pmask) * st_bytes)) + lane_off;
            }
            int n = tok0 + first_row + lane_row;
            if (CLAMP) n = min(n, c_end - 1);
            const uint32_t slot = PM == PM_TILE ? (uint32_t)(n & pmask) : (uint32_t)(p.page_shift < 0 ? n % p.page_size : (n & pmask));
            const uint32_t pg = (uint32_t)(PM == PM_TILE ? pg_id : __shfl(pg_id, n - tok0, 64));
            return plane + ((uint64_t)pg * sp_bytes + (uint64_t)(slot * st_bytes)) + lane_byte;
        };
        // ---- direct loads: 16 bytes per lane from memory to LDS byte (dst + 16 lane), dst wave-uniform.  The
        // compiler does not see these loads (it would wait for ALL loads under way in front of every LDS read that follows
        // one): the tile loop places its own waits, see there. ----
        auto load_to_lds16 = [&](const char* ptr, uint32_t dst) {
            if (REUSE) asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(ptr), "s"(dst) : "memory");
            else asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(ptr), "s"(dst) : "memory");
        };
        constexpr int kLoadsPerTile = KS0 + KS1 + VS0 + VS1;        // load instructions of a tile that a wavefront issues
        const uint32_t lds0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)lds;    // the LDS byte address of lds[0]
        // Tile t into the staged tile at LDS byte dst.  A lane fetches the chunk that the swizzle of the staged tile
        // (k_off, v_off) wants where its bytes land: first segments, one row per instruction: chunk lane ^ swizzle(row);
        // second K segment, eight rows of eight chunks per instruction: chunk (lane & 7) ^ (row & 7) of row lane >> 3.
        auto issue_direct = [&](auto clamp_tag, int t, int32_t pg_id, uint32_t dst) {
            const int tok0 = c_start + t * kTile;
            int ln = lane;
            asm volatile("" : "+v"(ln));
            ln &= 63;
#pragma unroll
            for (int s = 0; s < KS0; ++s) {
                const int j = slot_instr(s, RK::NJ0);
                const uint32_t byte = (uint32_t)((ln ^ (j & 7)) << 4);
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j, 0, byte, byte, kplane, ksp_bytes, kst_bytes), dst + j * 1024);
            }
#pragma unroll
            for (int s = 0; s < KS1; ++s) {
                const int j = slot_instr(s, RK::NJ1);
                const uint32_t byte = (uint32_t)(RK::D0 * ES + (((ln & 7) ^ ((ln >> 3) & 7)) << 4));
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j * 8, ln >> 3, (uint32_t)(ln >> 3) * kst_bytes + byte, byte, kplane,
                                      ksp_bytes, kst_bytes), dst + kK1Base + j * 1024);
            }
#pragma unroll
            for (int s = 0; s < VS0; ++s) {
                const int j = slot_instr(s, RV::NJ0);
                const uint32_t byte = (uint32_t)((ln ^ ((j & 3) << 1)) << 4);
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j, 0, byte, byte, vplane, vsp_bytes, vst_bytes), dst + kTile * RBK + j * 1024);
            }
        };
        // ---- e4m3 rows through raw tiles (kRaw): load instruction j of a segment covers rows j RPL .. (a lane: row j RPL + lane /
        // LPR, 16 bytes from byte (lane % LPR) 16 of the segment); it fills 1 KB of the raw tile, first K
        // segments, second K segment, V rows.  convert_raw reads back exactly the bytes this wavefront requested. ----
        // Two raw tiles of first K segments and V rows, each wavefront reading back only what it requested itself; the
        // second K segment, one instruction that every wavefront issues and converts alike (so that all issue the same
        // number of loads), has four places of its own: a wavefront requests tile t + 4's into the place of tile t's, which
        // every wavefront converted two barriers ago - with two places a fast wavefront would overwrite what a slow one has
        // yet to read.
        constexpr int kRawTile = (RK::NJ0 + RV::NJ0) * 1024;
        const uint32_t raw_lds = (uint32_t)(kStaged * kTileBytes + 16 + 2 * NW * 1024);      // offset of the raw tiles from lds[0]
        const uint32_t raw1_lds = raw_lds + 2 * kRawTile;                                    // ... and of the second K segments
        auto issue_raw = [&](auto clamp_tag, int t, int32_t pg_id) {
            const int tok0 = c_start + t * kTile;
            const uint32_t dst = lds0 + raw_lds + (uint32_t)(t & 1) * kRawTile;
            int ln = lane;
            asm volatile("" : "+v"(ln));
            ln &= 63;
#pragma unroll
            for (int s = 0; s < KS0; ++s) {
                const int j = slot_instr(s, RK::NJ0);
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j * RK::RPL0, ln / RK::LPR0, k_lane0, (ln % RK::LPR0) * 16, kplane,
                                      ksp_bytes, kst_bytes), dst + j * 1024);
            }
#pragma unroll
            for (int s = 0; s < KS1; ++s) {
                const int j = slot_instr(s, RK::NJ1);
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j * RK::RPL1, ln / RK::LPR1, k_lane1, RK::D0 * ES + (ln % RK::LPR1) * 16,
                                      kplane, ksp_bytes, kst_bytes), lds0 + raw1_lds + (uint32_t)(t & 3) * (RK::NJ1 * 1024) + j * 1024);
            }
#pragma unroll
            for (int s = 0; s < VS0; ++s) {
                const int j = slot_instr(s, RV::NJ0);
                load_to_lds16(row_ptr(clamp_tag, tok0, pg_id, j * RV::RPL0, ln / RV::LPR0, v_lane0, (ln % RV::LPR0) * 16, vplane,
                                      vsp_bytes, vst_bytes), dst + (RK::NJ0 + j) * 1024);
            }
        };
        // 16 one-byte values -> two 16-byte chunks of 16-bit values (K: times the head's scale, see above; V: exact)
        auto widen = [&](const uint4 in, auto is_k, uint4& lo, uint4& hi) {
            constexpr bool K = decltype(is_k)::value;
            const uint32_t r[4] = {in.x, in.y, in.z, in.w};
            uint32_t o[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                if (!K) {
                    o[2 * w] = P2::from_fp8(r[w], false);
                    o[2 * w + 1] = P2::from_fp8(r[w], true);
                } else if (fold) {
                    o[2 * w] = P2::from_fp8(r[w], false, kconv);
                    o[2 * w + 1] = P2::from_fp8(r[w], true, kconv);
                } else {
                    const f32x2_t k01 = __builtin_amdgcn_cvt_pk_f32_fp8(r[w], false);
                    const f32x2_t k23 = __builtin_amdgcn_cvt_pk_f32_fp8(r[w], true);
                    o[2 * w] = P2::pack(k01.x * kscale, k01.y * kscale);
                    o[2 * w + 1] = P2::pack(k23.x * kscale, k23.y * kscale);
                }
            }
            lo = make_uint4(o[0], o[1], o[2], o[3]);
            hi = make_uint4(o[4], o[5], o[6], o[7]);
        };
        auto convert_raw = [&](int t, char* buf) {
            const char* raw = lds + raw_lds + (t & 1) * kRawTile;
            const char* raw1 = lds + raw1_lds + (t & 3) * (RK::NJ1 * 1024);
            int ln = lane;
            asm volatile("" : "+v"(ln));
            ln &= 63;
            uint4 lo, hi;
#pragma unroll
            for (int s = 0; s < KS0; ++s) {
                const int j = slot_instr(s, RK::NJ0);
                const int row = j * RK::RPL0 + ln / RK::LPR0, piece = ln % RK::LPR0;
                widen(*reinterpret_cast<const uint4*>(raw + j * 1024 + ln * 16), BoolTag<true>(), lo, hi);
                char* at = buf + row * kK0Row;
                *reinterpret_cast<uint4*>(at + (((2 * piece) ^ (row & 7)) << 4)) = lo;
                *reinterpret_cast<uint4*>(at + (((2 * piece + 1) ^ (row & 7)) << 4)) = hi;
            }
#pragma unroll
            for (int s = 0; s < KS1; ++s) {
                const int j = slot_instr(s, RK::NJ1);
                const int row = j * RK::RPL1 + ln / RK::LPR1, piece = ln % RK::LPR1;
                widen(*reinterpret_cast<const uint4*>(raw1 + j * 1024 + ln * 16), BoolTag<true>(), lo, hi);
                char* at = buf + kK1Base + row * kK1Row;
                *reinterpret_cast<uint4*>(at + (((2 * piece) ^ (row & 7)) << 4)) = lo;
                *reinterpret_cast<uint4*>(at + (((2 * piece + 1) ^ (row & 7)) << 4)) = hi;
            }
#pragma unroll
            for (int s = 0; s < VS0; ++s) {
                const int j = slot_instr(s, RV::NJ0);
                const int row = j * RV::RPL0 + ln / RV::LPR0, piece = ln % RV::LPR0;
                widen(*reinterpret_cast<const uint4*>(raw + (RK::NJ0 + j) * 1024 + ln * 16), BoolTag<false>(), lo, hi);
                char* lv = buf + kTile * RBK;
                *reinterpret_cast<uint4*>(lv + v_off<RBV>(row, 2 * piece)) = lo;
                *reinterpret_cast<uint4*>(lv + v_off<RBV>(row, 2 * piece + 1)) = hi;
            }
        };
        // Page numbers per row (PM_ROW) for the direct loads.  A vector load that the compiler sees would make it wait, in
        // front of the first use of the numbers, for every row requested since - so they take the same road as the rows:
        // global_load_lds_dword puts the page numbers of a tile's 16 rows (lane i: row i & 15; rows past the end repeat the
        // last token) into one of eight slots behind the exchange area, and the requests for the rows read them from there,
        // by then long landed (see the tile loop).  All wavefronts write the same numbers to the same place.
        constexpr int kPageSlots = 8;
        const uint32_t pg_lds = (uint32_t)(kStaged * kTileBytes + 16 + 2 * NW * 1024 + (kRaw ? 2 * (RK::NJ0 + RV::NJ0) * 1024 + 4 * 1024 : 0));    // offset of the slots from lds[0] (behind the raw tiles)
        auto issue_pages = [&](int t) {
            const int n = min(c_start + t * kTile + (lane & 15), c_end - 1);
            const int idx = p.page_shift < 0 ? n / p.page_size : n >> p.page_shift;
            const int32_t* ptr = p.block_table + (int64_t)b * p.tbl_sb + idx;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(ptr), "s"(lds0 + pg_lds + (uint32_t)(t & (kPageSlots - 1)) * 256)
                         : "memory");
        };
        // e4m3 rows with page numbers per row: every lane reads the number of its row from the slot.
        auto issue_raw_rows = [&](int t) {
            const int tok0 = c_start + t * kTile;
            const int32_t* pages = reinterpret_cast<const int32_t*>(lds + pg_lds + (t & (kPageSlots - 1)) * 256);
            const uint32_t dst = lds0 + raw_lds + (uint32_t)(t & 1) * kRawTile;
            int ln = lane;
            asm volatile("" : "+v"(ln));
            ln &= 63;
            auto place = [&](int n) { return p.page_shift < 0 ? (uint32_t)(n % p.page_size) : (uint32_t)(n & pmask); };
            static_assert(!kRaw || (KS0 == 1 && KS1 == 1 && VS0 == 1), "one instruction per segment and wavefront");
            const int j0 = slot_instr(0, RK::NJ0), j1 = slot_instr(0, RK::NJ1), jv = slot_instr(0, RV::NJ0);
            const int row0 = j0 * RK::RPL0 + ln / RK::LPR0, row1 = j1 * RK::RPL1 + ln / RK::LPR1, rowv = jv * RV::RPL0 + ln / RV::LPR0;
            const uint32_t pg0 = (uint32_t)pages[row0], pg1 = (uint32_t)pages[row1], pgv = (uint32_t)pages[rowv];
            const uint32_t pl0 = place(min(tok0 + row0, c_end - 1)), pl1 = place(min(tok0 + row1, c_end - 1)),
                           plv = place(min(tok0 + rowv, c_end - 1));
            load_to_lds16(kplane + ((uint64_t)pg0 * ksp_bytes + (uint64_t)(pl0 * kst_bytes)) + (ln % RK::LPR0) * 16, dst + j0 * 1024);
            load_to_lds16(kplane + ((uint64_t)pg1 * ksp_bytes + (uint64_t)(pl1 * kst_bytes)) + (RK::D0 * ES + (ln % RK::LPR1) * 16),
                          lds0 + raw1_lds + (uint32_t)(t & 3) * (RK::NJ1 * 1024) + j1 * 1024);
            load_to_lds16(vplane + ((uint64_t)pgv * vsp_bytes + (uint64_t)(plv * vst_bytes)) + (ln % RV::LPR0) * 16, dst + (RK::NJ0 + jv) * 1024);
        };
        // Tile t with page numbers per row.  A first-segment instruction covers ONE row: its page number, read from the slot
        // by every lane alike, its place in the page and with them its address are wave-uniform.  The instruction of the
        // second K segment covers eight rows: a lane reads the number of its own.
        auto issue_direct_rows = [&](int t, uint32_t dst) {
            const int tok0 = c_start + t * kTile;
            const int32_t* pages = reinterpret_cast<const int32_t*>(lds + pg_lds + (t & (kPageSlots - 1)) * 256);
            int ln = lane;
            asm volatile("" : "+v"(ln));
            ln &= 63;
            auto place = [&](int n) { return p.page_shift < 0 ? (uint32_t)(n % p.page_size) : (uint32_t)(n & pmask); };
            // (all page numbers first: every request for rows is an asm statement that no LDS read may cross, and a read
            // in front of each would cost its round trip each time)
            static_assert(KS0 == VS0 && RK::NJ0 == RV::NJ0 && KS1 <= 1, "K and V rows of the first segments pair up");
            int32_t pg_row[KS0], pg_lane = 0;
#pragma unroll
            for (int s = 0; s < KS0; ++s) pg_row[s] = pages[slot_instr(s, RK::NJ0)];
            const int j1 = slot_instr(0, RK::NJ1 > 0 ? RK::NJ1 : 1);
            if (KS1) pg_lane = pages[j1 * 8 + (ln >> 3)];
            uint64_t k_base[KS0], v_base[KS0];                      // wave-uniform: page and place of the row
#pragma unroll
            for (int s = 0; s < KS0; ++s) {
                const int n = min(tok0 + slot_instr(s, RK::NJ0), c_end - 1);
                const uint32_t pg = (uint32_t)__builtin_amdgcn_readfirstlane(pg_row[s]);
                const uint32_t pl = place(n);
                k_base[s] = (uint64_t)pg * ksp_bytes + (uint64_t)(pl * kst_bytes);
                v_base[s] = (uint64_t)pg * vsp_bytes + (uint64_t)(pl * vst_bytes);
            }
#pragma unroll
            for (int s = 0; s < KS0; ++s) {
                const int j = slot_instr(s, RK::NJ0);
                load_to_lds16(kplane + k_base[s] + (uint32_t)((ln ^ (j & 7)) << 4), dst + j * 1024);
            }
            if (KS1) {
                const int n = min(tok0 + j1 * 8 + (ln >> 3), c_end - 1);
                const uint32_t byte = (uint32_t)(RK::D0 * ES + (((ln & 7) ^ ((ln >> 3) & 7)) << 4));
                load_to_lds16(kplane + ((uint64_t)(uint32_t)pg_lane * ksp_bytes + (uint64_t)(place(n) * kst_bytes)) + byte,
                              dst + kK1Base + j1 * 1024);
            }
#pragma unroll
            for (int s = 0; s < VS0; ++s) {
                const int j = slot_instr(s, RV::NJ0);
                load_to_lds16(vplane + v_base[s] + (uint32_t)((ln ^ ((j & 3) << 1)) << 4), dst + kTile * RBK + j * 1024);
            }
        };
        // Online softmax against a REFERENCE maximum that moves rarely.  The output tile lives in the accumulation
        // registers, which only the matrix cores reach directly; a rescale by exp2(old max - new max) goes through the
        // vector ALU, i.e. through copies of all 128 registers, and with the rescale inside the tile loop the compiler
        // keeps the tile in vector registers for part of every iteration (256 copies per tile, and everything else
        // spilled).  So the loop over the tiles holds no rescale: probabilities are exp2(logit - m_ref) with a reference
        // m_ref that may lie up to kSlack below the true running maximum (p <= 2^8, no problem for fp32 sums nor for P
        // rounded to 16 bits), and a tile whose logits exceed m_ref + kSlack leaves the loop, moves the reference
        // (move_reference, the rare path) and is done again.  l, the output and the lse are exact whatever the reference
        // is: lse = m_ref + log2(sum of exp2(logit - m_ref)).
        constexpr float kSlack = 8.f;
        float m_ref = -INFINITY, l_run = 0.f;        // for head c; l_run is this lane group's share of the sum
        float mx_seen = 0.f;                          // the tile maximum that made try_compute give up
        f32x4_t acc[DB];                              // acc[db][i] = O[h = c][16 db + 4 a + i]
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        auto move_reference = [&]() {
            const float m_new = fmaxf(m_ref, mx_seen);               // finite: a tile holds a valid token
            const float alpha = fast_exp2(m_ref - m_new);            // 0 the first time (m_ref = -inf)
            l_run *= alpha;
            // (eight blocks at a time: all 128 registers at once would push everything else out of the vector registers)
#pragma unroll
            for (int g = 0; g < DB / 8; ++g) {
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[8 * g + i] *= alpha;
                __builtin_amdgcn_sched_barrier(0);
            }
            m_ref = m_new;
        };

        // The two halves of a tile's arithmetic: qk_tile, the dot products q . k of the tile's tokens with this wavefront's
        // heads, and softmax_pv, everything after them.
        // Where a lane reads its MFMA operands in the staged tile.  The swizzle XORs the low bits of the
            // 16-byte chunk index with the low bits of the row, so the chunks of one lane are 128 bytes apart within
            // each class of the low bits: two base addresses for K (k-steps of either parity), four for V (output blocks
            // modulo four), and constant steps - not one address per operand, which at 18 k-steps and 32 output blocks
            // would be fifty registers held across the tile loop.
            //   K operand of k-step ks: row c, chunk 4 ks + a  ->  chunk ^ (c & 7) = 8 (ks >> 1) + ((4 (ks & 1) + a) ^ (c & 7))
            //   V operand of block db (transposed read): row 4 a + (c >> 2), chunk 2 db + ((c & 3) >> 1)
            //                                            ->  2 (4 (db >> 2) + ((db & 3) ^ (row & 3))) + ((c & 3) >> 1)
        // Direct loads: this wavefront's half of the dot products, k-steps kq_first, kq_first + 2, ...: the operands of its
        // parity class are 128 bytes apart from ONE base address (the last k-step lies in the second K segment).
        auto qk_half = [&](const char* buf) {
            constexpr int KSEG0 = RK::D0 / 32;
            const char* k_at = buf + c * kK0Row + (((4 * kq_first + a) ^ (c & 7)) << 4);
            const int k1_delta = kK1Base + c * (kK1Row - kK0Row) - KSEG0 / 2 * 128;
            constexpr int QG = 3, NQG = KQ / QG;
            static_assert(KQ % QG == 0, "k-steps in whole groups");
            f32x4_t s3[QG];
#pragma unroll
            for (int i = 0; i < QG; ++i) s3[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            uint4 ka[KQ];
#pragma unroll
            for (int i = 0; i < KQ; ++i)        // (k-step 2 i + kq_first: chunk group i; from KSEG0 on in the second segment)
                ka[i] = *reinterpret_cast<const uint4*>(k_at + (2 * i >= KSEG0 ? k1_delta : 0) + i * 128);
#pragma unroll
            for (int g = 0; g < NQG; ++g) {
#pragma unroll
                for (int i = 0; i < QG; ++i) s3[i] = M::qk(ka[g * QG + i], qreg[g * QG + i], s3[i]);
            }
            f32x4_t s = s3[0];
#pragma unroll
            for (int i = 1; i < QG; ++i) s += s3[i];
            return s;
        };
        // False: a logit of the tile exceeds the reference by more than the slack; nothing has been changed.
        auto softmax_pv = [&](int t, const char* buf, const f32x4_t s, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            const int tok0 = c_start + t * kTile;
            const int k4 = c >> 2, cc = c & 3;
            const int vrow = 4 * a + k4;
            const char* lv = buf + kTile * RBK + vrow * RBV + (cc >> 1) * 16 + (cc & 1) * 8 + whalf * (DB / 4) * 128;   // (+ this wavefront's columns)
            const char* v_at[4] = {lv + ((0 ^ (vrow & 3)) << 5), lv + ((1 ^ (vrow & 3)) << 5), lv + ((2 ^ (vrow & 3)) << 5),
                                   lv + ((3 ^ (vrow & 3)) << 5)};
            float sv[4] = {s.x, s.y, s.z, s.w};
            if (softcap) {
#pragma unroll
                for (int i = 0; i < 4; ++i) sv[i] = soft_cap_fn(sv[i] * logit_scale, p.soft_cap, inv_cap) * kLog2e;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) sv[i] *= logit_scale_log2;
            }
            if (MASKED) {                         // the last tile of the piece may be partial
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (tok0 + 4 * a + i >= c_end) sv[i] = -INFINITY;
            }
            const float mx = max_across_rows(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));     // finite: token tok0 is valid
            if (__builtin_amdgcn_ballot_w64(mx > m_ref + kSlack) != 0) {
                mx_seen = mx;
                return false;
            }
            float pr[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) pr[i] = fast_exp2(sv[i] - m_ref);
            l_run += (pr[0] + pr[1]) + (pr[2] + pr[3]);
            // P^T as B operand, rounded to the cache dtype as the reference does before its second dot (flash_decode.py:230)
            const uint2 pb = make_uint2(P2::pack(pr[0], pr[1]), P2::pack(pr[2], pr[3]));
            // ---- O^T[d][head] += V^T P^T ----
            constexpr int VG = DB < 16 ? DB : 16, NVG = DB / VG;
            static_assert(DB % VG == 0, "output blocks in whole groups");
            uint2 va[2][VG];
            auto read_v = [&](int g, int to) {
#pragma unroll
                for (int i = 0; i < VG; ++i)
                    va[to][i] = M::read_tr(v_at[(g * VG + i) & 3] + ((g * VG + i) >> 2) * 128);
            };
            read_v(0, 0);
#pragma unroll
            for (int g = 0; g < NVG; ++g) {
                if (g + 1 < NVG) read_v(g + 1, (g + 1) & 1);
#pragma unroll
                for (int i = 0; i < VG; ++i) acc[g * VG + i] = M::pv(va[g & 1][i], pb, acc[g * VG + i]);
                __builtin_amdgcn_sched_barrier(0);
            }
            return true;
        };

        // ---- the tiles of the piece: the loads of tiles t + 1 and t + 2 are under way while all wavefronts work on tile t
        // (two register tiles by the parity of t; the memory system's latency is longer than the arithmetic of one tile).
        // Page numbers are requested two tiles further ahead, BEFORE the rows of the tile in between: vector loads return
        // in order, so waiting for a number then never waits for rows requested after it.
        // (A wavefront that leaves the inner loop to move its reference does so after the tile's barrier and comes back for
        // the next tile: every wavefront passes exactly one barrier per tile.) ----
        {
            // Direct loads, four staged tiles (tile t in buffer t % 4), and the arithmetic of two tiles in one step: the dot
            // products of tile t + 1 next to the softmax and the PV product of tile t, which do not depend on each other - the
            // matrix cores work on the one while the vector ALU and the LDS round trips of the other are under way (with one
            // tile per step a wavefront's MFMA, softmax and MFMA again each wait for the one before).
            // Step t: wait until this wavefront's loads of tile t + 1 have landed; barrier (every wavefront's have, and every
            // wavefront is done with tile t - 1); request tile t + 3 into the buffer of tile t - 1; q . k of tile t + 1,
            // softmax and PV of tile t.  Loads return in order and every wavefront issues kLoadsPerTile of them per tile:
            // "tile t + 1 has landed" is "at most kLoadsPerTile loads under way" while tile t + 2 has been requested, "none
            // under way" otherwise.  (Loads that the compiler sees - page numbers per row, PM_ROW - only make these waits,
            // and the compiler's own, wait for more than they need.)
            const int n_full = (c_end - c_start) / kTile;          // tiles without rows past the end
            auto staged = [&](int t) { return lds + (t % kStaged) * kTileBytes; };
            auto issue_tile = [&](int t, int32_t pg_id) {
                const uint32_t dst = lds0 + (uint32_t)(t % kStaged) * kTileBytes;
                if constexpr (kRaw) {
                    if (PM == PM_ROW) {
                        if (t < n_tiles) issue_raw_rows(t);
                    } else if (t < n_full) {
                        issue_raw(BoolTag<false>(), t, pg_id);
                    } else if (t < n_tiles) {
                        issue_raw(BoolTag<true>(), t, pg_id);
                    }
                } else if (PM == PM_ROW) {
                    if (t < n_tiles) issue_direct_rows(t, dst);
                } else if (t < n_full) {
                    issue_direct(BoolTag<false>(), t, pg_id, dst);
                } else if (t < n_tiles) {
                    issue_direct(BoolTag<true>(), t, pg_id, dst);
                }
            };
            // the staged tiles are free: no wavefront still reads the previous piece's, none of its loads is under way
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            int32_t pg_hold = 0;
            // kRaw: one round of a tile's bytes - wait until this wavefront's share of tile u has landed in its raw tile (its
            // loads return in order: all but those of tile u + 1), convert it into the staged tile, request tile u + 2 into
            // the raw tile just read.
            // (Page numbers per row: a round requests the bytes of tile u + 2 and then the page numbers of tile u + 4; what
            // has to have landed at its top are the bytes of tile u and the page numbers of tile u + 2, requested two rounds
            // ago in that order: everything but the loads of the round before.)
            auto advance_raw = [&](int u) {
                if (PM == PM_ROW) {
                    if (u + 1 < n_tiles) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerTile + 1) : "memory");
                    else asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
                    if (u < n_tiles) convert_raw(u, staged(u));
                    issue_tile(u + 2, 0);
                    issue_pages(u + 4);
                } else {
                    if (u + 1 < n_tiles) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerTile) : "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    if (u < n_tiles) convert_raw(u, staged(u));
                    const int32_t pg_now = pg_hold;
                    pg_hold = page_id(u + 3);
                    issue_tile(u + 2, pg_now);
                }
            };
            if constexpr (kRaw) {
                if (PM == PM_ROW) {
                    issue_pages(0);
                    issue_pages(1);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    issue_tile(0, 0);
                    issue_pages(2);
                    issue_tile(1, 0);
                    issue_pages(3);
                } else {
                    issue_tile(0, page_id(0));
                    issue_tile(1, page_id(1));
                    pg_hold = page_id(2);
                }
                advance_raw(0);
                advance_raw(1);
            } else if (PM == PM_ROW) {
                // page numbers per row come through LDS as well (issue_pages), two steps ahead of the rows that need them
#pragma unroll
                for (int t = 0; t < 5; ++t) issue_pages(t);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                issue_tile(0, 0);
                issue_tile(1, 0);
                issue_tile(2, 0);
            } else {
                issue_tile(0, page_id(0));
                issue_tile(1, page_id(1));
                issue_tile(2, page_id(2));
                pg_hold = page_id(3);
            }
            load_q();
            // Q^T has to have arrived HERE: the compiler would otherwise wait for its loads where they are first used, inside
            // the tile loop, by counting down to "no load under way" - in every iteration, and the rows requested for the
            // tiles ahead are loads it does not know of.  (An empty asm that takes the registers as operands is such a use.)
#pragma unroll
            for (int i = 0; i < KQ; ++i) asm volatile("" : "+v"(qreg[i].x), "+v"(qreg[i].y), "+v"(qreg[i].z), "+v"(qreg[i].w));
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");          // tile 0 is there
            static_assert(kLoadsPerTile == (kRaw ? 3 : 5), "the waits below count the loads of one tile");
            // (the barrier also waits for this wavefront's LDS operations: its half of the next tile's dot products is in
            // the exchange area, its reads of the partner's half of the tile before are done)
            // PM_ROW: a step requests the rows of tile t + 3 and then the page numbers of tile t + 5, one load more; what has
            // to have landed at the top of step t are the rows of tile t + 1 and the page numbers of tile t + 3, both requested
            // in step t - 2: everything but the loads of step t - 1, which are six, or the one of the page numbers alone.
            auto step = [&](int t) {
                if constexpr (kRaw) {
                    // (every wavefront has converted its share of tile t + 1 and is done with tile t - 1, whose staged tile
                    // takes tile t + 2)
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    advance_raw(t + 2);
                } else if (PM == PM_ROW) {
                    if (t + 2 < n_tiles) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    issue_tile(t + 3, 0);
                    issue_pages(t + 5);
                } else {
                    if (t + 2 < n_tiles) asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    const int32_t pg_now = pg_hold;
                    pg_hold = page_id(t + 4);
                    issue_tile(t + 3, pg_now);
                }
            };
            // The halves of a tile's dot products cross between the two wavefronts of a head tile through the exchange area
            // behind the staged tiles: [tile parity][wavefront][lane] x 16 bytes.  A wavefront writes its half of tile t + 1
            // in step t and reads the partner's after the barrier of step t + 1; the same place is written again in step
            // t + 2, after a barrier that the partner reaches only when that read is done.
            char* const xch = lds + kStaged * kTileBytes + 16;
            auto put_half = [&](int t, const f32x4_t s) {
                *reinterpret_cast<float4*>(xch + (((t & 1) * NW + wave) * 64 + lane) * 16) = make_float4(s.x, s.y, s.z, s.w);
            };
            auto whole = [&](int t, const f32x4_t mine) {
                const float4 o = *reinterpret_cast<const float4*>(xch + (((t & 1) * NW + (wave ^ 1)) * 64 + lane) * 16);
                return f32x4_t{mine.x + o.x, mine.y + o.y, mine.z + o.z, mine.w + o.w};
            };
            f32x4_t s_mine = {0.f, 0.f, 0.f, 0.f}, s_cur = {0.f, 0.f, 0.f, 0.f};
            if (active) {
                s_mine = qk_half(staged(0));
                put_half(0, s_mine);
            }
            int t = 0;
            for (;;) {
                bool gave_up = false;
                for (; t < n_full; ++t) {
                    step(t);
                    if (active) {
                        s_cur = whole(t, s_mine);
                        if (t + 1 < n_tiles) {
                            s_mine = qk_half(staged(t + 1));
                            put_half(t + 1, s_mine);
                        }
                        if (!softmax_pv(t, staged(t), s_cur, BoolTag<false>())) {
                            gave_up = true;
                            break;
                        }
                    }
                }
                if (!gave_up) break;
                do move_reference(); while (!softmax_pv(t, staged(t), s_cur, BoolTag<false>()));
                ++t;
            }
            if (n_full < n_tiles) {                                 // the partial last tile
                step(n_full);
                if (active) {
                    s_cur = whole(n_full, s_mine);
                    while (!softmax_pv(n_full, staged(n_full), s_cur, BoolTag<true>())) move_reference();
                }
            }
        }
        if (!active) return;

        // ---- this wavefront's 16 heads are its own: no merge across wavefronts, results go out from the registers ----
        l_run += __shfl_xor(l_run, 16, 64);
        l_run += __shfl_xor(l_run, 32, 64);
        if (c < heads_here) {
            const int hq = head0 + c;
            const float norm = FP8 ? vscale * fast_rcp(l_run) : fast_rcp(l_run);   // l_run > 0: the piece holds a token
            const float lse_nat = (m_ref + fast_log2(l_run)) * kLn2;
            const int64_t prow = prow0 + (int64_t)(16 * wtile + c) * prow_step;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const float4 o = make_float4(acc[db].x * norm, acc[db].y * norm, acc[db].z * norm, acc[db].w * norm);
                const int d0 = 16 * (whalf * DB + db) + 4 * a;
                if (p.direct) store_out4(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + d0, o, p.out_dtype);
                else *reinterpret_cast<float4*>(p.part_o + prow * DV + d0) = o;
            }
            if (a == 0 && whalf == 0) {
                if (p.direct) {
                    if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse_nat;
                    if (p.pack_lse) store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + DV, lse_nat, p.out_dtype);
                } else {
                    p.part_lse[prow] = lse_nat;
                }
            }
        }
    };   // run_piece

#include "fdk_splitkv_mfma_work.h"
}

// Launch of the shared-tile kernels.  The plan counts head tiles of kSharedTileHeads q heads and one kv head per
// workgroup for them (mfma_heads_per_wg, mfma_kv_heads_per_wg).
template <int QDT, int DK, int DV, int MODE, bool FP8>
int launch_shared(const SplitParams& p_in, hipStream_t stream) {
    if (mfma_work_mode(p_in) != MODE || p_in.fused || p_in.probe || p_in.hg_per_wg != 1 || p_in.tile_heads != kSharedTileHeads)
        return (int)hipErrorInvalidValue;
    constexpr int kTileBytes = 2 * kTile * (DK + DV);
    SplitParams p = p_in;
    p.head_tiles = (p.group + kSharedTileHeads - 1) / kSharedTileHeads;
    p.hg_blocks = p.hkv;
    // staged tiles, the next work item, the exchange area of the half dot products, ...
    const int pm = (p.page_shift >= 0 && p.page_size % kTile == 0) ? PM_TILE : PM_ROW;
    const size_t lds_bytes = !FP8 ? 4 * (size_t)kTileBytes + 16 + 2 * kSharedWaves * 1024 + 8 * 256      // (+ page numbers)
                           : 3 * (size_t)kTileBytes + 16 + 2 * kSharedWaves * 1024 + 2 * 16384 + 4 * 1024 + 8 * 256;   // (+ raw tiles, page numbers)
    p.total_items = (int32_t)((int64_t)p.batch * p.num_splits * p.hg_blocks * p.head_tiles);
    // (the work queue: as many workgroups as are resident at once - one per compute unit at this size - and never more
    // than there are pieces: every workgroup of the queue has to take one, or it would not be counted among the
    // finished ones and the queue's counters would not be put back to zero)
    const int resident = min(p.num_cus > 0 ? p.num_cus : 256, p.total_items);
    p.persistent = MODE == WM_QUEUE ? 1 : 0;
    const unsigned units = (unsigned)(p.hg_blocks * p.head_tiles);
    const dim3 grid = p.balanced ? dim3(units, (unsigned)p.workgroups / units)
                    : p.persistent ? dim3((unsigned)resident)
                                   : dim3(units, (unsigned)p.num_splits, (unsigned)p.batch);
    const dim3 block(64 * kSharedWaves);
    p.shares = (int32_t)grid.y;
    p.grid_x = (int32_t)grid.x;
    p.wavefronts = kSharedWaves;
    const bool reuse = p.head_tiles > 1;
#define FDK_SHARED_LAUNCH(PMV, RU)                                                                                        \
    do {                                                                                                                  \
        const hipError_t e = hipFuncSetAttribute(                                                                         \
            reinterpret_cast<const void*>(&splitkv_mfma_shared_kernel<QDT, PMV, DK, DV, MODE, RU, FP8>),                  \
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);                                                  \
        if (e != hipSuccess) return (int)e;                                                                               \
        hipLaunchKernelGGL((splitkv_mfma_shared_kernel<QDT, PMV, DK, DV, MODE, RU, FP8>), grid, block, lds_bytes, stream, p); \
    } while (0)
    if (pm == PM_TILE) {
        if (reuse) FDK_SHARED_LAUNCH(PM_TILE, true);
        else FDK_SHARED_LAUNCH(PM_TILE, false);
    } else {
        if (reuse) FDK_SHARED_LAUNCH(PM_ROW, true);
        else FDK_SHARED_LAUNCH(PM_ROW, false);
    }
#undef FDK_SHARED_LAUNCH
    return (int)hipGetLastError();
}

template <int DK, int DV, int MODE>
int launch_mfma_shared(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream) {
    if (kv_dtype == FDK_FP8_E4M3)
        return q_dtype == FDK_BF16 ? launch_shared<FDK_BF16, DK, DV, MODE, true>(p, stream) : launch_shared<FDK_FP16, DK, DV, MODE, true>(p, stream);
    if (kv_dtype != q_dtype) return (int)hipErrorInvalidValue;
    return q_dtype == FDK_BF16 ? launch_shared<FDK_BF16, DK, DV, MODE, false>(p, stream) : launch_shared<FDK_FP16, DK, DV, MODE, false>(p, stream);
}

}  // namespace

}  // namespace fdk
