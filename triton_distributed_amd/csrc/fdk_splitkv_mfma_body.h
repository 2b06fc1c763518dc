// The body of the matrix-core split-KV kernels (fdk_splitkv_mfma.h includes this file inside each of its two kernel
// definitions, which supply: QDT, FP8, PM, NBUF, PROBE, MODE, REUSE, kPairedRows, DK = values per q and K row, DV = values
// per V and output row, and the argument block p).  Kept as text shared by the two kernels rather than as a function they
// call: the kernel arguments then stay where the compiler reads them with scalar loads.
    constexpr bool BAL = MODE == WM_SHARES;
    using M = Mma<QDT>;
    using P2 = Pack2<QDT>;
    using R = Regs<FP8, DK, DV>;
    using RK = typename R::K;
    using RV = typename R::V;
    // K and V rows alike and of one power-of-two segment (head_dim 64, 128, 256): K and V loads pair up, every load
    // instruction covers the same rows, and all page modes, fp8 caches, two register buffers and the single-launch
    // form are built.  Otherwise (192, 576 / 512 ...): one buffer, page numbers per tile or per row.
    // (kPairedRows, from the kernel definition: false in the kernels that take every row length through the general code)
    constexpr bool kOneSegment = kPairedRows && DK == DV && RK::D1 == 0;
    // One-byte rows of 192 values are one and a half 128-byte lines: neighbouring kv heads of a token share a line, and
    // workgroups with an odd number of kv heads are mapped so that those neighbours run on one XCD (one L2 fetches the
    // line once; spread over the XCDs in dispatch order every head's L2 fetched both of its partial lines).
    constexpr bool kRowsShareLines = !kOneSegment && FP8 && (DK % 128 != 0 || DV % 128 != 0);
    static_assert(kOneSegment || (NBUF == 1 && !PROBE && (PM == PM_TILE || PM == PM_ROW)), "not built");
    static_assert(DK >= DV && DK % 32 == 0 && DV % 16 == 0, "K rows at least as long as V rows");
    constexpr int NJ = R::NJ;                  // (one segment)
    constexpr int LPR = R::LPR;                // lanes per cache row (one segment)
    constexpr int RPL = R::RPL;                // rows per load instruction (one segment)
    constexpr int NJK = RK::NJ, NJV = RV::NJ;  // load instructions per tile
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int RBK = 2 * DK, RBV = 2 * DV;  // bytes of a staged (16-bit) row
    constexpr int KS = DK / 32;                // k-steps of the QK product
    constexpr int DB = DV / 16;                // 16-column blocks of the output
    constexpr int kScratch = kTile * (RBK + RBV);   // LDS bytes per wavefront: K tile + V tile; also 16 fp32 output rows

#ifdef FDK_TIMELINE
    long long ts[4] = {0, 0, 0, 0};
#endif
    FDK_STAMP(0);
    extern __shared__ __attribute__((aligned(16))) char lds[];      // [nw][kScratch] then m[nw][16], l[nw][16]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int kTileHeads = 16;             // q heads per head tile: the 16 columns of an MFMA tile
    constexpr bool kFirstPieceStraight = true; // (fdk_splitkv_mfma_work.h)
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
    constexpr bool kOnePageId = PM == PM_TILE || PM == PM_ROW;
    struct PageIds { int32_t pg[kOnePageId ? 1 : NJ]; };
    auto page_of_token = [&](int n) { return tbl[p.page_shift < 0 ? n / p.page_size : n >> p.page_shift]; };   // PM_ROW
    // Page numbers of tile t, for any t: positions are clamped to the table only, not to the sequence, so that
    // nothing here waits for kv_len.  The numbers of positions past the end are never used (a full tile has
    // none; the partial last tile asks again, clamped to its last token).
    auto pages_ahead = [&](int t, PageIds& pi) {
        const int tok0 = c_start + t * kTile;
        if (PM == PM_TILE) {
            pi.pg[0] = tbl[min(tok0, p.max_tokens - 1) >> p.page_shift];
        } else if (PM == PM_ROW) {
            pi.pg[0] = page_of_token(min(tok0 + c, p.max_tokens - 1));            // lane (c, any a): row c of the tile
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * RPL;
                if (PM >= PM_LANE) n += lrow;
                n = min(n, p.max_tokens - 1);
                pi.pg[kOnePageId ? 0 : j] = tbl[PM == PM_LANE_DIV ? n / p.page_size : n >> p.page_shift];
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
    // (A scale that is a power of two needs neither: the conversion instruction applies it as an exponent, which is the
    // exact k8 * scale - the code of the folded form with the scale in the conversion instead of in the logit scale.)
    const bool by_exponent = FP8 && !p.fp8_fold && is_pow2_scale(kscale);
    const bool fold = FP8 && (p.fp8_fold || by_exponent);
    const float kconv = by_exponent ? kscale : 1.0f;      // the scale operand of the K conversions of the folded form
    const float logit_scale_log2 = fold && !by_exponent ? p.scale_log2 * kscale : p.scale_log2;
    const float logit_scale = fold && !by_exponent ? p.sm_scale * kscale : p.sm_scale;

    const char* kbase = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES + lpiece * 16;
    const char* vbase = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES + lpiece * 16;
    const uint32_t ksp_bytes = (uint32_t)(p.k_sp * ES), vsp_bytes = (uint32_t)(p.v_sp * ES);
    const uint32_t kst_bytes = (uint32_t)(p.k_st * ES), vst_bytes = (uint32_t)(p.v_st * ES);
    char* my_lds = lds + wave * kScratch;
    char* lds_k = my_lds;
    char* lds_v = my_lds + kTile * RBK;
    const char* kplane = reinterpret_cast<const char*>(p.k) + ((int64_t)kvh * p.k_sh) * ES;   // wave-uniform
    const char* vplane = reinterpret_cast<const char*>(p.v) + ((int64_t)kvh * p.v_sh) * ES;
    // Rows of two segments: the row of the tile and the byte of the cache row that this lane's 16 bytes of load
    // instruction j start at (j is a constant wherever these are used)
    // (rows of two segments) K / V rows that several workgroups read - the q-head tiles of one kv head, which share an
    // XCD, see tiles_on_one_xcd - come by plain loads, so that they stay in that XCD's L2 for the other tiles; rows
    // that are read once, with the non-temporal hint
    auto load_rows16 = [&](const void* ptr) { return REUSE ? *reinterpret_cast<const uint4*>(ptr) : load_stream16(ptr); };
    auto k_row = [&](int j) { return RK::row0(j) + lane / RK::lpr(j); };
    auto v_row = [&](int j) { return RV::row0(j) + lane / RV::lpr(j); };
    auto k_byte = [&](int j) { return RK::seg_byte(j) + (lane % RK::lpr(j)) * 16; };
    auto v_byte = [&](int j) { return RV::seg_byte(j) + (lane % RV::lpr(j)) * 16; };

    auto pages_of = [&](int t, PageIds& pi) {        // clamped to the sequence: for the partial last tile
        const int tok0 = c_start + t * kTile;
        if (PM == PM_TILE) {
            pi.pg[0] = tbl[min(tok0, c_end - 1) >> p.page_shift];      // clamped: any tile index may be asked for
        } else if (PM == PM_ROW) {
            pi.pg[0] = page_of_token(min(tok0 + c, c_end - 1));
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * RPL;
                if (PM >= PM_LANE) n += lrow;
                n = min(n, c_end - 1);
                pi.pg[kOnePageId ? 0 : j] = tbl[PM == PM_LANE_DIV ? n / p.page_size : n >> p.page_shift];
            }
        }
    };
    auto issue = [&](int t, const PageIds& pi, R& rg, auto clamp_tag) {
        const int tok0 = c_start + t * kTile;
        if constexpr (kOneSegment) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                int n = tok0 + j * RPL + lrow;
                if (decltype(clamp_tag)::value) n = min(n, c_end - 1);     // partial tile: always a valid, finite row
                const uint32_t slot = PM == PM_LANE_DIV ? n % p.page_size : (n & pmask);
                // page number x page stride: one 32 x 32 -> 64 bit multiply-add per address (the strides, in bytes, fit
                // 32 bits; a page number is never negative where it is used)
                const uint32_t pg = (uint32_t)pi.pg[kOnePageId ? 0 : j];
                put(rg.k[j], load_stream16(kbase + ((uint64_t)pg * ksp_bytes + (uint64_t)(slot * kst_bytes))));
                put(rg.v[j], load_stream16(vbase + ((uint64_t)pg * vsp_bytes + (uint64_t)(slot * vst_bytes))));
            }
        } else {
            // where row `row` of the tile lies in a pool: its page (per tile, or from the lane that fetched the row's
            // number) and its slot in the page
            auto row_at = [&](int row, uint32_t sp_bytes, uint32_t st_bytes) {
                int n = tok0 + row;
                if (decltype(clamp_tag)::value) n = min(n, c_end - 1);
                const uint32_t slot = p.page_shift < 0 ? n % p.page_size : (n & pmask);
                const uint32_t pg = (uint32_t)(PM == PM_TILE ? pi.pg[0] : __shfl(pi.pg[0], row, 64));
                return (uint64_t)pg * sp_bytes + (uint64_t)(slot * st_bytes);
            };
#pragma unroll
            for (int j = 0; j < NJK; ++j) put(rg.k[j], load_rows16(kplane + k_byte(j) + row_at(k_row(j), ksp_bytes, kst_bytes)));
#pragma unroll
            for (int j = 0; j < NJV; ++j) put(rg.v[j], load_rows16(vplane + v_byte(j) + row_at(v_row(j), vsp_bytes, vst_bytes)));
        }
    };

    // PM_TILE: a tile never leaves its page, so a load address is (page base + first slot of the tile), which
    // is wave-uniform, plus a per-lane byte offset that is the same for every full tile.
    // Per-lane byte offsets of the NJ loads.  Up to head_dim 128 they are kept in registers; the widest rows need
    // the registers elsewhere and add a wave-uniform step per load instead (slightly slower).
    // (Rows of two segments: one offset per segment - the lane's place in the segment's first load - and a
    // wave-uniform step per load.)
    constexpr bool kOffsetsInRegs = kOneSegment && DK <= 128;
    constexpr int kOffsets = kOffsetsInRegs ? NJ : kOneSegment ? 1 : 2;
    uint32_t koff[kOffsets], voff[kOffsets];
    if constexpr (kOneSegment) {
#pragma unroll
        for (int j = 0; j < kOffsets; ++j) {
            koff[j] = (uint32_t)(((int64_t)(j * RPL + lrow) * p.k_st) * ES + lpiece * 16);
            voff[j] = (uint32_t)(((int64_t)(j * RPL + lrow) * p.v_st) * ES + lpiece * 16);
        }
    } else {
        koff[0] = (uint32_t)((int64_t)(lane / RK::LPR0) * p.k_st * ES + k_byte(0));
        koff[1] = RK::NJ1 ? (uint32_t)((int64_t)(lane / RK::LPR1) * p.k_st * ES + k_byte(RK::NJ0)) : 0;
        voff[0] = (uint32_t)((int64_t)(lane / RV::LPR0) * p.v_st * ES + v_byte(0));
        voff[1] = RV::NJ1 ? (uint32_t)((int64_t)(lane / RV::LPR1) * p.v_st * ES + v_byte(RV::NJ0)) : 0;
    }
    const int64_t kstep = (int64_t)RPL * p.k_st * ES;                                 // per load, wave-uniform
    const int64_t vstep = (int64_t)RPL * p.v_st * ES;
    auto issue_full = [&](int t, const PageIds& pi, R& rg) {
        if (PM == PM_TILE) {
            const int tok0 = c_start + t * kTile;
            const int64_t pg = pi.pg[0];
            const int slot0 = tok0 & pmask;
            const char* kp = kplane + (pg * p.k_sp + (int64_t)slot0 * p.k_st) * ES;
            const char* vp = vplane + (pg * p.v_sp + (int64_t)slot0 * p.v_st) * ES;
            if constexpr (kOneSegment) {
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    put(rg.k[j], load_stream16(kOffsetsInRegs ? kp + koff[j] : kp + j * kstep + koff[0]));
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    put(rg.v[j], load_stream16(kOffsetsInRegs ? vp + voff[j] : vp + j * vstep + voff[0]));
            } else {
#pragma unroll
                for (int j = 0; j < NJK; ++j)
                    put(rg.k[j], load_rows16(kp + (int64_t)RK::row0(j) * p.k_st * ES + koff[j < RK::NJ0 ? 0 : 1]));
#pragma unroll
                for (int j = 0; j < NJV; ++j)
                    put(rg.v[j], load_rows16(vp + (int64_t)RV::row0(j) * p.v_st * ES + voff[j < RV::NJ0 ? 0 : 1]));
            }
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
        } else if (FP8 && !kOneSegment) {
            // rows of two segments: K and V have their own load instructions; 16 one-byte values become two 16-byte
            // chunks of 16-bit values (chunk = value index / 8)
            auto k_dequant = [&](const uint32_t (&in)[4], uint32_t (&o)[8]) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if (fold) {
                        o[2 * w] = P2::from_fp8(in[w], false, kconv);
                        o[2 * w + 1] = P2::from_fp8(in[w], true, kconv);
                    } else {
                        const f32x2_t k01 = __builtin_amdgcn_cvt_pk_f32_fp8(in[w], false);
                        const f32x2_t k23 = __builtin_amdgcn_cvt_pk_f32_fp8(in[w], true);
                        o[2 * w] = P2::pack(k01.x * kscale, k01.y * kscale);
                        o[2 * w + 1] = P2::pack(k23.x * kscale, k23.y * kscale);
                    }
                }
            };
#pragma unroll
            for (int j = 0; j < NJK; ++j) {
                uint32_t ko[8];
                k_dequant(rg.k[j], ko);
#pragma unroll
                for (int half = 0; half < 2; ++half)
                    *reinterpret_cast<uint4*>(lds_k + k_off<RBK>(k_row(j), (k_byte(j) >> 3) + half)) =
                        make_uint4(ko[4 * half], ko[4 * half + 1], ko[4 * half + 2], ko[4 * half + 3]);
            }
#pragma unroll
            for (int j = 0; j < NJV; ++j) {
                uint32_t vo[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    vo[2 * w] = P2::from_fp8(rg.v[j][w], false);
                    vo[2 * w + 1] = P2::from_fp8(rg.v[j][w], true);
                }
#pragma unroll
                for (int half = 0; half < 2; ++half)
                    *reinterpret_cast<uint4*>(lds_v + v_off<RBV>(v_row(j), (v_byte(j) >> 3) + half)) =
                        make_uint4(vo[4 * half], vo[4 * half + 1], vo[4 * half + 2], vo[4 * half + 3]);
            }
        } else if (FP8) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int r = j * RPL + lrow;
                uint32_t ko[8], vo[8];
                if (fold) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        ko[2 * w] = P2::from_fp8(rg.k[j][w], false, kconv);
                        ko[2 * w + 1] = P2::from_fp8(rg.k[j][w], true, kconv);
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
                    *reinterpret_cast<uint4*>(lds_k + k_off<RBK>(r, ch)) =
                        make_uint4(ko[4 * half], ko[4 * half + 1], ko[4 * half + 2], ko[4 * half + 3]);
                    *reinterpret_cast<uint4*>(lds_v + v_off<RBV>(r, ch)) =
                        make_uint4(vo[4 * half], vo[4 * half + 1], vo[4 * half + 2], vo[4 * half + 3]);
                }
            }
        } else if constexpr (kOneSegment) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int r = j * RPL + lrow;
                *reinterpret_cast<uint4*>(lds_k + k_off<RBK>(r, lpiece)) = get(rg.k[j]);
                *reinterpret_cast<uint4*>(lds_v + v_off<RBV>(r, lpiece)) = get(rg.v[j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NJK; ++j) *reinterpret_cast<uint4*>(lds_k + k_off<RBK>(k_row(j), k_byte(j) >> 4)) = get(rg.k[j]);
#pragma unroll
            for (int j = 0; j < NJV; ++j) *reinterpret_cast<uint4*>(lds_v + v_off<RBV>(v_row(j), v_byte(j) >> 4)) = get(rg.v[j]);
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
        constexpr bool kReadVEarly = kOneSegment && DK <= 128 && !FP8;
        const int k4 = c >> 2, cc = c & 3;
        const int vrow = 4 * a + k4;
        uint2 va[DB];
        if (kReadVEarly) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) ka[ks] = *reinterpret_cast<const uint4*>(lds_k + k_off<RBK>(c, 4 * ks + a));
#pragma unroll
            for (int db = 0; db < DB; ++db) va[db] = M::read_tr(lds_v + v_off<RBV>(vrow, 2 * db + (cc >> 1)) + (cc & 1) * 8);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (!kReadVEarly) ka[ks] = *reinterpret_cast<const uint4*>(lds_k + k_off<RBK>(c, 4 * ks + a));
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
        // (finite: token tok0 is valid.  Without the LDS crossbar where the vector ALU and the LDS are what a kernel waits
        // for - one-byte caches, the general row code; the 16-bit one-segment kernels wait for memory and stay as they are)
        if constexpr (FP8 || !kPairedRows) {
            mx = max_across_rows(mx);
        } else {
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        }
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
            if (!kReadVEarly) va[db] = M::read_tr(lds_v + v_off<RBV>(vrow, 2 * db + (cc >> 1)) + (cc & 1) * 8);
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
                    float* dst = p.part_o + (prow0 + (int64_t)c * prow_step) * DV + d0;
                    if (p.fused) {
                        st_agent2(dst, o.x, o.y);
                        st_agent2(dst + 2, o.z, o.w);
                    } else {
                        *reinterpret_cast<float4*>(dst) = o;
                    }
                }
            }
        };
        constexpr bool kSmallTiles = kOneSegment ? kTile * (DK + DV) * (FP8 ? 1 : 2) <= 4096 : rows2_eight_share(FP8, DK, DV);
        if (ti_n == 1) merge(IntTag<1>());
        else if (ti_n == 2) merge(IntTag<2>());
        else if (ti_n == 4 || !kSmallTiles) merge(IntTag<4>());
        else merge(IntTag<kSmallTiles ? 8 : 4>());
        if (tix == 0 && a == 0) {
            if (p.direct) {
                if (p.lse) p.lse[(int64_t)b * p.lse_sb + hq] = lse_nat;
                if (p.pack_lse) store_out(p.out, (int64_t)b * p.out_sb + (int64_t)hq * p.out_sh + DV, lse_nat, p.out_dtype);
            } else if (p.fused) {
                st_agent1(p.part_lse + prow0 + (int64_t)c * prow_step, lse_nat);
            } else {
                p.part_lse[prow0 + (int64_t)c * prow_step] = lse_nat;
            }
        }
    }
    if constexpr (kOneSegment) {                          // (the single-launch form is built for these head dims only)
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
                merge_rows<DV, NR>(p, row0, hq_of, min(NR, n_rows - r0), mr.piece_step, mr.live, b, lane);
            }
        }
    }
    }
    FDK_STAMP(3);
#ifdef FDK_TIMELINE
    timeline_out();
#endif

    };   // run_piece
