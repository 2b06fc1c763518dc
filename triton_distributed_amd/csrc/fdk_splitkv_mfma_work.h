// How the pieces of a call are handed out to the workgroups of the matrix-core split-KV kernels: the second half of
// each kernel's body (the kernel definitions include this file after they have defined run_piece, write_empty_rows
// and: p, lane, wave, nh = kv heads per workgroup, hl = this wavefront's kv head within the block, tix = its index among
// the wavefronts of that head, s_next = an int in LDS, kTileHeads = q heads per head tile, kOneSegment, MODE,
// kFirstPieceStraight = whether a share's first piece gets straight-line code of its own, see below).
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
            int split = blockIdx.y, pb = blockIdx.z;
            int ht = 0, hgb = blockIdx.x;
#ifdef FDK_TIMELINE
            if (p.head_tiles == 1) hgb = (int)((blockIdx.x + (unsigned)p.timeline_rotate) % (unsigned)p.grid_x);
#endif
            if constexpr (kOneSegment) {
                if (p.head_tiles > 1) {
                    ht = blockIdx.x % p.head_tiles;
                    hgb = blockIdx.x / p.head_tiles;
                }
            } else if (kRowsShareLines && (nh & 1) && p.hg_blocks > 1) {
                // every unit of a (sequence, split) on one XCD: neighbouring kv heads share 128-byte lines
                int row, unit;
                tiles_on_one_xcd((int)(blockIdx.x + p.grid_x * (blockIdx.y + p.num_splits * blockIdx.z)),
                                 p.num_splits * p.batch, p.grid_x, row, unit);
                ht = unit % p.head_tiles;
                hgb = unit / p.head_tiles;
                split = row % p.num_splits;
                pb = row / p.num_splits;
            } else if (p.head_tiles > 1) {
                // the q-head tiles of a (sequence, split, kv-head block) on one XCD: see tiles_on_one_xcd
                int row;
                tiles_on_one_xcd((int)(blockIdx.x + p.grid_x * (blockIdx.y + p.num_splits * blockIdx.z)),
                                 p.hg_blocks * p.num_splits * p.batch, p.head_tiles, row, ht);
                hgb = row % p.hg_blocks;
                row /= p.hg_blocks;
                split = row % p.num_splits;
                pb = row / p.num_splits;
            }
            // the last split runs to the end of the sequence: a max_kv_len hint that was too small costs balance, not tokens
            const int64_t unit_row0 = ((int64_t)pb * p.hq + hgb * nh * p.group + ht * kTileHeads) * p.num_splits;
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
            int64_t prow0 = ((int64_t)pb * p.hq + (hgb * nh + hl) * p.group + ht * kTileHeads) * p.num_splits + split;
            MergeRows mr;
            mr.live = 0;                                              // from kv_len, inside run_piece
            mr.base = ((int64_t)pb * p.hq + hgb * nh * p.group + ht * kTileHeads) * p.num_splits;
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
        int wc_of_wg = blockIdx.y, bu_of_wg = blockIdx.x;   // grid = (units, shares)
        if constexpr (!kOneSegment) {
            if (kRowsShareLines && (nh & 1) && p.hg_blocks > 1) {   // every unit of a share on one XCD
                tiles_on_one_xcd((int)(blockIdx.x + p.grid_x * blockIdx.y), p.shares, p.grid_x, wc_of_wg, bu_of_wg);
            } else if (p.head_tiles > 1) {                  // the q-head tiles of a (share, kv-head block) on one XCD
                int row, tile;
                tiles_on_one_xcd((int)(blockIdx.x + p.grid_x * blockIdx.y), p.hg_blocks * p.shares, p.head_tiles, row, tile);
                bu_of_wg = (row % p.hg_blocks) * p.head_tiles + tile;
                wc_of_wg = row / p.hg_blocks;
            }
        }
        const int wc = wc_of_wg, bu = bu_of_wg;
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
                    write_empty_rows(b0 + __builtin_ctzll(empty), ((bu / p.head_tiles) * nh + hl) * p.group + ht_e * kTileHeads,
                                     min(kTileHeads, p.group - ht_e * kTileHeads));
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
        if constexpr (kFirstPieceStraight) {
            const Piece first = piece_of(piece_end);
            if (first.c_limit > first.c_start) run_piece(first.pb, first.hgb, first.ht, first.c_start, first.c_limit, first.prow0, 1, first.mr);
            if (!next_piece(first, piece_end)) return;
            for (;;) {
                __syncthreads();                                      // the LDS scratch is reused by the next piece
                const Piece pp = piece_of(piece_end);
                if (pp.c_limit > pp.c_start) run_piece(pp.pb, pp.hgb, pp.ht, pp.c_start, pp.c_limit, pp.prow0, 1, pp.mr);
                if (!next_piece(pp, piece_end)) return;
            }
        } else {
            // (kernels whose piece needs every register: one copy of it, in the loop)
            for (;;) {
                const Piece pp = piece_of(piece_end);
                if (pp.c_limit > pp.c_start) run_piece(pp.pb, pp.hgb, pp.ht, pp.c_start, pp.c_limit, pp.prow0, 1, pp.mr);
                if (!next_piece(pp, piece_end)) return;
                __syncthreads();                                      // the LDS scratch is reused by the next piece
            }
        }
    }
