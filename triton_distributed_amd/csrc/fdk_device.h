// Shared device-side definitions for the flash-decode kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fdk.h"

namespace fdk {

constexpr int kHeadDim = 128;       // head dimension of the vector path (the matrix-core path: see mfma_supported)
constexpr int kWaveSize = 64;
constexpr int kBalanceGranule = 16;  // tokens per unit of the balanced partition: one 16-token tile (with 64 tokens a share of a
                                     // few hundred tokens was up to an eighth longer than its neighbours)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Kernel arguments of the split kernels (passed by value).
struct SplitParams {
    const void* q;
    const void* k;
    const void* v;
    const int32_t* block_table;
    const int32_t* kv_lens;
    const float* k_scale;
    const float* v_scale;
    float* part_o;    // [B, Hq, S, D] fp32 (S > 1)
    float* part_lse;  // [B, Hq, S]    fp32 (S > 1)
    void* out;        // final output, written directly when S == 1
    float* lse;       // may be null
    int32_t* counters;  // zeroed scratch counters of the work queue: [0] head, [1] finished workgroups
    int2* slot_desc;    // balanced mode: where the pieces of (sequence, unit) are - {first share, live pieces} - written
                        // by the piece that holds the sequence's first token, read by the combine
    int64_t q_sb, q_sh;
    int64_t k_sp, k_st, k_sh;  // page / token / head strides, elements
    int64_t v_sp, v_st, v_sh;
    int64_t tbl_sb;
    int64_t out_sb, out_sh, lse_sb;
    int32_t batch, hq, hkv, group, head_dim;
    int32_t v_head_dim;             // values per V / output row (head_dim: per q / K row)
    int32_t page_size, page_shift;  // page_shift = log2(page_size) or -1
    int32_t num_splits, chunk;
    int32_t chunk_floor;            // chunk mode, > 0: chunks follow each sequence's own length (chunk_tokens_of)
    int32_t max_tokens;             // block_table columns * page_size: kv_len is clamped to it
    int32_t head_tiles;             // ceil(group / heads-per-workgroup)
    int32_t hg_per_wg, hg_blocks;   // kv-head groups per workgroup / workgroups along the kv-head axis
    int32_t out_dtype;              // fdk_dtype
    int32_t pack_lse;
    int32_t direct;                 // 1: single split, write the final (out, lse) instead of partials
    int32_t persistent, total_items, num_cus;
    int32_t balanced, workgroups;   // balanced mode: the KV ranges are cut into `workgroups` equal shares
    // What the launch was given, as arguments: the kernels must not read gridDim / blockDim where a result is on the way
    // to the first loads - those live in the hidden arguments, which are fetched only when first used, and a fetch from
    // the argument buffer that is not part of the batch at kernel entry costs a round trip of its own (measured 1.4 us).
    int32_t shares;                 // balanced mode: gridDim.y
    int32_t grid_x;                 // gridDim.x
    int32_t wavefronts;             // blockDim.x / 64
    int32_t rows_per_slot, heads_per_tile;   // balanced mode: partial rows per slot, q heads per tile (<= tile_heads)
    int32_t piece_cost;             // balanced mode: granules a sequence counts for on top of its own
    int32_t tune_wavefronts, tune_buffers;   // 0: chosen by the launcher; else the caller's override (measurements)
    int32_t* length_feedback;       // set where this kernel ends the call: {min, max of the clamped kv_lens, epoch, batch} goes here
    int32_t feedback_epoch;
    long long* timeline;            // timeline build only (see the split kernel): eight int64 per wavefront
    int64_t timeline_len;
    int32_t timeline_rotate;        // timeline build only: rotation of the head blocks over the workgroups
    int32_t fp8_fold;               // fp8 cache, matrix-core path: the K scale multiplies the logits (see the kernel)
    int32_t probe;                  // 1: load pipeline only (measurement aid), no results
    uint32_t ws_bytes;              // fused: bytes of the workspace (part_o onwards), below 2^32
    int32_t fused;                  // 1: the last piece of a (sequence, head block, head tile) to finish merges its
                                    // pieces into (out, lse); tickets at counters[2 + ...], no combine launch
    float scale_log2;               // sm_scale * log2(e)
    float soft_cap;                 // > 0: on (applied to natural-unit logits)
    float sm_scale;
    int32_t tile_heads;             // q heads of a kv head that one workgroup covers: 16 (an MFMA tile), or 64 in the
                                    // kernels whose wavefronts share the staged tiles (fdk_splitkv_mfma_shared.h)
};

struct CombineParams {
    const float* part_o;
    const float* part_lse;
    const int2* slot_desc;          // balanced mode: as in SplitParams
    const int32_t* kv_lens;
    void* out;
    float* lse;
    int64_t out_sb, out_sh, lse_sb;
    int32_t batch, hq, head_dim;    // head_dim: values per output row
    int32_t num_splits, chunk;
    int32_t chunk_floor;            // as in SplitParams
    int32_t max_tokens;
    int32_t out_dtype;
    int32_t pack_lse;
    // balanced mode (see the split kernel): where the pieces of a (sequence, head) row are
    int32_t balanced, workgroups;
    int32_t group, kv_heads_per_wg, head_tiles, hg_blocks, rows_per_slot, heads_per_tile, piece_cost;
    int32_t rows_per_pass;          // balanced mode: rows of a slot the workgroup covers at once (blockDim.x / (head_dim / 4))
    int32_t tile_heads;             // as in SplitParams
    int32_t* length_feedback;       // as in SplitParams (null: nothing is stored)
    int32_t feedback_epoch;
};

struct CombineRanksParams {
    const void* partial;
    const float* partial_lse;
    const int32_t* kv_lens;
    void* out;
    float* lse;
    int64_t stride_r, stride_b, stride_h;
    int64_t lse_stride_r, lse_stride_b;
    int64_t out_sb, out_sh, lse_sb_out;
    int32_t num_ranks, batch, hq, head_dim;
    int32_t partial_dtype, out_dtype, packed;
};

struct KvAppendParams {
    const void* qkv;
    const void* q_weight;
    const void* k_weight;
    const float* cos;
    const float* sin;
    const int32_t* block_table;
    const int32_t* kv_lens;
    const float* k_scale;
    const float* v_scale;
    void* k_cache;
    void* v_cache;
    void* q_out;
    int64_t qkv_sb, qkv_st, qkv_sh;
    int64_t cs_sb, cs_sp;
    int64_t tbl_sb;
    int64_t k_sp, k_st, k_sh, v_sp, v_st, v_sh;
    int64_t qo_sb, qo_st, qo_sh;
    int32_t batch, new_tokens, hq, hkv, head_dim;
    int32_t page_size, max_pages, num_pages, max_positions;
    float q_eps, k_eps;
};

// Launchers implemented in the .hip files; return hipError_t as int.
int launch_kv_append(const KvAppendParams& p, int qkv_dtype, int kv_dtype, hipStream_t stream);
int launch_splitkv_valu(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);
int launch_splitkv_mfma(const SplitParams& p, int q_dtype, int kv_dtype, hipStream_t stream);
int launch_splitkv_mfma_probe(const SplitParams& p, int kv_dtype, hipStream_t stream);      // head_dim 128
// (sink: four writable bytes for a checksum that is practically never stored; keeps the loads alive)
int launch_linear_read(const void* buf, size_t bytes, int nontemporal, int workgroups, uint32_t* sink, hipStream_t stream);
int launch_combine(const CombineParams& p, hipStream_t stream);
int launch_combine_ranks(const CombineRanksParams& p, hipStream_t stream);
bool valu_supported(int q_dtype, int kv_dtype, int group, int head_dim);
// workgroups per (sequence, split) of the VALU path for this head layout
int valu_units_per_seq(int hkv, int group, bool heads_contiguous, int kv_dtype);
bool mfma_supported(int q_dtype, int kv_dtype, int group, int head_dim, int v_head_dim);
int valu_heads_per_wg(int group);
int mfma_heads_per_wg(int group, int row_values, int kv_dtype);   // q heads of a kv head per workgroup (SplitParams.tile_heads)
int mfma_kv_heads_per_wg(int batch, int hkv, int group, int num_cus, int row_values, int kv_dtype);   // row_values: head_dim + v_head_dim
int mfma_units_per_seq(int hkv, int group, int kv_heads_per_wg, int tile_heads);

#if defined(__HIPCC__)

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// 16-byte load of cache data that is read once: the non-temporal hint keeps the stream out of the caches'
// replacement order, which on MI355X is worth about a tenth of the achievable read bandwidth.
__device__ __forceinline__ uint4 load_stream16(const void* p) {
    const u32x4_t x = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(x.x, x.y, x.z, x.w);
}

// Whether an fp8 dequantisation scale is a power of two within 2^-40 .. 2^40 (1.0, the usual value of an unscaled cache,
// among them): then k8 * scale is exactly what the conversion instruction gives with the scale as its exponent operand.
__device__ __forceinline__ bool is_pow2_scale(float s) {
    const uint32_t b = __builtin_bit_cast(uint32_t, s);
    return (b & 0x007fffffu) == 0 && (b >> 23) >= 127u - 40u && (b >> 23) <= 127u + 40u;
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of LANES lanes (LANES in {4, 8, 16}); every lane of the group gets the total.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
    x += dpp_mov<0xB1>(x);                 // quad_perm [1,0,3,2]
    x += dpp_mov<0x4E>(x);                 // quad_perm [2,3,0,1]
    if (LANES >= 8) x += dpp_mov<0x141>(x);   // row_half_mirror
    if (LANES >= 16) x += dpp_mov<0x140>(x);  // row_mirror
    return x;
}

// Inclusive prefix sum over the 64 lanes with DPP row shifts and row broadcasts (no LDS traffic).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_add_i32(int x) {
    // lanes outside ROW_MASK and shifted-in positions contribute 0
    return x + __builtin_amdgcn_update_dpp(0, x, CTRL, ROW_MASK, 0xF, ROW_MASK == 0xF);
}
__device__ __forceinline__ int wave_scan_i32(int x) {
    x = dpp_add_i32<0x111, 0xF>(x);   // row_shr:1
    x = dpp_add_i32<0x112, 0xF>(x);   // row_shr:2
    x = dpp_add_i32<0x114, 0xF>(x);   // row_shr:4
    x = dpp_add_i32<0x118, 0xF>(x);   // row_shr:8  -> scan within each row of 16
    x = dpp_add_i32<0x142, 0xA>(x);   // row_bcast:15 into rows 1 and 3
    x = dpp_add_i32<0x143, 0xC>(x);   // row_bcast:31 into rows 2 and 3
    return x;
}
__device__ __forceinline__ int wave_sum_i32(int x) { return __builtin_amdgcn_readlane(wave_scan_i32(x), 63); }

// Length feedback (one wavefront): the smallest and the largest of the clamped kv_lens, for a host that cannot read
// them otherwise.  The four values go out as one 16-byte store.
__device__ __forceinline__ void store_length_bounds(int32_t* feedback, const int32_t* kv_lens, int batch, int max_tokens,
                                                    int epoch, int lane) {
    int lo = 0x7fffffff, hi = 0;
    for (int b0 = 0; b0 < batch; b0 += 64) {
        if (b0 + lane < batch) {
            const int n = max(min(kv_lens[b0 + lane], max_tokens), 0);
            lo = min(lo, n);
            hi = max(hi, n);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off, 64));
        hi = max(hi, __shfl_xor(hi, off, 64));
    }
    if (lane == 0) *reinterpret_cast<int4*>(feedback) = make_int4(lo, hi, epoch, batch);
}

// Chunk mode: tokens per split of a sequence that holds kv_len tokens.  chunk_floor == 0: the plan's chunk, whatever
// the sequence holds (the plan sized it for the longest sequence the host expects).  chunk_floor > 0: the sequence's
// own length in num_splits equal parts of whole 16-token tiles, at least chunk_floor and at most the plan's chunk
// tokens each - as the reference cuts a sequence (flash_decode.py:151-153: cdiv(kv_len, NUM_KV_SPLITS)), so that a
// sequence shorter than the host's bound still spreads over all the workgroups it was given.
__device__ __forceinline__ int chunk_tokens_of(int kv_len, int num_splits, int chunk, int chunk_floor) {
    if (chunk_floor == 0) return chunk;
    const int even = ((kv_len + num_splits - 1) / num_splits + 15) & ~15;
    return min(max(even, chunk_floor), chunk);
}

// Reductions over the 64 lanes with DPP only (no LDS traffic): butterflies inside each row of 16, then the row
// results are passed down the rows (row_bcast:15 into rows 1 and 3, row_bcast:31 into rows 2 and 3), so that
// lane 63 holds the total, which every lane then reads.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_rows(float old, float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, x),
                                                                 CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float lane63(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}
__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_mov<0xB1>(x));                 // quad_perm [1,0,3,2]   (permutations: every lane has a source)
    x = fmaxf(x, dpp_mov<0x4E>(x));                 // quad_perm [2,3,0,1]
    x = fmaxf(x, dpp_mov<0x141>(x));                // row_half_mirror
    x = fmaxf(x, dpp_mov<0x140>(x));                // row_mirror
    x = fmaxf(x, dpp_rows<0x142, 0xA>(x, x));       // rows that take no part keep their own value
    x = fmaxf(x, dpp_rows<0x143, 0xC>(x, x));
    return lane63(x);
}
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_mov<0xB1>(x);
    x += dpp_mov<0x4E>(x);
    x += dpp_mov<0x141>(x);
    x += dpp_mov<0x140>(x);
    x += dpp_rows<0x142, 0xA>(0.f, x);              // rows that take no part add nothing
    x += dpp_rows<0x143, 0xC>(0.f, x);
    return lane63(x);
}

// soft cap: cap * tanh(x / cap), tanh(y) = 1 - 2 / (exp(2y) + 1)
__device__ __forceinline__ float soft_cap_fn(float x, float cap, float inv_cap) {
    float e = fast_exp2(2.0f * kLog2e * x * inv_cap);
    return cap * (1.0f - 2.0f * fast_rcp(e + 1.0f));
}

// dtype helpers -----------------------------------------------------------------------------------
template <int DT> struct Pack2;  // two 16-bit floats in a dword
template <> struct Pack2<FDK_BF16> {
    using vec = bf16x2_t;
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(vec, a), __builtin_bit_cast(vec, b), c, false);
    }
    static __device__ __forceinline__ float lo(uint32_t a) { return __builtin_bit_cast(float, a << 16); }
    static __device__ __forceinline__ float hi(uint32_t a) { return __builtin_bit_cast(float, a & 0xffff0000u); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        vec r = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, r);
    }
    // bytes 0,1 (hi = false) or 2,3 (hi = true) of four e4m3 values, converted exactly, in one instruction
    // (v_cvt_scalef32_pk_bf16_fp8 applies only the exponent of its scale operand; 1.0 leaves the value alone)
    static __device__ __forceinline__ uint32_t from_fp8(uint32_t four, bool hi) {
        return __builtin_bit_cast(uint32_t, hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(four, 1.0f, true)
                                               : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(four, 1.0f, false));
    }
    // ... times 2^e, e the exponent of `pow2` (a power of two): still exact, e4m3 values have four significant bits
    static __device__ __forceinline__ uint32_t from_fp8(uint32_t four, bool hi, float pow2) {
        return __builtin_bit_cast(uint32_t, hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(four, pow2, true)
                                               : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(four, pow2, false));
    }
};
template <> struct Pack2<FDK_FP16> {
    using vec = f16x2_t;
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(vec, a), __builtin_bit_cast(vec, b), c, false);
    }
    static __device__ __forceinline__ float lo(uint32_t a) { return (float)__builtin_bit_cast(vec, a).x; }
    static __device__ __forceinline__ float hi(uint32_t a) { return (float)__builtin_bit_cast(vec, a).y; }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        vec r = {(_Float16)a, (_Float16)b};
        return __builtin_bit_cast(uint32_t, r);
    }
    static __device__ __forceinline__ uint32_t from_fp8(uint32_t four, bool hi) {
        return __builtin_bit_cast(uint32_t, hi ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(four, 1.0f, true)
                                               : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(four, 1.0f, false));
    }
    static __device__ __forceinline__ uint32_t from_fp8(uint32_t four, bool hi, float pow2) {
        return __builtin_bit_cast(uint32_t, hi ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(four, pow2, true)
                                               : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(four, pow2, false));
    }
};

// Store one output element in the requested dtype.
__device__ __forceinline__ void store_out(void* base, int64_t idx, float x, int dtype) {
    if (dtype == FDK_BF16) {
        reinterpret_cast<__bf16*>(base)[idx] = (__bf16)x;
    } else if (dtype == FDK_FP16) {
        reinterpret_cast<_Float16*>(base)[idx] = (_Float16)x;
    } else {
        reinterpret_cast<float*>(base)[idx] = x;
    }
}

// Store four consecutive output elements; one vector store when the address allows it.
__device__ __forceinline__ void store_out4(void* base, int64_t idx, float4 x, int dtype) {
    if (dtype == FDK_FP32) {
        float* q = reinterpret_cast<float*>(base) + idx;
        if ((reinterpret_cast<uintptr_t>(q) & 15u) == 0) {
            *reinterpret_cast<float4*>(q) = x;
        } else {
            q[0] = x.x; q[1] = x.y; q[2] = x.z; q[3] = x.w;
        }
        return;
    }
    uint16_t* q = reinterpret_cast<uint16_t*>(base) + idx;
    const uint2 v = dtype == FDK_BF16 ? make_uint2(Pack2<FDK_BF16>::pack(x.x, x.y), Pack2<FDK_BF16>::pack(x.z, x.w))
                                      : make_uint2(Pack2<FDK_FP16>::pack(x.x, x.y), Pack2<FDK_FP16>::pack(x.z, x.w));
    if ((reinterpret_cast<uintptr_t>(q) & 7u) == 0) {
        *reinterpret_cast<uint2*>(q) = v;
    } else {
        q[0] = (uint16_t)v.x; q[1] = (uint16_t)(v.x >> 16); q[2] = (uint16_t)v.y; q[3] = (uint16_t)(v.y >> 16);
    }
}

#endif  // __HIPCC__

}  // namespace fdk
