/*
 * fdk - measurement aids of the benchmark.  Not part of the decode path and without a counterpart in the
 * reference: nothing here changes a result.  A product caller includes fdk.h only and leaves
 * fdk_decode_args.measure null.
 *
 *   fdk_measure_args        overrides of how the matrix-core split kernel is shaped, the load-only probe of that
 *                           kernel, and the per-wavefront clock readings of the timeline build
 *   fdk_probe_linear_read   a plain streaming read, the ceiling the decode kernels are compared with
 */
#ifndef FDK_MEASURE_H_
#define FDK_MEASURE_H_

#include "fdk.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct fdk_measure_args {
    uint32_t struct_size; /* = sizeof(fdk_measure_args); grows at the end like the structs of fdk.h */
    uint32_t probe_loads; /* 1: run only the load pipeline of the split kernel (same pieces, addresses and load
                             instructions, no arithmetic); out / lse / workspace are left undefined and no combine
                             runs.  Matrix-core path, head_dim 128 */

    /* 0 = let the library choose (what a caller wants).  Wavefronts per workgroup of the matrix-core split kernel
     * (4 or 8) and register buffers per wavefront (1 or 2), i.e. how many tiles of loads a compute unit keeps under
     * way.  A value the kernel cannot run with the plan's head blocks is ignored.  shares_per_cu (1..4): balanced
     * mode's workgroups per compute unit, which changes the plan (workgroups, workspace).  They change timing
     * only, never results. */
    int32_t wavefronts;
    int32_t buffers;
    int32_t shares_per_cu;

    /* Timeline build only (python -m triton_distributed_amd.build --timeline -> libfdk_timeline.so; the product
     * library ignores all three).  rotate_heads = r: workgroup x of a sequence takes head block (x + r) mod (head
     * blocks) instead of x (chunk mode and single pass, one q-head tile): which XCD reads which head's rows then
     * changes, the rows themselves do not.  timeline: eight int64 per wavefront of the matrix-core split kernel,
     * at [8 * (linear workgroup * wavefronts + wavefront)]: the 100 MHz clock at kernel entry, before the first
     * K/V loads of the wavefront's last piece, after that piece's last tile, after its merge and stores (0 if the
     * wavefront left earlier); the XCD, the kv head, the sequence, the linear workgroup index.  8-byte aligned;
     * wavefronts beyond timeline_len / 8 store nothing. */
    int32_t rotate_heads;
    int64_t* timeline;
    int64_t timeline_len;

    /* 1: plan equal shares of the whole batch (balanced mode) wherever the matrix-core path can run them (two or more
     * sequences), whatever the length hints say - for timing that plan against the one the library chooses
     * (bench.py --op plan-sweep).  Changes the plan (workgroups, workspace), never results. */
    int32_t force_balanced;
    int32_t reserved;
} fdk_measure_args;

/* A streaming read of buf[0, bytes) by `workgroups` workgroups of 256 threads with 16-byte loads (non-temporal if
 * `nontemporal`); buf is not written.  Its rate is the ceiling the decode kernels are compared with
 * (bench.py --op ceiling). */
int fdk_probe_linear_read(const void* buf, size_t bytes, int nontemporal, int workgroups, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* FDK_MEASURE_H_ */
