/*
 * A C99 caller of libfdk.so that uses nothing but the HIP runtime's C API and include/fdk.h: the form in which
 * a non-Python host (the reference's AOT launcher is C, python/triton_dist/tools/compile/compile.c) would bind
 * the decode path.  Builds a small paged bf16 problem on the host, runs fdk_plan / fdk_workspace_bytes /
 * fdk_decode on the GPU and compares the result with a naive double-precision attention over the same
 * (bf16-rounded) inputs.  Prints "OK" and returns 0 on success.
 *
 *   gcc -std=c99 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -I<repo>/include fdk_c_client.c \
 *       -L<repo>/triton_distributed_amd/lib -lfdk -L/opt/rocm/lib -lamdhip64 -lm -o fdk_c_client
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fdk.h"

#define CHECK_HIP(x)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                \
            return 2;                                                                     \
        }                                                                                 \
    } while (0)

static uint16_t f2bf(float f) { /* round to nearest even */
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float bf2f(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static float frand(uint32_t* s) { /* uniform in [-1, 1) */
    *s = *s * 1664525u + 1013904223u;
    return (float)((*s >> 8) & 0xffff) / 32768.0f - 1.0f;
}

enum { B = 3, HQ = 8, HKV = 2, D = 128, P = 4, MAXP = 40, POOL = 64 };

int main(void) {
    static const int32_t lens[B] = {37, 5, 150};
    const float scale = 1.0f / sqrtf((float)D);
    uint32_t seed = 12345u;
    size_t nq = (size_t)B * HQ * D, nkv = (size_t)POOL * P * HKV * D;
    uint16_t *q = malloc(nq * 2), *k = malloc(nkv * 2), *v = malloc(nkv * 2), *out = malloc(nq * 2);
    float* lse = malloc((size_t)B * HQ * 4);
    int32_t* table = malloc((size_t)B * MAXP * 4);
    if (!q || !k || !v || !out || !lse || !table) return 2;
    for (size_t i = 0; i < nq; ++i) q[i] = f2bf(frand(&seed));
    for (size_t i = 0; i < nkv; ++i) k[i] = f2bf(frand(&seed));
    for (size_t i = 0; i < nkv; ++i) v[i] = f2bf(frand(&seed));
    /* pages handed out back to front, unused table entries poisoned */
    int next = POOL - 1;
    for (int b = 0; b < B; ++b)
        for (int j = 0; j < MAXP; ++j) table[b * MAXP + j] = (j * P < lens[b]) ? next-- : -12345;

    void *dq, *dk, *dv, *dout, *dlse, *dtable, *dlens, *dws = NULL;
    CHECK_HIP(hipMalloc(&dq, nq * 2));
    CHECK_HIP(hipMalloc(&dk, nkv * 2));
    CHECK_HIP(hipMalloc(&dv, nkv * 2));
    CHECK_HIP(hipMalloc(&dout, nq * 2));
    CHECK_HIP(hipMalloc(&dlse, (size_t)B * HQ * 4));
    CHECK_HIP(hipMalloc(&dtable, (size_t)B * MAXP * 4));
    CHECK_HIP(hipMalloc(&dlens, B * 4));
    CHECK_HIP(hipMemcpy(dq, q, nq * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dk, k, nkv * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dv, v, nkv * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dtable, table, (size_t)B * MAXP * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dlens, lens, B * 4, hipMemcpyHostToDevice));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));

    if (fdk_abi_version() != FDK_ABI_VERSION) {
        fprintf(stderr, "ABI version %d != header %d\n", fdk_abi_version(), FDK_ABI_VERSION);
        return 1;
    }
    fdk_decode_args a;
    memset(&a, 0, sizeof a);
    a.struct_size = sizeof a;
    a.q = dq; a.q_stride_b = HQ * D; a.q_stride_h = D; a.q_dtype = FDK_BF16;
    a.kv_dtype = FDK_BF16; a.k_cache = dk; a.v_cache = dv;
    a.k_stride_page = a.v_stride_page = P * HKV * D;
    a.k_stride_tok = a.v_stride_tok = HKV * D;
    a.k_stride_head = a.v_stride_head = D;
    a.block_table = dtable; a.table_stride_b = MAXP; a.kv_lens = dlens;
    a.batch = B; a.num_q_heads = HQ; a.num_kv_heads = HKV; a.head_dim = D;
    a.page_size = P; a.max_pages = MAXP; a.sm_scale = scale;
    a.out = dout; a.out_stride_b = HQ * D; a.out_stride_h = D; a.out_dtype = FDK_BF16;
    a.lse = dlse; a.lse_stride_b = HQ;

    /* a rejected call: negative code, a message, nothing launched */
    a.head_dim = 96;
    if (fdk_decode(&a, stream) != FDK_EUNSUPPORTED || strlen(fdk_last_error()) == 0) {
        fprintf(stderr, "head_dim 96 was not rejected as expected\n");
        return 1;
    }
    a.head_dim = D;

    for (int forced = 0; forced <= 1; ++forced) {   /* the library's own plan (splits), then a forced single pass */
        fdk_plan_t plan;
        a.num_splits = forced;
        if (fdk_plan(&a, 0, &plan) != FDK_OK) { fprintf(stderr, "plan: %s\n", fdk_last_error()); return 1; }
        size_t ws = plan.num_splits > 1 ? fdk_workspace_bytes(B, HQ, D, plan.num_splits) : 0;
        if (dws) CHECK_HIP(hipFree(dws));
        dws = NULL;
        if (ws) CHECK_HIP(hipMalloc(&dws, ws));
        a.workspace = dws; a.workspace_bytes = ws;
        CHECK_HIP(hipMemsetAsync(dout, 0xff, nq * 2, stream));
        int rc = fdk_decode(&a, stream);
        if (rc != FDK_OK) { fprintf(stderr, "fdk_decode rc=%d: %s\n", rc, fdk_last_error()); return 1; }
        CHECK_HIP(hipStreamSynchronize(stream));
        CHECK_HIP(hipMemcpy(out, dout, nq * 2, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(lse, dlse, (size_t)B * HQ * 4, hipMemcpyDeviceToHost));

        double worst_o = 0.0, worst_l = 0.0;
        for (int b = 0; b < B; ++b)
            for (int h = 0; h < HQ; ++h) {
                const int kvh = h / (HQ / HKV), n = lens[b];
                double logit[256], m = -1e300, l = 0.0, acc[D];
                for (int t = 0; t < n; ++t) {
                    const size_t row = ((size_t)table[b * MAXP + t / P] * P + t % P) * HKV * D + (size_t)kvh * D;
                    double s = 0.0;
                    for (int d = 0; d < D; ++d) s += (double)bf2f(q[((size_t)b * HQ + h) * D + d]) * bf2f(k[row + d]);
                    logit[t] = s * scale;
                    if (logit[t] > m) m = logit[t];
                }
                for (int d = 0; d < D; ++d) acc[d] = 0.0;
                for (int t = 0; t < n; ++t) {
                    const size_t row = ((size_t)table[b * MAXP + t / P] * P + t % P) * HKV * D + (size_t)kvh * D;
                    const double p = exp(logit[t] - m);
                    l += p;
                    for (int d = 0; d < D; ++d) acc[d] += p * bf2f(v[row + d]);
                }
                for (int d = 0; d < D; ++d) {
                    const double got = bf2f(out[((size_t)b * HQ + h) * D + d]), want = acc[d] / l;
                    const double err = fabs(got - want) - 2e-2 * fabs(want);
                    if (err > worst_o) worst_o = err;
                }
                const double el = fabs((double)lse[b * HQ + h] - (m + log(l)));
                if (el > worst_l) worst_l = el;
            }
        printf("plan: splits=%d chunk=%d balanced=%d algo=%d  worst |out err| - 2e-2|ref| = %.4f  worst |lse err| = %.2e\n",
               plan.num_splits, plan.chunk_tokens, plan.balanced, plan.algo, worst_o, worst_l);
        if (worst_o > 2e-2 || worst_l > 1e-3) { fprintf(stderr, "mismatch\n"); return 1; }
    }
    printf("OK\n");
    return 0;
}
