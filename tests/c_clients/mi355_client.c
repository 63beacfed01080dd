/* A C caller of libmi355_matmul.so that includes only include/mi355_matmul.h:
 * the same u8 x s8 -> s32 problem through the thin C ABI (descriptor + device
 * pointers + stream), checked against a plain integer loop.  Built with gcc by
 * tests/test_gpu_c_clients.py.  Prints "ok" and exits 0 when every element
 * matches. */
#include <stdio.h>
#include <string.h>

#include "mi355_matmul.h"

#define CHECK(call) \
    do { \
        int s_ = (call); \
        if (s_ != MI355_SUCCESS) { \
            fprintf(stderr, "%s -> status %d: %s (line %d)\n", #call, s_, mi355_last_error(), __LINE__); \
            return 1; \
        } \
    } while (0)

enum { M = 64, N = 64, K = 64 };

int main(void) {
    static unsigned char src[M * K];
    static signed char wei[K * N];
    static int want[M * N], got[M * N];
    unsigned seed = 777u;
    for (int i = 0; i < M * K; ++i) { seed = seed * 1664525u + 1013904223u; src[i] = (unsigned char)(seed >> 24); }
    for (int i = 0; i < K * N; ++i) { seed = seed * 1664525u + 1013904223u; wei[i] = (signed char)((seed >> 24) % 255 - 127); }
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            int acc = 0;
            for (int k = 0; k < K; ++k) acc += ((int)src[m * K + k] - 128) * (int)wei[k * N + n];
            want[m * N + n] = acc;
        }
    int count = 0;
    CHECK(mi355_device_count(&count));
    if (count < 1) { fprintf(stderr, "no device\n"); return 1; }
    CHECK(mi355_device_set(0));

    mi355_matmul_desc_t d;
    memset(&d, 0, sizeof(d));
    d.batch = 1; d.M = M; d.N = N; d.K = K;
    d.src_dt = MI355_DT_U8; d.wei_dt = MI355_DT_S8; d.dst_dt = MI355_DT_S32; d.bias_dt = MI355_DT_UNDEF;
    d.src_stride[0] = M * K; d.src_stride[1] = K; d.src_stride[2] = 1;
    d.wei_stride[0] = K * N; d.wei_stride[1] = N; d.wei_stride[2] = 1;
    d.dst_stride[0] = M * N; d.dst_stride[1] = N; d.dst_stride[2] = 1;
    mi355_quant_t *qs[] = {&d.src_scale, &d.wei_scale, &d.dst_scale, &d.src_zp, &d.wei_zp, &d.dst_zp, &d.src_pr};
    for (unsigned i = 0; i < sizeof(qs) / sizeof(qs[0]); ++i) { qs[i]->dt = MI355_DT_UNDEF; qs[i]->group[0] = qs[i]->group[1] = 1; }
    d.src_zp.dt = MI355_DT_S32; d.src_zp.mask = 0;
    d.impl = MI355_IMPL_AUTO;

    int impl = 0;
    CHECK(mi355_matmul_query(&d, MI355_IMPL_AUTO, &impl));
    size_t scratch_bytes = 0;
    CHECK(mi355_matmul_scratch_bytes(&d, &scratch_bytes));

    void *dsrc, *dwei, *ddst, *dzp, *scratch = NULL;
    const int zp = 128;
    CHECK(mi355_mem_alloc(&dsrc, sizeof(src))); CHECK(mi355_mem_alloc(&dwei, sizeof(wei)));
    CHECK(mi355_mem_alloc(&ddst, sizeof(got))); CHECK(mi355_mem_alloc(&dzp, sizeof(zp)));
    if (scratch_bytes) CHECK(mi355_mem_alloc(&scratch, scratch_bytes));
    void *stream;
    CHECK(mi355_stream_create(&stream));
    CHECK(mi355_mem_h2d(dsrc, src, sizeof(src), stream)); CHECK(mi355_mem_h2d(dwei, wei, sizeof(wei), stream));
    CHECK(mi355_mem_h2d(dzp, &zp, sizeof(zp), stream));

    mi355_matmul_args_t a;
    memset(&a, 0, sizeof(a));
    a.src = dsrc; a.wei = dwei; a.dst = ddst; a.src_zp = dzp;
    CHECK(mi355_matmul_launch(&d, &a, scratch, stream));
    CHECK(mi355_mem_d2h(got, ddst, sizeof(got), stream));
    long bad = 0;
    for (int i = 0; i < M * N; ++i) bad += got[i] != want[i];
    /* and once more through the allocation-free entry point */
    CHECK(mi355_mem_set(ddst, 0, sizeof(got), stream));
    CHECK(mi355_matmul_launch_noalloc(&d, &a, stream));
    CHECK(mi355_mem_d2h(got, ddst, sizeof(got), stream));
    for (int i = 0; i < M * N; ++i) bad += got[i] != want[i];

    CHECK(mi355_stream_destroy(stream));
    CHECK(mi355_mem_free(dsrc)); CHECK(mi355_mem_free(dwei)); CHECK(mi355_mem_free(ddst)); CHECK(mi355_mem_free(dzp));
    CHECK(mi355_mem_free(scratch));
    if (bad) { fprintf(stderr, "%ld elements differ (%s)\n", bad, mi355_matmul_impl_name(impl)); return 1; }
    printf("ok %s\n", mi355_matmul_impl_name(impl));
    return 0;
}
