/* A C caller of libdnnl_amd.so that includes only include/dnnl_amd.h: u8 x s8 ->
 * s32 matmul, 64 x 64 x 64, src zero point 128, through the dnnl_* C API on a
 * GPU engine, checked against a plain integer loop.  Built with gcc by
 * tests/test_gpu_c_clients.py: struct layouts, enum values and calling
 * conventions of the header are what a compiled caller sees.
 * Prints "ok" and exits 0 when every element matches. */
#include <stdio.h>
#include <stdlib.h>

#include "dnnl_amd.h"

#define CHECK(call) \
    do { \
        dnnl_status_t s_ = (call); \
        if (s_ != dnnl_success) { \
            fprintf(stderr, "%s -> status %d (line %d)\n", #call, (int)s_, __LINE__); \
            return 1; \
        } \
    } while (0)

enum { M = 64, N = 64, K = 64 };

int main(void) {
    static unsigned char src[M * K];
    static signed char wei[K * N];
    static int want[M * N];
    unsigned seed = 12345u;
    for (int i = 0; i < M * K; ++i) { seed = seed * 1664525u + 1013904223u; src[i] = (unsigned char)(seed >> 24); }
    for (int i = 0; i < K * N; ++i) { seed = seed * 1664525u + 1013904223u; wei[i] = (signed char)((seed >> 24) % 255 - 127); }
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            int acc = 0;
            for (int k = 0; k < K; ++k) acc += ((int)src[m * K + k] - 128) * (int)wei[k * N + n];
            want[m * N + n] = acc;
        }

    dnnl_engine_t eng;
    dnnl_stream_t strm;
    CHECK(dnnl_engine_create(&eng, dnnl_gpu, 0));
    CHECK(dnnl_stream_create(&strm, eng, dnnl_stream_default_flags));

    dnnl_dims_t sd = {M, K}, wd = {K, N}, dd = {M, N}, one = {1};
    dnnl_memory_desc_t src_md, wei_md, dst_md, zp_md;
    CHECK(dnnl_memory_desc_create_with_tag(&src_md, 2, sd, dnnl_u8, dnnl_ab));
    CHECK(dnnl_memory_desc_create_with_tag(&wei_md, 2, wd, dnnl_s8, dnnl_ab));
    CHECK(dnnl_memory_desc_create_with_tag(&dst_md, 2, dd, dnnl_s32, dnnl_ab));
    CHECK(dnnl_memory_desc_create_with_tag(&zp_md, 1, one, dnnl_s32, dnnl_a));

    dnnl_primitive_attr_t attr;
    CHECK(dnnl_primitive_attr_create(&attr));
    CHECK(dnnl_primitive_attr_set_zero_points_mask(attr, DNNL_ARG_SRC, 0));

    dnnl_primitive_desc_t pd;
    CHECK(dnnl_matmul_primitive_desc_create(&pd, eng, src_md, wei_md, NULL, dst_md, attr));
    const char *impl = NULL; /* owned by the primitive descriptor */
    CHECK(dnnl_primitive_desc_query(pd, dnnl_query_impl_info_str, 0, &impl));
    char impl_name[64];
    snprintf(impl_name, sizeof(impl_name), "%s", impl ? impl : "?");
    dnnl_primitive_t prim;
    CHECK(dnnl_primitive_create(&prim, pd));

    dnnl_memory_t src_m, wei_m, dst_m, zp_m;
    CHECK(dnnl_memory_create(&src_m, src_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&wei_m, wei_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&dst_m, dst_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&zp_m, zp_md, eng, DNNL_MEMORY_ALLOCATE));
    void *p;
    CHECK(dnnl_memory_map_data(src_m, &p));
    for (int i = 0; i < M * K; ++i) ((unsigned char *)p)[i] = src[i];
    CHECK(dnnl_memory_unmap_data(src_m, p));
    CHECK(dnnl_memory_map_data(wei_m, &p));
    for (int i = 0; i < K * N; ++i) ((signed char *)p)[i] = wei[i];
    CHECK(dnnl_memory_unmap_data(wei_m, p));
    CHECK(dnnl_memory_map_data(zp_m, &p));
    ((int *)p)[0] = 128;
    CHECK(dnnl_memory_unmap_data(zp_m, p));

    dnnl_exec_arg_t args[4] = {{DNNL_ARG_SRC, src_m}, {DNNL_ARG_WEIGHTS, wei_m}, {DNNL_ARG_DST, dst_m},
            {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, zp_m}};
    CHECK(dnnl_primitive_execute(prim, strm, 4, args));
    CHECK(dnnl_stream_wait(strm));

    CHECK(dnnl_memory_map_data(dst_m, &p));
    long bad = 0;
    for (int i = 0; i < M * N; ++i) bad += ((int *)p)[i] != want[i];
    CHECK(dnnl_memory_unmap_data(dst_m, p));

    CHECK(dnnl_primitive_destroy(prim));
    CHECK(dnnl_primitive_desc_destroy(pd));
    CHECK(dnnl_primitive_attr_destroy(attr));
    CHECK(dnnl_memory_destroy(src_m)); CHECK(dnnl_memory_destroy(wei_m));
    CHECK(dnnl_memory_destroy(dst_m)); CHECK(dnnl_memory_destroy(zp_m));
    CHECK(dnnl_memory_desc_destroy(src_md)); CHECK(dnnl_memory_desc_destroy(wei_md));
    CHECK(dnnl_memory_desc_destroy(dst_md)); CHECK(dnnl_memory_desc_destroy(zp_md));
    CHECK(dnnl_stream_destroy(strm));
    CHECK(dnnl_engine_destroy(eng));
    if (bad) {
        fprintf(stderr, "%ld of %d elements differ (impl %s)\n", bad, M * N, impl_name);
        return 1;
    }
    printf("ok %s\n", impl_name);
    return 0;
}
