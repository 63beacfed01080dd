/* A C caller of libdnnl_amd.so that includes only include/dnnl_amd.h: an inner
 * product u8 x s8 -> s32 on channels-last tensors (src nhwc 64 x 16 x 2 x 2,
 * weights ohwi 64 x 16 x 2 x 2) through dnnl_inner_product_forward_primitive_desc_create
 * on a GPU engine, checked against a plain integer loop over the logical
 * indices.  Built with gcc by tests/test_gpu_c_clients.py.
 * Prints "ok <implementation>" and exits 0 when every element matches. */
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

enum { MB = 64, IC = 16, H = 2, W = 2, OC = 64, K = IC * H * W };

/* offset of logical (n, c, h, w) in a channels-last tensor */
static int cl(int n, int c, int h, int w) { return ((n * H + h) * W + w) * IC + c; }

int main(void) {
    static unsigned char src[MB * K];
    static signed char wei[OC * K];
    static int want[MB * OC];
    unsigned seed = 777u;
    for (int i = 0; i < MB * K; ++i) { seed = seed * 1664525u + 1013904223u; src[i] = (unsigned char)(seed >> 24); }
    for (int i = 0; i < OC * K; ++i) { seed = seed * 1664525u + 1013904223u; wei[i] = (signed char)((seed >> 24) % 255 - 127); }
    for (int n = 0; n < MB; ++n)
        for (int o = 0; o < OC; ++o) {
            int acc = 0;
            for (int c = 0; c < IC; ++c)
                for (int h = 0; h < H; ++h)
                    for (int w = 0; w < W; ++w) acc += (int)src[cl(n, c, h, w)] * (int)wei[cl(o, c, h, w)];
            want[n * OC + o] = acc;
        }

    dnnl_engine_t eng;
    dnnl_stream_t strm;
    CHECK(dnnl_engine_create(&eng, dnnl_gpu, 0));
    CHECK(dnnl_stream_create(&strm, eng, dnnl_stream_default_flags));

    dnnl_dims_t sd = {MB, IC, H, W}, wd = {OC, IC, H, W}, dd = {MB, OC};
    dnnl_memory_desc_t src_md, wei_any_md, dst_md;
    const_dnnl_memory_desc_t wei_md;
    CHECK(dnnl_memory_desc_create_with_tag(&src_md, 4, sd, dnnl_u8, dnnl_nhwc));
    CHECK(dnnl_memory_desc_create_with_tag(&wei_any_md, 4, wd, dnnl_s8, dnnl_format_tag_any));
    CHECK(dnnl_memory_desc_create_with_tag(&dst_md, 2, dd, dnnl_s32, dnnl_nc));

    dnnl_primitive_desc_t pd;
    CHECK(dnnl_inner_product_forward_primitive_desc_create(&pd, eng, dnnl_forward_inference, src_md, wei_any_md, NULL,
            dst_md, NULL));
    dnnl_primitive_kind_t kind;
    CHECK(dnnl_primitive_desc_query(pd, dnnl_query_primitive_kind, 0, &kind));
    if (kind != dnnl_inner_product) { fprintf(stderr, "primitive kind %d\n", (int)kind); return 1; }
    /* weights given as `any` take src's order of dims: ohwi */
    wei_md = dnnl_primitive_desc_query_md(pd, dnnl_query_weights_md, 0);
    dnnl_dims_t *ws = NULL;
    CHECK(dnnl_memory_desc_query(wei_md, dnnl_query_strides, &ws));
    if ((*ws)[0] != K || (*ws)[1] != 1 || (*ws)[2] != W * IC || (*ws)[3] != IC) {
        fprintf(stderr, "weights strides %ld %ld %ld %ld\n", (long)(*ws)[0], (long)(*ws)[1], (long)(*ws)[2], (long)(*ws)[3]);
        return 1;
    }
    const char *impl = NULL; /* owned by the primitive descriptor */
    CHECK(dnnl_primitive_desc_query(pd, dnnl_query_impl_info_str, 0, &impl));
    char impl_name[64];
    snprintf(impl_name, sizeof(impl_name), "%s", impl ? impl : "?");
    dnnl_primitive_t prim;
    CHECK(dnnl_primitive_create(&prim, pd));

    dnnl_memory_t src_m, wei_m, dst_m;
    CHECK(dnnl_memory_create(&src_m, src_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&wei_m, wei_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&dst_m, dst_md, eng, DNNL_MEMORY_ALLOCATE));
    void *p;
    CHECK(dnnl_memory_map_data(src_m, &p));
    for (int i = 0; i < MB * K; ++i) ((unsigned char *)p)[i] = src[i];
    CHECK(dnnl_memory_unmap_data(src_m, p));
    CHECK(dnnl_memory_map_data(wei_m, &p));
    for (int i = 0; i < OC * K; ++i) ((signed char *)p)[i] = wei[i];
    CHECK(dnnl_memory_unmap_data(wei_m, p));

    dnnl_exec_arg_t args[3] = {{DNNL_ARG_SRC, src_m}, {DNNL_ARG_WEIGHTS, wei_m}, {DNNL_ARG_DST, dst_m}};
    CHECK(dnnl_primitive_execute(prim, strm, 3, args));
    CHECK(dnnl_stream_wait(strm));

    CHECK(dnnl_memory_map_data(dst_m, &p));
    long bad = 0;
    for (int i = 0; i < MB * OC; ++i) bad += ((int *)p)[i] != want[i];
    CHECK(dnnl_memory_unmap_data(dst_m, p));

    CHECK(dnnl_primitive_destroy(prim));
    CHECK(dnnl_primitive_desc_destroy(pd));
    CHECK(dnnl_memory_destroy(src_m)); CHECK(dnnl_memory_destroy(wei_m)); CHECK(dnnl_memory_destroy(dst_m));
    CHECK(dnnl_memory_desc_destroy(src_md)); CHECK(dnnl_memory_desc_destroy(wei_any_md));
    CHECK(dnnl_memory_desc_destroy(dst_md));
    CHECK(dnnl_stream_destroy(strm));
    CHECK(dnnl_engine_destroy(eng));
    if (bad) {
        fprintf(stderr, "%ld of %d elements differ (impl %s)\n", bad, MB * OC, impl_name);
        return 1;
    }
    printf("ok %s\n", impl_name);
    return 0;
}
