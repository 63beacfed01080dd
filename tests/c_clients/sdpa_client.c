/* A C caller of libdnnl_amd.so that includes only include/dnnl_amd.h: scaled
 * dot-product attention on f32 tensors (2 batches x 3 heads, 10 queries x 24 keys,
 * head size 16, one key / value head shared by the query heads, keys stored
 * [b][1][sk][d] and handed over as the transposed view, a causal mask from the
 * bottom right, scale 0.25) through dnnl_amd_sdpa_primitive_desc_create on a GPU
 * engine, checked against a double-precision loop.  Built with gcc by
 * tests/test_gpu_c_clients.py.  Prints "ok <implementation>" and exits 0 when every
 * element is within 1e-5 of the loop's value. */
#include <math.h>
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

enum { B = 2, H = 3, SQ = 10, SK = 24, D = 16, DV = 16 };

static float frand(unsigned *seed) {
    *seed = *seed * 1664525u + 1013904223u;
    return (float)((int)(*seed >> 20) - 2048) / 1024.f; /* [-2, 2) in steps of 2^-10 */
}

int main(void) {
    static float q[B * H * SQ * D], k[B * SK * D], v[B * SK * DV];
    static double want[B * H * SQ * DV];
    unsigned seed = 4242u;
    for (int i = 0; i < B * H * SQ * D; ++i) q[i] = frand(&seed);
    for (int i = 0; i < B * SK * D; ++i) k[i] = frand(&seed);
    for (int i = 0; i < B * SK * DV; ++i) v[i] = frand(&seed);
    const float scale = 0.25f;
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h)
            for (int i = 0; i < SQ; ++i) {
                double s[SK], mx = -1e300, sum = 0;
                const int last = i + (SK - SQ); /* causal, diagonal from the bottom right */
                for (int j = 0; j <= last; ++j) {
                    double acc = 0;
                    for (int e = 0; e < D; ++e) acc += (double)q[((b * H + h) * SQ + i) * D + e] * k[(b * SK + j) * D + e];
                    s[j] = acc * scale;
                    if (s[j] > mx) mx = s[j];
                }
                for (int j = 0; j <= last; ++j) { s[j] = exp(s[j] - mx); sum += s[j]; }
                for (int e = 0; e < DV; ++e) {
                    double acc = 0;
                    for (int j = 0; j <= last; ++j) acc += s[j] / sum * v[(b * SK + j) * DV + e];
                    want[((b * H + h) * SQ + i) * DV + e] = acc;
                }
            }

    dnnl_engine_t eng;
    dnnl_stream_t strm;
    CHECK(dnnl_engine_create(&eng, dnnl_gpu, 0));
    CHECK(dnnl_stream_create(&strm, eng, dnnl_stream_default_flags));

    dnnl_dims_t qd = {B, H, SQ, D}, kd = {B, 1, D, SK}, ks = {SK * D, SK * D, 1, D}, vd = {B, 1, SK, DV};
    dnnl_dims_t dd = {B, H, SQ, DV}, one = {1};
    dnnl_memory_desc_t q_md, k_md, v_md, d_md, s_md;
    CHECK(dnnl_memory_desc_create_with_tag(&q_md, 4, qd, dnnl_f32, dnnl_abcd));
    CHECK(dnnl_memory_desc_create_with_strides(&k_md, 4, kd, dnnl_f32, ks)); /* [b][1][sk][d] storage, transposed view */
    CHECK(dnnl_memory_desc_create_with_tag(&v_md, 4, vd, dnnl_f32, dnnl_abcd));
    CHECK(dnnl_memory_desc_create_with_tag(&d_md, 4, dd, dnnl_f32, dnnl_abcd));
    CHECK(dnnl_memory_desc_create_with_tag(&s_md, 1, one, dnnl_f32, dnnl_a));

    dnnl_primitive_desc_t pd;
    CHECK(dnnl_amd_sdpa_primitive_desc_create(&pd, eng, q_md, k_md, v_md, d_md, NULL, s_md, /*invert_scale*/ 0,
            /*kv_head_number*/ 1, /*attn_mask_type: bottom right*/ 3, dnnl_softmax_accurate, dnnl_forward_inference, NULL, NULL,
            NULL, NULL));
    dnnl_primitive_kind_t kind;
    CHECK(dnnl_primitive_desc_query(pd, dnnl_query_primitive_kind, 0, &kind));
    if (kind != dnnl_amd_sdpa) { fprintf(stderr, "primitive kind %d\n", (int)kind); return 1; }
    const char *impl = NULL;
    CHECK(dnnl_primitive_desc_query(pd, dnnl_query_impl_info_str, 0, &impl));
    char impl_name[96];
    snprintf(impl_name, sizeof(impl_name), "%s", impl ? impl : "?");
    dnnl_primitive_t prim;
    CHECK(dnnl_primitive_create(&prim, pd));

    dnnl_memory_t q_m, k_m, v_m, d_m, s_m;
    CHECK(dnnl_memory_create(&q_m, q_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&k_m, k_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&v_m, v_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&d_m, d_md, eng, DNNL_MEMORY_ALLOCATE));
    CHECK(dnnl_memory_create(&s_m, s_md, eng, DNNL_MEMORY_ALLOCATE));
    void *p;
    CHECK(dnnl_memory_map_data(q_m, &p));
    for (int i = 0; i < B * H * SQ * D; ++i) ((float *)p)[i] = q[i];
    CHECK(dnnl_memory_unmap_data(q_m, p));
    CHECK(dnnl_memory_map_data(k_m, &p));
    for (int i = 0; i < B * SK * D; ++i) ((float *)p)[i] = k[i];
    CHECK(dnnl_memory_unmap_data(k_m, p));
    CHECK(dnnl_memory_map_data(v_m, &p));
    for (int i = 0; i < B * SK * DV; ++i) ((float *)p)[i] = v[i];
    CHECK(dnnl_memory_unmap_data(v_m, p));
    CHECK(dnnl_memory_map_data(s_m, &p));
    ((float *)p)[0] = scale;
    CHECK(dnnl_memory_unmap_data(s_m, p));

    dnnl_exec_arg_t args[5] = {{DNNL_ARG_QUERIES, q_m}, {DNNL_ARG_KEYS, k_m}, {DNNL_ARG_VALUES, v_m}, {DNNL_ARG_DST, d_m},
            {DNNL_ARG_SCALE, s_m}};
    CHECK(dnnl_primitive_execute(prim, strm, 5, args));
    CHECK(dnnl_stream_wait(strm));

    CHECK(dnnl_memory_map_data(d_m, &p));
    long bad = 0;
    double worst = 0;
    for (int i = 0; i < B * H * SQ * DV; ++i) {
        const double e = fabs((double)((float *)p)[i] - want[i]);
        if (e > worst) worst = e;
        bad += !(e <= 1e-5);
    }
    CHECK(dnnl_memory_unmap_data(d_m, p));

    CHECK(dnnl_primitive_destroy(prim));
    CHECK(dnnl_primitive_desc_destroy(pd));
    CHECK(dnnl_memory_destroy(q_m)); CHECK(dnnl_memory_destroy(k_m)); CHECK(dnnl_memory_destroy(v_m));
    CHECK(dnnl_memory_destroy(d_m)); CHECK(dnnl_memory_destroy(s_m));
    CHECK(dnnl_memory_desc_destroy(q_md)); CHECK(dnnl_memory_desc_destroy(k_md)); CHECK(dnnl_memory_desc_destroy(v_md));
    CHECK(dnnl_memory_desc_destroy(d_md)); CHECK(dnnl_memory_desc_destroy(s_md));
    CHECK(dnnl_stream_destroy(strm));
    CHECK(dnnl_engine_destroy(eng));
    if (bad) {
        fprintf(stderr, "%ld of %d elements off by more than 1e-5 (worst %g, impl %s)\n", bad, B * H * SQ * DV, worst, impl_name);
        return 1;
    }
    printf("ok %s\n", impl_name);
    return 0;
}
