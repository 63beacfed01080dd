// Internal interface between the C-ABI dispatcher (api.hip) and the kernel
// families.  Each family exports a predicate (can it compute this problem
// exactly?), its scratch need and a launcher.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/mi355_matmul.h"
#include "mi355_device.hpp"

namespace mi355 {

int ref_supported(const mi355_matmul_desc_t &d);
int ref_launch(const problem_t &P, hipStream_t stream);

int i8_supported(const mi355_matmul_desc_t &d);
size_t i8_scratch_bytes(const mi355_matmul_desc_t &d);
int i8_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream);

int f8_supported(const mi355_matmul_desc_t &d);
size_t f8_scratch_bytes(const mi355_matmul_desc_t &d);
int f8_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream);
int h16_supported(const mi355_matmul_desc_t &d);
size_t h16_scratch_bytes(const mi355_matmul_desc_t &d);
int h16_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream);

int mxf4_supported(const mi355_matmul_desc_t &d);
size_t mxf4_scratch_bytes(const mi355_matmul_desc_t &d);
int mxf4_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream);

int woq_supported(const mi355_matmul_desc_t &d);
size_t woq_scratch_bytes(const mi355_matmul_desc_t &d);
int woq_launch(const mi355_matmul_desc_t &d, const problem_t &P, void *scratch,
        hipStream_t stream);

// the same decode over weights in the 64-column packing
int woqp_supported(const mi355_matmul_desc_t &d);
int woqp_launch(const mi355_matmul_desc_t &d, const problem_t &P, hipStream_t stream);

// hip:mfma_f8 on 256 x 128 tiles of four wavefronts; fa / fb: 1 = e5m2 src / weights, 0 = e4m3 (a translation unit of its own: the build runs
// the family's instantiations side by side); bt = the weights as [N][K] bytes, K contiguous
int f8_launch_narrow(int fa, int fb, const problem_t &P, const char *bt, long ldb, long bt_bstride, unsigned batch, hipStream_t stream);

void set_error(const char *fmt, ...);

// Tuning switches (tests and measurements force a tile geometry where several can run a problem).  Each starts from
// the environment variable of its name, read once per process, and changes only through mi355_tuning_set: no getenv on a
// launch path.  Values: 0 = the library's own choice.
enum tune_key_t { TUNE_I8_TILES = 0, TUNE_F8_TILES, TUNE_H16_TILES, TUNE_GROUPED_IMPL, TUNE_GEMM_ORDER, TUNE_COUNT };
enum { TUNE_AUTO = 0, TUNE_LARGE = 1, TUNE_WIDE = 2, TUNE_SMALL = 3, TUNE_REF = 4, TUNE_SHORT = 5, TUNE_TALL = 6, TUNE_NARROW = 7 };
int tuning(tune_key_t key);

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) for a kernel, once per
// (kernel, device, size) of this process.  Safe to call from several host
// threads.
int ensure_dynamic_lds(const void *kernel, int bytes, const char *who);

// A 4-bit dst (f4_e2m1 / s4 / u4) in the GEMM tiles' epilogue: four consecutive columns of a row leave as two whole
// bytes, so rows are contiguous, every group of four is whole and starts a byte.
inline bool tile_nibble_dst_ok(const mi355_matmul_desc_t &d) {
    return d.dst_stride[2] == 1 && d.N % 4 == 0 && d.dst_stride[1] % 4 == 0 && d.dst_stride[0] % 4 == 0;
}

// [R][C] bytes (row pitch ld_in) -> [C][R] bytes (row pitch ld_out), per batch
void transpose_bytes(const void *in, long R, long C, long ld_in, long in_bstride, void *out,
        long ld_out, long out_bstride, long batches, hipStream_t stream);

inline bool is_int8_dt(int dt) { return dt == MI355_DT_S8 || dt == MI355_DT_U8; }
inline bool is_int4_dt(int dt) { return dt == MI355_DT_S4 || dt == MI355_DT_U4; }
inline bool is_f8_dt(int dt) { return dt == MI355_DT_F8_E4M3 || dt == MI355_DT_F8_E5M2; }
inline bool quant_absent(const mi355_quant_t &q) { return q.dt == MI355_DT_UNDEF; }
// a problem whose weights can be in the MI355_WEI_PACK_WOQ64 layout
inline bool woq64_layout_ok(const mi355_matmul_desc_t &d) {
    return d.wei_packing == MI355_WEI_PACK_WOQ64 && is_int4_dt(d.wei_dt) && d.batch == 1 && d.K % 32 == 0
            && d.N % 64 == 0 && d.K > 0 && d.N > 0;
}
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

} // namespace mi355
