// hip:mfma_f8 for problems of few tiles: the family's kernel on 256 x 128 tiles of four wavefronts, two workgroups a
// CU (geo_t<4, 128>).  A wavefront's part (128 x 64), its fragments and the epilogue are those of the
// eight-wavefront 256 x 256 geometry; twice as many workgroups share a problem.  Kept apart from kern_f8.hip so that
// the two sets of instantiations compile side by side.
#include "f8_family.hpp"

namespace mi355 {

int f8_launch_narrow(int fa, int fb, const problem_t &P, const char *bt, long ldb, long bt_bstride, unsigned batch, hipStream_t stream) {
    using narrow_t = geo_t<4, 128>;
    f8_extra_t X {};
    X.bt = bt;
    X.ldb = ldb;
    X.bt_bstride = bt_bstride;
    X.tiles_m = (int)((P.M + BM - 1) / BM);
    X.tiles_n = (int)((P.N + narrow_t::BN - 1) / narrow_t::BN);
    const dim3 grid((unsigned)(X.tiles_m * X.tiles_n), 1, batch);
    constexpr int smem_bytes = narrow_t::NSTAGE * narrow_t::STAGE_BYTES + NTAB_BYTES;
    auto go = [&](auto kern) -> int {
        if (const int st = ensure_dynamic_lds((const void *)kern, smem_bytes, "mfma_f8")) return st;
        hipLaunchKernelGGL(kern, grid, dim3(narrow_t::NT), smem_bytes, stream, P, X);
        return hipGetLastError() == hipSuccess ? MI355_SUCCESS : MI355_RUNTIME_ERROR;
    };
    // fa / fb: 1 = e5m2, 0 = e4m3
    if (fa && fb) return go(f8_gemm_kernel<f8_mma_t<1, 1, narrow_t>>);
    if (fa) return go(f8_gemm_kernel<f8_mma_t<1, 0, narrow_t>>);
    if (fb) return go(f8_gemm_kernel<f8_mma_t<0, 1, narrow_t>>);
    return go(f8_gemm_kernel<f8_mma_t<0, 0, narrow_t>>);
}

} // namespace mi355
