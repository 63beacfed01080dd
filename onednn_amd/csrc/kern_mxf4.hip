#include "kernels.hpp"
namespace mi355 {
int mxf4_supported(const mi355_matmul_desc_t &) { return MI355_UNIMPLEMENTED; }
size_t mxf4_scratch_bytes(const mi355_matmul_desc_t &) { return 0; }
int mxf4_launch(const mi355_matmul_desc_t &, const problem_t &, void *, hipStream_t) { return MI355_UNIMPLEMENTED; }
}
