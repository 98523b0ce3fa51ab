// Instantiates one share of the fp32 MFMA matrix-product kernels (see gemm_kernel.hpp, gemm.hip).
#include "gemm_kernel.hpp"

namespace cnt {

void gemm_dispatch_va1r(const GemmArgs &a, dim3 grid, hipStream_t s, int vb, bool bk, int tile) {
    launch_vb<1, false>(a, grid, s, vb, bk, tile);
}

}  // namespace cnt
