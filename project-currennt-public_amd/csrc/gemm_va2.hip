// Instantiates one share of the fp32 MFMA matrix-product kernels (see gemm_kernel.hpp, gemm.hip).
#include "gemm_kernel.hpp"

namespace cnt {

void gemm_dispatch_va2(const GemmArgs &a, dim3 grid, hipStream_t s, bool ak, int vb, bool bk, int tile) {
    launch_ak<2>(a, grid, s, ak, vb, bk, tile);
}

}  // namespace cnt
