// Error plumbing and the entry points that are not tied to one layer.
#include "common.hpp"

#include <cstring>

namespace cnt {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *last_error() { return g_error; }
}  // namespace cnt

extern "C" {

int cnt_version(void) { return 1; }
const char *cnt_last_error(void) { return cnt::last_error(); }

int cnt_matrix_product(void *stream, float *C, int m, int n, int k, const float *A, int transA, const float *B,
                       int transB, int accumulate) {
    using namespace cnt;
    CNT_REQUIRE(C && A && B, "matrix_product: null argument");
    // helpers/Matrix.cu has no functor for this combination either
    CNT_REQUIRE(!(transA && transB), "matrix_product: transposing both operands is not supported");
    return gemm_simple(static_cast<hipStream_t>(stream), C, m, n, k, A, transA != 0, B, transB != 0,
                       accumulate != 0);
}

}  // extern "C"
