// Instantiates the row kernels for one element type (bf16) so the three types compile in parallel.
#include "tde_rows.h"

namespace tde {

hipError_t launch_rows_bf16(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s) {
    return launch_rows_e<ElemBF16>(n, vpt, q, wn, a, g, s);
}

hipError_t launch_reduce_bf16(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows,
                             hipStream_t s) {
    return launch_reduce_e<ElemBF16>(n, a, row_bytes, first_row, row_step, rows, s);
}

} // namespace tde
