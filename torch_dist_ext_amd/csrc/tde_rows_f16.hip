// Instantiates the row kernels for one element type (f16) so the three types compile in parallel.
#include "tde_rows.h"

namespace tde {

hipError_t launch_rows_f16(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s) {
    return launch_rows_e<ElemF16>(n, vpt, q, wn, a, g, s);
}

hipError_t launch_reduce_f16(int n, const RowArgs &a, int64_t total_vecs, hipStream_t s) {
    return launch_reduce_e<ElemF16>(n, a, total_vecs, s);
}

} // namespace tde
