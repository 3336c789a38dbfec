// Traffic skeleton of the row kernel: the same workgroups, lane mapping, load order and cache policies, the
// same bytes read and written per row, and no arithmetic beyond an exclusive-or that keeps every load alive.
// What it writes is meaningless.  Timed next to the real kernel it shows how much of a launch is the memory
// pattern itself; RowArgs::probe_parts switches the input streams, the T-typed output rows and the code rows
// on and off separately, which shows what each part of the
// pattern costs alone.
#include <hip/hip_runtime.h>

#include "tde_rows.h"

namespace tde {

// CODE_BYTES: bytes of quantized output per 16-byte input vector (0 none, 4 for fp32 rows, 8 for 2-byte rows).
template <int N, int VPT, int CODE_BYTES, bool WN>
__global__ void __launch_bounds__(1024 / VPT)
    __attribute__((amdgpu_waves_per_eu(VPT == 1 ? 8 : (VPT == 2 ? 5 : 3)))) traffic_kernel(const RowArgs a, uint32_t row_bytes) {
    constexpr int NP = (N == 0) ? 1 : N;
    const int tid = threadIdx.x;
    const int tpr = a.threads_per_row;
    const int group = __builtin_amdgcn_readfirstlane(tid / tpr);
    const int t = tid - group * tpr;
    const void *part[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) part[r] = a.part[r];
    if (a.table != nullptr) {
#pragma unroll
        for (int r = 0; r < NP; ++r) {
            const void *from_table = a.table[r];
            part[r] = (part[r] != nullptr) ? part[r] : from_table;
        }
    }
    uint32_t lane_off[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) lane_off[j] = (uint32_t)(j * tpr + t) * 16u;

    {
        const int64_t row = (int64_t)xcd_chunked_block(blockIdx.x, gridDim.x, (uint32_t)a.xcd_chunk) * a.rows_per_block + group;
        const uint32_t bytes = (row < a.tokens) ? row_bytes : 0u;
        const int64_t row_byte = row * (int64_t)row_bytes;
        // The two output parts are switched through the sizes of their buffer resources, not through branches: a store
        // to a resource of size 0 is dropped, so the store instructions are the same whatever is switched on (with
        // branches around the stores of each vector the skeleton measured 1.1 us slower on 8 x [2048, 8192] than the
        // same traffic without them).  The loads are skipped as a whole when the inputs are switched off.
        const uint32_t row_wr_bytes = (a.probe_parts & 2) ? bytes : 0u;
        const bool wr_codes = (a.probe_parts & 4) != 0;
        RowLoads<NP, VPT> d;
        if (a.probe_parts & 1) {
#pragma unroll
            for (int r = 0; r < NP; ++r) {
                const rsrc_t rs = row_rsrc(part[r], row_byte, bytes);
#pragma unroll
                for (int j = 0; j < VPT; ++j) d.p[j][r] = rsrc_load16(rs, lane_off[j]);
            }
            const rsrc_t rr = row_rsrc(a.residual_in, row_byte, bytes);
#pragma unroll
            for (int j = 0; j < VPT; ++j) d.r[j] = rsrc_load16(rr, lane_off[j]);
        } else {
#pragma unroll
            for (int j = 0; j < VPT; ++j) {
                d.r[j] = u32x4{(uint32_t)tid, (uint32_t)j, 0x9e3779b9u, 0x7f4a7c15u};
#pragma unroll
                for (int r = 0; r < NP; ++r) d.p[j][r] = u32x4{0u, 0u, 0u, 0u};
            }
        }

        const rsrc_t res_out = row_rsrc(a.residual_out, row_byte, row_wr_bytes);
        const rsrc_t norm_out = row_rsrc(a.norm_out, row_byte, WN ? row_wr_bytes : 0u);
        const uint32_t code_row = row_bytes / 16u * (uint32_t)CODE_BYTES;
        const rsrc_t q_out = row_rsrc(a.q_out, row * (int64_t)code_row, (CODE_BYTES != 0 && bytes != 0u && wr_codes) ? code_row : 0u);
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            u32x4 x = d.r[j];
#pragma unroll
            for (int r = 0; r < NP; ++r) x ^= d.p[j][r];
            rsrc_store16(res_out, lane_off[j], x);
            if constexpr (WN) rsrc_store16(norm_out, lane_off[j], x);
            if constexpr (CODE_BYTES == 8) {
                const u32x2 w = {x[0] ^ x[2], x[1] ^ x[3]};
                __builtin_amdgcn_raw_buffer_store_b64(w, q_out, (int)(lane_off[j] / 2u), 0, kAuxStore);
            } else if constexpr (CODE_BYTES == 4) {
                __builtin_amdgcn_raw_buffer_store_b32(x[0] ^ x[1] ^ x[2] ^ x[3], q_out, (int)(lane_off[j] / 4u), 0, kAuxStore);
            }
        }
    }
}

template <int N, int VPT>
hipError_t launch_traffic_nv(int code_bytes, bool wn, const RowArgs &a, const Geometry &g, uint32_t row_bytes, hipStream_t s) {
    const dim3 grid((unsigned)g.grid), block((unsigned)g.block_threads);
    // The LDS the row kernel of this geometry allocates (never touched here), padding included, and its
    // wavefronts-per-SIMD bound: the skeleton then fills a compute unit with as many workgroups as the kernel does.
    const size_t lds = (size_t)g.lds_bytes;
#define TDE_TRAFFIC(CB, WNB)                                                                   \
    if (lds > kDefaultMaxDynamicLds) {                                                         \
        const hipError_t e = allow_large_lds<traffic_kernel<N, VPT, CB, WNB>>();               \
        if (e != hipSuccess) return e;                                                         \
    }                                                                                          \
    hipLaunchKernelGGL((traffic_kernel<N, VPT, CB, WNB>), grid, block, lds, s, a, row_bytes); \
    return hipGetLastError();
    if (code_bytes == 0) { TDE_TRAFFIC(0, true) }
    if (code_bytes == 8) { if (wn) { TDE_TRAFFIC(8, true) } else { TDE_TRAFFIC(8, false) } }
    if (code_bytes == 4) { if (wn) { TDE_TRAFFIC(4, true) } else { TDE_TRAFFIC(4, false) } }
#undef TDE_TRAFFIC
    return hipErrorInvalidValue;
}

template <int N>
hipError_t launch_traffic_n(int vpt, int code_bytes, bool wn, const RowArgs &a, const Geometry &g, uint32_t row_bytes,
                            hipStream_t s) {
    if (vpt == 1) return launch_traffic_nv<N, 1>(code_bytes, wn, a, g, row_bytes, s);
    if (vpt == 2) return launch_traffic_nv<N, 2>(code_bytes, wn, a, g, row_bytes, s);
    if (vpt == 4) return launch_traffic_nv<N, 4>(code_bytes, wn, a, g, row_bytes, s);
    return hipErrorInvalidValue;
}

hipError_t launch_traffic(int n, int vpt, int code_bytes, bool wn, const RowArgs &a, const Geometry &g, uint32_t row_bytes,
                          hipStream_t s) {
    switch (n) {
    case 2: return launch_traffic_n<2>(vpt, code_bytes, wn, a, g, row_bytes, s);
    case 4: return launch_traffic_n<4>(vpt, code_bytes, wn, a, g, row_bytes, s);
    case 8: return launch_traffic_n<8>(vpt, code_bytes, wn, a, g, row_bytes, s);
    }
    return hipErrorInvalidValue;
}

} // namespace tde
