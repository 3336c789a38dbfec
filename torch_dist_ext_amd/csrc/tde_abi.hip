// C ABI of libtde_hip.so: validation, launch geometry, kernel dispatch and the emulated peer
// workspace.  Declarations and the reference interfaces they replace are in include/tde_abi.h.
#include <hip/hip_runtime.h>

#include <algorithm>

#include <cstdint>
#include <cstring>
#include <mutex>
#include <new>

#include "tde_abi.h"
#include "tde_rows.h"

// Stage buffer of tde_reduce_rms_static_stage: part of the library's device image, one copy per GPU, held
// until the process ends.  Host code never uses this name as an address: static_stage_ptr() asks the
// runtime for the current device's copy once and keeps the answer.
static __device__ __align__(256) unsigned char scratch[TDE_STATIC_STAGE_BYTES];

namespace {

thread_local int g_last_hip_error = 0;

int hip_fail(hipError_t e) {
    g_last_hip_error = (int)e;
    return TDE_EHIP;
}

int elem_bytes(int dtype) {
    switch (dtype) {
    case TDE_BF16:
    case TDE_F16: return 2;
    case TDE_F32: return 4;
    case TDE_F64: return 8;
    }
    return 0;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_stage_ptr(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return TDE_EINVAL;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e);
        if (ptr == nullptr) return TDE_EINVAL;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return TDE_OK;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kMaxBlock = 1024;
constexpr int64_t kLoadsInFlightPerCu = 128 * 1024; // target for the limit on resident workgroups (see validate)
// launches with fewer workgroups per compute unit are not limited: 24 with 8 partials, 32 with 4 (whose launches are
// shorter), i.e. 6144 and 8192 workgroups on the 256 CUs of an unpartitioned MI355X
constexpr int64_t kLimitFromWorkgroupsPerCu8 = 24, kLimitFromWorkgroupsPerCu4 = 32;
constexpr int kDefaultComputeUnits = 256; // MI355X; used when no device can be asked (planning on a host without one)

// Compute units of the current device, asked once per device and thread (no lock on the launch path).
int compute_units() {
    thread_local int cached_dev = -1, cached_cu = 0;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
        (void)hipGetLastError();
        return kDefaultComputeUnits;
    }
    if (dev != cached_dev) {
        int cu = 0;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) {
            (void)hipGetLastError();
            cu = kDefaultComputeUnits;
        }
        cached_dev = dev;
        cached_cu = cu;
    }
    return cached_cu;
}

int validate(const tde_problem *p, tde::Geometry *geo) {
    if (p == nullptr) return TDE_EINVAL;
    const int eb = elem_bytes(p->dtype);
    if (eb == 0) return TDE_EDTYPE;
    if (!(p->nranks == 2 || p->nranks == 4 || p->nranks == 8)) return TDE_ENRANKS;
    if (p->rank < 0 || p->rank >= p->nranks) return TDE_ERANK;
    if (p->tokens < 0 || p->hidden <= 0) return TDE_ESHAPE;
    if (p->hidden > kMaxBlock * 16) return TDE_EHIDDEN; // also keeps hidden * eb far from overflow
    if ((p->hidden * eb) % 16 != 0) return TDE_ESHAPE;
    if (p->quant < TDE_QUANT_NONE || p->quant > TDE_QUANT_FP8_STATIC) return TDE_EQUANT;
    if (p->quant == TDE_QUANT_FP8_STATIC && !(p->static_scale > 0.0f && p->static_scale <= 3.0e38f)) return TDE_EQUANT;
    if (p->quant == TDE_QUANT_FP8_GROUP && p->hidden % TDE_QUANT_GROUP != 0) return TDE_EQUANT;
    if (p->algo < TDE_ALGO_AUTO || p->algo > TDE_ALGO_STAGED_OWNED) return TDE_EALGO;
    if (p->dtype == TDE_F64 && p->quant != TDE_QUANT_NONE) return TDE_EQUANT; // doubles: no quantized output
    const int vec = 16 / eb;
    const int64_t nvec = p->hidden / vec;
    if (nvec > kMaxBlock) return TDE_EHIDDEN; // as the reference: one 16-byte vector per thread, 1024 threads
    int64_t total_bytes = 0; // tokens * hidden * elem must be addressable with 64-bit signed offsets
    if (__builtin_mul_overflow(p->tokens, p->hidden * eb, &total_bytes)) return TDE_ESHAPE;

    // Vectors per thread, from sweeps on MI355X over hidden 1024..8192 in steps of 1024, 2/4/8 partials, 128..32768 rows
    // and three output modes (bf16 and fp16 agree); only differences that held on two devices and across the row
    // counts between the swept powers of two are in here.  Four vectors per thread (small workgroups, many loads in
    // flight per thread, few wavefronts to synchronize per row, partials summed while the later ones are still
    // arriving) win on long rows and wherever eight partials meet full wavefronts, two in the longest launches of
    // mid-length rows; elsewhere one vector per thread is as fast or faster.
    int vpt = 1;
    if (nvec >= 896) {
        // Few rows are latency-bound and the widest row groups have the shortest dependent chain; from 256 rows
        // up four vectors per thread are 4-13 % faster than one (8 partials, hidden 8192).  With two partials
        // and up to 2048 rows two vectors per thread are another 2-7 % faster.
        vpt = p->tokens >= 256 ? 4 : (p->tokens >= 128 ? 2 : 1);
        if (p->nranks == 2 && p->tokens >= 256 && p->tokens <= 2048) vpt = 2;
    } else if (nvec == 512 && p->nranks >= 8 && p->tokens >= 1024) {
        vpt = p->tokens >= 16384 ? 2 : 4; // four: 3-4 % over one; from 16384 rows two are another 4-7 % ahead
    } else if (nvec == 256 && p->nranks >= 8 && p->tokens >= 2048) {
        // four: 3-6 % over one (with fewer partials or rows one is 3-16 % faster); from 32768 rows two: another 4-6 %
        vpt = p->tokens >= 32768 ? 2 : 4;
    } else if (nvec == 256 && p->nranks == 4 && p->tokens >= 32768) {
        vpt = 2; // 3-4 % over one
    } else if (nvec == 768 && p->nranks >= 8 && p->tokens >= 2048) {
        // rows of 6144 2-byte elements: twelve wavefronts with one vector each lose to three with four vectors
        // (2048 to 5600 rows: 1.5-2.3 %) and, in long launches, to six with two (3-6 % from 8192 rows)
        if (p->tokens >= 8192) vpt = 2;
        else if (p->tokens < 5632) vpt = 4;
    } else if (nvec == 768 && p->nranks == 4 && p->tokens >= 1024 && p->tokens < 2048) {
        vpt = 4; // 1-5 %
    } else if (nvec == 384 && p->nranks >= 8 && p->tokens >= 8192 && p->quant != TDE_QUANT_NONE) {
        vpt = p->tokens >= 32768 ? 2 : 4; // 4-5 % over one with quantized output; with T-typed output one is 2 % ahead
    } else if (nvec == 128 && p->nranks >= 8 && p->tokens >= 4096 && p->tokens < 8192) {
        vpt = 2; // 1-3 % over one
    } else if (nvec == 640) {
        // Ten wavefronts per row leave the compute units unevenly filled: from 640 rows up five wavefronts with two
        // vectors each are 10-21 % faster until there are enough rows to even that out (2048 with eight partials,
        // 16384 with four; with two partials one vector per thread stays 16 % behind at any size).  With four partials
        // and 16384+ rows all three choices are within 1 %; four vectors per thread is the one whose launches take the
        // same time from the first on (with one, launches 5 to 50 of a cold run took up to 30 % longer).
        const int64_t even_from = p->nranks >= 8 ? 2048 : (p->nranks == 4 ? 16384 : INT64_MAX);
        if (p->tokens >= 640 && p->tokens < even_from) vpt = 2;
        else if (p->nranks == 4 && p->tokens >= even_from) vpt = 4;
        else if (p->nranks >= 8 && p->tokens >= 16384) vpt = 2; // eight partials, long launches: 2 % over one
    }
    if (p->tune_vecs_per_thread != 0) {
        if (p->tune_vecs_per_thread != 1 && p->tune_vecs_per_thread != 2 && p->tune_vecs_per_thread != 4) return TDE_EINVAL;
        vpt = p->tune_vecs_per_thread;
    }
    if (p->tune_rows_per_block < 0) return TDE_EINVAL;
    if (p->tune_workgroups_per_cu < -1 || p->tune_workgroups_per_cu > 8 || p->reserved != 0) return TDE_EINVAL;
    if (p->dtype == TDE_F64) vpt = 1;
    const int64_t lanes = (nvec + vpt - 1) / vpt;
    const int tpr = (int)((lanes + 63) / 64 * 64);
    int rpb = 256 / tpr; // pack short rows so a workgroup has at least four wavefronts
    if (rpb * tpr > kMaxBlock / vpt) rpb = (kMaxBlock / vpt) / tpr; // never beyond the kernel's launch bound
    const int cus = compute_units();
    while (rpb > 1 && (p->tokens + rpb - 1) / rpb < 2 * cus) rpb /= 2; // keep every CU busy first
    if (rpb < 1) rpb = 1;
    if (p->tune_rows_per_block > 0 && p->tune_rows_per_block * tpr <= kMaxBlock / vpt) rpb = p->tune_rows_per_block;
    if (p->tokens > 0 && rpb > p->tokens) rpb = (int)p->tokens;
    const int64_t grid = (p->tokens + rpb - 1) / rpb; // one workgroup per group of rows, no loop
    if (grid > 0x7fffffff) return TDE_ESHAPE;

    // Resident workgroups per compute unit.  Left alone, a CU takes as many workgroups as its registers and LDS hold
    // (3-6 here), each with all of its rows' loads in flight.  On MI355X long launches run fastest with 120-160 KiB
    // of loads in flight per CU: more costs 1-8 % from 8192 rows up with 4 or 8 partials (32768 x 8192: 7.5 % with
    // 4 partials, 4.5 % with 8; 16384 rows: 1-3 %; 8192 rows with 8 partials: 1 %), fewer than two workgroups or
    // eight wavefronts per CU leave the arithmetic of one row uncovered by the loads of another.  Short launches (a
    // few generations of workgroups) gain nothing and can lose 1-3 %, and with 2 partials no limit helps.  At the
    // threshold itself the gain is small: 4 x [8192, 7168] with per-group scales 0.4 % on a device that has been under
    // load for 20 ms (0.9 % slower in the first milliseconds after idling).
    int wgs_per_cu = 0;
    const bool staged = p->algo == TDE_ALGO_STAGED || p->algo == TDE_ALGO_STAGED_OWNED; // its row kernel reads 2 streams
    if (p->dtype != TDE_F64 && !staged && p->nranks >= 4 && grid >= (p->nranks >= 8 ? kLimitFromWorkgroupsPerCu8 : kLimitFromWorkgroupsPerCu4) * cus) {
        const int64_t per_wg = (int64_t)rpb * (p->nranks + 1) * nvec * 16; // bytes of loads one workgroup keeps in flight
        const int waves = tpr * rpb / 64;
        // per-group scales are the heaviest arithmetic per row and four partials the shortest loads to cover it
        const int need_waves = (p->quant == TDE_QUANT_FP8_GROUP && p->nranks <= 4) ? 12 : 8;
        const int at_least = std::max(2, (need_waves + waves - 1) / waves);
        wgs_per_cu = (int)std::min<int64_t>(8, std::max<int64_t>(at_least, (kLoadsInFlightPerCu + per_wg / 2) / per_wg));
    }
    if (p->tune_workgroups_per_cu != 0 && p->dtype != TDE_F64) wgs_per_cu = p->tune_workgroups_per_cu < 0 ? 0 : p->tune_workgroups_per_cu;

    if (geo) {
        geo->wgs_per_cu = wgs_per_cu;
        size_t lds = tde::sumsq_lds_bytes(tpr * rpb, vpt, vec);
        if (wgs_per_cu > 0) {
            lds = std::max(lds, tde::lds_bytes_for_workgroups_per_cu(wgs_per_cu)); // never with doubles
            // what the launch enforces: a geometry whose own LDS is larger than the padding admits fewer still
            // (64: the kernels' static LDS)
            geo->wgs_per_cu = (int)std::min<size_t>((size_t)wgs_per_cu, tde::kLdsPerCu / (lds + 64));
        }
        geo->lds_bytes = (int)lds;
        geo->vec_elems = vec;
        geo->nvec = (int)nvec;
        geo->vpt = vpt;
        geo->threads_per_row = tpr;
        geo->rows_per_block = rpb;
        geo->block_threads = tpr * rpb;
        geo->grid = grid;
        // Row groups per XCD chunk of the row mapping (tde_rows.h: xcd_chunked_block); 16 measured best with 8
        // partials, 8 with 4.
        geo->xcd_chunk = p->nranks >= 8 ? 16 : 8;
        // Eight partials, four vectors per thread, no limit asked for or planned, and 4 to 24 workgroups per CU: the
        // row kernel's two-wavefronts-per-SIMD instantiation (tde_rows.h: WIDE) is 0.2-2.2 % faster there; it is
        // reported as the limit of two workgroups per CU that its registers amount to.
        geo->wide = p->nranks == 8 && vpt == 4 && p->dtype != TDE_F64 && !staged && wgs_per_cu == 0 &&
                    p->tune_workgroups_per_cu == 0 && grid >= 4 * (int64_t)cus;
        if (geo->wide) geo->wgs_per_cu = 2;
    }
    return TDE_OK;
}

int64_t algorithmic_bytes(const tde_problem *p, int64_t *scale_elems) {
    const int64_t e = elem_bytes(p->dtype);
    const int64_t T = p->tokens, H = p->hidden, N = p->nranks;
    int64_t out = 0, scales = 0;
    switch (p->quant) {
    case TDE_QUANT_NONE: out = T * H * e; break;
    case TDE_QUANT_FP8_TOKEN:
    case TDE_QUANT_INT8_TOKEN: scales = T; out = T * H + 4 * scales; break;
    case TDE_QUANT_FP8_GROUP: scales = T * (H / TDE_QUANT_GROUP); out = T * H + 4 * scales; break;
    case TDE_QUANT_FP8_STATIC: out = T * H; break;
    }
    if (p->quant != TDE_QUANT_NONE && p->write_norm) out += T * H * e;
    if (scale_elems) *scale_elems = scales;
    return (N + 1) * T * H * e + H * e + T * H * e + out;
}

// Calibration kernel: plain 16-byte copy (known traffic for scaling the profiler's memory counters,
// and the practical copy ceiling of the device).
__global__ void __launch_bounds__(256) copy_kernel(const void *src, void *dst, int64_t total_vecs) {
    using tde::u32x4;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vecs; v += stride) {
        const u32x4 x = __builtin_nontemporal_load((const TDE_GLOBAL u32x4 *)((const TDE_GLOBAL char *)src + v * 16));
        __builtin_nontemporal_store(x, (TDE_GLOBAL u32x4 *)((TDE_GLOBAL char *)dst + v * 16));
    }
}

// Nothing: what one dispatch costs when it does no work.
__global__ void __launch_bounds__(64) empty_kernel() {}

// Streaming-rate probes: one 256-thread workgroup per 4 KiB, no loop (the shape that measured fastest for
// both directions).  MODE 0 reads only (the loaded words feed a store that never executes for real data),
// 1 writes only, 2 copies.
template <int MODE>
__global__ void __launch_bounds__(256) stream_kernel(const void *src, void *dst, int64_t total_bytes) {
    using tde::u32x4;
    const int64_t base = (int64_t)blockIdx.x * 4096;
    const int64_t left = total_bytes - base;
    const uint32_t bytes = left < 4096 ? (uint32_t)left : 4096u;
    const uint32_t off = threadIdx.x * 16u;
    u32x4 x = {threadIdx.x, blockIdx.x, 0x9e3779b9u, 0x7f4a7c15u};
    if (MODE != 1) x = tde::rsrc_load16(tde::row_rsrc(src, base, bytes), off);
    if (MODE == 0) {
        // keeps the load alive; random data never matches, so nothing is written
        if ((x[0] ^ x[1]) == 0x5bd1e995u && (x[2] ^ x[3]) == 0x27d4eb2fu) tde::rsrc_store16(tde::row_rsrc(dst, 0, 16), 0, x);
    } else {
        __builtin_amdgcn_raw_buffer_store_b128(x, tde::row_rsrc(dst, base, bytes), (int)off, 0, MODE == 1 ? tde::kAuxDefault : tde::kAuxStore);
    }
}

} // namespace

struct tde_workspace {
    int32_t nranks;
    int32_t nblocks;
    int64_t slot_bytes;
    void *slots[TDE_MAX_RANKS];
    void *flags;   // nranks regions of nblocks*nranks ints, zeroed (layout parity only: no kernel here reads them)
    int32_t *cells; // 5 int cells: counter, two-shot clock, one-shot clock, one-shot size, one-shot clear
};

extern "C" {

int tde_abi_version(void) { return TDE_ABI_VERSION; }

const char *tde_status_string(int status) {
    switch (status) {
    case TDE_OK: return "ok";
    case TDE_EINVAL: return "invalid argument (null pointer or malformed struct)";
    case TDE_ENRANKS: return "nranks must be 2, 4 or 8";
    case TDE_EDTYPE: return "unsupported dtype (bf16, f16, f32, f64)";
    case TDE_ESHAPE: return "bad shape: hidden*elem_size must be a positive multiple of 16 bytes, tokens >= 0";
    case TDE_EHIDDEN: return "hidden too large for the one-pass row kernel (max 1024 16-byte vectors per row: 8192 bf16/f16, 4096 f32, 2048 f64)";
    case TDE_EALIGN: return "buffer not 16-byte aligned";
    case TDE_EQUANT: return "bad quant mode, per-group quant with hidden not a multiple of 128, or static scale not > 0";
    case TDE_EALGO: return "bad algorithm, or staged algorithm without a stage buffer";
    case TDE_EHIP: return "HIP runtime error (see tde_last_hip_error)";
    case TDE_ERANK: return "rank outside [0, nranks)";
    case TDE_ENOMEM: return "device allocation failed";
    case TDE_ETOOBIG: return "tokens*hidden*elem_size exceeds the library's static stage (TDE_STATIC_STAGE_BYTES)";
    }
    return "unknown status";
}

int tde_last_hip_error(void) { return g_last_hip_error; }

int tde_probe_copy(void *dst, const void *src, int64_t bytes, void *hip_stream) {
    if (dst == nullptr || src == nullptr || bytes < 0 || bytes % 16 != 0) return TDE_EINVAL;
    if (!aligned16(dst) || !aligned16(src)) return TDE_EALIGN;
    if (bytes == 0) return TDE_OK;
    const int64_t vecs = bytes / 16;
    int64_t blocks = (vecs + 255) / 256;
    if (blocks > compute_units() * 16) blocks = compute_units() * 16;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(hip_stream), src, dst, vecs);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TDE_OK : hip_fail(e);
}

int tde_probe_launch(void *hip_stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(hip_stream));
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TDE_OK : hip_fail(e);
}

int tde_probe_stream(void *dst, const void *src, int64_t bytes, int32_t mode, void *hip_stream) {
    if (dst == nullptr || src == nullptr || bytes < 0 || bytes % 16 != 0 || mode < 0 || mode > 2) return TDE_EINVAL;
    if (!aligned16(dst) || !aligned16(src)) return TDE_EALIGN;
    if (bytes == 0) return TDE_OK;
    const int64_t blocks = (bytes + 4095) / 4096;
    if (blocks > 0x7fffffff) return TDE_ESHAPE;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const dim3 grid((unsigned)blocks), block(256);
    switch (mode) {
    case 0: hipLaunchKernelGGL(stream_kernel<0>, grid, block, 0, s, src, dst, bytes); break;
    case 1: hipLaunchKernelGGL(stream_kernel<1>, grid, block, 0, s, src, dst, bytes); break;
    default: hipLaunchKernelGGL(stream_kernel<2>, grid, block, 0, s, src, dst, bytes); break;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TDE_OK : hip_fail(e);
}

int tde_device_info(tde_device_info_out *out) {
    if (out == nullptr) return TDE_EINVAL;
    std::memset(out, 0, sizeof(*out));
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    int cu = 0, khz = 0, bits = 0;
    e = hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return hip_fail(e);
    // Clock and width are optional: a runtime that does not report them leaves zeros.
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeMemoryClockRate, dev) != hipSuccess) khz = 0;
    if (hipDeviceGetAttribute(&bits, hipDeviceAttributeMemoryBusWidth, dev) != hipSuccess) bits = 0;
    (void)hipGetLastError();
    size_t free_b = 0, total_b = 0;
    e = hipMemGetInfo(&free_b, &total_b);
    if (e != hipSuccess) return hip_fail(e);
    out->compute_units = cu;
    out->memory_clock_khz = khz;
    out->memory_bus_bits = bits;
    out->total_memory_bytes = (int64_t)total_b;
    return TDE_OK;
}

int tde_plan(const tde_problem *problem, tde_plan_out *plan) {
    if (plan == nullptr) return TDE_EINVAL;
    tde::Geometry g{};
    const int st = validate(problem, &g);
    if (st != TDE_OK) return st;
    std::memset(plan, 0, sizeof(*plan));
    plan->algo = (problem->algo == TDE_ALGO_STAGED || problem->algo == TDE_ALGO_STAGED_OWNED) ? problem->algo : TDE_ALGO_FUSED;
    plan->reference_algo = (problem->tokens <= 128) ? 1 : 2;
    plan->vec_elems = g.vec_elems;
    plan->block_threads = g.block_threads;
    plan->vecs_per_thread = g.vpt;
    plan->rows_per_block = g.rows_per_block;
    plan->grid_blocks = (int32_t)g.grid;
    plan->xcd_chunk = g.xcd_chunk;
    plan->workgroups_per_cu = g.wgs_per_cu;
    plan->lds_bytes = g.lds_bytes;
    plan->algorithmic_bytes = algorithmic_bytes(problem, &plan->scale_elems);
    return TDE_OK;
}

namespace {
enum : int { kPhaseReduce = 1, kPhaseNorm = 2, kTrafficOnly = 4 };

int run_phases(const tde_problem *p, const tde_buffers *b, void *hip_stream, int phases, int probe_parts = 7) {
    tde::Geometry g{};
    const int st = validate(p, &g);
    if (st != TDE_OK) return st;
    if (b == nullptr) return TDE_EINVAL;
    if (p->tokens == 0) return TDE_OK; // nothing to do; empty buffers may be null
    const bool quant = p->quant != TDE_QUANT_NONE;
    const bool wn = !quant || p->write_norm != 0;
    const bool staged = p->algo == TDE_ALGO_STAGED || p->algo == TDE_ALGO_STAGED_OWNED;
    const bool traffic = phases == kTrafficOnly;
    if (traffic) {
        if (staged) return TDE_EALGO; // the skeleton mirrors the fused kernel only
        phases = kPhaseReduce | kPhaseNorm;
    }
    const bool both = phases == (kPhaseReduce | kPhaseNorm);
    if (!both && !staged) return TDE_EALGO; // a single phase exists only in the staged algorithms
    const bool reads_partials = !staged || (phases & kPhaseReduce);

    for (int r = 0; reads_partials && r < p->nranks; ++r) {
        if (b->partial[r] == nullptr && b->partial_table == nullptr) return TDE_EINVAL;
        if (!aligned16(b->partial[r])) return TDE_EALIGN;
    }
    if (phases & kPhaseNorm) {
        if (!b->residual_in || !b->residual_out || !b->gamma) return TDE_EINVAL;
        if (wn && !b->norm_out) return TDE_EINVAL;
        if (quant && !b->q_out) return TDE_EINVAL;
        if (quant && p->quant != TDE_QUANT_FP8_STATIC && !b->scale_out) return TDE_EINVAL;
    }
    if (staged && !b->stage) return TDE_EALGO;
    if (!aligned16(b->residual_in) || !aligned16(b->residual_out) || !aligned16(b->gamma) ||
        !aligned16(b->norm_out) || !aligned16(b->stage) || !aligned16(b->partial_table))
        return TDE_EALIGN;
    if (quant && ((reinterpret_cast<uintptr_t>(b->q_out) & 7u) || (reinterpret_cast<uintptr_t>(b->scale_out) & 3u)))
        return TDE_EALIGN;

    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    tde::RowArgs a{};
    for (int r = 0; r < p->nranks; ++r) a.part[r] = b->partial[r];
    a.table = b->partial_table;
    a.residual_in = b->residual_in;
    a.residual_out = b->residual_out;
    a.norm_out = b->norm_out;
    a.gamma = b->gamma;
    a.q_out = b->q_out;
    a.scale_out = b->scale_out;
    a.stage_out = b->stage;
    a.tokens = p->tokens;
    a.hidden = (int32_t)p->hidden;
    a.nvec = g.nvec;
    a.threads_per_row = g.threads_per_row;
    a.rows_per_block = g.rows_per_block;
    a.xcd_chunk = g.xcd_chunk;
    a.eps = p->eps;
    a.hidden_f = (float)p->hidden;
    a.static_scale = p->static_scale;
    a.probe_parts = probe_parts;

    int n = p->nranks;
    hipError_t e = hipSuccess;
    if (traffic && p->dtype == TDE_F64) return TDE_EDTYPE;
    if (traffic) {
        const int code_bytes = quant ? (elem_bytes(p->dtype) == 4 ? 4 : 8) : 0;
        e = tde::launch_traffic(n, g.vpt, code_bytes, wn, a, g, (uint32_t)g.nvec * 16u, stream);
        return e == hipSuccess ? TDE_OK : hip_fail(e);
    }
    if (staged && (phases & kPhaseReduce)) {
        // All rows as one span of bytes, or only this rank's share (rows == rank mod nranks) row by row.
        const int64_t row_bytes = (int64_t)g.nvec * 16;
        int64_t span_bytes = p->tokens * row_bytes, first = 0, step = 1, rows = 1;
        if (p->algo == TDE_ALGO_STAGED_OWNED) {
            span_bytes = row_bytes;
            first = p->rank;
            step = p->nranks;
            rows = (p->tokens - p->rank + p->nranks - 1) / p->nranks;
        }
        switch (p->dtype) {
        case TDE_BF16: e = tde::launch_reduce_bf16(n, a, span_bytes, first, step, rows, stream); break;
        case TDE_F16: e = tde::launch_reduce_f16(n, a, span_bytes, first, step, rows, stream); break;
        case TDE_F32: e = tde::launch_reduce_f32(n, a, span_bytes, first, step, rows, stream); break;
        case TDE_F64: e = tde::launch_reduce_f64(n, a, span_bytes, first, step, rows, stream); break;
        }
        if (e != hipSuccess) return hip_fail(e);
    }
    if (!(phases & kPhaseNorm)) return TDE_OK;
    if (staged) {
        for (int r = 0; r < tde::kMaxKernelRanks; ++r) a.part[r] = nullptr;
        a.part[0] = b->stage;
        a.table = nullptr;
        n = 0;
    }
    switch (p->dtype) {
    case TDE_BF16: e = tde::launch_rows_bf16(n, g.vpt, p->quant, wn, a, g, stream); break;
    case TDE_F16: e = tde::launch_rows_f16(n, g.vpt, p->quant, wn, a, g, stream); break;
    case TDE_F32: e = tde::launch_rows_f32(n, g.vpt, p->quant, wn, a, g, stream); break;
    case TDE_F64: e = tde::launch_rows_f64(n, a, g, stream); break;
    }
    if (e != hipSuccess) return hip_fail(e);
    return TDE_OK;
}
} // namespace

int tde_reduce_rms(const tde_problem *p, const tde_buffers *b, void *hip_stream) {
    return run_phases(p, b, hip_stream, kPhaseReduce | kPhaseNorm);
}

int tde_stage_reduce(const tde_problem *p, const tde_buffers *b, void *hip_stream) {
    return run_phases(p, b, hip_stream, kPhaseReduce);
}

int tde_stage_norm(const tde_problem *p, const tde_buffers *b, void *hip_stream) {
    return run_phases(p, b, hip_stream, kPhaseNorm);
}

int tde_reduce_rms_static_stage(const tde_problem *p, const tde_buffers *b, void *hip_stream) {
    if (p == nullptr || b == nullptr) return TDE_EINVAL;
    if (p->algo != TDE_ALGO_AUTO && p->algo != TDE_ALGO_STAGED) return TDE_EALGO;
    tde_problem staged = *p;
    staged.algo = TDE_ALGO_STAGED;
    const int st = validate(&staged, nullptr);
    if (st != TDE_OK) return st;
    // validate() has bounded hidden and checked that tokens * hidden * elem does not overflow
    if (p->tokens * p->hidden * elem_bytes(p->dtype) > (int64_t)TDE_STATIC_STAGE_BYTES) return TDE_ETOOBIG;
    void *stage = nullptr;
    const int sp = static_stage_ptr(&stage);
    if (sp != TDE_OK) return sp;
    tde_buffers with_stage = *b;
    with_stage.stage = stage;
    return run_phases(&staged, &with_stage, hip_stream, kPhaseReduce | kPhaseNorm);
}

int tde_probe_rows(const tde_problem *p, const tde_buffers *b, void *hip_stream) {
    return run_phases(p, b, hip_stream, kTrafficOnly);
}

int tde_probe_rows_parts(const tde_problem *p, const tde_buffers *b, int32_t parts, void *hip_stream) {
    if (parts < 1 || parts > 7) return TDE_EINVAL;
    return run_phases(p, b, hip_stream, kTrafficOnly, parts);
}

// ---- emulated peer workspace ----------------------------------------------------------------

int tde_workspace_create(int32_t nranks, int32_t nblocks, int64_t slot_bytes, tde_workspace **out) {
    if (out == nullptr) return TDE_EINVAL;
    *out = nullptr;
    if (!(nranks == 2 || nranks == 4 || nranks == 8)) return TDE_ENRANKS;
    if (nblocks < 1 || nblocks > 65536) return TDE_EINVAL;
    if (slot_bytes <= 0 || slot_bytes % 16 != 0) return TDE_ESHAPE;
    tde_workspace *ws = new (std::nothrow) tde_workspace();
    if (ws == nullptr) return TDE_ENOMEM;
    ws->nranks = nranks;
    ws->nblocks = nblocks;
    ws->slot_bytes = slot_bytes;
    hipError_t e = hipSuccess;
    for (int r = 0; r < nranks && e == hipSuccess; ++r) e = hipMalloc(&ws->slots[r], (size_t)slot_bytes * 2);
    // one flag region per rank, each nblocks * nranks ints as the reference sizes it (src/ops/all_reduce_fusion.cpp:72)
    const size_t flag_bytes = (size_t)nranks * nblocks * nranks * sizeof(int32_t);
    if (e == hipSuccess) e = hipMalloc(&ws->flags, flag_bytes);
    if (e == hipSuccess) e = hipMemset(ws->flags, 0, flag_bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ws->cells), 5 * 64);
    if (e == hipSuccess) e = hipMemset(ws->cells, 0, 5 * 64);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        tde_workspace_destroy(ws);
        g_last_hip_error = (int)e;
        return (e == hipErrorOutOfMemory) ? TDE_ENOMEM : TDE_EHIP;
    }
    *out = ws;
    return TDE_OK;
}

int tde_workspace_destroy(tde_workspace *ws) {
    if (ws == nullptr) return TDE_OK;
    for (int r = 0; r < TDE_MAX_RANKS; ++r)
        if (ws->slots[r]) (void)hipFree(ws->slots[r]);
    if (ws->flags) (void)hipFree(ws->flags);
    if (ws->cells) (void)hipFree(ws->cells);
    delete ws;
    return TDE_OK;
}

void *tde_workspace_slot(const tde_workspace *ws, int32_t r) {
    if (ws == nullptr || r < 0 || r >= ws->nranks) return nullptr;
    return ws->slots[r];
}

void *tde_workspace_stage(const tde_workspace *ws, int32_t r) {
    if (ws == nullptr || r < 0 || r >= ws->nranks) return nullptr;
    return static_cast<char *>(ws->slots[r]) + ws->slot_bytes;
}

int64_t tde_workspace_slot_bytes(const tde_workspace *ws) { return ws ? ws->slot_bytes : 0; }
int32_t tde_workspace_nranks(const tde_workspace *ws) { return ws ? ws->nranks : 0; }

int tde_workspace_fill_table(const tde_workspace *ws, void **table, int32_t entries) {
    if (ws == nullptr || table == nullptr) return TDE_EINVAL;
    const int n = ws->nranks;
    if (entries != 3 * n + 5) return TDE_EINVAL;
    for (int r = 0; r < n; ++r) {
        table[r] = ws->slots[r];
        table[n + r] = static_cast<char *>(ws->flags) + (size_t)r * ws->nblocks * n * sizeof(int32_t);
        table[2 * n + r] = ws->slots[r];
    }
    for (int c = 0; c < 5; ++c) table[3 * n + c] = reinterpret_cast<char *>(ws->cells) + 64 * c;
    return TDE_OK;
}

} // extern "C"
