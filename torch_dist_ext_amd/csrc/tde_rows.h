// Row kernels for gfx950 (MI355X): N-way partial reduce + residual add + RMSNorm + dynamic quant,
// one pass per row with the row held in registers.
//
// Arithmetic contract (what the reference's torch-eager composition computes,
// test/test_all_reduce_fusion.py:23-28,75-76, with the reduce order of
// src/common/all_reduce_fusion_impl.h:280-298):
//   s   = T( ((0 + p_0) + p_1) + ... + p_{N-1} )      fp32 accumulate in rank order, one rounding to T
//   x   = T( float(s) + float(residual_in) )           -> residual_out            (impl.h:271-278)
//   rs  = 1 / sqrt( sum(float(x)^2) / H + eps )        fp32, IEEE divide and sqrt; the sum in the order of
//                                                      torch's CPU reduction (sumsq_torch_order below)
//   y1  = T( float(x) * rs )
//   y   = T( float(gamma) * float(y1) )                -> norm_out
//   per-token fp8 : scale = amax|y| / 448, code = e4m3( clamp(float(y)/scale, +-448) )
//   per-group fp8 : the same over each 128-column group
//   per-token int8: scale = amax|y| / 127, code = clamp(rne(float(y)/scale), +-127)
//   static fp8    : code = e4m3( clamp(float(y)/static_scale, +-448) ), no scale written
//
// Included by one translation unit per element type; nothing here is exported.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "tde_abi.h"

namespace tde {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kMaxWavesPerBlock = 16;
constexpr int kMaxKernelRanks = 8;

// Kernel argument block (passed by value in kernarg memory).
struct RowArgs {
    const void *part[kMaxKernelRanks]; // host-known partial pointers (or the stage buffer in [0])
    const void *const *table;          // optional device pointer table; entry r used when part[r] == null
    const void *residual_in;
    void *residual_out;
    void *norm_out;
    const void *gamma;
    void *q_out;
    float *scale_out;
    void *stage_out; // stage A destination
    int64_t tokens;
    int32_t hidden;
    int32_t nvec;           // 16-byte vectors per row
    int32_t threads_per_row; // multiple of 64
    int32_t rows_per_block;
    int32_t xcd_chunk; // workgroups per XCD chunk of the row mapping (power of two; 0 or 1 = rows in launch order)
    float eps;
    float hidden_f;
    float static_scale;
    int32_t probe_parts; // traffic skeleton only: bit 0 read the inputs, bit 1 write the T-typed rows, bit 2 write the code rows
};

// ---------------------------------------------------------------------------------------------
// Element traits: a 16-byte vector <-> VEC floats.  pack() rounds to nearest even.
// ---------------------------------------------------------------------------------------------
struct ElemBF16 {
    static constexpr int VEC = 8;
    static constexpr int BYTES = 2;
    static __device__ __forceinline__ void unpack(u32x4 raw, float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __builtin_bit_cast(float, raw[i] << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, raw[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 raw;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x2 v = {f[2 * i], f[2 * i + 1]};
            raw[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
        }
        return raw;
    }
    // fp32 bit pattern of a non-negative element given by its own bits
    static __device__ __forceinline__ uint32_t magnitude_to_f32_bits(uint32_t m) { return m << 16; }
};

struct ElemF16 {
    static constexpr int VEC = 8;
    static constexpr int BYTES = 2;
    static __device__ __forceinline__ void unpack(u32x4 raw, float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = raw[i]; // copy first: bit_cast applied straight to a vector element reads lane 0
            const f16x2 h = __builtin_bit_cast(f16x2, w);
            f[2 * i] = (float)h[0];
            f[2 * i + 1] = (float)h[1];
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 raw;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f16x2 h = {(_Float16)f[2 * i], (_Float16)f[2 * i + 1]};
            raw[i] = __builtin_bit_cast(uint32_t, h);
        }
        return raw;
    }
    static __device__ __forceinline__ uint32_t magnitude_to_f32_bits(uint32_t m) {
        return __builtin_bit_cast(uint32_t, (float)__builtin_bit_cast(_Float16, (uint16_t)m)); // NaN stays NaN
    }
};

struct ElemF32 {
    static constexpr int VEC = 4;
    static constexpr int BYTES = 4;
    static __device__ __forceinline__ void unpack(u32x4 raw, float (&f)[VEC]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = raw[i]; // copy first: bit_cast applied straight to a vector element reads lane 0
            f[i] = __builtin_bit_cast(float, w);
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[VEC]) {
        u32x4 raw;
#pragma unroll
        for (int i = 0; i < 4; ++i) raw[i] = __builtin_bit_cast(uint32_t, f[i]);
        return raw;
    }
    static __device__ __forceinline__ uint32_t magnitude_to_f32_bits(uint32_t m) { return m; }
};

// Largest magnitude of a row's elements, taken on the bit patterns: for non-negative floats of one format the
// unsigned order of the bits is the order of the values with every NaN above infinity, so an unsigned maximum of
// |x| propagates NaN as torch's amax does (a float maximum would drop it) and costs no more.  The 2-byte types keep
// two running 16-bit maxima in one register (one packed instruction per two elements).
//   amax_fold: folds a 16-byte vector into the running maximum (start from 0)
//   amax_f32_bits: the fp32 bit pattern of the largest magnitude folded in (a NaN pattern if any element was NaN)
__device__ __forceinline__ uint32_t max_u32(uint32_t a, uint32_t b) { return a > b ? a : b; }

template <class E>
__device__ __forceinline__ uint32_t amax_fold(uint32_t acc, u32x4 raw) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = raw[i]; // copy first: bit_cast applied straight to a vector element reads lane 0
        if constexpr (E::BYTES == 2) {
            const u16x2 a = __builtin_bit_cast(u16x2, acc), b = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
            acc = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
        } else {
            acc = max_u32(acc, w & 0x7fffffffu);
        }
    }
    return acc;
}

template <class E>
__device__ __forceinline__ uint32_t amax_f32_bits(uint32_t acc) {
    if constexpr (E::BYTES == 2) acc = max_u32(acc >> 16, acc & 0xffffu);
    return E::magnitude_to_f32_bits(acc);
}

// ---------------------------------------------------------------------------------------------
// 64-lane wavefront reductions: four DPP steps inside each 16-lane row, then the four row
// results are combined through v_readlane.  Every lane ends with the same value.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, dpp_move_u32<CTRL>(__builtin_bit_cast(uint32_t, v)));
}

// Unsigned maximum over each 16-lane row (the maxima here are bit patterns of magnitudes, see amax_fold).
__device__ __forceinline__ uint32_t row16_max(uint32_t v) {
    v = max_u32(v, dpp_move_u32<0xB1>(v));  // quad_perm [1,0,3,2]
    v = max_u32(v, dpp_move_u32<0x4E>(v));  // quad_perm [2,3,0,1]
    v = max_u32(v, dpp_move_u32<0x141>(v)); // row_half_mirror
    v = max_u32(v, dpp_move_u32<0x140>(v)); // row_mirror
    return v;
}

__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ uint32_t wave_max(uint32_t v) {
    v = row16_max(v);
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16),
                   c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max_u32(max_u32(a, b), max_u32(c, d));
}

// Maximum over the `waves_per_row` wavefronts that share a row.  `slots` is an LDS buffer indexed by wavefront
// number inside the block, used once per kernel (one barrier).  Identity is 0 (bit patterns of magnitudes).
__device__ __forceinline__ uint32_t row_max(uint32_t v, uint32_t *slots, int wave, int lane, int first_wave, int waves_per_row) {
    v = wave_max(v);
    if (waves_per_row == 1) return v;
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    const int k = lane & 15;
    const uint32_t t = (k < waves_per_row) ? slots[first_wave + k] : 0u;
    return row16_max(t);
}

// ---------------------------------------------------------------------------------------------
// Sum of a row's squares in the order of torch's CPU reduction.
//
// The eager composition computes x.float().pow(2).mean(-1) (test/test_all_reduce_fusion.py:25).  On x86 hosts
// torch reduces a contiguous row of n floats with 8-lane vectors and four interleaved vector accumulators
// (its cascade sum): with V = n / 8 vectors, I = V / 4,
//   chain (m, k), m = 0..7, k = 0..3, takes the elements 8 * (4 * i + k) + m, i = 0..I-1;
//   every 16 consecutive i form a block that is summed left to right from zero; the block sums of a chain are
//   summed left to right (a last block shorter than 16 included);
//   p[m] = chain(m,0) + the V % 4 vectors left over + chain(m,1) + chain(m,2) + chain(m,3), left to right;
//   sum  = the n % 8 scalars left over, then p[0] .. p[7], left to right from zero.
// (Rows shorter than 8 floats use four interleaved scalars instead; rows beyond 8192 floats would add a cascade
// level and do not occur: a row has at most 1024 16-byte vectors.)  Following that order makes the reciprocal RMS,
// and with it every normed element, scale and code, bit-identical to the eager composition's.
//
// The row's squares are laid out in LDS in element order (`img`); one thread sums one block of one chain
// (16 reads 32 floats apart), the block sums go through LDS (`bs`), and lanes 4m+k of every wavefront finish chain
// (m, k).  With 8 floats per 16-byte vector (2-byte element types) a block of 64 vectors is exactly what one
// wavefront loaded with one load instruction, so the first step needs no workgroup barrier (WAVE_BLOCKS).
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float quad_bcast(float v) {
    return dpp_move<CTRL>(v);
}

// Dynamic LDS a kernel that calls sumsq_torch_order needs.
inline size_t sumsq_lds_bytes(int block_threads, int vpt, int vec_floats) {
    return ((size_t)block_threads * vpt * vec_floats + 1024) * sizeof(float);
}

// A compute unit of gfx950 has 160 KiB of LDS; a workgroup that asks for this much dynamic LDS (the kernels' 64
// static bytes and the allocation granule fit in the slack) shares its CU with at most `wgs` - 1 others.
constexpr size_t kLdsPerCu = 160 * 1024;
constexpr size_t kDefaultMaxDynamicLds = 64 * 1024; // what a kernel may ask for without raising its attribute
inline size_t lds_bytes_for_workgroups_per_cu(int wgs) { return (kLdsPerCu / (size_t)wgs - 1024) & ~(size_t)255; }

// Raises KERNEL's dynamic-LDS ceiling to (nearly) the whole CU, once per device (a launch asking for more than 64 KiB
// fails otherwise).  Not a stream operation; the first launch of a kernel on a device that needs it pays for it.
template <auto KERNEL>
hipError_t allow_large_lds() {
    static std::atomic<uint64_t> done{0}; // bit d: set on device d
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t{1} << dev) : 0;
    if (bit != 0 && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    // the most a launch here asks for; the kernel's static LDS must still fit beside it
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes_for_workgroups_per_cu(1));
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    else (void)hipGetLastError(); // reported through the return value, not left behind for the next call
    return e;
}

// Returns `v`, but only once `after` exists: index arithmetic built on the result cannot be hoisted above the
// row loads, whose registers leave no room for it.
__device__ __forceinline__ int not_before(int v, uint32_t after) {
    asm volatile("; index math stays behind the row loads" : "+v"(v) : "v"(after));
    return v;
}

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Block `b` of chain `cl` (= 4m + k): the first `terms` (0..16) of 16 elements 32 floats apart, summed left to
// right.  GUARD: never read past the last term (rows whose LDS image ends inside the block).
template <bool GUARD>
__device__ __forceinline__ float chain_block_sum(const float *img, int b, int cl, int terms) {
    const float *src = img + 512 * b + 8 * (cl & 3) + (cl >> 2);
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = src[(!GUARD || i < terms) ? 32 * i : 0];
    float acc = 0.0f;
    if (__builtin_amdgcn_ballot_w64(terms != 16) == 0) { // every lane of the wavefront has a full block
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += v[i];
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += (i < terms) ? v[i] : 0.0f;
    }
    return acc;
}

// Wavefront-uniform variant of not_before (the value comes back in a scalar register).
__device__ __forceinline__ int uniform_not_before(int v, uint32_t after) {
    return __builtin_amdgcn_readfirstlane(not_before(v, after));
}

// The squares of this thread's vector j (vector index j * tpr + t of the row) go to their place in the row group's
// image, which holds the row's squares in element order.  `after`: a word of the data the squares were computed from.
template <int VPT, int VECF>
__device__ __forceinline__ void sumsq_put(float *lds_img, int j, int tpr, int group, int t, const float (&sq)[VECF], uint32_t after) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int vec = not_before(group * (tpr * VPT) + j * tpr + t, after);
    float *dst = lds_img + vec * VECF;
    if constexpr (VECF % 4 == 0) {
#pragma unroll
        for (int c = 0; c < VECF; c += 4) *reinterpret_cast<f32x4 *>(dst + c) = f32x4{sq[c], sq[c + 1], sq[c + 2], sq[c + 3]};
    } else {
#pragma unroll
        for (int c = 0; c < VECF; ++c) dst[c] = sq[c];
    }
}

// After every thread of the row group has put its squares: the sum, the same value in every thread.
// lds_img: one float per element the workgroup holds (threads * VPT * VECF), lds_bs: 1024 floats (32 per block),
// both shared by the workgroup's row groups (sumsq_lds_bytes gives the total).
// Contains workgroup barriers when a row spans several wavefronts: all threads of the workgroup must call it together.
template <int VPT, int VECF, bool WAVE_BLOCKS>
__device__ __forceinline__ float sumsq_torch_order(float *lds_img, float *lds_bs, int n, int t, int tpr, int group, int lane,
                                                   uint32_t after) {
    n = uniform_not_before(n, after);
    tpr = uniform_not_before(tpr, after);
    group = uniform_not_before(group, after);
    t = not_before(t, after);
    lane = not_before(lane, after);
    const int waves_per_row = tpr >> 6;
    const int cap = tpr * VPT * VECF;        // floats this row group can hold
    const int cap_blocks = (cap + 511) >> 9; // 64-vector blocks this row group can hold (<= 16)
    float *img = lds_img + group * cap;
    float *bs = lds_bs + group * (cap_blocks * 32);
    const int V = n >> 3, tail = n & 7, I = V >> 2, L = V & 3, NB = (I + 15) >> 4;

    const int cl = lane & 31;
    int blocks = NB; // block sums that exist in `bs`
    if constexpr (WAVE_BLOCKS) {
        static_assert(VECF == 8, "one wavefront load = one block of 64 eight-float vectors");
        // Block j * waves_per_row + w is what wavefront w wrote for its vector j: no other wavefront is involved.
        // Blocks past the row's end sum to zero, and adding zero to a sum of squares changes nothing.
        wave_lds_fence();
        const int w = t >> 6;
        if constexpr (VPT == 1) {
            if (lane < 32) { // one block per wavefront: half of its lanes have a chain
                int terms = I - 16 * w;
                terms = terms < 0 ? 0 : (terms > 16 ? 16 : terms);
                bs[w * 32 + cl] = chain_block_sum<false>(img, w, cl, terms);
            }
        } else {
            // two blocks at a time, one per half of the wavefront; their reads and sums interleave
            float sum[VPT / 2];
            int b[VPT / 2];
#pragma unroll
            for (int s = 0; s < VPT / 2; ++s) {
                b[s] = ((lane >> 5) + 2 * s) * waves_per_row + w;
                int terms = I - 16 * b[s];
                terms = terms < 0 ? 0 : (terms > 16 ? 16 : terms);
                sum[s] = chain_block_sum<false>(img, b[s], cl, terms);
            }
#pragma unroll
            for (int s = 0; s < VPT / 2; ++s) bs[b[s] * 32 + cl] = sum[s];
        }
        blocks = cap_blocks;
    } else {
        if (waves_per_row > 1) __syncthreads(); else wave_lds_fence();
        for (int c = t; c < 32 * NB; c += tpr) {
            const int b = c >> 5;
            int terms = I - 16 * b;
            terms = terms > 16 ? 16 : terms;
            bs[c] = chain_block_sum<true>(img, b, c & 31, terms);
        }
    }
    if (waves_per_row > 1) __syncthreads(); else wave_lds_fence();

    // Lane 4m + k of every wavefront sums the blocks of chain (m, k); the quad then holds the four chains of m.
    float chain = 0.0f;
    if (blocks == 16) {
        float v[16];
#pragma unroll
        for (int b2 = 0; b2 < 16; ++b2) v[b2] = bs[b2 * 32 + cl];
#pragma unroll
        for (int b2 = 0; b2 < 16; ++b2) chain += v[b2];
    } else if (blocks <= 8) {
        float v[8];
#pragma unroll
        for (int b2 = 0; b2 < 8; ++b2) v[b2] = bs[(b2 < blocks ? b2 : 0) * 32 + cl];
#pragma unroll
        for (int b2 = 0; b2 < 8; ++b2) chain += (b2 < blocks) ? v[b2] : 0.0f;
    } else {
        float v[16];
#pragma unroll
        for (int b2 = 0; b2 < 16; ++b2) v[b2] = bs[(b2 < blocks ? b2 : 0) * 32 + cl];
#pragma unroll
        for (int b2 = 0; b2 < 16; ++b2) chain += (b2 < blocks) ? v[b2] : 0.0f;
    }
    const int m = cl >> 2;
    float p = quad_bcast<0x00>(chain);
    for (int l = 0; l < L; ++l) p += img[8 * (4 * I + l) + m];
    p += quad_bcast<0x55>(chain);
    p += quad_bcast<0xAA>(chain);
    p += quad_bcast<0xFF>(chain);

    float sum = 0.0f;
    if (V == 0) {
        // fewer than 8 floats: four interleaved scalars, the first of them also takes what is left over
        if (n < 4) {
            for (int e = 0; e < n; ++e) sum += img[e];
        } else {
            sum = img[0];
            for (int e = 4; e < n; ++e) sum += img[e];
            sum += img[1];
            sum += img[2];
            sum += img[3];
        }
    } else {
        for (int e = 0; e < tail; ++e) sum += img[8 * V + e];
    }
#pragma unroll
    for (int mm = 0; mm < 8; ++mm) sum += read_lane(p, 4 * mm);
    return sum;
}

// Every buffer is device (global) memory: the few accesses that do not go through a buffer resource
// are typed as address space 1, so they never take the flat aperture check.
#define TDE_GLOBAL __attribute__((address_space(1)))

// Row-sized buffer resources.  A row is addressed as (wavefront-uniform 128-bit resource in SGPRs)
// + (32-bit lane offset in one VGPR).  The resource's size is the row's byte length, or 0 for a row
// past the end: the hardware then returns zeros for loads and drops stores, so neither partially
// filled wavefronts nor tail rows need a branch.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kRsrcFlags = 0x00020000; // raw buffer, 32-bit data format (gfx9 family encoding)
constexpr int kAuxStream = 2; // nt on loads and stores: streamed once, do not keep in cache.
// Measured on MI355X with inputs and outputs rotated far beyond the 256 MB memory-side cache:
// nt loads 7.0 vs 6.4 TB/s read ceiling; nt stores 1-2 % faster than sc1 and 8 % faster than the
// default policy on the 6:1 read/write mix.  (With outputs small enough to stay in that cache,
// sc1 stores measure faster; that is not the HBM-bound case.)
constexpr int kAuxStore = 2;
constexpr int kAuxDefault = 0;

__device__ __forceinline__ rsrc_t row_rsrc(const void *base, int64_t byte_off, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)(static_cast<const char *>(base) + byte_off), 0, (int)bytes,
                                             kRsrcFlags);
}
__device__ __forceinline__ u32x4 rsrc_load16(rsrc_t r, uint32_t off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, kAuxStream);
}
__device__ __forceinline__ void rsrc_store16(rsrc_t r, uint32_t off, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)off, 0, kAuxStore);
}

// Pack VEC fp32 values (already clamped to +-448) to OCP e4m3 bytes, round to nearest even.
template <int VEC>
__device__ __forceinline__ void pack_fp8(const float (&q)[VEC], uint32_t (&out)[VEC / 4]) {
#pragma unroll
    for (int w = 0; w < VEC / 4; ++w) {
        int word = 0;
        word = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * w], q[4 * w + 1], word, false);
        word = __builtin_amdgcn_cvt_pk_fp8_f32(q[4 * w + 2], q[4 * w + 3], word, true);
        out[w] = (uint32_t)word;
    }
}

template <int VEC>
__device__ __forceinline__ void pack_int8(const float (&q)[VEC], uint32_t (&out)[VEC / 4]) {
#pragma unroll
    for (int w = 0; w < VEC / 4; ++w) {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int code = (int)__builtin_rintf(q[4 * w + b]); // ties to even
            word |= ((uint32_t)code & 0xffu) << (8 * b);
        }
        out[w] = word;
    }
}

// y / d, correctly rounded, for a divisor shared by many elements.  `rcp` must be the correctly
// rounded 1/d.  q0 = RN(y*rcp) is within one ulp of the quotient; the residual y - q0*d is exact
// in one fma; adding residual*rcp back in a second fma rounds to the correctly rounded quotient
// (Markstein's division theorem) as long as nothing underflows.  Callers take this path only when
// d is far from the subnormal and overflow ranges and use a plain division otherwise.
// The residual is taken as q0*d - y and subtracted, not as y - q0*d and added: the same value for every non-zero y,
// and for y = -0 the result is then -0 like the quotient's (the other form ends in (+0) + (-0) = +0).
__device__ __forceinline__ float div_shared(float y, float d, float rcp) {
    const float q0 = y * rcp;
    const float e = __builtin_fmaf(q0, d, -y);
    return __builtin_fmaf(-e, rcp, q0);
}

// min(max(q, -limit), limit) that keeps NaN, as torch.clamp does (the float minimum and maximum drop it).
__device__ __forceinline__ float clamp_keep_nan(float q, float limit) {
    const float c = fminf(fmaxf(q, -limit), limit);
    return (q != q) ? q : c;
}

// Which row group a workgroup takes.  Workgroups are handed to the 8 XCDs round-robin, so in launch order
// every XCD (every L2) walks all of every buffer in 16 KiB steps.  Remapped in groups of 8*chunk, XCD k
// instead takes `chunk` consecutive row groups of each group, i.e. a contiguous piece of every buffer:
// measured 0.5-1.5 % faster with chunks of 8-16 rows (c3 58.4 -> 57.5 us), slower again beyond 64, and 2 %
// slower when each XCD owns one contiguous eighth of the tensor.  A grid tail shorter than a group keeps
// launch order, so the mapping stays one-to-one.
__device__ __forceinline__ uint32_t xcd_chunked_block(uint32_t bid, uint32_t grid, uint32_t chunk) {
    if (chunk > 1) {
        const uint32_t span = 8u * chunk; // power of two
        if (bid < (grid & ~(span - 1u))) {
            const uint32_t w = bid & (span - 1u);
            bid = (bid - w) + (w & 7u) * chunk + (w >> 3);
        }
    }
    return bid;
}

// The loads of one row: N partial vectors and one residual vector per owned 16-byte column slot.
template <int NP, int VPT>
struct RowLoads {
    u32x4 p[VPT][NP];
    u32x4 r[VPT];
};

// ---------------------------------------------------------------------------------------------
// The row kernel.
//   E      element traits
//   N      number of partials summed per element; N == 0 means "the sum was staged":
//          part[0] already holds s (a T-typed [tokens,hidden] buffer)
//   VPT    16-byte vectors per thread per row (1, 2 or 4)
//   Q      tde_quant
//   WN     write the T-typed normed row (always true for Q == NONE)
//   WIDE   compiled for two wavefronts per SIMD (256 registers) instead of three, with gamma requested ahead of the
//          row also for eight partials: two workgroups per CU whose gamma never waits.  Launched for eight partials
//          with four vectors per thread at 4 to 24 workgroups per CU (launch_rows_nv, Geometry::wide)
// Block layout: rows_per_block row groups of threads_per_row threads; thread t of a row group
// owns vectors t, t + threads_per_row, ... (coalesced 1 KiB per wavefront per load).
// ---------------------------------------------------------------------------------------------
template <class E, int N, int VPT, int Q, bool WN, bool WIDE = false>
__global__ void __launch_bounds__(1024 / VPT)
    __attribute__((amdgpu_waves_per_eu(VPT == 1 ? 8 : (VPT == 2 ? 5 : (WIDE ? 2 : 3))))) row_kernel(const RowArgs a) {
    constexpr int VEC = E::VEC;
    constexpr int NP = (N == 0) ? 1 : N;
    // residual_out is stored together with the row's other output at the end, one write burst per row: against storing
    // it as soon as the sum is known that measures 0.9 % faster on 8 x [2048, 8192] bf16 -> fp8, 0.4 % on 4 x [8192, 7168]
    // -> fp8 per group, 2.6 % on 2 x [8192, 8192], 7 % on 4 x [512, 7168], and the same within noise elsewhere.
    // Dynamic LDS: the workgroup's squares (one float per element it holds), then 1024 floats of block sums.
    extern __shared__ __attribute__((aligned(16))) float lds_dyn[];
    float *const lds_img = lds_dyn;
    float *const lds_bs = lds_dyn + blockDim.x * (VPT * VEC);
    __shared__ uint32_t lds_max[kMaxWavesPerBlock];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tpr = a.threads_per_row;
    const int waves_per_row = tpr >> 6;
    const int group = __builtin_amdgcn_readfirstlane(tid / tpr); // uniform inside a wavefront
    const int first_wave = group * waves_per_row;
    const uint32_t row_bytes = (uint32_t)a.hidden * E::BYTES;

    // Partial pointers: from the argument block, or (one uniform branch, batched scalar loads)
    // from the device pointer table for the entries the host left null.
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

    uint32_t lane_off[VPT]; // byte offset of this thread's vector j inside a row
#pragma unroll
    for (int j = 0; j < VPT; ++j) lane_off[j] = (uint32_t)(j * tpr + tid - group * tpr) * 16u;
// Thread index inside the row group and lane index, rebuilt from the first load offset where they are needed:
// the thread id itself does not stay in a register through the load phase, which has none to spare.
#define TDE_T ((int)(lane0 >> 4))
#define TDE_LANE ((int)(lane0 >> 4) & (kWave - 1))

    auto issue_loads = [&](RowLoads<NP, VPT> &d, int64_t row) {
        const uint32_t bytes = (row < a.tokens) ? row_bytes : 0u;
        const int64_t row_byte = row * (int64_t)row_bytes;
#pragma unroll
        for (int r = 0; r < NP; ++r) {
            const rsrc_t rs = row_rsrc(part[r], row_byte, bytes);
#pragma unroll
            for (int j = 0; j < VPT; ++j) d.p[j][r] = rsrc_load16(rs, lane_off[j]);
        }
        const rsrc_t rr = row_rsrc(a.residual_in, row_byte, bytes);
#pragma unroll
        for (int j = 0; j < VPT; ++j) d.r[j] = rsrc_load16(rr, lane_off[j]);
    };

    // One workgroup, one group of rows: the grid covers every row (no loop; a looping wavefront waits for its
    // own stores, a fresh workgroup does not).
    const int64_t row0 = (int64_t)xcd_chunked_block(blockIdx.x, gridDim.x, (uint32_t)a.xcd_chunk) * a.rows_per_block;

    // The row's loads go out before anything else touches memory -- except gamma where it pays to have it first:
    // with up to four partials of a 2-byte type, several vectors per thread and a per-token scale, the registers are
    // there to hold gamma through the load phase, and requested ahead of the row (it is served from L2) it is never
    // waited for behind the row's own traffic.  Measured against requesting it after the accumulate phase, alternating
    // two builds in one process: 4 x [32768, 5120] fp16 -> int8 per token -1.0 %, 4 x [8192, 7168] bf16 -> fp8 per
    // token -1.4 %, 2 x [8192, 8192] -0.6 %, 4 x [2048, 7168] -0.7 %; with per-group scales (no second barrier to
    // cover) +0.9 to +2.7 %, with T-typed output or fp32 rows equal to +0.4 %, so those keep the late request.
    // With eight partials the 16 registers are one too many for three wavefronts per SIMD (169 against 168: spilling
    // costs 2 us on 8 x [2048, 8192], and gamma ahead of the row for three of the four vectors gains 0.1 us); the WIDE
    // instantiation takes them and runs two workgroups per CU: 8 x [2048, 8192] bf16 -> fp8 56.8 us against 57.3,
    // -0.8 % from 1024 to 4096 rows, -1.5 % for rows of 7168, -2.2 % for 4096 rows of 2048, nothing from 6144 rows on
    // (where the launch is limited to two workgroups per CU anyway) and +0.8 to +1.8 % below 1024 rows.  The other
    // eight-partial kernels gain less but none loses (per-group scales -1.0 %, T-typed output -0.3 to -0.8 %, fp32 rows
    // -0.2 to -0.9 %), so WIDE carries gamma ahead of the row for all of them.
    const rsrc_t gamma_rsrc = row_rsrc(a.gamma, 0, row_bytes);
    constexpr bool GAMMA_FIRST =
        VPT > 1 && N != 0 &&
        (WIDE || (N <= 4 && E::BYTES == 2 && (Q == TDE_QUANT_FP8_TOKEN || Q == TDE_QUANT_INT8_TOKEN)));
    u32x4 gamma_first[GAMMA_FIRST ? VPT : 1];
    if constexpr (GAMMA_FIRST) {
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            gamma_first[j] = __builtin_amdgcn_raw_buffer_load_b128(gamma_rsrc, (int)lane_off[j], 0, kAuxDefault);
        __builtin_amdgcn_sched_barrier(0);
    }
    RowLoads<NP, VPT> cur;
    issue_loads(cur, row0 + group);
    u32x4 gamma_early = u32x4{0, 0, 0, 0};
    if constexpr (VPT == 1) {
        __builtin_amdgcn_sched_barrier(0);
        gamma_early = __builtin_amdgcn_raw_buffer_load_b128(gamma_rsrc, (int)lane_off[0], 0, kAuxDefault);
    }
    // From here on only the first offset stays in a register (the compiler cannot see where it came from, so it
    // keeps neither the thread index nor the other offsets alive through the load phase); the others are one
    // addition away.
    uint32_t lane0 = lane_off[0];
    asm volatile("" : "+v"(lane0));
    const uint32_t vec_stride = (uint32_t)tpr * 16u;
#define TDE_OFF(j) (lane0 + (uint32_t)(j) * vec_stride)

    {
        const int64_t row = row0 + group;
        const bool row_ok = row < a.tokens;
        const uint32_t bytes = row_ok ? row_bytes : 0u;
        const int64_t row_byte = row * (int64_t)row_bytes; // wavefront-uniform

        // ---- reduce, residual add, sum of squares ------------------------------------------------
        const rsrc_t res_out = row_rsrc(a.residual_out, row_byte, bytes);
        u32x4 xraw[VPT];
        // With four vectors per thread, or one, the partials are summed rank by rank as they arrive (the memory system
        // returns a wavefront's loads in the order it issued them), so that only the last partial's additions are
        // left when the row is complete.  The order of every element's additions is the same either way.  With two
        // vectors per thread the accumulators cost more occupancy than the overlap returns (8 partials, 1024 rows of
        // 5120: 21.5 us against 20.4), so those variants sum vector by vector.  With one vector per thread (the
        // decode-size geometries) waiting rank by rank is worth 0.5-1.5 % up to 512 rows and nothing beyond.
        constexpr bool RANK_MAJOR = (N >= 4 && (VPT >= 4 || VPT == 1));
        float racc[RANK_MAJOR ? VPT : 1][VEC];
        if constexpr (RANK_MAJOR) {
            __builtin_amdgcn_sched_barrier(0);
            // The first two partials are taken together, vector by vector: their eight sums fit the registers the
            // two vectors arrived in, so the accumulators cost no registers while all other loads are in flight.
#pragma unroll
            for (int j = 0; j < VPT; ++j) {
                float p0[VEC], p1[VEC];
                E::unpack(cur.p[j][0], p0);
                E::unpack(cur.p[j][1], p1);
#pragma unroll
                for (int i = 0; i < VEC; ++i) racc[j][i] = (0.0f + p0[i]) + p1[i];
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 2; r < NP; ++r) {
#pragma unroll
                for (int j = 0; j < VPT; ++j) {
                    float p[VEC];
                    E::unpack(cur.p[j][r], p);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) racc[j][i] += p[i];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // From here on the wavefront has its row and only arithmetic, LDS and stores left: with up to four partials
        // (short load phases, three workgroups sharing the vector units about 60 % of the time) it goes ahead of the
        // wavefronts that are still summing partials.  4 x [32768, 5120] -0.5 %, 4 x [8192, 7168] -0.2 %; with eight
        // partials nothing at 2048+ rows and +0.7 % at 512 rows, so those stay at the default priority.
        if constexpr (N != 0 && N <= 4 && VPT == 4) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            float s[VEC];
            if constexpr (N == 0) {
                E::unpack(cur.p[j][0], s);
            } else if constexpr (RANK_MAJOR) {
                E::unpack(E::pack(racc[j]), s);
            } else {
                float acc[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
#pragma unroll
                for (int r = 0; r < NP; ++r) {
                    float p[VEC];
                    E::unpack(cur.p[j][r], p);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] += p[i];
                }
                E::unpack(E::pack(acc), s);
            }
            float res[VEC], x[VEC];
            E::unpack(cur.r[j], res);
#pragma unroll
            for (int i = 0; i < VEC; ++i) x[i] = s[i] + res[i];
            xraw[j] = E::pack(x);
            E::unpack(xraw[j], x);
            float sq[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) sq[i] = x[i] * x[i];
            sumsq_put<VPT, VEC>(lds_img, j, tpr, group, TDE_T, sq, xraw[j][0]);
        }
        // gamma (shared by all rows, served from L2).  With several vectors per thread it is requested
        // only now (unless it went out first, see GAMMA_FIRST): the registers of the row loads are free
        // again, and the reduction below covers its latency.  With one vector per thread registers are
        // plentiful and it was requested right behind the row loads (shortest dependent chain for small,
        // latency-bound inputs).
        u32x4 gamma_raw[VPT];
        if constexpr (GAMMA_FIRST) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) gamma_raw[j] = gamma_first[j];
        } else if constexpr (VPT > 1) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < VPT; ++j)
                gamma_raw[j] = __builtin_amdgcn_raw_buffer_load_b128(gamma_rsrc, (int)TDE_OFF(j), 0, kAuxDefault);
        } else {
            gamma_raw[0] = gamma_early;
        }
        const float sumsq = sumsq_torch_order<VPT, VEC, E::BYTES == 2>(lds_img, lds_bs, a.hidden, TDE_T, tpr, group, TDE_LANE, xraw[VPT - 1][0]);
        const float rs = 1.0f / __builtin_sqrtf(sumsq / a.hidden_f + a.eps);

        // ---- normalize ------------------------------------------------------------------------------
        u32x4 yraw[VPT];
        uint32_t amax[VPT]; // running maxima of the magnitudes' bit patterns (amax_fold), per vector
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            float x[VEC], g[VEC], y[VEC];
            E::unpack(xraw[j], x);
            E::unpack(gamma_raw[j], g);
#pragma unroll
            for (int i = 0; i < VEC; ++i) y[i] = x[i] * rs;
            E::unpack(E::pack(y), y);
#pragma unroll
            for (int i = 0; i < VEC; ++i) y[i] = g[i] * y[i];
            yraw[j] = E::pack(y);
            if constexpr (Q == TDE_QUANT_NONE || WN) {
                const rsrc_t norm_out = row_rsrc(a.norm_out, row_byte, bytes);
                rsrc_store16(norm_out, TDE_OFF(j), yraw[j]);
            }
            if constexpr (Q != TDE_QUANT_NONE && Q != TDE_QUANT_FP8_STATIC) amax[j] = amax_fold<E>(0u, yraw[j]);
        }

        if constexpr (Q == TDE_QUANT_NONE) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) rsrc_store16(res_out, TDE_OFF(j), xraw[j]);
        }

        // ---- dynamic quant epilogue ---------------------------------------------------------------
        if constexpr (Q != TDE_QUANT_NONE) {
            constexpr float QMAX = (Q == TDE_QUANT_INT8_TOKEN) ? 127.0f : 448.0f;
            float scale[VPT];
            if constexpr (Q == TDE_QUANT_FP8_GROUP) {
                constexpr int LANES_PER_GROUP = TDE_QUANT_GROUP / VEC; // 16 (2-byte types) or 32 (fp32)
                const int64_t groups_per_row = a.hidden / TDE_QUANT_GROUP;
                const rsrc_t sc_out = row_rsrc(a.scale_out, row * groups_per_row * 4, row_ok ? (uint32_t)groups_per_row * 4u : 0u);
#pragma unroll
                for (int j = 0; j < VPT; ++j) {
                    uint32_t m = row16_max(amax_f32_bits<E>(amax[j]));
                    if constexpr (LANES_PER_GROUP == 32) m = max_u32(m, (uint32_t)__shfl_xor((int)m, 16, kWave));
                    scale[j] = __builtin_bit_cast(float, m) / QMAX;
                    if ((TDE_LANE & (LANES_PER_GROUP - 1)) == 0)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, scale[j]), sc_out,
                                                              (int)((TDE_OFF(j) / 16u / LANES_PER_GROUP) * 4u), 0, kAuxDefault);
                }
            } else if constexpr (Q == TDE_QUANT_FP8_STATIC) {
#pragma unroll
                for (int j = 0; j < VPT; ++j) scale[j] = a.static_scale;
            } else {
                uint32_t m = amax[0];
#pragma unroll
                for (int j = 1; j < VPT; ++j) {
                    if constexpr (E::BYTES == 2) m = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, m), __builtin_bit_cast(u16x2, amax[j])));
                    else m = max_u32(m, amax[j]);
                }
                m = row_max(amax_f32_bits<E>(m), lds_max, wave, TDE_LANE, first_wave, waves_per_row);
                const float sc = __builtin_bit_cast(float, m) / QMAX;
#pragma unroll
                for (int j = 0; j < VPT; ++j) scale[j] = sc;
                if (row_ok && TDE_T == 0) ((TDE_GLOBAL float *)a.scale_out)[row] = sc;
            }
            const rsrc_t q_out = row_rsrc(a.q_out, row * (int64_t)a.hidden, row_ok ? (uint32_t)a.hidden : 0u);
#pragma unroll
            for (int j = 0; j < VPT; ++j) rsrc_store16(res_out, TDE_OFF(j), xraw[j]);
            // One wavefront-uniform decision for all of the thread's vectors, so the common path carries no per-lane
            // branch: the fast quotient needs every divisor far from the subnormal and overflow ranges.  A dynamic scale
            // that is NaN or infinite (a NaN or an infinity among the normed values) also takes the plain division.
            bool unsafe = false;
#pragma unroll
            for (int j = 0; j < VPT; ++j) unsafe = unsafe || !(scale[j] == 0.0f || (scale[j] > 0x1p-60f && scale[j] < 0x1p60f));
            const bool fast = __builtin_amdgcn_ballot_w64(unsafe) == 0;
            auto quantize = [&](auto use_fast) {
#pragma unroll
                for (int j = 0; j < VPT; ++j) {
                    float y[VEC], q[VEC];
                    E::unpack(yraw[j], y);
                    const float div = (scale[j] > 0.0f) ? scale[j] : 1.0f;
                    if constexpr (Q == TDE_QUANT_FP8_STATIC) {
                        // A caller's scale can be far below the row's values (the dynamic scales cannot: |y| <= QMAX *
                        // scale).  Beyond twice the largest code the quotient clamps to QMAX whatever it is, so y is cut
                        // there: the product y * rcp then stays finite and the correction never sees inf - inf.
                        const float ymax = (div < 0x1p60f) ? 2.0f * QMAX * div : 3.0e38f;
#pragma unroll
                        for (int i = 0; i < VEC; ++i) y[i] = clamp_keep_nan(y[i], ymax);
                    }
                    if constexpr (decltype(use_fast)::value) {
                        const float rcp = 1.0f / div;
                        if constexpr (Q == TDE_QUANT_FP8_STATIC) {
#pragma unroll
                            for (int i = 0; i < VEC; ++i) q[i] = clamp_keep_nan(div_shared(y[i], div, rcp), QMAX);
                        } else {
                            // |y| <= QMAX * scale up to two roundings: the quotient is within 1e-4 of +-QMAX at most,
                            // which the conversions below round to the largest code; nothing to clamp
#pragma unroll
                            for (int i = 0; i < VEC; ++i) q[i] = div_shared(y[i], div, rcp);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < VEC; ++i) q[i] = clamp_keep_nan(y[i] / div, QMAX);
                    }
                    uint32_t codes[VEC / 4];
                    if constexpr (Q == TDE_QUANT_INT8_TOKEN)
                        pack_int8<VEC>(q, codes);
                    else
                        pack_fp8<VEC>(q, codes);
                    const uint32_t code_off = (TDE_OFF(j) / 16u) * (uint32_t)VEC;
                    if constexpr (VEC == 8) {
                        u32x2 w = {codes[0], codes[1]};
                        __builtin_amdgcn_raw_buffer_store_b64(w, q_out, (int)code_off, 0, kAuxStore);
                    } else {
                        __builtin_amdgcn_raw_buffer_store_b32(codes[0], q_out, (int)code_off, 0, kAuxStore);
                    }
                }
            };
            if (fast)
                quantize(std::true_type{});
            else
                quantize(std::false_type{});
        }
    }
}
#undef TDE_T
#undef TDE_LANE
#undef TDE_OFF

// Stage A of the staged algorithm: s = T(sum of partials) for every element, no row structure.
// One workgroup of 256 threads reduces a contiguous span of 256*U vectors (U vectors per thread,
// all N*U loads in flight before the first add) and exits; spans past the end are cut by the buffer
// resource's size, so there is no loop and no tail branch.  U = 4 is the faster choice over the whole
// tensor (8 partials x 32 MiB: 50.5 us against 52.9 us with U = 2); for single 16 KiB rows it would
// leave one workgroup per row, and U = 2 (two per row) measures slightly faster there.
// Which bytes stage A covers: `row_bytes` long rows first_row, first_row + row_step, ...; each row is cut
// into spans_per_row spans.  The whole tensor as one long "row" (first_row 0) is the all-rows form; the
// reference's two-shot share of one rank is rows == rank (mod nranks) (impl.h:365-366).
struct ReduceSpan {
    int64_t row_bytes;
    int64_t first_row;
    int64_t row_step;
    int64_t spans_per_row;
    uint32_t xcd_chunk; // spans each XCD takes in a row (xcd_chunked_block); 16 over whole tensors, 1 for single rows
};

template <class E, int N, int U>
__global__ void __launch_bounds__(256) reduce_kernel(const RowArgs a, const ReduceSpan sp) {
    constexpr int VEC = E::VEC;
    constexpr uint32_t SPAN = 256u * U * 16u; // bytes per workgroup
    const void *part[N];
#pragma unroll
    for (int r = 0; r < N; ++r) part[r] = a.part[r];
    if (a.table != nullptr) {
#pragma unroll
        for (int r = 0; r < N; ++r) {
            const void *from_table = a.table[r];
            part[r] = (part[r] != nullptr) ? part[r] : from_table;
        }
    }
    const int64_t bid = xcd_chunked_block(blockIdx.x, gridDim.x, sp.xcd_chunk);
    const int64_t k = bid / sp.spans_per_row;
    const int64_t in_row = (bid - k * sp.spans_per_row) * SPAN;
    const int64_t base = (sp.first_row + k * sp.row_step) * sp.row_bytes + in_row;
    const int64_t left = sp.row_bytes - in_row;
    const uint32_t bytes = left < (int64_t)SPAN ? (uint32_t)left : SPAN;
    u32x4 raw[U][N];
#pragma unroll
    for (int r = 0; r < N; ++r) {
        const rsrc_t rs = row_rsrc(part[r], base, bytes);
#pragma unroll
        for (int u = 0; u < U; ++u) raw[u][r] = rsrc_load16(rs, (uint32_t)(u * 256 + threadIdx.x) * 16u);
    }
    const rsrc_t out = row_rsrc(a.stage_out, base, bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int r = 0; r < N; ++r) {
            float p[VEC];
            E::unpack(raw[u][r], p);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += p[i];
        }
        // The staged sum is re-read by stage B right away: default (cacheable) store.
        __builtin_amdgcn_raw_buffer_store_b128(E::pack(acc), out, (int)((u * 256 + threadIdx.x) * 16), 0, kAuxDefault);
    }
}

// ---------------------------------------------------------------------------------------------
// Host-side launch geometry shared by tde_plan and the launchers.
// ---------------------------------------------------------------------------------------------
struct Geometry {
    int wgs_per_cu; // limit on resident workgroups per compute unit (0 = none), enforced through lds_bytes
    int lds_bytes;  // dynamic LDS of the row kernel's launch
    int vec_elems;
    int nvec;
    int vpt;
    int threads_per_row;
    int rows_per_block;
    int block_threads;
    int64_t grid;
    int xcd_chunk;
    bool wide; // launch the row kernel's WIDE instantiation (eight partials, four vectors per thread)
};

// Per-dtype launchers, defined in tde_rows_<dtype>.hip.
hipError_t launch_rows_bf16(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s);
hipError_t launch_rows_f16(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s);
hipError_t launch_rows_f32(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s);
hipError_t launch_reduce_bf16(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows, hipStream_t s);
hipError_t launch_reduce_f16(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows, hipStream_t s);
hipError_t launch_reduce_f32(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows, hipStream_t s);

// Rows of doubles (tde_rows_f64.hip): one vector per thread, no quantized output.
hipError_t launch_rows_f64(int n, const RowArgs &a, const Geometry &g, hipStream_t s);
hipError_t launch_reduce_f64(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows, hipStream_t s);

// Traffic skeleton of the row kernel (tde_probe.hip): same geometry and bytes, no arithmetic.
hipError_t launch_traffic(int n, int vpt, int code_bytes, bool wn, const RowArgs &a, const Geometry &g, uint32_t row_bytes,
                          hipStream_t s);

// Instantiation + dispatch body used by the three per-dtype translation units.
template <class E, int N, int VPT>
hipError_t launch_rows_nv(int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s) {
    const dim3 grid((unsigned)g.grid), block((unsigned)g.block_threads);
    const size_t lds = (size_t)g.lds_bytes; // sumsq_lds_bytes of this geometry, padded where the launch limits workgroups per CU
#define TDE_LAUNCH(QM, WNB)                                                                              \
    if constexpr (N == 8 && VPT == 4) {                                                                  \
        if (g.wide) {                                                                                    \
            if (lds > kDefaultMaxDynamicLds) {                                                           \
                const hipError_t e = allow_large_lds<row_kernel<E, N, VPT, QM, WNB, true>>();            \
                if (e != hipSuccess) return e;                                                           \
            }                                                                                            \
            hipLaunchKernelGGL((row_kernel<E, N, VPT, QM, WNB, true>), grid, block, lds, s, a);        \
            return hipGetLastError();                                                                    \
        }                                                                                                \
    }                                                                                                    \
    if (lds > kDefaultMaxDynamicLds) {                                                                   \
        const hipError_t e = allow_large_lds<row_kernel<E, N, VPT, QM, WNB>>();                          \
        if (e != hipSuccess) return e;                                                                   \
    }                                                                                                    \
    hipLaunchKernelGGL((row_kernel<E, N, VPT, QM, WNB>), grid, block, lds, s, a);                      \
    return hipGetLastError();
    switch (q) {
    case TDE_QUANT_NONE: TDE_LAUNCH(TDE_QUANT_NONE, true)
    case TDE_QUANT_FP8_TOKEN:
        if (wn) { TDE_LAUNCH(TDE_QUANT_FP8_TOKEN, true) } else { TDE_LAUNCH(TDE_QUANT_FP8_TOKEN, false) }
    case TDE_QUANT_FP8_GROUP:
        if (wn) { TDE_LAUNCH(TDE_QUANT_FP8_GROUP, true) } else { TDE_LAUNCH(TDE_QUANT_FP8_GROUP, false) }
    case TDE_QUANT_INT8_TOKEN:
        if (wn) { TDE_LAUNCH(TDE_QUANT_INT8_TOKEN, true) } else { TDE_LAUNCH(TDE_QUANT_INT8_TOKEN, false) }
    case TDE_QUANT_FP8_STATIC:
        if (wn) { TDE_LAUNCH(TDE_QUANT_FP8_STATIC, true) } else { TDE_LAUNCH(TDE_QUANT_FP8_STATIC, false) }
    }
#undef TDE_LAUNCH
    return hipErrorInvalidValue;
}

template <class E, int N>
hipError_t launch_rows_n(int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s) {
    if (vpt == 1) return launch_rows_nv<E, N, 1>(q, wn, a, g, s);
    if (vpt == 2) return launch_rows_nv<E, N, 2>(q, wn, a, g, s);
    if (vpt == 4) return launch_rows_nv<E, N, 4>(q, wn, a, g, s);
    return hipErrorInvalidValue;
}

template <class E>
hipError_t launch_rows_e(int n, int vpt, int q, bool wn, const RowArgs &a, const Geometry &g, hipStream_t s) {
    switch (n) {
    case 0: return launch_rows_n<E, 0>(vpt, q, wn, a, g, s);
    case 2: return launch_rows_n<E, 2>(vpt, q, wn, a, g, s);
    case 4: return launch_rows_n<E, 4>(vpt, q, wn, a, g, s);
    case 8: return launch_rows_n<E, 8>(vpt, q, wn, a, g, s);
    }
    return hipErrorInvalidValue;
}

template <class E, int N, int U>
hipError_t launch_reduce_nu(const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows,
                            hipStream_t s) {
    constexpr int64_t span = 256 * U * 16;
    ReduceSpan sp{row_bytes, first_row, row_step, (row_bytes + span - 1) / span, rows == 1 ? 16u : 1u};
    const int64_t blocks = rows * sp.spans_per_row;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffff) return hipErrorInvalidValue; // grid dimension limit
    hipLaunchKernelGGL((reduce_kernel<E, N, U>), dim3((unsigned)blocks), dim3(256), 0, s, a, sp);
    return hipGetLastError();
}

template <class E, int N>
hipError_t launch_reduce_n(const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows,
                           hipStream_t s) {
    if (N >= 8 && row_bytes <= 256 * 4 * 16) return launch_reduce_nu<E, N, 2>(a, row_bytes, first_row, row_step, rows, s);
    return launch_reduce_nu<E, N, 4>(a, row_bytes, first_row, row_step, rows, s);
}

// Stage A over rows first_row, first_row + row_step, ... (`rows` of them), each row_bytes long.
template <class E>
hipError_t launch_reduce_e(int n, const RowArgs &a, int64_t row_bytes, int64_t first_row, int64_t row_step, int64_t rows,
                           hipStream_t s) {
    switch (n) {
    case 2: return launch_reduce_n<E, 2>(a, row_bytes, first_row, row_step, rows, s);
    case 4: return launch_reduce_n<E, 4>(a, row_bytes, first_row, row_step, rows, s);
    case 8: return launch_reduce_n<E, 8>(a, row_bytes, first_row, row_step, rows, s);
    }
    return hipErrorInvalidValue;
}

} // namespace tde
