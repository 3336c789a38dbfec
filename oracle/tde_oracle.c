/*
 * ORACLE — TEST INFRASTRUCTURE ONLY.  Never linked into or called from the product
 * (torch_dist_ext_amd/); only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it.
 *
 * Scalar C restatement, one element at a time, of one rank's reduce + residual + RMSNorm stage and
 * of this build's quant definitions.  Every dtype conversion is written out in integer arithmetic
 * (round to nearest even), so it shares no code with torch or with the HIP kernels.
 *
 * Reference lines followed:
 *   tdo_reduce_rms: sum     src/common/all_reduce_fusion_impl.h:280-298  fp32, rank order, one cast to T
 *                            (accumulator starts at +0 like test/test_all_reduce_fusion.py:75 `sum(dim=0)`)
 *                   residual src/common/all_reduce_fusion_impl.h:271-278  T(float(a)+float(b))
 *                   norm     test/test_all_reduce_fusion.py:23-28          x*rsqrt(mean(x^2)+eps) -> T -> weight*x -> T
 *                            (the kernel at impl.h:316-340 rounds once; the test composition, which is
 *                             the judged one, rounds twice — this file follows the test)
 *                   fp64 sum of squares as in test/unit_test.cpp:204-210 is mode TDO_SUMSQ_F64
 *                   mean    test/test_all_reduce_fusion.py:25 `x.float().pow(2).mean(-1)`: the arithmetic is in
 *                            torch (third party, not in the reference tree; 2.10.0 in this image).  Its CPU
 *                            kernel sums a contiguous row with 8-float vectors, four interleaved vector
 *                            accumulators and a cascade every 16 steps; tdo_torch_row_sum restates that order
 *                            (mode TDO_SUMSQ_TORCH) and tests/test_oracle.py pins it bit for bit against
 *                            torch.sum / torch.mean over every row length the tests and benchmarks use.
 *   quant (PARITY UNPINNED by the reference, which has no quant code): scale = amax/qmax,
 *                   code = rne(clamp(y/scale)), OCP e4m3 (bias 7, no infinities, NaN = 0x7f) or int8.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off, no fast-math)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define TDO_BF16 0
#define TDO_F16 1
#define TDO_F32 2

#define TDO_QUANT_NONE 0
#define TDO_QUANT_FP8_TOKEN 1
#define TDO_QUANT_FP8_GROUP 2
#define TDO_QUANT_INT8_TOKEN 3

#define TDO_SUMSQ_F32_SEQ 0  /* fp32 accumulator, left to right */
#define TDO_SUMSQ_F64 1      /* fp64 accumulator, rounded to fp32 once (closest to the exact mean) */
#define TDO_SUMSQ_F32_PAIRWISE 2 /* fp32 pairwise tree over the row */
#define TDO_SUMSQ_TORCH 3    /* the order of torch's CPU sum over a contiguous row (tdo_torch_row_sum) */

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- bfloat16 ---------------------------------------------------------------------------------- */
float tdo_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

uint16_t tdo_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb; /* round to nearest, ties to even */
    return (uint16_t)(u >> 16);
}

/* ---- IEEE half --------------------------------------------------------------------------------- */
float tdo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t tdo_f32_to_f16(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);         /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;                                 /* <= 2^-25 rounds to zero (tie to even) */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal half: value = m * 2^(e-23), unit 2^-24 */
        shift = (uint32_t)(-e - 1); /* m >> shift gives units of 2^-24: shift = 23 - (e + 24) */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1; /* carry into the exponent is correct by construction */
    return (uint16_t)(sign | (base + q));
}

/* ---- OCP fp8 e4m3 (e4m3fn): bias 7, max 448, no inf, NaN = S.1111.111 ---------------------------- */
float tdo_e4m3_to_f32(uint8_t c) {
    uint32_t sign = (c & 0x80u) ? 1u : 0u;
    uint32_t exp = (c >> 3) & 0xfu;
    uint32_t man = c & 7u;
    float v;
    if (exp == 15 && man == 7) return u2f(0x7fc00000u | (sign << 31));
    if (exp == 0) v = (float)man * (1.0f / 512.0f); /* man * 2^-9 */
    else v = ldexpf((float)(8 + man), (int)exp - 10); /* (1 + man/8) * 2^(exp-7) */
    return sign ? -v : v;
}

/* Round to nearest even; values that round above 448 become NaN (no saturation), like a plain
   cast.  Callers clamp to +-448 first. */
uint8_t tdo_f32_to_e4m3(float f) {
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    float x = u2f(a);
    if (x >= 464.0f) return (uint8_t)(sign | 0x7fu); /* 464 is the midpoint between 448 and the absent 480 */
    if (x < 0.0009765625f) return sign;              /* < 2^-10: half of the smallest subnormal 2^-9 -> 0; tie at 2^-10 goes to even (0) */
    if (x == 0.0009765625f) return sign;
    int e;
    (void)frexpf(x, &e); /* x = m * 2^e, m in [0.5,1) -> exponent of leading bit is e-1 */
    int le = e - 1;
    if (le < -6) le = -6; /* subnormal range uses the unit of exponent -6 */
    /* unit in the last place = 2^(le-3) */
    float ulp = ldexpf(1.0f, le - 3);
    float qf = x / ulp; /* exact: power-of-two scaling */
    float fl = floorf(qf);
    float rem = qf - fl;
    uint32_t q = (uint32_t)fl;
    if (rem > 0.5f || (rem == 0.5f && (q & 1u))) q += 1;
    /* q counts ulps: normal numbers have q in [8,16], subnormal q in [0,8] */
    uint32_t code;
    if (le == -6 && q < 8) code = q;                       /* subnormal */
    else {
        if (q == 16) { q = 8; le += 1; }
        code = ((uint32_t)(le + 7) << 3) | (q - 8);
    }
    if (code > 0x7eu) return (uint8_t)(sign | 0x7fu);
    return (uint8_t)(sign | code);
}

/* ---- generic element access ------------------------------------------------------------------- */
static float load_elem(int dtype, const void *p, int64_t i) {
    switch (dtype) {
    case TDO_BF16: return tdo_bf16_to_f32(((const uint16_t *)p)[i]);
    case TDO_F16: return tdo_f16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

static void store_elem(int dtype, void *p, int64_t i, float v) {
    switch (dtype) {
    case TDO_BF16: ((uint16_t *)p)[i] = tdo_f32_to_bf16(v); break;
    case TDO_F16: ((uint16_t *)p)[i] = tdo_f32_to_f16(v); break;
    default: ((float *)p)[i] = v; break;
    }
}

/* Round an fp32 value to the element type and back. */
static float round_elem(int dtype, float v) {
    switch (dtype) {
    case TDO_BF16: return tdo_bf16_to_f32(tdo_f32_to_bf16(v));
    case TDO_F16: return tdo_f16_to_f32(tdo_f32_to_f16(v));
    default: return v;
    }
}

/*
 * Sum of n floats in the order torch's CPU kernel uses for a reduction over a contiguous row on x86
 * (vector width 8 floats, four interleaved accumulators, partial sums flushed to the next cascade level
 * every 2^level_power steps).  Rows shorter than one vector take four interleaved scalars instead.
 */
static int ceil_log2_i64(int64_t x) {
    if (x <= 2) return 1;
    int n = 0;
    for (uint64_t v = (uint64_t)(x - 1); v; v >>= 1) ++n;
    return n;
}

/* nrows interleaved accumulators of `width` floats each over `size` steps; step i, accumulator k reads
   v[(i * nrows + k) * width + lane].  out[nrows][width]. */
static void cascade_rows(const float *v, int64_t size, int nrows, int width, float *out) {
    enum { LEVELS = 4 };
    float acc[LEVELS][4][8];
    memset(acc, 0, sizeof(acc));
    int level_power = ceil_log2_i64(size) / LEVELS;
    if (level_power < 4) level_power = 4;
    const int64_t level_step = (int64_t)1 << level_power;
    const int64_t level_mask = level_step - 1;
    int64_t i = 0;
    while (i + level_step <= size) {
        for (int64_t j = 0; j < level_step; ++j, ++i)
            for (int k = 0; k < nrows; ++k)
                for (int l = 0; l < width; ++l) acc[0][k][l] += v[(i * nrows + k) * width + l];
        for (int j = 1; j < LEVELS; ++j) {
            for (int k = 0; k < nrows; ++k)
                for (int l = 0; l < width; ++l) { acc[j][k][l] += acc[j - 1][k][l]; acc[j - 1][k][l] = 0.0f; }
            const int64_t mask = level_mask << (j * level_power);
            if ((i & mask) != 0) break;
        }
    }
    for (; i < size; ++i)
        for (int k = 0; k < nrows; ++k)
            for (int l = 0; l < width; ++l) acc[0][k][l] += v[(i * nrows + k) * width + l];
    for (int j = 1; j < LEVELS; ++j)
        for (int k = 0; k < nrows; ++k)
            for (int l = 0; l < width; ++l) acc[0][k][l] += acc[j][k][l];
    for (int k = 0; k < nrows; ++k)
        for (int l = 0; l < width; ++l) out[k * width + l] = acc[0][k][l];
}

/* One accumulator group of `width` lanes over `count` items of `width` floats: four interleaved partial sums,
   the items left over added to the first, then the other three added to it. */
static void row_sum_lanes(const float *v, int64_t count, int width, float *out) {
    float part[4 * 8];
    const int64_t size_ilp = count / 4;
    cascade_rows(v, size_ilp, 4, width, part);
    for (int64_t i = size_ilp * 4; i < count; ++i)
        for (int l = 0; l < width; ++l) part[l] += v[i * width + l];
    for (int k = 1; k < 4; ++k)
        for (int l = 0; l < width; ++l) part[l] += part[k * width + l];
    for (int l = 0; l < width; ++l) out[l] = part[l];
}

float tdo_torch_row_sum(const float *v, int64_t n) {
    enum { W = 8 };
    if (n < W) {
        float s;
        row_sum_lanes(v, n, 1, &s);
        return s;
    }
    float lanes[W];
    const int64_t vecs = n / W;
    row_sum_lanes(v, vecs, W, lanes);
    float s = 0.0f;
    for (int64_t k = vecs * W; k < n; ++k) s += v[k];
    for (int l = 0; l < W; ++l) s += lanes[l];
    return s;
}

static float pairwise_sum(const float *v, int64_t n) {
    if (n <= 8) {
        float s = 0.0f;
        for (int64_t i = 0; i < n; ++i) s += v[i];
        return s;
    }
    int64_t h = n / 2;
    return pairwise_sum(v, h) + pairwise_sum(v + h, n - h);
}

/*
 * The whole stage for [tokens, hidden].  parts: nranks pointers to [tokens*hidden] arrays of dtype.
 * norm_out may be NULL.  q_out / scale_out are required when quant != NONE.
 * Returns 0, or -1 on a bad argument.
 */
int tdo_reduce_rms(int dtype, int nranks, int64_t tokens, int64_t hidden, const void *const *parts,
                   const void *residual_in, const void *gamma, float eps, int quant, int sumsq_mode,
                   void *residual_out, void *norm_out, uint8_t *q_out, float *scale_out) {
    if (nranks < 1 || tokens < 0 || hidden <= 0 || !parts || !residual_in || !gamma || !residual_out) return -1;
    if (quant != TDO_QUANT_NONE && (!q_out || !scale_out)) return -1;
    if (quant == TDO_QUANT_FP8_GROUP && hidden % 128 != 0) return -1;
    float *x = (float *)malloc(sizeof(float) * (size_t)hidden);
    float *y = (float *)malloc(sizeof(float) * (size_t)hidden);
    float *sq = (float *)malloc(sizeof(float) * (size_t)hidden);
    if (!x || !y || !sq) { free(x); free(y); free(sq); return -1; }
    for (int64_t t = 0; t < tokens; ++t) {
        const int64_t base = t * hidden;
        /* reduce in rank order, one rounding; residual add, one rounding */
        for (int64_t h = 0; h < hidden; ++h) {
            float acc = 0.0f;
            for (int r = 0; r < nranks; ++r) acc += load_elem(dtype, parts[r], base + h);
            float s = round_elem(dtype, acc);
            float xr = round_elem(dtype, s + load_elem(dtype, residual_in, base + h));
            x[h] = xr;
            store_elem(dtype, residual_out, base + h, xr);
            sq[h] = xr * xr;
        }
        float sumsq;
        if (sumsq_mode == TDO_SUMSQ_F64) {
            double d = 0.0;
            for (int64_t h = 0; h < hidden; ++h) d += (double)sq[h];
            sumsq = (float)d;
        } else if (sumsq_mode == TDO_SUMSQ_F32_PAIRWISE) {
            sumsq = pairwise_sum(sq, hidden);
        } else if (sumsq_mode == TDO_SUMSQ_TORCH) {
            sumsq = tdo_torch_row_sum(sq, hidden);
        } else {
            sumsq = 0.0f;
            for (int64_t h = 0; h < hidden; ++h) sumsq += sq[h];
        }
        float mean = sumsq / (float)hidden;
        float rs = 1.0f / sqrtf(mean + eps);
        for (int64_t h = 0; h < hidden; ++h) {
            float y1 = round_elem(dtype, x[h] * rs);
            float yy = round_elem(dtype, load_elem(dtype, gamma, h) * y1);
            y[h] = yy;
            if (norm_out) store_elem(dtype, norm_out, base + h, yy);
        }
        if (quant == TDO_QUANT_NONE) continue;
        const int64_t group = (quant == TDO_QUANT_FP8_GROUP) ? 128 : hidden;
        const int64_t ngroups = hidden / group;
        const float qmax = (quant == TDO_QUANT_INT8_TOKEN) ? 127.0f : 448.0f;
        for (int64_t g = 0; g < ngroups; ++g) {
            float amax = 0.0f;
            for (int64_t h = g * group; h < (g + 1) * group; ++h) {
                float a = fabsf(y[h]);
                if (a > amax || a != a) amax = a; /* a NaN stays: torch's amax propagates it (no later `>` replaces it) */
            }
            float scale = amax / qmax;
            scale_out[t * ngroups + g] = scale;
            float div = scale > 0.0f ? scale : 1.0f;
            for (int64_t h = g * group; h < (g + 1) * group; ++h) {
                float q = y[h] / div;
                if (q > qmax) q = qmax;
                if (q < -qmax) q = -qmax;
                if (quant == TDO_QUANT_INT8_TOKEN) q_out[base + h] = (uint8_t)(int8_t)(int)nearbyintf(q);
                else q_out[base + h] = tdo_f32_to_e4m3(q);
            }
        }
    }
    free(x); free(y); free(sq);
    return 0;
}

/*
 * The reference's own CPU check, restated: fp32 data, fp32 rank-order sum, residual add, fp64 sum of
 * squares, beta = 1/sqrt(x2/H + eps) in double, out = x*beta then *= gamma (test/unit_test.cpp:175-217).
 */
int tdo_unit_test_ref(const float *allreduce_in, const float *residual_in, const float *gamma, int64_t size,
                      int64_t hidden, int nranks, float *residual_out, float *norm_out, float eps) {
    if (hidden <= 0 || size % hidden != 0) return -1;
    for (int64_t i = 0; i < size; ++i) {
        float acc = allreduce_in[i];
        for (int r = 1; r < nranks; ++r) acc += allreduce_in[(int64_t)r * size + i];
        acc += residual_in[i];
        residual_out[i] = acc;
    }
    for (int64_t t = 0; t < size / hidden; ++t) {
        double x2 = 0;
        for (int64_t h = 0; h < hidden; ++h) {
            float d = residual_out[t * hidden + h];
            x2 += d * d;
        }
        double beta = 1.0 / sqrt(x2 / hidden + eps);
        for (int64_t h = 0; h < hidden; ++h) {
            norm_out[t * hidden + h] = residual_out[t * hidden + h] * beta;
            norm_out[t * hidden + h] *= gamma[h];
        }
    }
    return 0;
}
