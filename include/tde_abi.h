/*
 * tde_abi.h — C ABI of the MI355X (gfx950) fused reduce + residual + RMSNorm (+ dynamic quant)
 * row kernels.  Plain pointers and sizes only: no torch types, no C++ types.
 *
 * The library behind this header (libtde_hip.so) computes ONE rank's reduce-and-normalize stage
 * of the reference's fused `allreduce_rms` operator.  The N peer partial buffers that the
 * reference reads through IPC-mapped peer memory are N ordinary device allocations here.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   - allreduce_rms_fusion_impl<T>(void** workspace, rank, nranks, size, hidden_dim, in, res_in,
 *     res_out, norm_out, gamma, eps, stream)       src/common/all_reduce_fusion_impl.h:500-535
 *   - AllReduceFusionParams<T>                      src/common/all_reduce_fusion_impl.h:300-314
 *   - allreduce_fusion_kernel_launcher<T,NRanks>    src/common/all_reduce_fusion_impl.h:476-498
 *   - CommWorkspace allocation + pointer table      src/ops/all_reduce_fusion.cpp:63-105,143-174
 *
 * Every function returns a tde_status (0 = success).  HIP runtime failures are returned as
 * TDE_EHIP; the HIP error code is then available from tde_last_hip_error().
 */
#ifndef TDE_ABI_H
#define TDE_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TDE_ABI_VERSION 4
#define TDE_MAX_RANKS 16 /* array bound, as MAX_RANKS in src/ops/all_reduce_fusion.h:8 */
#define TDE_QUANT_GROUP 128
#define TDE_STATIC_STAGE_BYTES (32 << 20) /* stage held inside the library for tde_reduce_rms_static_stage */

/* ---- status codes ------------------------------------------------------------------------- */
typedef enum tde_status {
    TDE_OK = 0,
    TDE_EINVAL = 1,     /* null pointer / malformed struct */
    TDE_ENRANKS = 2,    /* nranks not in {2,4,8}; reference: assert(false) impl.h:526-534 */
    TDE_EDTYPE = 3,     /* dtype not supported (tde_probe_rows: not for TDE_F64) */
    TDE_ESHAPE = 4,     /* hidden*elem not a multiple of 16 bytes, tokens<0, hidden<=0 (impl.h:479-480) */
    TDE_EHIDDEN = 5,    /* hidden larger than the row kernel supports (reference: pkg assert, __init__.py:69) */
    TDE_EALIGN = 6,     /* a buffer is not 16-byte aligned (vec_t alignment, impl.h:208) */
    TDE_EQUANT = 7,     /* unknown quant mode, group mode with hidden % 128 != 0, a static scale that is not > 0,
                           or any quant mode with TDE_F64 */
    TDE_EALGO = 8,      /* unknown algorithm, or staged algorithm without a stage buffer */
    TDE_EHIP = 9,       /* HIP runtime error; see tde_last_hip_error() */
    TDE_ERANK = 10,     /* rank outside [0,nranks) */
    TDE_ENOMEM = 11,    /* device allocation failed */
    TDE_ETOOBIG = 12    /* tde_reduce_rms_static_stage: the rows do not fit the library's static stage */
} tde_status;

/* ---- enums ---------------------------------------------------------------------------------- */
typedef enum tde_dtype {
    TDE_BF16 = 0, /* __bfloat16 in the reference dispatch, src/ops/all_reduce_fusion.cpp:19-22 */
    TDE_F16 = 1,  /* __half,                              src/ops/all_reduce_fusion.cpp:14-17 */
    TDE_F32 = 2,  /* float,                               src/ops/all_reduce_fusion.cpp:29-33 */
    TDE_F64 = 3   /* double, admitted by the same macro;  src/ops/all_reduce_fusion.cpp:29-33.  Summed and normed
                     in double as the eager composition does for double tensors (mean of squares in fp32,
                     test_all_reduce_fusion.py:25); TDE_QUANT_NONE only, every algorithm */
} tde_dtype;

typedef enum tde_quant {
    TDE_QUANT_NONE = 0,      /* normed output in the input dtype (the reference's only mode) */
    TDE_QUANT_FP8_TOKEN = 1, /* OCP e4m3 codes, one fp32 scale per row:  scale = rowamax/448 */
    TDE_QUANT_FP8_GROUP = 2, /* OCP e4m3 codes, one fp32 scale per [row, 128-column group]  */
    TDE_QUANT_INT8_TOKEN = 3, /* int8 codes, one fp32 scale per row:      scale = rowamax/127 */
    TDE_QUANT_FP8_STATIC = 4  /* OCP e4m3 codes with a caller-given per-tensor scale (tde_problem.static_scale);
                                 no scales are written.  The reference carries an unused `scale_factor` field for
                                 this (impl.h:313). */
} tde_quant;

typedef enum tde_algo {
    TDE_ALGO_AUTO = 0,   /* = TDE_ALGO_FUSED */
    TDE_ALGO_FUSED = 1,  /* one pass per row: reduce -> residual -> norm -> quant, row kept in registers
                            (the arithmetic of the one-shot body, impl.h:450-471) */
    TDE_ALGO_STAGED = 2, /* two launches: (A) N-way reduce of every row into `stage` (impl.h:365-377),
                            (B) residual + norm (+quant) reading `stage` (impl.h:381-393) */
    TDE_ALGO_STAGED_OWNED = 3 /* as STAGED, but (A) reduces only this rank's share, rows == rank (mod nranks), as one
                            rank of the reference's two-shot does (impl.h:366); the other rows of `stage` must already
                            hold their sums (in the reference the peers write them, impl.h:373-376) */
} tde_algo;

/* ---- problem / buffers ---------------------------------------------------------------------- */
typedef struct tde_problem {
    int32_t dtype;      /* tde_dtype of partials, residual, gamma, residual_out, norm_out */
    int32_t nranks;     /* number of partial buffers, {2,4,8} */
    int32_t rank;       /* index of the caller's own partial (informational; order is always 0..N-1) */
    int32_t quant;      /* tde_quant */
    int32_t algo;       /* tde_algo */
    int32_t write_norm; /* quant modes: also write the T-typed normed row to norm_out (0/1).
                           TDE_QUANT_NONE always writes norm_out. */
    int64_t tokens;     /* rows; 0 is allowed (no launch) */
    int64_t hidden;     /* columns per row */
    float eps;          /* added to mean(x^2) before the reciprocal square root */
    float static_scale; /* TDE_QUANT_FP8_STATIC: code = e4m3(clamp(y / static_scale, +-448)); must be > 0 and finite */
    /* Launch-geometry overrides for sweeps and tests, per call; 0 = automatic.  The reference's launcher
       hard-codes its geometry (impl.h:481-489) and has no counterpart. */
    int32_t tune_vecs_per_thread; /* 1, 2 or 4 16-byte vectors per thread per row (other non-zero values: TDE_EINVAL) */
    int32_t tune_rows_per_block;  /* rows side by side in one workgroup; ignored where it would exceed the
                                     kernel's launch bound of 1024 / vecs_per_thread threads */
    int32_t tune_workgroups_per_cu; /* at most this many workgroups resident per compute unit (1..8; enforced by
                                       padding the launch's dynamic LDS); -1 = no limit; other values: TDE_EINVAL */
    int32_t reserved;               /* must be 0 */
} tde_problem;

typedef struct tde_buffers {
    /* Device pointers, each a contiguous row-major [tokens, hidden] array of `dtype`.
       If partial_table is non-null it is a DEVICE array of nranks device pointers (the first
       nranks entries of the reference's workspace table, src/ops/all_reduce_fusion.cpp:159-162)
       and the kernel reads the pointers from it; entry `rank` is replaced by partial[rank]
       when partial[rank] is non-null (the caller's own allreduce_in, never staged). */
    const void *partial[TDE_MAX_RANKS];
    const void *const *partial_table;
    const void *residual_in;
    void *residual_out;
    void *norm_out;    /* may be null when quant != NONE and write_norm == 0 */
    const void *gamma; /* [hidden] of `dtype` */
    void *q_out;       /* [tokens, hidden] bytes (fp8 e4m3 / int8); null when quant == NONE */
    float *scale_out;  /* [tokens] or [tokens, hidden/128] fp32; null when quant == NONE or FP8_STATIC */
    void *stage;       /* [tokens, hidden] of `dtype`; required for TDE_ALGO_STAGED */
} tde_buffers;

typedef struct tde_plan_out {
    int32_t algo;            /* algorithm that will run (tde_algo, never AUTO) */
    int32_t reference_algo;  /* what the reference launcher would pick: 1 = one-shot (tokens <= 128),
                                2 = two-shot (impl.h:491) */
    int32_t vec_elems;       /* elements per 16-byte access: 8 (bf16/f16), 4 (f32); impl.h:478 */
    int32_t block_threads;   /* threads per workgroup (multiple of 64) */
    int32_t vecs_per_thread; /* 16-byte vectors each thread owns per row */
    int32_t rows_per_block;  /* rows a workgroup processes side by side (one wave group per row) */
    int32_t grid_blocks;     /* workgroups launched for the row kernel */
    int32_t xcd_chunk;       /* row groups each XCD takes in a row: workgroup b of every 8*xcd_chunk takes row group
                                (b % 8) * xcd_chunk + b / 8 of that span (1 = launch order) */
    int32_t workgroups_per_cu; /* limit on resident workgroups per compute unit the launch enforces through its LDS
                                  (0 = none); below a requested tune_workgroups_per_cu where the geometry's own LDS
                                  already admits fewer.  Also 2, without LDS padding, where the plan picks the row
                                  kernel built for two wavefronts per SIMD (eight partials, four vectors per thread,
                                  4 to 24 workgroups per CU, tune_workgroups_per_cu == 0): its registers admit two */
    int32_t lds_bytes;         /* dynamic LDS per workgroup of the row kernel's launch, padding included */
    int64_t algorithmic_bytes; /* (N+1)*T*H*e + H*e + T*H*e + OUT, OUT as documented for the quant mode */
    int64_t scale_elems;       /* number of fp32 scales written */
} tde_plan_out;

/* ---- entry points --------------------------------------------------------------------------- */

/* Library / ABI version (TDE_ABI_VERSION of the build). */
int tde_abi_version(void);

/* Human-readable text for a tde_status. Never null. */
const char *tde_status_string(int status);

/* HIP error code of the most recent TDE_EHIP on this thread (0 if none). */
int tde_last_hip_error(void);

/* Pure host: validates the problem exactly as tde_reduce_rms does and reports launch geometry and
   algorithmic bytes.  Launches nothing; the geometry is sized for the current device's compute-unit
   count (asked once per device), or for 256 compute units where no device is present.  Replaces the
   shape/nranks asserts and the grid/block/algorithm selection of allreduce_fusion_kernel_launcher
   (impl.h:476-498, 526-534). */
int tde_plan(const tde_problem *problem, tde_plan_out *plan);

/* Enqueue the row kernel(s) on `hip_stream` (a hipStream_t, null = default stream) of the current
   device and return without synchronizing.  Replaces allreduce_rms_fusion_impl<T>
   (impl.h:500-535) for the arithmetic of one rank; quant outputs extend it. */
int tde_reduce_rms(const tde_problem *problem, const tde_buffers *buffers, void *hip_stream);

/* The two launches of the staged algorithms (problem->algo must be TDE_ALGO_STAGED or TDE_ALGO_STAGED_OWNED,
   else TDE_EALGO), one at a time, for a caller that puts its own exchange between them as the reference's
   two-shot kernel does with its barrier (impl.h:377-380):
   tde_stage_reduce = the reduce-scatter body (impl.h:365-377): sums the partials of all rows, or of rows ==
   rank (mod nranks), into buffers->stage; only partial[], partial_table and stage are read from `buffers`.
   tde_stage_norm = the body after the barrier (impl.h:381-393): residual add + norm (+quant) of every row of
   buffers->stage; partial[] and partial_table are ignored.
   tde_reduce_rms with the same problem is exactly tde_stage_reduce followed by tde_stage_norm. */
int tde_stage_reduce(const tde_problem *problem, const tde_buffers *buffers, void *hip_stream);
int tde_stage_norm(const tde_problem *problem, const tde_buffers *buffers, void *hip_stream);

/* tde_reduce_rms with the staged algorithm (TDE_ALGO_STAGED; TDE_ALGO_AUTO means the same here, any other
   algorithm is TDE_EALGO) and the stage buffer taken from a fixed array inside the library's device image
   instead of buffers->stage (which is ignored).  After its first call on a device (which looks the array's
   address up) it calls no allocator and nothing that allocates: for callers that cannot allocate -- code under
   HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
   reference, whose stage lives in the CommWorkspace allocation (src/ops/all_reduce_fusion.cpp:70-74).
   Limit: tokens * hidden * elem_size <= TDE_STATIC_STAGE_BYTES (32 MiB, e.g. 2048 x 8192 bf16), else
   TDE_ETOOBIG.  Every GPU the library runs on holds one copy of the array until the process ends -- 32 MiB of
   device memory per GPU for every process that loads the library, whether it calls this entry point or not -- and
   every call on a GPU uses that copy: calls that overlap on one GPU (different streams, different threads) race,
   silently; the library keeps no record of the streams it was given and cannot tell.
   Each call overwrites the part of the array it reads, so nothing needs clearing between calls.
   Note the meaning of TDE_ALGO_AUTO: the staged algorithm here, the fused one in tde_reduce_rms. */
int tde_reduce_rms_static_stage(const tde_problem *problem, const tde_buffers *buffers, void *hip_stream);

/* Calibration: enqueue a plain copy of `bytes` (multiple of 16) from src to dst on `hip_stream`.
   Known traffic (bytes read + bytes written) for scaling profiler memory counters and for
   measuring the device's practical streaming ceiling.  No counterpart in the reference. */
int tde_probe_copy(void *dst, const void *src, int64_t bytes, void *hip_stream);

/* Measurement aid: enqueue one empty kernel (one wavefront, no memory access).  Back-to-back calls timed on a stream
   give the cost of a dispatch itself, the floor under the small, latency-bound problems.  No counterpart in the
   reference. */
int tde_probe_launch(void *hip_stream);

/* Measurement aid: the device's practical streaming rates.  mode 0 reads `bytes` from src (dst, at least 16
   bytes, is not written for any realistic data), 1 writes `bytes` to dst (src is not read), 2 copies; one
   workgroup per 4 KiB, no loop.  `bytes` a multiple of 16.  No counterpart in the reference. */
int tde_probe_stream(void *dst, const void *src, int64_t bytes, int32_t mode, void *hip_stream);

/* Measurement aid: the memory traffic of tde_reduce_rms for the same problem and buffers with the arithmetic
   removed -- same workgroups, lane mapping, load order and cache policies, every input byte read and every
   output byte (scales excepted) written once, contents meaningless.  OVERWRITES residual_out, norm_out and
   q_out.  Fused algorithm only (TDE_EALGO for the staged ones).  Timing it next to tde_reduce_rms shows how
   far the kernel is from what its access pattern alone achieves.  No counterpart in the reference. */
int tde_probe_rows(const tde_problem *problem, const tde_buffers *buffers, void *hip_stream);

/* tde_probe_rows with parts of the traffic switched off, to measure what each part of the access pattern costs on its
   own in the same process as the kernel: `parts` is a bit set -- 1 read the N partial rows and the residual row,
   2 write the T-typed output rows (residual_out, and norm_out where the problem writes it), 4 write the code rows;
   7 is tde_probe_rows.  With bit 1 clear nothing is read (the rows written are a thread pattern); with bits 2 and 4
   clear nothing is written for any realistic data.  TDE_EINVAL outside 1..7.  No counterpart in the reference. */
int tde_probe_rows_parts(const tde_problem *problem, const tde_buffers *buffers, int32_t parts, void *hip_stream);

/* Properties of the current device as the HIP runtime reports them, for printing next to measured rates:
   compute units, memory clock (kHz), memory bus width (bits; 0 where the runtime reports none) and total
   device memory.  The clock is the runtime's figure, not the per-pin data rate: MI355X reports 2 000 000 kHz
   x 8192 bits for HBM3E rated 8 TB/s, i.e. 3.9 transfers per reported clock.  No counterpart in the
   reference, which hard-codes its block counts (impl.h:481-489). */
typedef struct tde_device_info_out {
    int32_t compute_units;
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int32_t reserved;
    int64_t total_memory_bytes;
} tde_device_info_out;
int tde_device_info(tde_device_info_out *out);

/* ---- emulated peer workspace ----------------------------------------------------------------
   One allocation per emulated rank plays the role of that rank's IPC-mapped comm buffer
   (CommWorkspace, src/ops/all_reduce_fusion.cpp:63-96).  Each slot is 2*slot_bytes large: the
   first half holds the rank's partial, the second half is the gathered/staged region
   (comm_bufs[r] + size, impl.h:375,387). */
typedef struct tde_workspace tde_workspace;

/* nblocks: workgroups the reference's kernels would synchronize (1..65536; its package passes 256,
   torch_dist_ext/__init__.py:24); it sizes the per-rank flag regions of the pointer table exactly as the reference
   does, nblocks * nranks ints each (src/ops/all_reduce_fusion.cpp:72).  No kernel of this library reads the flags. */
int tde_workspace_create(int32_t nranks, int32_t nblocks, int64_t slot_bytes, tde_workspace **out);
int tde_workspace_destroy(tde_workspace *ws);
/* Device pointer of slot r (first half). */
void *tde_workspace_slot(const tde_workspace *ws, int32_t r);
/* Device pointer of the stage half of slot r. */
void *tde_workspace_stage(const tde_workspace *ws, int32_t r);
int64_t tde_workspace_slot_bytes(const tde_workspace *ws);
int32_t tde_workspace_nranks(const tde_workspace *ws);
/* Fill `table` (host array, (3*nranks+5) entries) with the reference's pointer-table layout
   (src/ops/all_reduce_fusion.cpp:159-169): [0,N) slot pointers, [N,2N) flag regions,
   [2N,3N) one-shot regions (alias the slots here), then 5 scalar cells. */
int tde_workspace_fill_table(const tde_workspace *ws, void **table, int32_t entries);

#ifdef __cplusplus
}
#endif
#endif /* TDE_ABI_H */
