/*
 * muon_amd.h -- C ABI of libmuon_amd.so: the MI355X (gfx950) Muon optimizer step.
 *
 * The reference (thib-s/Muon) has no FFI of its own: its boundary is the Python module
 * surface of muon.py.  The entry points below are what a ctypes binding of that module needs
 * to replace the reference's device work; each one cites the reference lines it replaces.
 *
 * Conventions
 *   - every entry point returns 0 on success and a negative MUON_AMD_E* code on failure;
 *     muon_amd_last_error() returns a thread-local message for the last failure;
 *   - nothing here allocates or frees device memory, synchronises the device or the stream,
 *     or keeps a pointer after returning: tensors, descriptor tables and workspace are owned
 *     by the caller, and all work is enqueued asynchronously on `stream` (a hipStream_t);
 *   - pointers named *_dev are device pointers; descriptor tables passed as *_dev must stay
 *     valid until the enqueued kernels have run;
 *   - matrices are row-major; "bf16" storage is uint16_t holding the upper half of an fp32.
 */
#ifndef MUON_AMD_H
#define MUON_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUON_AMD_ABI_VERSION 3

#define MUON_AMD_OK        0
#define MUON_AMD_EINVAL   (-1)   /* bad argument (null pointer, bad size, misaligned table) */
#define MUON_AMD_ELAUNCH  (-2)   /* HIP reported an error while enqueuing */
#define MUON_AMD_EDEVICE  (-3)   /* current device is not gfx950 */

/* Newton-Schulz rounding policy (flags argument of the GEMM / norm entry points). */
#define MUON_AMD_ROUND_REFERENCE 1  /* round every intermediate to bf16 exactly where the
                                       reference's bf16 tensor expression does (muon.py:282-287) */
#define MUON_AMD_ROUND_FUSED     0  /* one bf16 rounding per stored output (closer to fp32) */
#define MUON_AMD_NORM_UNIT       2  /* muon_amd_norm_finalize only: denom = 1 (no Frobenius
                                       pre-scale; the AOL variant rescales by rows instead) */
#define MUON_AMD_GEMM_ROWSUM     4  /* muon_amd_ns_gemm only, for a mirrored product without addend
                                       (A = X X^T): also leave, per row of the result, partial sums
                                       of |A_ij| in MuonGemmDesc.rowsum (muon.py:779-781 fused into
                                       the product's epilogue) */
#define MUON_AMD_GEMM_Q_KMAJOR   8  /* muon_amd_ns_gemm: every descriptor of the launch gives its second
                                       operand k-major (MuonGemmDesc.q_kmajor = 1); muon_amd_ns_gemm_apply
                                       always takes it that way */

/* How muon_amd_aol_rescale scales the Gram matrix (mode argument). */
#define MUON_AMD_AOL_SYMMETRIC   0  /* A <- diag(r) A diag(r): the Gram matrix of the rescaled X   */
#define MUON_AMD_AOL_ROWS_ONLY   1  /* A <- diag(r)^2 A = A / s, rows only, as muon.py:785 writes it */

/* Storage type of the caller's tensors of one matrix / Adam tensor: gradient, optimizer state and
 * parameter share it, as they do in the reference (state is zeros_like(p), muon.py:95-96,
 * 250-252).  Arithmetic is fp32 either way; with bf16 storage every tensor expression of the
 * reference rounds to bf16, and so do the kernels. */
#define MUON_AMD_SRC_F32   0
#define MUON_AMD_SRC_BF16  1

/* ------------------------------------------------------------------------------------------
 * Descriptor of one Muon matrix (the 2-D view rows x cols of a parameter; 4-D conv filters are
 * viewed as (d0, d1*d2*d3) by the caller, muon.py:11-12).  Arrays of these live in device
 * memory; the elementwise kernels index them by matrix.
 *
 * Workspace roles.  m = min(rows, cols), n = max(rows, cols); *_p are those sizes rounded up to
 * the GEMM tile of the chunk (zero padded; zero rows/columns stay zero through the iteration).
 *   direct : rows_p x cols_p  bf16, the matrix in the orientation of the parameter
 *   transp : cols_p x rows_p  bf16, its transpose
 * (each with its own leading dimension, which may exceed the padded width so that rows do not
 * sit a power of two apart in memory)
 * For a wide matrix (rows <= cols) X = direct and X^T = transp; for a tall one the roles swap,
 * which is how the reference's transpose-if-tall (muon.py:278-279, 289-290) is folded into
 * indexing instead of a pass of its own.
 * ------------------------------------------------------------------------------------------ */
typedef struct MuonMatDesc {
    void*     grad;        /* rows*cols of src_dtype: gradient / NS input                     */
    void*     momentum;    /* rows*cols of src_dtype: momentum buffer, or NULL (plain NS)     */
    void*     param;       /* rows*cols of src_dtype: parameter, or NULL                      */
    uint16_t* out;         /* rows*cols bf16 functional output, or NULL                       */
    uint16_t* u;           /* rows*cols bf16 scratch: update before normalisation             */
    uint16_t* direct;      /* rows_p x cols_p bf16 normalised matrix, parameter orientation   */
    uint16_t* transp;      /* cols_p x rows_p bf16 normalised matrix, transposed              */
    const uint16_t* result;/* rows_p x cols_p bf16: NS output in parameter orientation        */
    float*    partials;    /* per-block partial sums of squares, indexed by global block id   */
    float*    denom;       /* one float: (||u||_F + eps) as the reference forms it            */
    int32_t   rows, cols;
    int32_t   rows_p, cols_p;
    int32_t   ld_direct;   /* leading dimension (elements) of direct and result, >= cols_p    */
    int32_t   ld_transp;   /* leading dimension (elements) of transp, >= rows_p               */
    int32_t   src_dtype;   /* MUON_AMD_SRC_*: storage type of grad, momentum and param        */
    float     scale;       /* max(1, grad.size(-2)/grad.size(-1))**0.5  (muon.py:14)          */
    int32_t   part_begin;  /* first global block id of this matrix in the momentum launch     */
    int32_t   part_end;    /* one past the last                                               */
} MuonMatDesc;

/* One GEMM  acc[i][j] = sum_k P[i][k] * Q[j][k]  ("NT": both operands row-major along k; with
 * q_kmajor = 1 the second operand is given as Q[k][j], leading dimension ldq >= colsn, so that
 * a X + B X reads X itself and no transposed copy of X is kept) over a padded matrix, with the epilogue
 *     t1 = alpha*acc ; t2 = beta*D[i][j] ; (both rounded to bf16 under ROUND_REFERENCE)
 *     o  = bf16(t1 + t2)          -> C[i][j]  and  CT[j][i]
 *     o2 = bf16(gamma * o)        -> C2[i][j] and  C2T[j][i]
 * Any of D, C, CT, C2, C2T may be NULL.  When CT == C the job list only covers tiles with
 * their column block on or above their row block and the kernel mirrors them (tiles inside a
 * diagonal block are stored directly and never mirrored: MuonTileJob.diag).
 * Replaces the functional roles of the reference's three Triton kernels:
 *   ns_line_1 (A = X X^T, muon.py:349-456), ns_line_2 (alpha A A^T + beta A, muon.py:464-588),
 *   ns_line_3 (a X + B X, muon.py:639-746).                                                   */
typedef struct MuonGemmDesc {
    const uint16_t* P;  const uint16_t* Q;  const uint16_t* D;
    uint16_t* C;  uint16_t* CT;  uint16_t* C2;  uint16_t* C2T;
    int32_t ldp, ldq, ldd, ldc, ldct;   /* leading dimensions in elements, multiples of 8     */
    int32_t K;                          /* multiple of 64                                     */
    int32_t rows, colsn;                /* padded extent of the output (multiples of the tile) */
    /* MUON_AMD_GEMM_ROWSUM: rows x ld_rowsum floats; entry [i][s] receives the sum of |o_ij| over
     * the 64 columns j of slot s (every entry with s < colsn / 64 is written exactly once per
     * launch, some with zero; adding a row's entries in slot order gives sum_j |o_ij|).       */
    float*  rowsum;
    int32_t ld_rowsum;                  /* >= colsn / 64                                       */
    int32_t q_kmajor;                   /* 0: Q is colsn x K, rows along k; 1: Q is K x colsn   */
} MuonGemmDesc;

/* One output tile of one matrix, or one share of its reduction.  A tile whose K is long and
 * whose launch would leave most of the GPU idle (the one 128 x 128 tile of X X^T for a
 * 128 x 16384 matrix) is given to `count` jobs, each reducing k0..k1; each parks its fp32
 * accumulators in slot part_base + index of the split workspace, and the job that arrives last
 * adds the slots in slot order and writes the tile (the result does not depend on arrival order). */
typedef struct MuonTileJob {
    int32_t desc;      /* index into the MuonGemmDesc table of the launch */
    int32_t i0;        /* first output row  (multiple of the tile rows)   */
    int32_t j0;        /* first output col  (multiple of the tile cols)   */
    int32_t diag;      /* 1 when a mirrored (symmetric) GEMM's tile lies in a diagonal block */
    int32_t k0, k1;    /* reduction range of this job, multiples of 64; 0 and K when unsplit */
    int32_t part_base; /* first slot of the tile's split group (also its counter); unused when unsplit */
    int32_t split;     /* 0 when unsplit, else index | (count << 16) */
} MuonTileJob;

/* One tensor of the auxiliary Adam group. */
typedef struct MuonAdamDesc {
    void* param;         /* numel of dtype, or NULL when `update` is used instead             */
    const void* grad;    /* numel of dtype                                                    */
    void* exp_avg;       /* numel of dtype                                                    */
    void* exp_avg_sq;    /* numel of dtype                                                    */
    void* update;        /* numel of dtype: functional output (adam_update's return), or NULL */
    int64_t numel;
    int32_t dtype;       /* MUON_AMD_SRC_*: storage type of all five tensors                  */
    int32_t reserved;    /* 0                                                                 */
} MuonAdamDesc;

/* One matrix of the AOL rescaling step of the 4-iteration variant (muon.py:776-785), in the
 * wide orientation: X is m_p x n_p with m_p <= n_p (zero padded).                           */
typedef struct MuonAolDesc {
    uint16_t* xr;     /* m_p x n_p bf16 (leading dimension ld_n): X, scaled by r along rows     */
    uint16_t* xc;     /* n_p x m_p bf16 (ld_m): X^T, scaled by r along columns                  */
    uint16_t* gram;   /* m_p x m_p bf16 (ld_m): A = X X^T, becomes diag(r) A diag(r)            */
    float*    rvec;   /* m_p floats: r_i = max(sum_j |A_ij|, eps)^-1/2                          */
    const float* rowsum; /* m_p x ld_rowsum partial row sums left by the X X^T launch, or NULL      */
    int32_t   m_p, n_p, ld_n, ld_m;
    int32_t   ld_rowsum, reserved;
} MuonAolDesc;

int         muon_amd_abi_version(void);
const char* muon_amd_last_error(void);
/* One-time set-up on the current device: checks that it is a gfx950 (MUON_AMD_EDEVICE if not),
 * raises the dynamic LDS limit of the GEMM kernels and looks up the device's static scratch
 * array.  Optional -- the first GEMM launch on a device does it too -- but required before
 * recording launches into a HIP graph, because it is not a stream operation.                */
int         muon_amd_init(void);

/* sizeof() of the structs above, so that a binding can check its own layout. */
size_t muon_amd_sizeof_mat_desc(void);
size_t muon_amd_sizeof_gemm_desc(void);
size_t muon_amd_sizeof_tile_job(void);
size_t muon_amd_sizeof_adam_desc(void);
size_t muon_amd_sizeof_aol_desc(void);

/* Elements each block of the flat elementwise launches covers (momentum, apply, adam), and
 * the edge of the square tile of the normalise/transposing launch. */
int muon_amd_elementwise_block_elems(void);
int muon_amd_normalize_tile(void);

/* GEMM tile classes (rows x cols of the output tile a workgroup computes):
 *   0: 128 x 128 (4 waves, two workgroups per CU)   1: 256 x 256 (8 waves, one workgroup per CU)
 * Padded matrix sizes must be multiples of the larger of the two.  Return the tile extent, or
 * a negative code for an unknown class. */
int muon_amd_gemm_tile_rows(int tile_class);
int muon_amd_gemm_tile_cols(int tile_class);

/* ---- host-side validation (no GPU work): checks host copies of the tables a launch will
 *      use against what the kernels assume.  Call before uploading them.                 ---- */
int muon_amd_validate_gemm(const MuonGemmDesc* descs_host, int ndesc,
                           const MuonTileJob* jobs_host, int njobs, int tile_class,
                           int split_slots /* slots of the split workspace the jobs may use */);
int muon_amd_validate_mats(const MuonMatDesc* descs_host, int nmat,
                           const int32_t* block_prefix_host, const int32_t* tile_prefix_host,
                           int tile_edge);

/* The last update product of the iteration with the parameter step fused into its epilogue
 * (muon.py:287 followed by muon.py:14, 98-99, 15): for every matrix k of the launch, with
 * o = bf16(alpha*acc + beta*D) as above,
 *     update = bf16(o * mats[k].scale);
 *     mats[k].param <- mats[k].param * wd_factor - lr * update     (if param)
 *     mats[k].out   <- update                                      (if out)
 * in the storage type mats[k].src_dtype, at the unpadded extent mats[k].rows x mats[k].cols.
 * X is the parameter itself for a wide matrix (rows <= cols) and its transpose for a tall one; the
 * C / CT / C2 / C2T pointers of the descriptors are ignored (nothing else is written), jobs are
 * never split.  mats_dev is the table of the elementwise launches; it is indexed by
 * MuonTileJob.desc.  scalars_dev: NULL or device memory holding {lr, wd_factor} (see
 * muon_amd_momentum).                                                                        */
int muon_amd_ns_gemm_apply(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                           int tile_class, float alpha, float beta, int flags,
                           const MuonMatDesc* mats_dev, float lr, float wd_factor,
                           const float* scalars_dev, void* stream);

/* The same launch for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The fp32 slots and counters of split reductions live in a static device array inside the
 * library (MUON_AMD_NOALLOC_MAX_SPLIT_SLOTS slots of 128 x 128 floats plus one counter each,
 * 16 MiB + 1 KiB per GPU, held until the process ends) instead of caller-owned memory; the call
 * clears the counters it uses with a small fill kernel on `stream`, then enqueues the same
 * kernel as muon_amd_ns_gemm.  split_slots = number of slots the job list addresses (0 when no
 * job is split; the value given to muon_amd_validate_gemm); more than the maximum is refused
 * with MUON_AMD_EINVAL.  It allocates and frees nothing.  All calls on one GPU share that GPU's
 * array: two calls with split jobs whose kernels overlap on one GPU (different streams, or
 * different threads) race; calls on one stream are ordered and safe.                          */
#define MUON_AMD_NOALLOC_MAX_SPLIT_SLOTS 256
int muon_amd_noalloc_max_split_slots(void);
int muon_amd_ns_gemm_noalloc(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                             int tile_class, float alpha, float beta, float gamma, int flags,
                             int split_slots, void* stream);

/* ---- Muon elementwise stages ------------------------------------------------------------ */

/* Momentum EMA + Nesterov blend + bf16 cast + per-block sum of squares
 * (muon.py:9-10 and the cast of muon.py:277).  block_prefix_dev[nmat+1] maps block -> matrix.
 *   momentum <- lerp(momentum, grad, one_minus_beta);
 *   u = nesterov ? lerp(grad, momentum, beta) : momentum       (lerp = torch's two-branch rule)
 * With mutate_grad != 0 and nesterov, u is also written back into grad as the reference does.
 * A matrix whose descriptor has momentum == NULL is only cast (u = grad).
 * The launch may cover a run of the table instead of all of it (descs_dev + first, nmat = count,
 * a prefix table of count + 1 entries that starts at 0): the sums of squares go to the slots
 * part_begin + block-within-matrix either way.  A caller uses this to run the stage for one
 * matrix as soon as its gradient exists, ahead of the rest of the step.
 * scalars_dev (here and in muon_amd_apply / muon_amd_adam): NULL, or device memory holding the
 * float arguments of the call in their order ({one_minus_beta, beta} here), which the kernel then
 * reads at run time in place of the by-value ones -- a launch recorded into a HIP graph can so
 * be replayed with new hyper-parameters after a small copy into that memory.               */
int muon_amd_momentum(const MuonMatDesc* descs_dev, const int32_t* block_prefix_dev, int nmat,
                      int nblocks, float one_minus_beta, float beta, int nesterov,
                      int mutate_grad, const float* scalars_dev, void* stream);

/* denom = ||u||_F + eps per matrix from the partial sums (muon.py:282).  Under
 * MUON_AMD_ROUND_REFERENCE the norm and the sum are rounded to bf16 as the reference's bf16
 * tensors are. */
int muon_amd_norm_finalize(const MuonMatDesc* descs_dev, int nmat, float eps, int flags,
                           void* stream);

/* direct = bf16(u / denom) (zero padded), transp = direct^T (muon.py:278-282).
 * tile_prefix_dev[nmat+1] maps block -> matrix over (rows_p/T)*(cols_p/T) tiles. */
int muon_amd_normalize(const MuonMatDesc* descs_dev, const int32_t* tile_prefix_dev, int nmat,
                       int ntiles, void* stream);

/* One grouped GEMM launch over a tile job list (see MuonGemmDesc).  split_partials_dev (slots of
 * tile_rows * tile_cols floats) and split_counters_dev (one int32 per slot, zero before the
 * first launch; every launch leaves them zero) are needed only when a job is split, else NULL. */
int muon_amd_ns_gemm(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                     int tile_class, float alpha, float beta, float gamma, int flags,
                     float* split_partials_dev, int32_t* split_counters_dev, void* stream);

/* result -> update = bf16(result * scale) (muon.py:14);  if param: param <- param*wd_factor
 * - lr*update (muon.py:98-99); if out: out <- update (what muon_update returns, muon.py:15). */
int muon_amd_apply(const MuonMatDesc* descs_dev, const int32_t* block_prefix_dev, int nmat,
                   int nblocks, float lr, float wd_factor, const float* scalars_dev /* {lr, wd_factor} */,
                   void* stream);

/* ---- AOL rescaling (muon.py:776-785; no counterpart kernel in the reference, which leaves
 *      these tensor expressions to torch.compile) ------------------------------------------- */
/* Rows each block of the two launches below covers (one wavefront per row). */
int muon_amd_aol_rows_per_block(void);
/* Host-side check of the tables: row_prefix_host[nmat+1] counts blocks over the rows of each
 * Gram matrix, seg_prefix_host[3*nmat+1] over the rows of X, X^T and A of each matrix.        */
int muon_amd_validate_aol(const MuonAolDesc* descs_host, int nmat, const int32_t* row_prefix_host,
                          const int32_t* seg_prefix_host);
/* rvec_i = max(bf16(sum_j |A_ij|), eps)^-1/2 for every row of every Gram matrix, from a pass
 * over the stored A.                                                                          */
int muon_amd_aol_rowsum(const MuonAolDesc* descs_dev, const int32_t* row_prefix_dev, int nmat,
                        int nblocks, float eps, void* stream);
/* The same from the partial row sums that the X X^T launch left under MUON_AMD_GEMM_ROWSUM
 * (MuonAolDesc.rowsum): no pass over A.  The slots of a row are added in a fixed order.       */
int muon_amd_aol_rowsum_finalize(const MuonAolDesc* descs_dev, const int32_t* row_prefix_dev, int nmat,
                                 int nblocks, float eps, void* stream);
/* X <- diag(r) X in both stored orientations, in place, and the Gram matrix rescaled in place:
 * MUON_AMD_AOL_SYMMETRIC  A <- diag(r) A diag(r), the Gram matrix of the rescaled X that the
 *                         iteration assumes;
 * MUON_AMD_AOL_ROWS_ONLY  A <- A / s (s = r^-2) by rows only, as muon.py:785 writes it: A is
 *                         then no longer symmetric, and the polynomial launch that follows must
 *                         cover every tile (no mirrored store).                               */
int muon_amd_aol_rescale(const MuonAolDesc* descs_dev, const int32_t* seg_prefix_dev, int nmat,
                         int nblocks, int mode, void* stream);

/* ---- auxiliary Adam (muon.py:104-109 and 255-258) ---------------------------------------- */
/* m <- lerp(m, g, w1); v <- lerp(v, g*g, w2)  with w1 = 1-beta1, w2 = 1-beta2;
 * upd = (m/bias1) / (sqrt(v/bias2) + eps);  param <- param*wd_factor - lr*upd  (or update<-upd)
 * w1, w2, bias1 = 1-beta1**step and bias2 = 1-beta2**step are computed by the caller in double
 * (as the reference's Python does) and passed rounded to float. */
int muon_amd_adam(const MuonAdamDesc* descs_dev, const int32_t* block_prefix_dev, int ntensors,
                  int nblocks, float lr, float wd_factor, float w1, float w2, float eps,
                  float bias1, float bias2,
                  const float* scalars_dev /* {lr, wd_factor, w1, w2, eps, bias1, bias2} */,
                  void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MUON_AMD_H */
