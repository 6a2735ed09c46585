/*
 * flashmuon.h -- C ABI of libflashmuon_hip.so, the gfx950 (MI355X) kernel library behind
 * matmul_transpose / matmul_transpose_assign / fast_newtonschulz / Muon.step.
 *
 * The reference (nil0x9/flash-muon) has no FFI: its device boundary is a Triton JIT launch
 * (flash_muon/matmul_transpose_triton.py:91-101) and torch eager ops (flash_muon/muon.py:23-29,
 * 87-89, 99-100).  Each entry point below names the reference lines it replaces.
 *
 * Conventions, common to every entry point:
 *   - plain C types only; every pointer is device memory owned by the caller;
 *   - leading dimensions and strides are in ELEMENTS, not bytes;
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it and the call returns
 *     without synchronising; nothing is allocated or freed;
 *   - the return value is an fm_status; 0 is success; bad arguments are reported before any
 *     launch; asynchronous device faults surface at the caller's next synchronisation;
 *   - `ws`/`ws_bytes` is caller-provided scratch of at least the size the matching
 *     *_workspace_bytes() function returns (it may be NULL when that size is 0).
 *   - the entry points keep no state between calls and are re-entrant; two calls that share a
 *     workspace must be ordered on one stream.  The exceptions are process-global: the tuning
 *     knobs (fm_set_knob: one setting for all threads, to be changed only while no other thread is
 *     inside a call) and the device array of fm_syrk_bf16_static.
 */
#ifndef FLASHMUON_H
#define FLASHMUON_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* fm_stream_t; /* hipStream_t */

/* every entry point is exported; everything else in the library has hidden visibility */
#define FM_API __attribute__((visibility("default")))

enum fm_status {
  FM_OK = 0,
  FM_ERR_NULL = 1,        /* a required pointer is NULL */
  FM_ERR_SHAPE = 2,       /* a dimension is negative, zero where forbidden, or inconsistent */
  FM_ERR_STRIDE = 3,      /* a leading dimension is smaller than the row it must hold, or output
                             strides that map two elements to one address */
  FM_ERR_DTYPE = 4,       /* dtype code not one of FM_BF16 / FM_F16 / FM_F32 */
  FM_ERR_ALIAS = 5,       /* an output overlaps an input it must not overlap */
  FM_ERR_WORKSPACE = 6,   /* ws is NULL or ws_bytes too small */
  FM_ERR_LAUNCH = 7,      /* hipLaunchKernel reported an error */
  FM_ERR_ALIGN = 8        /* a pointer is not aligned to its element size */
};

enum fm_dtype { FM_BF16 = 0, FM_F16 = 1, FM_F32 = 2 };

/* Human-readable text for a status code (static storage). */
FM_API const char* fm_status_string(int status);

/* Library version, "major.minor.patch". */
FM_API const char* fm_version(void);

/* Tuning knobs, for experiments and for tests that have to reach a particular schedule.  A
 * negative value gives the decision back to the library.  The environment variables
 * FLASHMUON_GRID, FLASHMUON_KSPLIT, FLASHMUON_FAST_MIN_UNITS, FLASHMUON_NO_MID, FLASHMUON_NO_SUB64, FLASHMUON_HALF,
 * FLASHMUON_DIAG_LAST and FLASHMUON_NO_TICKETS set the initial
 * values; they are read once, when the library is first used, never per call.  No counterpart in
 * the reference (its tuning is Triton's autotune table, flash_muon/matmul_transpose_triton.py:6-18).
 */
enum fm_knob {
  FM_KNOB_GRID = 0,            /* workgroups per launch of the 256x256 schedule (at most one per CU) */
  FM_KNOB_KSPLIT = 1,          /* parts every tile of that schedule, or of the 128x128 one, is cut into along k */
  FM_KNOB_FAST_MIN_UNITS = 2,  /* take the 256x256 schedule when tiles * k-stages >= this (0: whenever the shape allows) */
  FM_KNOB_NO_MID = 3,          /* 1: never take the 128x128 copy-fed schedule */
  FM_KNOB_NO_SUB64 = 4,        /* 1: cut the tiles left after the last full round along k (fp32 parts, second
                                  kernel) even where 64x64 sub-tiles over the whole k would do, and never run
                                  a whole product on such sub-tiles; 0: run every product of at most a
                                  sixteenth as many 256x256 tiles as workgroups on them (by estimate otherwise) */
  FM_KNOB_HALF = 5,            /* 1: always, 0: never run the 256x256 schedule on 128x256 half tiles (taken by
                                  itself when all of them fit into one round of workgroups) */
  FM_KNOB_DIAG_LAST = 6,       /* 0: the tiles left after the last full round of a symmetric product are the
                                  last of the blocked tile order, whatever they are (otherwise: diagonal tiles,
                                  which need one operand panel each and 10 of their 16 sub-tiles) */
  FM_KNOB_NO_TICKETS = 7       /* 1: sub-tile w of the last round goes to workgroup w even where a workspace is
                                  there to hand them out in (otherwise: in the order the workgroups arrive) */
};
FM_API int fm_set_knob(int knob, long long value);

/* ---------------------------------------------------------------------------------------------
 * Scratch for the three GEMM-shaped entry points below, by the shape of their OUTPUT: (M, M) for
 * fm_syrk_bf16, fm_syrk_f16, fm_syrk_f32 and fm_syrk_poly_bf16, (M, K) for fm_gemm_axpby_bf16.  It holds the
 * fp32 partial tiles of output tiles whose k range is split over several workgroups: 256 KiB per
 * part, at most 256 parts (64 MiB) when the output has more 256x256 tiles than the GPU has CUs,
 * at most 768 (192 MiB) below that; 16 MiB (256 parts of 64 KiB) for outputs of at most 128 tiles
 * of 128x128 that are not whole 256x256 tiles, and 0 for shapes that never take such a schedule.
 * Sizes for the 256x256 schedule include 256 bytes at the end of the workspace whose first 8 hold a
 * counter: the 64x64 sub-tiles that the tiles left after the last full round are cut into are drawn
 * from it in the order the workgroups arrive (upper 48 bits: the launch the count belongs to, lower
 * 16: tickets drawn).  The word needs no initialisation and no reset between calls (a launch takes
 * it over with an atomic maximum; a word it cannot take over only means sub-tile w goes to workgroup
 * w, with the same bits in the output), and must not be written by others while a call is in flight.
 * The calls also run with ws == NULL (or a smaller ws) on a slower schedule that needs none.
 */
FM_API size_t fm_gemm_workspace_bytes(int rows_out, int cols_out);

/* ---------------------------------------------------------------------------------------------
 * Y = X * X^T, X is M x K bf16 (row stride ldx, unit column stride), Y is M x M bf16 with
 * arbitrary strides (ldy_row, ldy_col).  Only tiles on or above the diagonal are computed; every
 * tile above it is written twice, directly and mirrored, from the same accumulators, and Y == Y^T
 * holds bit for bit.  fp32 accumulation, one round-to-nearest-even to bf16.  Y must not overlap X,
 * and the larger of |ldy_row|, |ldy_col| must be at least M times the smaller (no two elements of
 * Y at one address).
 * Replaces mmt_kernel + its launch: flash_muon/matmul_transpose_triton.py:20-75, 90-101.
 */
FM_API int fm_syrk_bf16(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col,
                 int M, int K, void* ws, size_t ws_bytes, fm_stream_t stream);

/* Scratch for fm_syrk_bf16 and fm_syrk_f16 by the shape of X: fm_gemm_workspace_bytes(M, M), and for
 * an X whose sides are not whole multiples of 128 also room for a zero-padded copy of X and the padded
 * product, so that such shapes run on the tiled schedules too (copied in, multiplied, the M x M part
 * copied out: three launches) instead of the general one.  With less than this the calls still run,
 * on the schedule that the scratch they get allows.  No counterpart in the reference, whose masked
 * loads and stores take any shape (flash_muon/matmul_transpose_triton.py:48-52, 70-75).
 */
FM_API size_t fm_syrk_workspace_bytes(int M, int K);

/* fm_syrk_bf16 for callers that cannot allocate or hand over scratch memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments as fm_syrk_bf16 minus ws / ws_bytes, and the results of fm_syrk_bf16
 * called with a workspace of 64 MiB: the partial tiles go to a 64 MiB array (256 slots of 256 KiB)
 * that the library holds in the device memory of every GPU it is used on, from the first use until
 * the process ends.  (Outputs of few tiles with a long k, which fm_syrk_bf16 cuts deeper along k when
 * it is given the up to 192 MiB of fm_gemm_workspace_bytes, are cut as far as 256 slots allow; their
 * fp32 sums then run in another order.  Sides that are not whole tiles run on the general schedule,
 * without padded copies.)  Nothing is allocated, freed or synchronised; the first call on
 * a device looks the array's address up (do that once outside a graph capture).
 * Limits: M <= FM_STATIC_MAX_M and K <= FM_STATIC_MAX_K, otherwise FM_ERR_SHAPE.  All calls on one
 * GPU share the array, which keeps the last call's contents (nothing in it has to start at zero:
 * every part is written before it is read): calls that overlap in time on one GPU, i.e. on
 * different streams, race with each other and must be ordered by the caller.
 */
#define FM_STATIC_MAX_M 65536
#define FM_STATIC_MAX_K 1048576
FM_API int fm_syrk_bf16_static(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col,
                        int M, int K, fm_stream_t stream);

/* The same product for fp16 X and Y (the reference's kernel takes its element type from the
 * input: flash_muon/matmul_transpose_triton.py:63): fp32 accumulation, one round-to-nearest-even
 * to fp16, same arguments and schedule.
 */
FM_API int fm_syrk_f16(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col,
                int M, int K, void* ws, size_t ws_bytes, fm_stream_t stream);

/* The same product for fp32 X and Y, on fp32 MFMA (32x32x2): fp32 products and accumulation, no
 * rounding of the result.  Runs on the general tiled schedule for every shape; ws is not used.
 */
FM_API int fm_syrk_f32(const void* X, int64_t ldx, void* Y, int64_t ldy_row, int64_t ldy_col,
                int M, int K, void* ws, size_t ws_bytes, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * P = b*A + c*(A*A) for a SYMMETRIC M x M bf16 matrix A (row stride lda; the kernels read A[i][j]
 * and A[j][i] interchangeably).  Same triangular schedule and dual store as fm_syrk_bf16; the polynomial is evaluated on the fp32 accumulator
 * and rounded to bf16 once.  P must not overlap A.
 * If diag_out is not NULL it receives the M diagonal values of the polynomial in fp32 and the
 * diagonal of P is written as zero: the diagonal carries most of P's magnitude near convergence
 * (about -2.7 where the off-diagonal entries are O(1/sqrt(M))), so keeping it out of bf16 removes
 * the largest rounding error of a Newton-Schulz step.  fm_gemm_axpby_bf16 takes it back as
 * row_alpha.
 * Replaces the second symmetric product and the three elementwise ops after it:
 * flash_muon/muon.py:27-28.
 */
FM_API int fm_syrk_poly_bf16(const void* A, int64_t lda, void* P, int64_t ldp, int M, float b, float c,
                      float* diag_out, void* ws, size_t ws_bytes, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Xout = a*X + P*X for P (M x M, row stride ldp) and X (M x K, row stride ldx).  The
 * contraction runs over the rows of X, so the kernel reads X through its transpose
 * XT (K x M, row stride ldxt), which the caller supplies (fm_scale_cast_bf16 and this function
 * both produce it).  X and XT must hold the same values: on the 256x256 schedule the term a*X is
 * read through XT as well, on the other schedules through X.  Either output may be NULL, not both:
 * Xout is M x K (row stride ldo), XoutT is its transpose K x M (row stride ldot), written from the
 * same registers.
 * If row_alpha is not NULL (M floats), row i uses a + row_alpha[i] in place of a, i.e. the
 * kernel computes a*X + (P + diag(row_alpha))*X with the diagonal term in fp32.
 * No output may overlap an input.
 * Replaces flash_muon/muon.py:29 (`X = a * X + B @ X`: one GEMM and two elementwise ops).
 */
FM_API int fm_gemm_axpby_bf16(const void* P, int64_t ldp, const void* XT, int64_t ldxt,
                       const void* X, int64_t ldx, void* Xout, int64_t ldo,
                       void* XoutT, int64_t ldot, int M, int K, float a,
                       const float* row_alpha, void* ws, size_t ws_bytes, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * out[0] = sum over the rows x cols matrix G (row stride ldg) of bf16(G[i,j])^2, in fp32,
 * with a fixed reduction tree (bit-reproducible run to run).  ws needs fm_sumsq_workspace_bytes().
 * Replaces the reduction inside `X.norm(dim=(-2,-1))`: flash_muon/muon.py:15, 23.
 */
FM_API size_t fm_sumsq_workspace_bytes(void);
FM_API int fm_sumsq(const void* G, int dtype, int rows, int cols, int64_t ldg, float* out,
             void* ws, size_t ws_bytes, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * D = bf16(G) / (sqrt(sumsq[0]) + eps) and T = D^T.  G is rows x cols of `dtype` (row stride
 * ldg); D is rows x cols bf16 (row stride ldd); T is cols x rows bf16 (row stride ldt).  Either
 * output may be NULL, not both.
 * Replaces the cast, the transposed view, the division and the `.contiguous()` copy of it:
 * flash_muon/muon.py:15-17, 23 and flash_muon/matmul_transpose_triton.py:88.
 */
FM_API int fm_scale_cast_bf16(const void* G, int dtype, int rows, int cols, int64_t ldg,
                       const float* sumsq, float eps, void* D, int64_t ldd, void* T, int64_t ldt,
                       fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * The whole quintic Newton-Schulz orthogonalisation of one matrix: G is rows x cols of `dtype`
 * (row stride ldg), out is rows x cols bf16 (row stride ldout).  Runs fm_sumsq,
 * fm_scale_cast_bf16 and `steps` x (fm_syrk_bf16, fm_syrk_poly_bf16, fm_gemm_axpby_bf16) on
 * `stream`, iterating on the wide orientation (M = min(rows, cols)).  steps == 0 returns the
 * normalised input.  out must not overlap G.  A matrix whose sides are not whole multiples of 128
 * (of 256 where whole 256x256 tiles are estimated to pay for the padding) is iterated on zero-padded to whole tiles inside the workspace (zero rows and columns stay zero
 * through every step) and the rows x cols part is copied out at the end.
 * Replaces fast_newtonschulz: flash_muon/muon.py:6-33.
 */
FM_API size_t fm_newtonschulz_workspace_bytes(int rows, int cols);

/* ---------------------------------------------------------------------------------------------
 * The same for `batch` (1..32) matrices of one shape and dtype, with every GEMM-shaped stage run
 * as ONE launch over the whole batch, so that shapes whose tile count does not fill the chip
 * (M = 4096 gives 136 tiles for 256 CUs) are packed together.  G and out are HOST arrays of
 * `batch` device pointers; all inputs share ldg and all outputs ldout.  No out[i] may overlap
 * any G[j] or another out[j].  This is how the step over the same-shape parameters of
 * flash_muon/muon.py:90-103 is meant to call the path.
 */
FM_API size_t fm_newtonschulz_batched_workspace_bytes(int batch, int rows, int cols);
FM_API int fm_newtonschulz_batched_bf16(const void* const* G, int dtype, int batch, int rows, int cols,
                                        int64_t ldg, void* const* out, int64_t ldout, int steps,
                                        float a, float b, float c, float eps,
                                        void* ws, size_t ws_bytes, fm_stream_t stream);
FM_API int fm_newtonschulz_bf16(const void* G, int dtype, int rows, int cols, int64_t ldg,
                         void* out, int64_t ldout, int steps, float a, float b, float c, float eps,
                         void* ws, size_t ws_bytes, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * In place, elementwise over n elements of `dtype`:
 *     buf <- lerp(buf, g, w_buf)         (the reference passes w_buf = 1 - momentum)
 *     g   <- lerp(g, buf, w_nes)         (w_nes = momentum; only when nesterov != 0,
 *                                         otherwise g is left alone)
 * lerp(s, e, w) is s + w*(e - s) for |w| < 0.5 and e - (e - s)*(1 - w) otherwise, the form
 * torch's lerp_ uses.  Each line is computed in fp32 and rounded once to `dtype`, and the second
 * line reads the ROUNDED buf, as two successive torch lerp_ calls do.
 * Replaces flash_muon/muon.py:99-100.
 */
FM_API int fm_momentum_nesterov(void* g, void* buf, int dtype, int64_t n, float w_buf, float w_nes,
                         int nesterov, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * In place over n elements: p <- round(p * decay_mul) ; p <- round(p + alpha * u), with u bf16
 * and p of p_dtype; two roundings, as torch's mul_ followed by add_(alpha=) produce.
 * Replaces flash_muon/muon.py:87-89.
 */
FM_API int fm_weight_update(void* p, int p_dtype, const void* u_bf16, int64_t n, float decay_mul,
                     float alpha, fm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * The two updates above for `batch` (1..32) tensors of n elements each in one launch: g, buf, p and
 * u_bf16 are HOST arrays of `batch` device pointers; tensor i gets exactly what the single-tensor
 * call computes.  No tensor may overlap another.  For the loop over same-shape parameters:
 * flash_muon/muon.py:90-100 and 86-89.
 */
FM_API int fm_momentum_nesterov_batched(void* const* g, void* const* buf, int batch, int dtype, int64_t n,
                                 float w_buf, float w_nes, int nesterov, fm_stream_t stream);
FM_API int fm_weight_update_batched(void* const* p, int p_dtype, const void* const* u_bf16, int batch,
                             int64_t n, float decay_mul, float alpha, fm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHMUON_H */
