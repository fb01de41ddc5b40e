/*
 * libdlspm_hip -- fp32 CSR sparse kernels for AMD MI355X (gfx950): SpMM, CSR-sampled SDDMM and the
 * fused SDDMM->SpMM, behind a plain C ABI.
 *
 * Conventions shared by every entry point (they restate what the reference's drivers do around
 * their kernel launches, /root/reference paths relative to the reference tree):
 *   - every pointer is a DEVICE pointer owned by the caller (the reference allocates with
 *     sycl::malloc_device in main(), e.g. SPMM/spmm-esimd-fromfile2.cpp:172-180);
 *   - indices and sizes are 32-bit ints, CSR is zero-based, dense operands are row-major and
 *     contiguous (leading dimension = N or D);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls only enqueue
 *     work on it and return, they never synchronise;
 *   - the CSR structure (row_offsets, col_indices) is read-only: the library never writes it;
 *   - outputs are fully overwritten, including rows with no nonzero, so no pre-zeroing is needed
 *     (the reference kernels return early on empty rows and rely on the driver's memset,
 *     SPMM/spmmesimd2.hpp:90-91, SPMM/spmm-esimd-fromfile2.cpp:196);
 *   - no input needs padding (the reference over-allocates col/val by 2*VLC for its unmasked tail
 *     loads, SPMM/spmm-esimd-fromfile2.cpp:174-176);
 *   - any N / D >= 1 and any float-aligned dense operand is accepted (the reference rejects
 *     N % 16 != 0, SPMM/spmm-esimd-fromfile2.cpp:230-231): every width of at least 4 takes the
 *     dwordx4 path (those accesses need only dword alignment; a row's last lane reads and writes the
 *     row's last four floats), widths 1 to 3 a dword path of the same kernels;
 *   - results are deterministic: no floating-point atomics (the reference's SDDMM v4 uses them,
 *     SDDMM/sddmm-esimd-fromfile_v4.hpp:161,175);
 *   - errors are returned as a negative status, nothing is thrown across the ABI (the reference
 *     throws std::invalid_argument / std::logic_error on the host before launching).
 *   - `workspace` is optional device memory owned by the caller. NULL (or 0 bytes) is always valid and selects the
 *     schedule that needs none. What else can travel through (workspace, workspace_bytes) -- schedule memory, a row plan,
 *     a cut plan, or hints about the matrix in the upper byte of the size -- is decided in one place: dlspm_analyze looks
 *     at the matrix once, dlspm_advise says what to allocate, build and pass for an op and a width (below). The
 *     thresholds behind that advice live in the library's code only. A non-NULL workspace smaller than the call needs is
 *     refused with DLSPM_E_WORKSPACE. Schedule memory needs no initialisation and means nothing afterwards; two calls that
 *     share it must not overlap in time.
 *       schedule memory (dlspm_workspace_bytes() bytes, no hint): lets SpMM and the fused op use the flat schedule on large
 *         matrices (every wave owns a fixed run of nonzeros, however they are spread over the rows; a second kernel adds
 *         the partial rows kept in the workspace, in a fixed order: the faster schedule for very uneven rows, the slower
 *         one for even rows), and all three ops the column-sliced schedule where the dense operands gathered per nonzero
 *         exceed one L2 (the column ranges of the sparse matrix one after the other, so that the part of the operands in
 *         use fits the cache; partial rows per range in the workspace, added in range order; SDDMM keeps only the range
 *         boundaries there).
 *       DLSPM_HINT_ROWS_EVEN, with workspace NULL: the caller knows that no row is much longer than the mean (longest
 *         row at most one and a half times nnz / M). Tall matrices of long rows then run one whole row per wave, which
 *         is the faster split for even rows and the slower one for uneven rows. A hint about speed only: a wrong one
 *         costs time, never correctness (a row's products are added in a different, equally fixed order).
 *       DLSPM_HINT_ROW_PLAN: `workspace` holds the row plan of this matrix (dlspm_row_plan_build, below; at least
 *         dlspm_row_plan_bytes(M) bytes, else DLSPM_E_WORKSPACE) and the launch hands the rows out in the plan's order.
 *         The plan is only read.
 *       DLSPM_HINT_BANDED: the columns of every row lie in a window much narrower than K that moves down the columns
 *         with the row (sliding-window and block-diagonal attention masks, banded matrices). Neighbouring rows then
 *         gather neighbouring dense rows: the row blocks are dealt to the XCDs in contiguous runs, so that each L2
 *         fetches its own share of the K-side operands and not all of them, and the call runs as row blocks whatever
 *         memory comes with it. Measured on MI355X, K = V = 16384 x 128 floats, 128 columns per row: the fused op 104 us
 *         in column slices, 77 us with NULL, 74 us with this hint; the L2s fetch 33 MiB per launch instead of 145 MiB.
 *         A wrong hint costs time, never correctness: the bits are those of the call with NULL. May be combined with
 *         DLSPM_HINT_ROWS_EVEN; a row plan takes precedence. dlspm_advise detects bands from the matrix.
 *       DLSPM_HINT_ROWS_SKEWED: with a row plan, the longest row is at least twenty times the mean (the planned SDDMM
 *         and fused launches then run one row per workgroup at heights where they would keep rows grouped). With
 *         workspace NULL: long rows lie next to each other in a tall matrix of short rows (an embedding whose frequent
 *         tokens come first), and the launch groups at most four rows (fused: eight) into a workgroup instead of up to
 *         sixteen -- 33288 x 512 with 17.6 nonzeros per row and a run of rows of 300: SpMM at N = 256 57 -> 28 us.
 *         dlspm_advise gives it where one eighth of the rows holds 1.6 times its share of the nonzeros and the longest
 *         row eight times the mean. Not together with DLSPM_HINT_ROWS_EVEN (DLSPM_E_INVALID_ARG). About speed only.
 * Calls on different streams may run concurrently from different host threads (each with its own
 * workspace). The library's only mutable state is per host thread (the tuning overrides of dlspm_set_tuning and the
 * last HIP error), a cache of the devices' properties, and the static scratch array of spmm_csr_f32_static.
 */
#ifndef DLSPM_HIP_H
#define DLSPM_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default) /* what this header declares is what the library exports */
#endif

/* status codes */
#define DLSPM_OK              0
#define DLSPM_E_INVALID_ARG  (-1) /* negative size, NULL pointer for a non-empty operand, nnz/M/K inconsistent */
#define DLSPM_E_WORKSPACE    (-2) /* a workspace was passed, but smaller than dlspm_workspace_bytes()        */
#define DLSPM_E_LAUNCH       (-3) /* the HIP runtime refused the launch (see dlspm_last_hip_error)         */
#define DLSPM_E_INVALID_CSR  (-4) /* dlspm_csr_check found a malformed CSR structure                        */
#define DLSPM_E_NO_DEVICE    (-5) /* the current device is not a gfx950, or there is none                   */
#define DLSPM_E_STATIC_LIMIT (-6) /* spmm_csr_f32_static: the sizes need more scratch than the library holds   */

/* hints, or-ed into `workspace_bytes` (see above); the size proper is workspace_bytes & ~DLSPM_HINT_MASK */
#define DLSPM_HINT_ROWS_EVEN ((size_t)1 << 62)
#define DLSPM_HINT_ROW_PLAN  ((size_t)1 << 61)
#define DLSPM_HINT_BANDED    ((size_t)1 << 60)
#define DLSPM_HINT_CUT_PLAN  ((size_t)1 << 59)
#define DLSPM_HINT_ROWS_SKEWED ((size_t)1 << 58)
#define DLSPM_HINT_MASK      ((size_t)0xFF << 56)

/* Deprecated spelling of DLSPM_HINT_ROWS_EVEN, still accepted: this constant as `workspace` with workspace_bytes 0.
 * A pointer value that is no pointer is easy to forward by accident; new code passes the hint bit. */
#define DLSPM_ROWS_EVEN ((void*)1)

/* operation selectors for dlspm_workspace_bytes */
#define DLSPM_OP_SPMM   0
#define DLSPM_OP_SDDMM  1
#define DLSPM_OP_FUSED  2

/*
 * C[M x N] = A_csr[M x K] * B[K x N].
 * Replaces the kernel launch `SpmmEsimd<CH>(values_dev, row_offsets_dev, column_indices_dev,
 * rhs_matrix_dev, output_dev, item, MSZ, KSZ, NSZ)` of SPMM/spmm-esimd-fromfile2.cpp:199-228
 * (kernel: SPMM/spmmesimd2.hpp:63-147, launch sizing ComputeNT: SPMM/spmmesimd2.hpp:30-60) and
 * computes what the CPU loop Spmm of SPMM/spmm-esimd-fromfile2.cpp:63-83 computes.
 *   row_offsets[M+1], col_indices[nnz], values[nnz]; B is K x N, C is M x N, both row-major.
 */
int spmm_csr_f32(int M, int K, int N, int nnz,
                 const int* row_offsets, const int* col_indices, const float* values,
                 const float* B, float* C,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * out_values[j] = dot(lhs[i, :], rhs[col_indices[j], :]) for every CSR slot j of row i
 * (S .* (lhs * rhs^T) written in S's own CSR order; indices are neither copied nor permuted).
 * Replaces `Launcher(row_offsets, column_indices, lhs, rhs, out, NSZ, NT, nh_threads, queue)` of
 * SDDMM/sddmm-esimd-fromfile.hpp:180-212 (kernel :59-131; the small-K variant
 * SDDMM/sddmm-esimd-fromfile_v4.hpp:102-177) and computes what the CPU loop Sddmm of
 * SDDMM/sddmm-esimd-fromfile.cpp:18-36 computes. D is the inner (feature) dimension, called NSZ in
 * the reference's SDDMM files.
 *   lhs is M x D, rhs is K x D (the un-transposed storage of rhs^T), out_values[nnz].
 */
int sddmm_csr_f32(int M, int K, int D, int nnz,
                  const int* row_offsets, const int* col_indices,
                  const float* lhs, const float* rhs, float* out_values,
                  void* workspace, size_t workspace_bytes, void* stream);

/*
 * O[M x D] = (S .* (Q * Kmat^T) * scale) * V, with the sampled scores kept on chip.
 * Replaces `FusedEsimd(a_row_offsets, a_column_indices, c, b, d, e, item)` of
 * FUSED/fused-esimd_cb.cpp:100-189 (launch :318-331; c->Q, b->Kmat, d->V, e->O) and computes what
 * Sddmm followed by Spmm compute in FUSED/fused.cpp:47-89. scale = 1.0f gives exactly the
 * reference's semantics (it has no scale); the scores are fp32 between the two stages as there.
 *   Q is M x D, Kmat and V are K x D, O is M x D.
 */
int fused_sddmm_spmm_f32(int M, int K, int D, int nnz,
                         const int* row_offsets, const int* col_indices,
                         const float* Q, const float* Kmat, const float* V, float scale,
                         float* O,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * spmm_csr_f32 for callers that cannot allocate device memory and cannot size a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference (whose drivers
 * allocate everything up front in main()). It runs exactly what spmm_csr_f32 runs when it is handed
 * dlspm_workspace_bytes() bytes of workspace -- the flat schedule for matrices of half a million nonzeros and more, the
 * column-sliced schedule for a B beyond one L2, the row-block schedule otherwise -- and returns the same bits, but the
 * partial rows and slice boundaries live in a buffer that is part of the library itself: a static device array of
 * dlspm_static_scratch_bytes() = 8 MiB per GPU, held from the moment the library is loaded until the process ends.
 * The call allocates nothing, frees nothing and never synchronises (its first call on each device looks the array's
 * address up once). Sizes whose schedule needs more than that are refused with DLSPM_E_STATIC_LIMIT and nothing is
 * launched (call spmm_csr_f32 with NULL or with a workspace of your own then). Every call on one GPU shares that GPU's
 * array: calls that overlap in time on one GPU (two streams, two threads) race on it and must be ordered by the caller.
 * Nothing in the array needs to start at zero: every partial row that is read was written by the same call.
 */
int spmm_csr_f32_static(int M, int K, int N, int nnz,
                        const int* row_offsets, const int* col_indices, const float* values,
                        const float* B, float* C, void* stream);
size_t dlspm_static_scratch_bytes(void);

/*
 * Bytes of device workspace the op can use for these sizes (0 = none, as for small or short-row problems;
 * SDDMM uses one only for the slice boundaries of the column-sliced schedule; `workspace` may always be NULL).
 * Host-only. Takes the place of the host-side
 * launch sizing the reference does before each launch (SPMM/spmm-esimd-fromfile2.cpp:188-192,
 * SDDMM/sddmm-esimd-fromfile_v4.cpp:146-160).
 */
size_t dlspm_workspace_bytes(int op, int M, int K, int N_or_D, int nnz);

/*
 * Device-side restatement of the reference's SanityCheck (SPMM/spmm-esimd-fromfile2.cpp:36-61):
 * row_offsets[0] == 0, row_offsets[M] == nnz, offsets non-decreasing, no row longer than K, every
 * column index in [0, K). Synchronises `stream`. Returns DLSPM_OK or DLSPM_E_INVALID_CSR.
 * The compute entry points do not call it; a malformed CSR handed to them is undefined behaviour,
 * as it is for the reference's kernels.
 */
int dlspm_csr_check(int M, int K, int nnz, const int* row_offsets, const int* col_indices,
                    void* stream);

/*
 * One look at the matrix, one answer. The compute calls see sizes only; how a matrix should be launched also depends on
 * how uneven its rows are and on whether neighbouring rows gather neighbouring dense rows. These two calls hold every
 * such rule in one place (the thresholds live in the library's code, once):
 *   dlspm_analyze   one pass over the CSR structure on the device (synchronises `stream`; once per matrix structure, like
 *                   dlspm_csr_check): the longest row, the rows without nonzeros, the widest row (largest - smallest
 *                   column + 1), and, with the rows cut into eight contiguous eighths (the share of one XCD under
 *                   DLSPM_HINT_BANDED): the columns that the eighths span, summed, in thousandths of K (1000: a band that
 *                   moves down the columns with the row; 8000: every eighth reaches all columns), and the nonzeros of
 *                   the heaviest eighth in thousandths of the mean eighth.
 *   dlspm_advise    host only: for op (DLSPM_OP_*) at dense width N_or_D, what to allocate (`bytes` of device memory, 0:
 *                   pass NULL), what to build into it (`build`: nothing, dlspm_row_plan_build or
 *                   dlspm_row_plan_build_cut; nothing with bytes > 0: plain schedule memory, no initialisation), and
 *                   the hint bits to or into workspace_bytes (`hints`). A band is detected, not hinted; very uneven rows
 *                   in masks of 16 to 64 rows per compute unit get DLSPM_HINT_ROWS_SKEWED with their plan, and so do,
 *                   without a plan, tall matrices of short rows whose long rows lie next to each other.
 * Use:  dlspm_matrix_info mi; dlspm_call_plan cp;
 *       dlspm_analyze(M, K, nnz, row_offsets, col_indices, stream, &mi);   dlspm_advise(DLSPM_OP_SPMM, N, &mi, &cp);
 *       void* ws = NULL; if (cp.bytes) hipMalloc(&ws, cp.bytes);
 *       if (cp.build == DLSPM_BUILD_ROW_PLAN) dlspm_row_plan_build(M, row_offsets, ws, cp.bytes, stream);
 *       if (cp.build == DLSPM_BUILD_CUT_PLAN) dlspm_row_plan_build_cut(M, row_offsets, ws, cp.bytes, stream);
 *       spmm_csr_f32(M, K, N, nnz, ..., ws, cp.bytes | cp.hints, stream);    // as often as the structure is used
 * The finer-grained queries below (dlspm_csr_row_stats, dlspm_workspace_advice, dlspm_row_plan_advice,
 * dlspm_describe_*) remain for callers that know their matrices and for tuning reports.
 * No counterpart in the reference, whose launch sizing needs no knowledge of the matrix (SPMM/spmmesimd2.hpp:30-60) and
 * takes the rows as they come.
 */
typedef struct dlspm_matrix_info {
    int M, K, nnz;
    int max_row_len;             /* longest row                                                               */
    int empty_rows;              /* rows without nonzeros                                                     */
    int max_col_span;            /* widest row: largest - smallest column index + 1                           */
    int eighths_cover_permille;  /* sum over the eight eighths of the rows of the columns each spans, x 1000 / K */
    int eighths_nnz_permille;    /* nonzeros of the heaviest eighth x 1000 / those of the mean eighth         */
} dlspm_matrix_info;
#define DLSPM_BUILD_NOTHING   0
#define DLSPM_BUILD_ROW_PLAN  1
#define DLSPM_BUILD_CUT_PLAN  2
typedef struct dlspm_call_plan {
    int build;     /* DLSPM_BUILD_*: what to build into the memory before the first launch */
    size_t bytes;  /* device memory to pass as `workspace` (0: NULL)                       */
    size_t hints;  /* DLSPM_HINT_* bits to or into `workspace_bytes`                       */
} dlspm_call_plan;
int dlspm_analyze(int M, int K, int nnz, const int* row_offsets, const int* col_indices, void* stream,
                  dlspm_matrix_info* info);
int dlspm_advise(int op, int N_or_D, const dlspm_matrix_info* info, dlspm_call_plan* plan);

/*
 * Longest row and number of rows without nonzeros of a CSR structure that lives on the device (either result
 * pointer may be NULL). Synchronises `stream`; meant to be called once per matrix, like dlspm_csr_check. It
 * has no counterpart in the reference, whose launch sizing looks at M and N only
 * (SPMM/spmmesimd2.hpp:30-60).
 * Use: dlspm_workspace_advice and dlspm_row_plan_advice take the longest row (dlspm_analyze returns it too).
 */
int dlspm_csr_row_stats(int M, const int* row_offsets, void* stream, int* max_row_len, int* empty_rows);

/*
 * Row plan: the order in which a launch hands the rows of one matrix to its workgroups, built once per matrix
 * structure and passed with every launch as its workspace, with DLSPM_HINT_ROW_PLAN. Small matrices with uneven rows,
 * one row per workgroup and every workgroup on the device at once, finish when the compute unit that was handed the
 * most nonzeros does; the plan puts the long rows first and packs the rows that start together so that every compute
 * unit is handed about the same number of nonzeros (2048 x 512, lognormal row lengths, N = 256: 7.6 -> 6.1 us); larger
 * matrices with uneven rows gain as much from the rows being handed out longest first. Every row is summed by one
 * four-wave workgroup in a fixed order (no atomics): the result is bit-identical to the call with a NULL workspace
 * wherever that runs one row per workgroup too.
 *   dlspm_row_plan_bytes(M)  bytes of DEVICE memory for the plan of a matrix of M rows: 3 * M ints, and beyond 2048
 *                            rows as much again and a third for the sort (the launches read the first 3 * M ints).
 *   dlspm_row_plan_build     builds the plan from row_offsets (device) into `plan` (device, 8-byte aligned) with
 *                            kernels on `stream`: nothing is copied to the host, nothing synchronises, and the call may
 *                            be captured in a HIP graph together with the launches that use the plan (one launch up to
 *                            2048 rows, 3 + log2(M / 2048) beyond). A mask whose structure changes from call to call
 *                            can therefore be re-planned on the stream. DLSPM_E_WORKSPACE if plan_bytes is too small.
 *   the launches             spmm_csr_f32 / sddmm_csr_f32 / fused_sddmm_spmm_f32 with workspace = plan and
 *                            workspace_bytes = plan_bytes | DLSPM_HINT_ROW_PLAN. The plan must have been built from the
 *                            same row_offsets (a stale plan gives wrong values but stays inside the arrays). A planned
 *                            launch runs one row per workgroup also where the size rule would group a few rows, if the
 *                            rows are long enough (SDDMM and the fused op up to 2048 rows: whatever their length).
 *                            Short rows, column tiles of a B that fits one L2, widths below 4 (SDDMM and the fused
 *                            op: widths outside 16 < D <= 512, and rows that the size rule groups in masks of more
 *                            than 4096 rows, 8192 at D >= 128 and 128 nonzeros per row) ignore the plan and run as
 *                            with NULL. A planned launch is one kernel (no memset, no allocation, no
 *                            synchronisation); the plan is only read, so launches may share it.
 * No counterpart in the reference, whose kernels take the rows in matrix order (SPMM/spmmesimd2.hpp:63-75).
 */
size_t dlspm_row_plan_bytes(int M);
/*
 * Cut plan: a row plan that also cuts rows. A row that holds much more than a compute unit's share of the nonzeros
 * (share = nnz / compute units) sets the time of the launch by itself, through the one compute unit it runs on,
 * whatever the order of the rows. A cut plan hands every row above one share out in 2, 4, ... 256 equal pieces (the
 * fewest that are no longer than three quarters of a share) to as many workgroups. SDDMM pieces take a share of the row's nonzeros and write
 * their own CSR slots (same bits as any other schedule). SpMM at 33 ... 512 columns gives every piece ALL nonzeros of the
 * row and a share of its columns: one kernel, nothing to combine. The fused op, and SpMM at other widths, write one
 * partial row per piece into memory that follows the plan, and a second small kernel adds the pieces of every cut row
 * in piece order. No atomics, no fences anywhere: deterministic; rows that are not cut are summed as by the plain plan.
 * The plan has room for the most pieces any matrix of M rows can need -- M + 8/3 x compute units entries -- so its size
 * and the launches' grids depend on M, the width and the device only, never on the matrix, and building it needs no
 * look at the matrix from the host.
 *   dlspm_row_plan_bytes_for(op, M, N_or_D)  bytes of DEVICE memory for the cut plan of a matrix of M rows and the
 *                            partial rows of op at that dense width (SDDMM: none, the width is ignored). 0: no cut plan
 *                            at this height (more than 2^20 rows).
 *   dlspm_row_plan_build_cut builds it from row_offsets (device) into `plan` (device, 256-byte aligned) with kernels on
 *                            `stream` only, like dlspm_row_plan_build (two launches up to 2048 - 2 x compute units rows).
 *                            plan_bytes must be at least dlspm_row_plan_bytes_for(DLSPM_OP_SDDMM, M, 0); a plan that is
 *                            to serve SpMM or the fused op must have been sized for that op and width.
 *   the launches             the three compute entry points with workspace = plan and
 *                            workspace_bytes = plan_bytes | DLSPM_HINT_CUT_PLAN (DLSPM_E_WORKSPACE below
 *                            dlspm_row_plan_bytes_for(op, M, width)). SpMM and the fused op write the partial rows
 *                            behind the plan: launches that share a cut plan must not overlap in time. Sizes a planned
 *                            launch is not built for run as with NULL. The fused op (SpMM outside 33 ... 512 columns):
 *                            two kernels per launch.
 * dlspm_row_plan_advice returns 2 where it expects the cut plan to beat the plain one.
 * No counterpart in the reference (one hardware thread per row or row slice, SPMM/spmmesimd2.hpp:63-75).
 */
size_t dlspm_row_plan_bytes_for(int op, int M, int N_or_D);
int dlspm_row_plan_build_cut(int M, const int* row_offsets, void* plan, size_t plan_bytes, void* stream);
/* Whether a plan is worth building for op (DLSPM_OP_*) at these sizes and this longest row (-1: unknown): 0 no (the
 * planned launch is not built for the shape, the rows are known to be even, or the dense operands are so far beyond one
 * L2 that the column-sliced schedule's workspace matters more), 1 a row plan, 2 a cut plan. One of the questions
 * dlspm_advise asks; a caller that passes DLSPM_HINT_ROWS_SKEWED with the plan (longest row at least twenty times the
 * mean) gets the answer for that launch by passing such a longest row here. */
int dlspm_row_plan_advice(int op, int M, int K, int N_or_D, int nnz, int max_row_len);
int dlspm_row_plan_build(int M, const int* row_offsets, void* plan, size_t plan_bytes, void* stream);

/*
 * What to pass as `workspace` for a matrix of these sizes whose longest row has max_row_len nonzeros (from
 * dlspm_csr_row_stats, or known to the caller): DLSPM_PASS_NULL, DLSPM_PASS_ROWS_EVEN (NULL with DLSPM_HINT_ROWS_EVEN)
 * or DLSPM_PASS_WORKSPACE (dlspm_workspace_bytes() bytes of device memory): the memory where the column-sliced schedule
 * applies, or where the rows are very uneven and the flat schedule applies; the hint where the rows are even; NULL
 * otherwise. Host-only; a negative max_row_len means "unknown" and gives the memory only for the column-sliced
 * schedule. One of the questions dlspm_advise asks (after dlspm_row_plan_advice: where a plan applies it is the faster
 * answer). No counterpart in the reference.
 */
#define DLSPM_PASS_NULL       0
#define DLSPM_PASS_ROWS_EVEN  1
#define DLSPM_PASS_WORKSPACE  2
#define DLSPM_PASS_ROWS_SKEWED 3  /* (dlspm_describe_launch_rows only: NULL with DLSPM_HINT_ROWS_SKEWED) */
int dlspm_workspace_advice(int op, int M, int K, int N_or_D, int nnz, int max_row_len);

/*
 * Launch shape the library would use for these sizes, for tuning reports and for host-side models of the
 * schedule (the reference's SpmmEsimdCPU / FusedEsimdCPU, SPMM/spmm-esimd-v1.cpp:83-169 and
 * FUSED/fused.cpp:93-216, play that role for its kernels). Host-only, never touches the device.
 * shape[10] receives: [0] floats per lane per access (4 or 1), [1] G lanes per dense row (SpMM, fused stage 2; 0 for
 * SDDMM), [2] accesses per lane per dense row, [3] G1 lanes per dot product (SDDMM, fused stage 1; 0 for SpMM),
 * [4] accesses per lane per dot product (0 = run-time loop), [5] waves per workgroup, [6] rows per workgroup,
 * [7] column tiles, [8] nonzeros per wave of the flat schedule that a call WITH workspace would use (0 = such a call
 * uses the workgroup-per-row-block schedule too; SDDMM needs no workspace for it), [9] number of such waves.
 * Returns DLSPM_OK or DLSPM_E_INVALID_ARG.
 */
int dlspm_describe_launch(int op, int M, int K, int N_or_D, int nnz, int* shape);

/*
 * The same for a call that passes NULL, the even-rows hint or workspace memory (`passing` = DLSPM_PASS_NULL,
 * DLSPM_PASS_ROWS_EVEN, DLSPM_PASS_WORKSPACE, defined with dlspm_workspace_advice): the lane layout of SpMM
 * (column tiles narrower than 128 only without memory; tiles of 128 on a B of any height only with it, where the
 * column-sliced schedule cuts the tile's slab of B) and the rows per workgroup (more for rows known to be even)
 * depend on it. dlspm_describe_launch is the DLSPM_PASS_NULL case.
 */
int dlspm_describe_launch_rows(int op, int M, int K, int N_or_D, int nnz, int passing, int* shape);

/*
 * Column-sliced schedule that a call WITH workspace would use for these sizes: *slices = number of column ranges
 * the device works through one after the other (0 = that schedule is not used: dense operands of at most 4 MiB,
 * narrow dense rows, short rows), *rows_per_workgroup = rows of one slice handled by a four-wave
 * workgroup. Either pointer may be NULL. Host-only. No counterpart in the reference.
 */
int dlspm_describe_slices(int op, int M, int K, int N_or_D, int nnz, int* slices, int* rows_per_workgroup);

/*
 * Overrides of the launch rules, for tuning sweeps and tests; production callers never need them. One set per host
 * thread: dlspm_set_tuning changes the calling thread's, NULL goes back to the process default. That default is the
 * rules themselves unless the environment said otherwise when the library first looked, once per process:
 * DLSPM_SPLIT="W,R", DLSPM_FLAT, DLSPM_FLAT_CHUNK, DLSPM_SLICES, DLSPM_TILE_MAJOR, DLSPM_TILE_WIDTH, DLSPM_PLAN_ORDER,
 * DLSPM_XCD_CONTIGUOUS, DLSPM_STREAM_RESULTS
 * (so that the drivers can be swept from a shell). No launch reads the environment. An override that names a shape
 * the kernels are not built for is ignored. dlspm_workspace_bytes and the describe calls follow the overrides, so
 * set them before sizing a workspace. No counterpart in the reference (its knobs are -D macros, SPMM/spmmesimd.hpp:17-21).
 */
typedef struct dlspm_tuning {
    int split_w, split_r; /* waves and rows per workgroup of the row-block kernels; 0, 0 = the size rule           */
    int flat;             /* flat schedule of a call with workspace: -1 the size rule, 0 never, 1 always            */
    int flat_chunk;       /* nonzeros per wave of the flat schedule (>= 64); 0 = the rule                           */
    int slices;           /* column-sliced schedule: -1 the size rule, 0 never, n >= 2 that many slices             */
    int tile_major;       /* SpMM column tiles: -1 the rule, 0 row-major, 1 one after the other (tile-major), 2 / 3 every */
                          /* XCD on its own tiles, row- / tile-major within it (calls without memory, with tile_width)    */
    int tile_width;       /* SpMM column tile: 0 the rule, else 512, 256, 128, 64 or 32 (with tile_major = 0: tiles */
                          /* of this width in row-major order)                                                       */
    int plan_order;       /* dlspm_row_plan_build: 0 packed (the rule), 1 alternating groups, 2 longest first       */
    int xcd_contiguous;   /* 0 (the rule): neighbouring row blocks go to different XCDs, as the hardware deals them;   */
                          /* 1: each of the eight XCDs works on one contiguous run of row blocks, so that a banded    */
                          /* mask gathers a different eighth of the dense operands into each L2 (4x fewer bytes       */
                          /* fetched, 6 % faster on a 16384-row band; unsafe as a rule: rows whose length depends on   */
                          /* their position would load the XCDs unevenly). One column tile, no row plan, no slices.   */
                          /* (DLSPM_HINT_BANDED asks for the same per call.)                                          */
    int stream_results;   /* results stored with the non-temporal hint: -1 the size rule (dense result rows from one   */
                          /* L2's worth on, SDDMM results from one and a half), 0 never, 1 always                      */
    int cut_piece_pct;    /* cut plans: the longest piece, in per cent of a share (nnz / compute units); 0 = the rule, 75  */
    int cut_longest_pct;  /* ... and the longest row that stays whole; 0 = the rule, 100. Both 10 ... 1000; they enter the  */
                          /* size of a cut plan, so set them before dlspm_row_plan_bytes_for and keep them for the launches */
    int rules_off;        /* DLSPM_RULE_* bits: size rules switched off, to measure what each is worth; 0 = all on        */
    int compute_units;    /* 0 = the device's own; n (8 ... 1024, a multiple of 8): rules, grids and plans as on a device of n  */
                          /* compute units -- for tests of the rules on another size of device (a partition of an MI355X); */
                          /* results are right for any n, times are best for the true one                                  */
} dlspm_tuning;
/* rules that dlspm_tuning.rules_off can switch off (the others have a field of their own above) */
#define DLSPM_RULE_EIGHT_WAVES_FEW_ROWS         1  /* SDDMM, fused: eight waves per row below two rows per compute unit     */
#define DLSPM_RULE_SIXTEEN_WAVES_TALL_LONG_ROWS 2  /* SpMM: sixteen waves per row for very long rows in a tall matrix       */
#define DLSPM_RULE_MORE_WAVES_FEW_LONG_ROWS     4  /* SpMM: eight or sixteen waves per row for few rows of very many nonzeros */
#define DLSPM_RULE_GROUP_ROWS                   8  /* several short rows per workgroup in tall matrices                     */
#define DLSPM_RULE_ROW_ALIGNED_SPLIT           16  /* whole rows per wave where that is nearly as even as the even split    */
#define DLSPM_RULE_PLAN_UNGROUPS               32  /* a planned launch runs one row per workgroup where the size rule groups */
#define DLSPM_RULE_EXACT_WIDTH_KERNELS         64  /* SDDMM, fused: kernels without bounds handling for D = 16, 32, ... 512  */
#define DLSPM_RULE_CUT_ROWS_BY_COLUMNS        128  /* SpMM with a cut plan, 33 ... 512 columns: the pieces of a cut row share  */
                                                   /* its columns, not its nonzeros (no partial rows, no second kernel)       */
#define DLSPM_RULE_FINER_COLUMN_TILES         256  /* SpMM without memory or plan: narrower column tiles of B for few rows,   */
                                                   /* and for N above 512 in matrices of up to eight rows per compute unit   */
#define DLSPM_RULE_ROW_PIECES_FEW_ROWS        512  /* SDDMM without memory or plan: several workgroups share each row of a   */
                                                   /* mask of fewer rows than three quarters of the compute units, two up to */
                                                   /* one and a half times their number                                      */
#define DLSPM_RULE_MASK_BY_RANGE             1024  /* SDDMM, D a multiple of four up to 512 that no kernel is built for exactly */
                                                   /* (not 32, 64, 96, 128, 192, 256, 384, 512): rhs read as a buffer of 1 GiB    */
                                                   /* whose range check zeroes the lanes past D, where rhs fits (else: by selects); */
                                                   /* the fused op's first stage likewise at D = 260 ... 380                      */
void dlspm_tuning_default(dlspm_tuning* t);   /* fills *t with "follow the rules" */
int dlspm_set_tuning(const dlspm_tuning* t);  /* DLSPM_OK or DLSPM_E_INVALID_ARG (a field out of range) */
int dlspm_get_tuning(dlspm_tuning* t);        /* what the calling thread's launches currently use */

/*
 * What the library knows about the device that the calling thread has current (read from hipDeviceProp_t once per
 * device): compute units, bytes of one L2, and whether it is the gfx950 the kernels are built for. Any pointer may be
 * NULL. The launch rules scale with the first two (bins of a row plan = compute units, slices and column tiles from
 * the L2 size). Returns DLSPM_E_NO_DEVICE without a device (the figures are then those of a whole MI355X: 256, 4 MiB,
 * which is also what the host-only size queries use there); the compute entry points return DLSPM_E_NO_DEVICE when
 * the current device is not a gfx950.
 */
int dlspm_device_info(int* compute_units, long long* l2_bytes, int* is_gfx950);

/* Human-readable text for a status code (never NULL). */
const char* dlspm_status_string(int status);

/* hipError_t (as int) of the last failed HIP call made by this thread inside the library, 0 if none. */
int dlspm_last_hip_error(void);

/* "dlspm_hip <major>.<minor> gfx950" */
const char* dlspm_version(void);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* DLSPM_HIP_H */
