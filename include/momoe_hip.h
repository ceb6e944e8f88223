/* C ABI of libmomoe_hip.so: hand-written gfx950 (MI355X) kernels for the MoMoE
 * SwiGLU mixture-of-experts layer.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is DEVICE memory unless said
 *     otherwise; bf16 tensors are passed as `void*`/`const void*`.
 *   - nothing is allocated or freed; the caller owns every buffer and sizes the
 *     workspaces with the *_ints / *_bytes queries below.
 *   - work is only ENQUEUED on `stream` (a hipStream_t passed as void*); no entry
 *     point synchronises with the device.
 *   - the return value is a status code (MOMOE_OK or MOMOE_ERR_*); no C++
 *     exception crosses the boundary.  Entry points are re-entrant; the only state the
 *     library keeps is set once and never changed afterwards (the raised dynamic-LDS
 *     limit of each GEMM kernel, the per-device address of the fixed scratch array of
 *     momoe_index_build_static).
 *   - dimension letters: M tokens, D embedding, H expert hidden, N experts,
 *     K experts per token, Msum = M*K (token,expert) pairs = "sorted rows":
 *     the rows of expert i occupy [cumsums[i], cumsums[i+1]) in ascending token order.
 *
 * Each declaration cites the part of the reference (tilde-research/MoMoE-impl,
 * paths relative to its root) that it replaces.
 */
#ifndef MOMOE_HIP_H
#define MOMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOMOE_OK 0
#define MOMOE_ERR_BAD_ARG 1     /* null pointer, negative size, misaligned pointer */
#define MOMOE_ERR_UNSUPPORTED 2 /* shape outside what the kernels handle */
#define MOMOE_ERR_LAUNCH 3      /* the HIP runtime refused a launch */

/* Rows per row tile of the grouped GEMMs.  A tile table is built for one tile height
 * (momoe_index_build, momoe_tile_table_build).  momoe_lin1_swiglu_fwd, momoe_lin2_scale_fwd,
 * momoe_dgrad_h and momoe_dgrad_x take tables of any height up to MOMOE_TILE_ROWS: they hold
 * one code path for heights up to MOMOE_RECOMPUTE_TILE_ROWS and one for taller tiles, and follow
 * the table.  momoe_lin1_swiglu_bwd takes heights up to MOMOE_RECOMPUTE_TILE_ROWS (its epilogue
 * leaves no registers for a taller tile).  A kernel given a table of a greater height than it
 * takes returns without writing anything.
 * tile_rows = 0 in momoe_index_build lets the library choose between the two heights from the
 * routing itself, on the device: taller tiles when they save enough passes over the experts'
 * weights (e.g. experts of 513..640 rows: two row tiles instead of three), else the shorter. */
#define MOMOE_TILE_ROWS 320
#define MOMOE_RECOMPUTE_TILE_ROWS 256
/* column-block width of the partial row sums written by momoe_lin1_swiglu_bwd */
#define MOMOE_GS_BLOCK 128

int momoe_abi_version(void);
const char* momoe_status_string(int status);

/* Measurement aid, no counterpart in the reference.  ticks2: device pointer to two zeroed
 * 64-bit counters, or NULL to stop.  While set, one wavefront of every grouped-GEMM launch
 * (x.Wl1, h.Wl2, both data gradients, both weight gradients) adds the shader-clock ticks it ran
 * for to ticks2[0] and the ticks of the constant 100 MHz counter over the same interval to
 * ticks2[1]: 100 * ticks2[0] / ticks2[1] = average shader clock in MHz under those kernels.
 * Process-wide setting, meant for a benchmark harness: launches in flight when it changes may
 * use either value; the buffer must outlive every launch made while it is set.
 */
int momoe_set_clock_trace(unsigned long long* ticks2);

/* Measurement aid, no counterpart in the reference: what the matrix pipe of this machine
 * sustains on a given kind of operand data.  Launches one workgroup of 8 wavefronts per CU whose
 * waves do nothing but issue the GEMMs' MFMA (v_mfma_f32_32x32x16_bf16, the 2 x 4 fragment tile
 * of one wave) `iters` x 16 times on operands read once from operands_64KiB (4096 x 16 bytes of
 * bf16 values: the row-side operand's fragments come from the first half, the column-side
 * operand's from the second half).  The
 * rate depends on the data: the chip is power-limited under sustained MFMA load.
 * sink_512: 512 floats of scratch (not written in practice).  ticks2 (may be NULL): device
 * pointer to two 64-bit counters that receive the shader-clock ticks and the 100 MHz ticks of
 * one wavefront.  Returns the number of floating-point operations of the launch (time it with
 * events on `stream`), or -1 on a bad argument / failed launch.
 */
int64_t momoe_mfma_rate_probe(const void* operands_64KiB, float* sink_512, int iters,
                              unsigned long long* ticks2, void* stream);

/* Measurement aid, no counterpart in the reference: the rate at which this machine streams
 * weights from HBM when nothing else happens.  Reads `blocks` row-major bf16 matrices of
 * krows x ncol (consecutive in memory; krows a multiple of 32, ncol of 256, one matrix below
 * 4 GiB) exactly as the grouped GEMMs read expert weights -- global -> LDS transfers of 32 x 256
 * stages, four stages per workgroup in flight, one workgroup per CU -- and drops the data.
 * Returns the bytes read by the launch (time it with events on `stream`; use more bytes than
 * the 256 MiB last-level cache holds), or -1 on a bad argument / failed launch.
 */
int64_t momoe_hbm_stream_probe(const void* matrix, int64_t blocks, int64_t krows, int64_t ncol,
                               void* stream);

/* ---- routing index -------------------------------------------------------
 * Replaces find_used_experts + scatter_cols_kernel (momoe/momoe.py:821-842,
 * 760-815) and the torch.sum at :830.
 *
 * mask_NM: int32 0/1, element (i,m) at mask[i*stride_n + m*stride_m].
 * Outputs: sizes_N int64[N]; cumsums_N1 int32[N+1]; idx_Msum int32[M*K]
 * (token of each sorted row); which_Msum int32[M*K] (slot of the pair within its
 * token = number of lower-numbered experts holding the token); inv_MK
 * int32[M*K] (sorted row of token m's k-th pair); tile_table
 * int32[momoe_tile_table_ints()] (device-side list of (expert,row-block) tiles
 * so that no GEMM launch depends on host knowledge of the routing);
 * tile_rows: rows per row tile the table is built for, a multiple of 32 from 32 to
 * MOMOE_TILE_ROWS (anything else: MOMOE_ERR_UNSUPPORTED; the GEMMs deal whole 32-row fragment
 * rows to an expert's tiles), or 0: the library
 * picks MOMOE_RECOMPUTE_TILE_ROWS or MOMOE_TILE_ROWS on the device (table[1] holds the choice);
 * momoe_tile_table_ints(M, N, K, 0) sizes the table for either.
 * recompute_table (may be NULL; only with tile_rows = 0, MOMOE_ERR_BAD_ARG otherwise)
 * int32[momoe_tile_table_ints(M, N, K, MOMOE_RECOMPUTE_TILE_ROWS)]: receives the table for tiles of
 * MOMOE_RECOMPUTE_TILE_ROWS rows, which momoe_lin1_swiglu_bwd needs whatever height was chosen
 * for the others (the same contents as momoe_tile_table_build would give, without its launch).
 * violations int32[1] += number of tokens whose pair count differs from K
 * (caller zeroes it; if the total pair count exceeds M*K the tile table is
 * emptied so later kernels touch nothing).
 */
int64_t momoe_tile_table_ints(int64_t M, int64_t N, int64_t K, int tile_rows);
int64_t momoe_index_workspace_bytes(int64_t M, int64_t N);
int momoe_index_build(const int32_t* mask_NM, int64_t stride_n, int64_t stride_m,
                      int64_t M, int64_t N, int64_t K,
                      int64_t* sizes_N, int32_t* cumsums_N1, int32_t* idx_Msum,
                      int32_t* which_Msum, int32_t* inv_MK,
                      int32_t* tile_table, int tile_rows, int32_t* recompute_table,
                      void* workspace, int64_t workspace_bytes,
                      int32_t* violations, void* stream);

/* A tile table for another tile height, from the prefix sums of a finished momoe_index_build
 * (no counterpart in the reference: its launchers size their grids on the host).  Msum = M*K, the
 * rows the sorted matrices were allocated for; tile_table int32[momoe_tile_table_ints(M, N, K,
 * tile_rows)].  Same contents as the table momoe_index_build writes for that tile_rows (a
 * multiple of 32 from 32 to MOMOE_TILE_ROWS; 0 is not accepted here).
 */
int momoe_tile_table_build(const int32_t* cumsums_N1, int64_t N, int64_t Msum, int tile_rows,
                           int32_t* tile_table, void* stream);

/* momoe_index_build_static: momoe_index_build without the workspace arguments, for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The panel counts
 * go to a fixed array of MOMOE_INDEX_STATIC_SCRATCH_BYTES that is part of the library's device
 * code (each GPU the library runs on holds it until the process ends), so the call allocates
 * nothing and calls no allocating routine; inputs and outputs are still the caller's.
 * momoe_index_workspace_bytes(M, N) > MOMOE_INDEX_STATIC_SCRATCH_BYTES (e.g. M = 65536 tokens
 * with more than 240 experts) returns MOMOE_ERR_UNSUPPORTED.  Results are bit-identical to
 * momoe_index_build.  All calls on one GPU share that GPU's array: two calls that overlap on one
 * GPU (different streams) race; calls on one stream, or on different GPUs, do not.  The first
 * call on a device looks the array's address up (hipGetSymbolAddress), which must not happen
 * under stream capture: make one call per device beforehand.
 */
#define MOMOE_INDEX_STATIC_SCRATCH_BYTES 4194304
int momoe_index_build_static(const int32_t* mask_NM, int64_t stride_n, int64_t stride_m,
                             int64_t M, int64_t N, int64_t K,
                             int64_t* sizes_N, int32_t* cumsums_N1, int32_t* idx_Msum,
                             int32_t* which_Msum, int32_t* inv_MK,
                             int32_t* tile_table, int tile_rows, int32_t* recompute_table,
                             int32_t* violations, void* stream);

/* ---- experts forward -----------------------------------------------------
 * momoe_lin1_swiglu_fwd replaces lin1_kernel (momoe/momoe.py:69-152):
 *   [a|b] = x[idx[r]] @ Wl1[i]  (fp32 accumulate), h[r] = bf16(a * b * sigmoid(b)).
 * x_MD bf16 [M,D]; Wl1_ND2H bf16 [N,D,2H]; h_blocked bf16 [H/32][Msum][32]: h[r][j] at
 * [((j / 32) * Msum + r) * 32 + j % 32], the layout momoe_lin2_scale_fwd reads (its contraction
 * runs over j: 32 of them for consecutive rows are one contiguous block).  h_blocked may be NULL:
 * then only a|b is produced and row tiles entirely below ab_row_lo are skipped;
 * ab_rows bf16 [*,2H] indexed by the sorted row r (may be NULL): rows with
 * ab_row_lo <= r < ab_row_hi receive bf16(a)|bf16(b) (the selective save of
 * :141-145 with lo=0, hi=Msave).
 */
int momoe_lin1_swiglu_fwd(const void* x_MD, const void* Wl1_ND2H, const int32_t* idx_Msum,
                          const int32_t* tile_table, void* h_blocked,
                          void* ab_rows, int64_t ab_row_lo, int64_t ab_row_hi,
                          int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum, void* stream);

/* momoe_lin2_scale_fwd replaces lin2_kernel (momoe/momoe.py:161-237):
 *   ys[r] = bf16( (h[r] @ Wl2[i]) * s[i, idx[r]] ), rows kept in sorted order.
 * h_blocked as written by momoe_lin1_swiglu_fwd.
 * s_NM fp32, element (i,m) at s[i*s_stride_n + m*s_stride_m]. ys_MsumD bf16 [Msum,D].
 */
int momoe_lin2_scale_fwd(const void* h_blocked, const void* Wl2_NHD,
                         const float* s_NM, int64_t s_stride_n, int64_t s_stride_m,
                         const int32_t* idx_Msum, const int32_t* tile_table, void* ys_MsumD,
                         int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum, void* stream);

/* momoe_combine replaces y_KMD.sum(dim=0) / G_x_KMD.sum(dim=0) (momoe/momoe.py:290, :754):
 *   out[m] = bf16( sum_k rows[inv[m,k]] ) with fp32 accumulation, k ascending.
 */
int momoe_combine(const void* rows_MsumD, const int32_t* inv_MK, void* out_MD,
                  int64_t M, int64_t D, int64_t K, int64_t Msum, void* stream);

/* ---- experts backward ----------------------------------------------------
 * The reference's swiglu_backward_kernel (momoe/momoe.py:421-535) computes dL/dh = G_y.Wl2^T,
 * recomputes a|b = x.Wl1 for rows that were not saved, and applies the SwiGLU backward, in one
 * kernel; lin1_backward_kernel (:683-703) obtains the gate-weight gradient from a recomputed
 * down projection.  Here the same results come from three entry points:
 *
 * momoe_dgrad_h:  u[r] = bf16( G_y[idx[r]] @ Wl2[i]^T )  (fp32 accumulate over D), the
 *   gradient of h before the gate weight; u_MsumH bf16 [Msum,H] in sorted order.
 *
 * momoe_lin1_swiglu_bwd, for the sorted rows without saved a|b:
 *   a|b  = x[idx[r]] @ Wl1[i]   (fp32, kept in registers)
 *   s    = s_NM[i, idx[r]],  sig = sigmoid(b)
 *   gz[r] = bf16( s u b sig | s u a sig (1 + b (1 - sig)) )       [G_a | G_b], 2H columns
 *   hs    = bf16( s a b sig )       (h pre-scaled by the gate weight, for the Wl2 gradient)
 *   gs_part[p][r] = sum over the p-th block of MOMOE_GS_BLOCK hidden columns of u a b sig
 * (sum_p gs_part[p][r] = G_y[idx[r]] . (h[r] @ Wl2[i]) = dL/ds, by associativity).
 * gs_part fp32 [ceil(H/MOMOE_GS_BLOCK)][Msum].
 * gz is written k-blocked, gz_blocked bf16 [2H/32][Msum][32]: gz[r][j] at
 * [((j / 32) * Msum + r) * 32 + j % 32] -- the layout momoe_dgrad_x contracts over and
 * MOMOE_LAYOUT_KBLOCKED of momoe_wgrad.
 * hs is written in the layout MOMOE_LAYOUT_TRANSPOSED of momoe_wgrad, zero padding included:
 * hsT_GH32 bf16 [momoe_padded_rows(Msum, N) / 32][ld_hsT][32], ld_hsT >= H a multiple of 8.
 *
 * momoe_swiglu_bwd_saved: the same from the saved a|b (bf16) of the rows below Msave; the row
 * sum is spread over the first ceil(H/256) parts, the other parts get zeros
 * (nparts = ceil(H / MOMOE_GS_BLOCK)).
 *
 * Which of the two produces a row (the reference's own choice is per tile of its autotuned
 * height, momoe/momoe.py:486): rows are taken in groups of 32 counted from their expert's first
 * row; momoe_swiglu_bwd_saved produces the groups that lie entirely below Msave,
 * momoe_lin1_swiglu_bwd (row_lo = Msave) all others, so that up to 31 rows just below Msave
 * are recomputed although their a|b were saved.  Call both with the same Msave; either is a
 * no-op when it has no rows (Msave = 0, row_lo = Msum).
 */
int momoe_dgrad_h(const void* Gy_MD, const void* Wl2_NHD, const int32_t* idx_Msum,
                  const int32_t* tile_table, void* u_MsumH,
                  int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum, void* stream);

int momoe_lin1_swiglu_bwd(const void* x_MD, const void* Wl1_ND2H, const int32_t* idx_Msum,
                          const int32_t* tile_table, const void* u_MsumH,
                          const float* s_NM, int64_t s_stride_n, int64_t s_stride_m,
                          int64_t row_lo, void* gz_blocked, void* hsT_GH32, int64_t ld_hsT,
                          float* gs_part,
                          int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum, void* stream);

int momoe_swiglu_bwd_saved(const void* ab_save, const void* u_MsumH,
                           const float* s_NM, int64_t s_stride_n, int64_t s_stride_m,
                           const int32_t* idx_Msum, const int32_t* cumsums_N1, int64_t Msave,
                           void* gz_blocked, void* hsT_GH32, int64_t ld_hsT,
                           float* gs_part, int64_t nparts,
                           int64_t M, int64_t H, int64_t N, int64_t Msum, void* stream);

/* momoe_gs_scatter: Gs_NM[i, idx[r]] = sum_p gs_part[p][r] for every sorted row r of
 * expert i (momoe/momoe.py:699-703 without atomics).  Gs_NM fp32 contiguous [N,M],
 * zero-filled by the caller (:721).
 */
int momoe_gs_scatter(const float* gs_part, int64_t nparts, const int32_t* idx_Msum,
                     const int32_t* cumsums_N1, float* Gs_NM,
                     int64_t M, int64_t N, int64_t Msum, void* stream);

/* momoe_dgrad_x replaces the GEMM of lin1_backward_kernel (momoe/momoe.py:662-681):
 *   gxs[r] = bf16( gz[r] @ Wl1[i]^T ), rows kept in sorted order; follow with
 *   momoe_combine to obtain G_x.  gz_blocked as written by the SwiGLU backward entry points.
 */
int momoe_dgrad_x(const void* gz_blocked, const void* Wl1_ND2H, const int32_t* tile_table,
                  void* gxs_MsumD, int64_t M, int64_t D, int64_t H, int64_t N, int64_t Msum,
                  void* stream);

/* momoe_wgrad replaces weights_update_kernel (momoe/momoe.py:356-412):
 *   GW[i][x][y] = bf16( sum over sorted rows r of expert i of A(r, x) * B(r, y) ).
 * Each operand comes in one of two layouts:
 *   MOMOE_LAYOUT_ROWS        bf16 [row][feature] with row stride ld (>= features):
 *                            A(r, x) = A[ra(r) * lda + x], ra(r) = a_gather ? a_gather[r] : r.
 *   MOMOE_LAYOUT_TRANSPOSED  bf16 [padded sorted row / 32][ld][32] with ld >= features, no
 *                            gather: the sorted row r of expert i (whose first sorted row is
 *                            c = cumsums[i]) has the padded position
 *                            p = ((c + 31) & ~31) + 32 * i + (r - c) < momoe_padded_rows(Msum, N),
 *                            and its feature f sits at [(p / 32) * ld * 32 + f * 32 + p % 32];
 *                            the positions between an expert's last row and the next multiple of
 *                            32 must hold zeros.  This is how momoe_lin1_swiglu_bwd /
 *                            momoe_swiglu_bwd_saved write hs: the contraction index is the fast
 *                            one, which the kernel reads from LDS at twice the rate of the row
 *                            layout, and each 32-row stage of a tile is one contiguous block.
 *                            At most one operand may be transposed.
 *   MOMOE_LAYOUT_KBLOCKED    (B only) bf16 [features/32][ld][32] with ld >= Msum = rows of the
 *                            matrix, no gather: B(r, y) = B[((y / 32) * ld + r) * 32 + y % 32];
 *                            Y a multiple of 32.  This is how gz is written.  The eight
 *                            32-column blocks of a tile are addressed with 32-bit byte offsets:
 *                            8 * ld * 64 bytes must stay below 4 GiB, i.e. ld < 8 388 608 rows
 *                            (about one million tokens at K = 8), else MOMOE_ERR_UNSUPPORTED.
 * M = number of tokens (rows of a gathered matrix, and the most rows an expert can hold);
 * M * ld * 2 bytes (row layout) must stay below 4 GiB.  Experts without rows get exact zeros.
 * Wl2 gradient: A = hs (transposed, X=H), B = G_y gathered by idx (Y=D).
 * Wl1 gradient: A = x gathered by idx (X=D), B = gz (k-blocked, Y=2H).
 * workspace: device scratch (16-byte aligned, contents undefined on entry and exit) for
 * fp32 partial tiles of MOMOE_WGRAD_PARTIAL_BYTES each.  An expert that holds many times
 * the average number of rows is contracted in several pieces so that its tiles do not
 * outlast everything else in the launch; the pieces meet in the workspace and a second
 * kernel adds them.  Any size is accepted: momoe_wgrad_workspace_bytes() is the most the
 * library will use, a smaller workspace means coarser pieces, 0 (workspace may be NULL)
 * means none.  The result does not depend on the routing of other experts, but the
 * summation order of a cut expert differs from that of an uncut one.
 */
#define MOMOE_WGRAD_PARTIAL_BYTES 262144
#define MOMOE_LAYOUT_ROWS 0
#define MOMOE_LAYOUT_TRANSPOSED 1
#define MOMOE_LAYOUT_KBLOCKED 2
int64_t momoe_padded_rows(int64_t Msum, int64_t N);
int64_t momoe_wgrad_workspace_bytes(int64_t N, int64_t X, int64_t Y, int64_t Msum);
int momoe_wgrad(const void* A, int64_t lda, int a_layout, const int32_t* a_gather,
                const void* B, int64_t ldb, int b_layout, const int32_t* b_gather,
                const int32_t* cumsums_N1, void* GW_NXY,
                int64_t M, int64_t N, int64_t X, int64_t Y, int64_t Msum,
                void* workspace, int64_t workspace_bytes, void* stream);

/* ---- router ----------------------------------------------------------------
 * momoe_router_fwd replaces the elementwise part of TopKRouterFunction.forward
 * (momoe/topk_router.py:96-120), given the gate logits (the matmul of :95 stays a
 * library GEMM): fp32 softmax over the N-Ks routed and the Ks shared columns,
 * top-(K-Ks) of (probability + bias) with ties going to the lower index,
 * renormalisation.  logits_MN [M,N] row-major, bf16 (logits_f32=0) or fp32 (=1).
 * Outputs: mask_NM int32 [N,M] contiguous; s_MN fp32 [M,N] (its transpose view is
 * s_NM); p_sel_MN fp32 [M,N] (masked softmax probabilities, :106); Ng_M, Ks_M fp32 [M].
 */
int momoe_router_fwd(const void* logits_MN, int logits_f32, const float* biases_N,
                     int64_t M, int64_t N, int64_t K, int64_t Ks,
                     int32_t* mask_NM, float* s_MN, float* p_sel_MN, float* Ng_M, float* Ks_M,
                     void* stream);

/* momoe_router_bwd replaces normalize_backward_kernel (momoe/topk_router.py:11-56):
 * gradient w.r.t. the gate logits, bf16 [M,N] row-major.  Gs_NM fp32, element (i,m) at
 * Gs[i*gs_stride_n + m*gs_stride_m]; it is not modified.
 */
int momoe_router_bwd(const float* Gs_NM, int64_t gs_stride_n, int64_t gs_stride_m,
                     const float* p_sel_MN, const float* s_MN, const float* Ng_M, const float* Ks_M,
                     const int32_t* mask_NM, int64_t M, int64_t N, int64_t Ks,
                     void* Glogits_MN, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOMOE_HIP_H */
