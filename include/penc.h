/*
 * penc.h -- C ABI of the MI355X (gfx950) permutohedral-lattice hash encoding.
 *
 * One shared library (libpenc_hip.so) replaces the native half of the reference: the pybind11
 * class `EncodingWrapper` with its methods `forward`, `backward`,
 * `double_backward_from_positions` (reference: src/PyBridge.cxx:36-42,
 * include/permutohedral_encoding/Encoding.cuh:162-188) and the host launchers behind them
 * (reference: src/Encoding.cu:55-334).
 *
 * Conventions
 *  - Plain pointers and sizes only.  Unless a parameter says "host", every pointer is DEVICE
 *    memory of the GPU that is current on the calling thread; it is borrowed for the duration of
 *    the enqueued work.  The library never allocates or frees device memory and keeps no state.
 *  - All arrays are fp32, densely packed, row-major (F = nr_feat, the features per level: 2, 4 or 8):
 *        positions            [N][D]
 *        lattice_values       [L][C][F]      (8-byte aligned for F = 2, 16-byte for F = 4 and 8;
 *                                            binary16 or bfloat16 in the *_half entry points)
 *        scale_factor         [L][D]         (from penc_scale_factors)
 *        random_shift         [L][D]
 *        anneal_window        [L]
 *        sliced_values        [L+E][F][N]    E = ceil(D/F) if concat_points else 0
 *        grad_sliced_values   [L+E][F][N]    (levels >= L are ignored)
 *        lattice_values_grad  [L][C][F]      (8-byte aligned; the reference returns this logical shape as a
 *                                             permuted view of [L][2][C], src/Encoding.cu:141,204)
 *        positions_grad       [N][D]         (the reference returns this logical shape as a
 *                                             transposed view of [D][N], src/Encoding.cu:152,205)
 *  - `workspace` (optional, may be NULL) is device scratch memory of `workspace_bytes` bytes that
 *    the table-gradient scatter uses to turn its random atomics into streaming traffic; its
 *    contents on entry and exit are meaningless.  penc_scatter_workspace_bytes() suggests a size;
 *    any size works (a small one means more passes, none means direct atomics).  Results do not
 *    depend on it beyond the order of floating-point accumulation.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Work is enqueued and
 *    the call returns without synchronising, like the reference's launches on the current stream.
 *  - D = pos_dim in 2..8, nr_feat 2, 4 or 8 (reference: Encoding.cuh:139-156 supports 2..7 and 2 only;
 *    its instantiations for 4 and 8 features are commented out, src/Encoding.cu:362-363).  With more
 *    than two features the table gradient treats the feature pairs (0,1), (2,3), ... of a level like
 *    levels of their own.
 *  - Every function returns PENC_OK or one of the error codes below; penc_status_string() names it.
 */
#ifndef PENC_H_
#define PENC_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PENC_OK 0
#define PENC_ERR_NULL_POINTER 1        /* a required pointer is NULL */
#define PENC_ERR_BAD_SIZE 2            /* N, L or C is not positive, or a product overflows 2^31 elements */
#define PENC_ERR_UNSUPPORTED_POS_DIM 3 /* pos_dim outside 2..8 (reference: Encoding.cuh:155) */
#define PENC_ERR_UNSUPPORTED_NR_FEAT 4 /* nr_feat not 2, 4 or 8 (reference: Encoding.cuh:142 accepts 2 only) */
#define PENC_ERR_MISALIGNED 5          /* lattice_values not aligned to a slot, or a gradient array not to 8 bytes */
#define PENC_ERR_LAUNCH 6              /* the HIP runtime rejected a launch (hipGetLastError) */
#define PENC_ERR_SCRATCH_TOO_SMALL 7    /* penc_backward_static: the problem does not fit the static scratch */
#define PENC_ERR_WORKSPACE_TOO_SMALL 8  /* penc_backward_rowmajor with positions_grad, penc_forward_rowmajor: no room for the level-major array */
#define PENC_ERR_UNSUPPORTED_TABLE_FORMAT 9 /* the *_half entry points: table_format is neither PENC_TABLE_FP16 nor PENC_TABLE_BF16 */

const char* penc_status_string(int status);

/* Number of extra output levels that carry the raw positions when concat_points is set.
 * Replaces: src/Encoding.cu:71-74 and src/pytorch_modules/modules.py:95-103. */
int penc_extra_levels(int pos_dim, int nr_feat, int concat_points);

/* scale_factor_out[l][i] = fp32(1/sqrt((i+1)(i+2))) * (1.0f / sigmas[l]): the fp32 result of the
 * reference's "tensor element / host scalar", which ATen evaluates as a multiplication by the
 * rounded reciprocal.  Both arrays are HOST memory.
 * Replaces: EncodingFixedParams::compute_scale_factor_tensor, Encoding.cuh:55-69. */
int penc_scale_factors(int pos_dim, int nr_levels, const float* sigmas, float* scale_factor_out);

/* Suggested size of the `workspace` argument of the gradient calls below for binning
 * `levels_per_pass` levels at a time (<= 0: the library's default, all of them); 0 when the capacity
 * is too large for binning (above 2^25 slots).  `nr_levels` counts pairs of features: pass
 * nr_levels * nr_feat / 2.  Per level the workspace holds, for each of the ceil(capacity / 8192)
 * slot ranges (at most 512: above 2^22 slots a range spans 2^14 to 2^16 slots) and each group of
 * 4096 or 8192 points, a 4-byte count and room for the group's
 * expected share of the (pos_dim + 1) records per point plus three standard deviations; a record is
 * 10 bytes for pos_dim <= 5 and capacities up to 2^19 and 12 bytes otherwise: about 11.5 or
 * 13.5 * (pos_dim + 1) bytes per point and level (1.2 GiB for 2^20 points, 24 levels, pos_dim 3).
 * Any smaller workspace works too: the levels are then binned in several passes, and with none the
 * gradient is accumulated with direct atomics.  No counterpart in the reference (its scatter is one
 * atomicAdd per value, EncodingGPU.cuh:409-410). */
size_t penc_scatter_workspace_bytes(int pos_dim, int64_t nr_positions, int nr_levels, int capacity,
                                    int levels_per_pass);

/* Size of `workspace` that lets penc_backward compute positions_grad in groups of a few levels
 * (partial sums in the workspace, then one deterministic reduction) instead of one thread walking
 * all levels; 0 when there is nothing to gain.  A workspace serving both gradients needs the larger
 * of the two sizes.  No counterpart in the reference (it sums levels with atomics,
 * EncodingGPU.cuh:745-750). */
size_t penc_positions_workspace_bytes(int pos_dim, int64_t nr_positions, int nr_levels);

/* Slice: sliced_values[l][f][n] = sum over the D+1 simplex vertices of
 * lattice_values[l][slot][f] * barycentric * anneal_window[l]; extra levels copy
 * positions * points_scaling (zero-padded).
 * Replaces: Encoding<D,2>::forward, src/Encoding.cu:55-108 (kernel forward_gpu,
 * kernels/permutohedral_encoding/EncodingGPU.cuh:68-256). */
int penc_forward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                 const float* positions, const float* lattice_values, const float* scale_factor,
                 const float* random_shift, const float* anneal_window, float* sliced_values,
                 int concat_points, float points_scaling, void* stream);

/* penc_forward with the result as the layer after the encoding reads it: rows
 * sliced_rows[n][nr_feat*level + feature] of row_stride floats (>= nr_feat*(L+E)) instead of [L+E][F][N].
 * The gathering kernel keeps working a level at a time (one level's slice of the table stays in L2, its
 * stores are coalesced) into `workspace`, which must hold the [L+E][F][N] array
 * (penc_forward_rowmajor_workspace_bytes; PENC_ERR_WORKSPACE_TOO_SMALL otherwise), and an LDS-tiled
 * transpose then writes every row as one contiguous chunk, at streaming speed.
 * Replaces: Encoding<D,2>::forward (src/Encoding.cu:55-108) followed by the strided copy a consumer of
 * contiguous rows makes of the reference's permute + reshape (src/pytorch_modules/modules.py:87); a
 * consumer that takes the strided view as it is (a matrix multiplication) needs neither. */
size_t penc_forward_rowmajor_workspace_bytes(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int concat_points);
int penc_forward_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                          const float* positions, const float* lattice_values, const float* scale_factor,
                          const float* random_shift, const float* anneal_window, float* sliced_rows, int64_t row_stride,
                          int concat_points, float points_scaling, void* workspace, size_t workspace_bytes, void* stream);

/* First backward.  lattice_values_grad and positions_grad are each optional (NULL = not wanted,
 * the reference's require_*_grad flags); at least one must be given.  lattice_values_grad is
 * cleared by the library before the scatter-add; positions_grad is written, not accumulated.
 * Replaces: Encoding<D,2>::backward, src/Encoding.cu:112-215 (kernels backward_gpu and
 * backward_gpu_only_pos, EncodingGPU.cuh:259-414 and 530-769). */
int penc_backward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                  const float* positions, const float* lattice_values, const float* scale_factor,
                  const float* random_shift, const float* anneal_window,
                  const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                  void* workspace, size_t workspace_bytes, void* stream);

/* penc_backward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as penc_backward without the workspace: the scratch the table-gradient
 * scatter and the position-gradient partial sums use is a fixed array of
 * PENC_STATIC_SCRATCH_BYTES inside the library's code object (one copy per GPU, held until the
 * process ends).  The call allocates and frees nothing.
 *   - Limit: one level's slot-range records must fit, i.e.
 *     penc_scatter_workspace_bytes(pos_dim, nr_positions, nr_levels * nr_feat / 2, capacity, 1) <= PENC_STATIC_SCRATCH_BYTES
 *     (about 1.3 million points at pos_dim 3 and 2^18 slots, 0.7 million at 2^22 slots); larger problems return PENC_ERR_SCRATCH_TOO_SMALL
 *     and nothing is enqueued.  Levels are binned in as many passes as the scratch needs; position
 *     gradients whose partial sums do not fit are summed by one thread per point instead.
 *   - Every call on a GPU uses that GPU's one array, whose contents survive between calls; what
 *     has to start at zero (a flag per level and slot range) is cleared by the call's own fill kernel,
 *     and every count is written before it is read.  Calls that overlap on
 *     one GPU (two streams, two threads) race on it: serialise them. */
#define PENC_STATIC_SCRATCH_BYTES (64u << 20)
size_t penc_static_scratch_bytes(void);
int penc_backward_static(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                         const float* positions, const float* lattice_values, const float* scale_factor,
                         const float* random_shift, const float* anneal_window,
                         const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                         void* stream);

/* penc_backward reading the upstream gradient as the layer after the encoding produces it: rows
 * grad_rows[n][nr_feat*level + feature] of grad_row_stride floats (even, >= nr_feat*nr_levels; 8-byte
 * aligned) instead of [level][feature][n].  Same outputs and rules as penc_backward.
 *   - The table gradient reads the rows in place.
 *   - The position gradient gathers level by level and needs its upstream gradient in
 *     [level][feature][n] order: that copy (4*nr_feat*nr_levels*nr_positions bytes) is kept at the front of the
 *     workspace.  When the table gradient is wanted too, the scattering kernel writes it as a
 *     by-product of reading the rows; otherwise the rows are transposed first.  With positions_grad the
 *     workspace is therefore required: penc_backward_rowmajor_workspace_bytes() gives the size that also
 *     serves the scatter and the partial sums; PENC_ERR_WORKSPACE_TOO_SMALL if the copy does not fit.
 * Replaces: the strided `.contiguous()` copy of src/pytorch_modules/funcs.py:47 followed by
 * Encoding<D,2>::backward (src/Encoding.cu:112-215). */
size_t penc_backward_rowmajor_workspace_bytes(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                              int want_lattice_values_grad, int want_positions_grad);
int penc_backward_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                           const float* positions, const float* lattice_values, const float* scale_factor,
                           const float* random_shift, const float* anneal_window, const float* grad_rows,
                           int64_t grad_row_stride, float* lattice_values_grad, float* positions_grad,
                           void* workspace, size_t workspace_bytes, void* stream);

/* penc_backward_rowmajor for the table gradient alone (lattice_values is not needed). */
int penc_backward_table_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                 const float* positions, const float* scale_factor, const float* random_shift,
                                 const float* anneal_window, const float* grad_rows, int64_t grad_row_stride,
                                 float* lattice_values_grad, void* workspace, size_t workspace_bytes, void* stream);

/* Double backward from d(loss)/d(positions_grad): gradient w.r.t. lattice_values and w.r.t.
 * grad_sliced_values ([L+E][2][N], zeros in the extra levels).  Either output may be NULL.
 * lattice_values_grad is cleared by the library first.
 * Replaces: Encoding<D,2>::double_backward_from_positions, src/Encoding.cu:219-334 (kernels
 * double_backward_from_positions_gpu_1 / _2, EncodingGPU.cuh:1016-1257 and 1260-1493). */
int penc_double_backward_from_positions(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels,
                                        int capacity, const float* positions,
                                        const float* lattice_values, const float* scale_factor,
                                        const float* random_shift, const float* anneal_window,
                                        const float* double_positions_grad,
                                        const float* grad_sliced_values, float* lattice_values_grad,
                                        float* grad_grad_sliced_values, int concat_points, void* workspace,
                                        size_t workspace_bytes, void* stream);

/* penc_double_backward_from_positions with the upstream gradient of the first backward given as rows
 * grad_rows[n][2*level + feature] (see penc_backward_rowmajor), read in place by the scattering half.
 * grad_grad_sliced_values is written as [L+E][2][N] like before.
 * Replaces: the same reference code as penc_double_backward_from_positions, fed by funcs.py:47's copy. */
int penc_double_backward_from_positions_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels,
                                                 int capacity, const float* positions, const float* lattice_values,
                                                 const float* scale_factor, const float* random_shift,
                                                 const float* anneal_window, const float* double_positions_grad,
                                                 const float* grad_rows, int64_t grad_row_stride,
                                                 float* lattice_values_grad, float* grad_grad_sliced_values,
                                                 int concat_points, void* workspace, size_t workspace_bytes,
                                                 void* stream);

/* The three gathering entry points for a table kept in 16 bits per value: lattice_values_half is
 * [L][C][F] of IEEE binary16 (table_format PENC_TABLE_FP16) or of bfloat16 (PENC_TABLE_BF16),
 * aligned to one slot of 2F bytes.  The values are widened exactly on load and all arithmetic
 * stays fp32, so the results are those of the fp32 entry points on the widened table; sliced
 * values, both gradients and grad_grad_sliced_values are fp32 as before (the table gradient never
 * reads the table).  grad_row_stride selects the layout of the upstream gradient: 0 for
 * [L+E][F][N], otherwise rows of that many floats as in the *_rowmajor entry points (with their
 * workspace rules).
 * Replaces: nothing that runs in the reference; it carries the intent as a disabled switch
 * (LATTICE_HALF_PRECISION, kernels/permutohedral_encoding/EncodingGPU.cuh:12) beside the same
 * forward / backward / double_backward_from_positions (src/Encoding.cu:55-334). */
#define PENC_TABLE_FP16 1
#define PENC_TABLE_BF16 2
int penc_forward_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                      const float* positions, const void* lattice_values_half, int table_format,
                      const float* scale_factor, const float* random_shift, const float* anneal_window,
                      float* sliced_values, int concat_points, float points_scaling, void* stream);
int penc_backward_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                       const float* positions, const void* lattice_values_half, int table_format,
                       const float* scale_factor, const float* random_shift, const float* anneal_window,
                       const float* grad, int64_t grad_row_stride, float* lattice_values_grad, float* positions_grad,
                       void* workspace, size_t workspace_bytes, void* stream);
int penc_double_backward_from_positions_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                             const float* positions, const void* lattice_values_half, int table_format,
                                             const float* scale_factor, const float* random_shift,
                                             const float* anneal_window, const float* double_positions_grad,
                                             const float* grad, int64_t grad_row_stride, float* lattice_values_grad,
                                             float* grad_grad_sliced_values, int concat_points, void* workspace,
                                             size_t workspace_bytes, void* stream);

/* One AdamW step (decoupled weight decay, no amsgrad) on n fp32 values in a single kernel, with the
 * formulas and the order of operations of torch.optim.AdamW; `step` counts from 1.  With
 * skip_zero_gradients an entry whose gradient is exactly 0 keeps its value and both moments: on a
 * hash table most slots receive no gradient in a step, and the update then reads the gradient and
 * touches the rest only where something arrived.
 * No counterpart in the reference library; its training script steps the whole table with
 * torch.optim.AdamW (examples/performance.py:99-101, 161). */
int penc_adamw_step(float* params, const float* grads, float* exp_avg, float* exp_avg_sq, int64_t n, double lr,
                    double beta1, double beta2, double eps, double weight_decay, int64_t step, int skip_zero_gradients,
                    void* stream);

/* The table gradient for tables that dwarf the batch: the caller keeps ONE gradient array and a map of
 * the slot ranges that hold anything across calls, and no call touches more of either than the batch does.
 *   touched  uint32 [L * F/2][R], R = ceil(capacity / penc_touched_range_slots(capacity)) slot ranges per level
 *            and pair of features (penc_touched_map_entries() entries in all): nonzero where the gradient
 *            may be nonzero.
 * Contract: wherever `touched` is 0 the gradient is 0 (both start zeroed by the caller; penc_clear_touched and
 * penc_adamw_step_sparse restore that state).  penc_backward_sparse and
 * penc_double_backward_from_positions_sparse then ADD their sums into lattice_values_grad (so the two calls of a
 * training step accumulate into the one array, which is what autograd would do with a second dense add) and mark
 * the ranges they reached; they clear nothing.  Everything else is as in penc_backward /
 * penc_backward_rowmajor (grad_row_stride 0 or a row stride) and penc_double_backward_from_positions.
 * penc_adamw_step_sparse applies penc_adamw_step with skip_zero_gradients to the touched ranges only and, with
 * `clear`, zeroes the gradients it used and the map; penc_clear_touched only does the clearing.  Both cost one
 * workgroup per (range, level) that leaves at once where nothing was added: the step on a 2^22-slot, 24-level
 * table follows what the batch touched instead of reading 768 MiB of gradient.
 * Replaces: the `zeros` of the whole gradient in every call (src/Encoding.cu:141, 246), autograd's dense
 * accumulation of the two table gradients, and the full-table optimizer step of the reference's training
 * protocol (examples/performance.py:99-101). */
size_t penc_touched_map_entries(int nr_feat, int nr_levels, int capacity);
int penc_touched_range_slots(int capacity);
int penc_backward_sparse(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                         const float* positions, const float* lattice_values, const float* scale_factor,
                         const float* random_shift, const float* anneal_window, const float* grad, int64_t grad_row_stride,
                         float* lattice_values_grad, uint32_t* touched, float* positions_grad, void* workspace,
                         size_t workspace_bytes, void* stream);
int penc_double_backward_from_positions_sparse(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                               const float* positions, const float* lattice_values,
                                               const float* scale_factor, const float* random_shift,
                                               const float* anneal_window, const float* double_positions_grad,
                                               const float* grad, int64_t grad_row_stride, float* lattice_values_grad,
                                               uint32_t* touched, float* grad_grad_sliced_values, int concat_points,
                                               void* workspace, size_t workspace_bytes, void* stream);
int penc_adamw_step_sparse(float* params, float* grads, float* exp_avg, float* exp_avg_sq, int nr_feat, int nr_levels,
                           int capacity, uint32_t* touched, double lr, double beta1, double beta2, double eps,
                           double weight_decay, int64_t step, int clear, void* stream);
int penc_clear_touched(float* grads, int nr_feat, int nr_levels, int capacity, uint32_t* touched, void* stream);

/* dst[c][r] = src[r][c] for a dense row-major rows x cols matrix with cols <= 255 (2 * levels):
 * turns the row-major upstream gradient (N, 2(L+E)) into the grad_sliced_values layout
 * [L+E][2][N] at streaming speed.
 * Replaces: the strided `.contiguous()` copy of src/pytorch_modules/funcs.py:47. */
int penc_transpose(const float* src, float* dst, int64_t rows, int cols, void* stream);

/* Introspection for parity checks: what the kernels derive from each (level, point) before they
 * touch the table.  Outputs are [L][N][D+1]; each may be NULL.
 *   rem0, rank : the remainder-0 lattice point and the residual ranks after the hyperplane wrap
 *   slot       : hashed table index of each of the D+1 vertices
 *   barycentric: the D+1 interpolation weights
 * The kernels share one routine for rem0 and rank and have two equivalent routines for slots and
 * weights; gather_path picks which one is reported: 0 = the compare-and-select chains of the
 * scattering and position-gradient kernels, 1 = the rank sort through LDS of the forward and
 * grad-of-grad kernels (reference: EncodingGPU.cuh:130-223). */
int penc_simplex_debug(int pos_dim, int64_t nr_positions, int nr_levels, int capacity,
                       const float* positions, const float* scale_factor, const float* random_shift,
                       int gather_path, int* rem0, int* rank, int* slot, float* barycentric, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PENC_H_ */
