/*
 * distdl_hip.h -- C ABI of libdistdl_hip.so (gfx950 / MI355X).
 *
 * One rank's local share of the DistDL data-parallel hot path: the strided
 * pack / unpack copies of Repartition and HaloExchange, and the local-shard
 * compute of DistributedLayerNorm, DistributedEmbedding and DistributedLinear.
 *
 * Conventions (every entry point):
 *   - plain pointers and sizes only; every pointer named "device" is a device
 *     address owned by the caller, every other pointer is host memory that is
 *     only read during the call;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work
 *     is enqueued asynchronously, nothing synchronises, nothing allocates;
 *   - the return value is 0 on success, a positive hipError_t if the runtime
 *     refused a launch, or a negative DDL_E_* code for a rejected argument;
 *     ddl_last_error() gives the message of the calling thread's last failure;
 *   - shapes, starts and strides are int64 counts of ELEMENTS, row-major order
 *     of dimensions (dimension 0 slowest) unless strides say otherwise.
 *
 * Citations are paths below the reference's src/distdl/ (or tests/, examples/).
 */
#ifndef DISTDL_HIP_H
#define DISTDL_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DDL_MAX_DIMS 8

#define DDL_E_ARG      (-1)  /* null pointer, negative size, bad enum        */
#define DDL_E_DIMS     (-2)  /* ndim outside [1, DDL_MAX_DIMS]               */
#define DDL_E_ALIGN    (-3)  /* pointer not aligned to the element size      */
#define DDL_E_SHAPE    (-4)  /* box outside its tensor / inconsistent shape  */
#define DDL_E_UNSUPP   (-5)  /* valid request this build does not implement  */

/* Library identification: "distdl_hip <version> gfx950". */
const char* ddl_version(void);

/* Message for the last non-zero return on the calling thread ("" if none). */
const char* ddl_last_error(void);

/* ------------------------------------------------------------------------ *
 * Box copies (Repartition / HaloExchange pack, unpack, self-copy)
 * ------------------------------------------------------------------------ */

/* One rectangular box copied between two strided device tensors.  `src` and
 * `dst` point at the FIRST element of the box on each side. */
typedef struct ddl_box {
    const void* src;                   /* device */
    void*       dst;                   /* device */
    int32_t     ndim;                  /* 1..DDL_MAX_DIMS */
    int32_t     reserved;
    int64_t     shape[DDL_MAX_DIMS];
    int64_t     src_stride[DDL_MAX_DIMS];
    int64_t     dst_stride[DDL_MAX_DIMS];
} ddl_box_t;

#define DDL_OP_COPY 0   /* dst  = src                                          */
#define DDL_OP_ADD  1   /* dst += src  (needs `dtype`; boxes must not alias)   */

#define DDL_DT_BITS 0   /* opaque elements of elem_size bytes (copy only)      */
#define DDL_DT_F32  1
#define DDL_DT_F64  2
#define DDL_DT_BF16 3
#define DDL_DT_F16  4
#define DDL_DT_I32  5   /* box accumulation only; sums wrap around             */
#define DDL_DT_I64  6   /* box accumulation only; sums wrap around             */

/* Copies (or accumulates) `nbox` boxes in as few launches as possible (16
 * boxes per launch).  Boxes of one call must not overlap each other on the
 * destination side.  Zero-volume boxes are skipped.
 *
 * Replaces the strided self-copy of Repartition,
 *   backends/mpi_numpy/functional/repartition.py:179-190 (np.copyto(output[ysl], input[xsl])),
 *   backends/nccl_cupy/functional/repartition.py:186,
 * and, with DDL_OP_ADD, the adjoint accumulation of HaloExchange,
 *   backends/mpi_numpy/functional/halo_exchange.py:138,140 (grad_output[lbs] += lbb). */
int ddl_copy_boxes(const ddl_box_t* boxes, int nbox, int elem_size,
                   int op, int dtype, void* stream);

/* One box summed over `nsrc` sources (1..64) in one pass:
 *   dst[box] = (srcs[0][box] / divisor) + (srcs[1][box] / divisor) + ...
 * added in the order of `srcs`, quotients and partial sums rounded to the
 * element type, i.e. bit for bit what element-wise divisions followed by
 * accumulating box copies give -- but every source is read once and the
 * destination written once.  `box` supplies dst, shape, dst_stride and the
 * src_stride shared by all sources (its src field is ignored); srcs[q] points
 * at the first element of the box in source q, all a multiple of 16 bytes
 * apart.  dst may be one of the sources (same strides) but must not overlap
 * them otherwise.  Integer dtypes take divisor 1 only.  The 16-bit types are
 * divided and added in fp32 and rounded to nearest even after every operation
 * (a NaN stays a NaN, whatever its payload); a divisor that is a power of two
 * is applied as a product with its exact reciprocal, which gives the same bits.
 *
 * Replaces the local reduction and re-layout of ReduceScatter,
 *   backends/mpi_numpy/functional/reduce_scatter.py:86-119 (rearrange + MPI.SUM
 *   into the own slab), the sum of AllSumReduce, all_sum_reduce.py:77-92, and
 * the scaling of gradients ahead of the adjoint sums,
 *   all_gather.py:188-190, all_sum_reduce.py:127-128, broadcast.py:208-209
 *   (grad_output / scale_backward). */
int ddl_sum_boxes(const ddl_box_t* box, const void* const* srcs, int nsrc,
                  int elem_size, int dtype, double divisor, void* stream);

/* Pack: for b in [0,nbox): bufs[b] (contiguous, C order, shape box_shape[b])
 *       = tensor[box_start[b] : box_start[b]+box_shape[b]].
 * `tensor_strides` are the element strides of the (possibly non-contiguous)
 * source tensor whose extent is `tensor_shape`.  box_start / box_shape are
 * [nbox][ndim] row-major.  bufs[b] may be NULL to skip a box.
 *
 * Replaces  np.copyto(xfer_buff, input.detach()[sl].cpu().numpy())
 *   backends/mpi_numpy/functional/repartition.py:158-171 (forward), :300-312 (adjoint),
 *   xfer_buff.copy_(input.detach()[sl])  backends/nccl_cupy/functional/repartition.py:164,
 * and the halo bulk-slab pack
 *   backends/mpi_numpy/functional/halo_exchange.py:50-53 (forward), :115-119 (adjoint). */
int ddl_pack_boxes(const void* tensor, const int64_t* tensor_shape,
                   const int64_t* tensor_strides, int ndim, int elem_size,
                   int nbox, const int64_t* box_start, const int64_t* box_shape,
                   void* const* bufs, void* stream);

/* Unpack: tensor[box_start[b] : +box_shape[b]] (op)= bufs[b]; the mirror of
 * ddl_pack_boxes.  op = DDL_OP_COPY or DDL_OP_ADD (then `dtype` != DDL_DT_BITS).
 *
 * Replaces  np.copyto(output[sl], xfer_buff)
 *   backends/mpi_numpy/functional/repartition.py:192-208 (forward), :335-349 (adjoint),
 *   output[sl] = xfer_buff.detach().clone()  backends/nccl_cupy/functional/repartition.py:205,
 * and the halo ghost-slab unpack
 *   backends/mpi_numpy/functional/halo_exchange.py:70-74 (forward), :136-140 (adjoint, add). */
int ddl_unpack_boxes(void* tensor, const int64_t* tensor_shape,
                     const int64_t* tensor_strides, int ndim, int elem_size,
                     int nbox, const int64_t* box_start, const int64_t* box_shape,
                     const void* const* bufs, int op, int dtype, void* stream);

/* Sets every element of each box of `tensor` to zero bits.
 * Replaces  grad_output[lgs] = 0.0  backends/mpi_numpy/functional/halo_exchange.py:116,119
 * and the zero initialisation of the Repartition output, repartition.py:175-177. */
int ddl_zero_boxes(void* tensor, const int64_t* tensor_shape,
                   const int64_t* tensor_strides, int ndim, int elem_size,
                   int nbox, const int64_t* box_start, const int64_t* box_shape,
                   void* stream);

/* ------------------------------------------------------------------------ *
 * Fused halo staging: zero-pad + ghost fill + send-slab pack in one pass
 * ------------------------------------------------------------------------ */

/* Writes the padded, exchanged tensor `xpad` (contiguous, shape
 * x_shape[d] + pad[d][0] + pad[d][1]) from the local shard `x` (contiguous,
 * shape x_shape) and, in the same pass, the send slabs.
 *
 *   pad   [ndim][2]  total padding = explicit zero padding + halo width
 *   recv  [ndim][2]  ghost (receive) widths, left/right, in xpad coordinates
 *   send  [ndim][2]  bulk  (send)    widths, left/right
 *   ghost_bufs [ndim][2]  contiguous received slabs (NULL where width is 0)
 *   bulk_bufs  [ndim][2]  contiguous slabs to send   (NULL where width is 0)
 *
 * Slab geometry is that of HaloExchange._assemble_slices, nn/halo_exchange.py:37-99:
 * for exchange dimension i, dimensions j<i span all of xpad, j==i the
 * ghost/bulk strip, j>i the bulk range [recv[j][0], size-recv[j][1]).
 * The result equals F.pad (nn/conv_feature.py:400-407) followed by the
 * dimension-ordered pack / unpack loop of
 * backends/mpi_numpy/functional/halo_exchange.py:30-76 when the ghost slabs
 * are those the neighbours send: an element lying in the ghost strips of
 * several dimensions takes the slab of the highest such dimension, and a bulk
 * slab of dimension i sees the ghosts of dimensions < i.
 * Only when every ghost slab is available before the call (one-GPU stub
 * exchange, or `ghost_bufs` all NULL for phase 0 of a real exchange).
 *
 * `kernel` chooses between the library's two implementations, whose results
 * are identical (no counterpart in the reference; tests run every case on
 * both).  DDL_HALO_AUTO: tensors of 2-, 4- or 8-byte elements whose shard rows
 * hold at least 32 elements (8-byte ones count as two) are assembled through
 * LDS and stored in whole 128-byte lines, everything else is written row by
 * row.  DDL_HALO_LINES lowers that row threshold to 1, DDL_HALO_ROWS always
 * writes row by row.  Whatever the choice, 1-byte elements, padded rows shorter
 * than 32 elements, outputs not aligned to 16 bytes and tensors of 2^31
 * elements or more are written row by row. */
#define DDL_HALO_AUTO  0
#define DDL_HALO_ROWS  1
#define DDL_HALO_LINES 2
int ddl_halo_pad_exchange(const void* x, void* xpad, const int64_t* x_shape,
                          int ndim, int elem_size,
                          const int64_t* pad, const int64_t* recv,
                          const int64_t* send,
                          const void* const* ghost_bufs, void* const* bulk_bufs,
                          int kernel, void* stream);

/* ------------------------------------------------------------------------ *
 * DistributedLayerNorm local shard (fp32, bf16 or fp16 elements; fp32 sums)
 * ------------------------------------------------------------------------ */

/* Per-row partial statistics of the local shard x[rows, cols] (row stride
 * `ld` elements, dtype DDL_DT_F32 / _BF16 / _F16): stats[r] = { mean_r, M2_r }
 * with M2 = sum (x - mean_r)^2, fp32 accumulation.  One read of x.
 *
 * Replaces the local halves of DistributedLayerNorm._compute_mean / _compute_var,
 *   nn/layernorm.py:230 (input.mean(dim, keepdim)) and :246-247. */
int ddl_ln_partial_stats(const void* x, int dtype, int64_t rows, int64_t cols,
                         int64_t ld, float* stats /*[rows][2]*/, void* stream);

/* Combines the partial statistics of the `nparts` workers that share a row and
 * normalises the local shard:
 *   mean = (1/P) sum_p mean_p
 *   var  = (1/P) sum_p (M2_p + n_p (mean_p - mean)^2) / n_p      (biased)
 *   y    = (x - mean) / sqrt(var + eps) [* gamma + beta]
 * which is the reference's mean-of-local-means / mean-of-local-variances,
 *   nn/layernorm.py:230-233, :246-247, :298-302, :309,
 * with the two all-reduces replaced by one gather of {mean, M2}.
 *   x, y, gamma, beta   elements of `dtype`
 *   part_stats [nparts][rows][2]  fp32 (this worker's own partials included)
 *   part_cols  [nparts]           host array: columns n_p held by each worker
 *   gamma/beta [cols] or NULL (both or neither)
 *   mean_out/rstd_out [rows] fp32 or NULL: the combined statistics, for backward. */
int ddl_ln_normalize_affine(const void* x, int dtype, int64_t rows, int64_t cols,
                            int64_t ld, const float* part_stats,
                            int nparts, const int64_t* part_cols,
                            const void* gamma, const void* beta,
                            float eps, void* y, int64_t ldy,
                            float* mean_out, float* rstd_out, void* stream);

/* Layer norm of rows that this worker holds whole, in ONE launch and one read
 * of x:  y = (x - mean) / sqrt(var + eps) [* gamma + beta]  with the row's own
 * mean and biased variance.  Replaces
 *   torch.nn.functional.layer_norm(input, normalized_shape, weight, bias, eps)
 * in the branch of DistributedLayerNorm.forward that runs when the normalised
 * dimensions are not partitioned, nn/layernorm.py:310-319.  Arguments as above. */
int ddl_layer_norm(const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld,
                   const void* gamma, const void* beta, float eps,
                   void* y, int64_t ldy, float* mean_out, float* rstd_out,
                   void* stream);

/* ddl_ln_partial_stats and ddl_ln_normalize_affine in ONE launch, for a worker
 * whose peers' statistics are in memory before the launch: slots p != my_part
 * of part_stats[nparts][rows][2] are read, slot my_part is written (the pair
 * ddl_ln_partial_stats would store), and y, mean_out, rstd_out are what
 * ddl_ln_normalize_affine would return for the completed table, bit for bit.
 * The row stays in registers between the two halves, so x is read once.
 * The same reference lines, nn/layernorm.py:230-233, :246-247, :298-302, :309;
 * which of the two forms applies is decided by where the all-reduces of
 * :231 and :247 stand in time: a peer whose pair can only arrive after this
 * worker's own has been sent needs the two launches.
 * Limits: nparts <= 64; rows of at most 16384 columns, columns and pitches
 * multiples of 4, 4-element-aligned pointers (else DDL_E_UNSUPP: take the two
 * launches).  part_cols[my_part] must equal cols. */
int ddl_ln_stats_normalize(const void* x, int dtype, int64_t rows, int64_t cols,
                           int64_t ld, float* part_stats, int nparts,
                           int my_part, const int64_t* part_cols,
                           const void* gamma, const void* beta, float eps,
                           void* y, int64_t ldy, float* mean_out,
                           float* rstd_out, void* stream);

/* The fp32 forms of the first two (dtype = DDL_DT_F32). */
int ddl_ln_partial_stats_f32(const float* x, int64_t rows, int64_t cols,
                             int64_t ld, float* stats /*[rows][2]*/,
                             void* stream);
int ddl_ln_normalize_affine_f32(const float* x, int64_t rows, int64_t cols,
                                int64_t ld, const float* part_stats,
                                int nparts, const int64_t* part_cols,
                                const float* gamma, const float* beta,
                                float eps, float* y, int64_t ldy,
                                float* mean_out, float* rstd_out,
                                void* stream);

/* Backward of the LayerNorm shard: what autograd derives from the reference's
 * forward (nn/layernorm.py:230-247, 295-309, all-reduces included).  With
 * g = dy * gamma (gamma NULL = 1), xhat = (x - mean) * rstd (mean, rstd as
 * ddl_ln_normalize_affine returned them) and a = 1 / (P * columns of this
 * worker), P = workers sharing a row:
 *
 *   ddl_ln_bwd_partial   sums[r] = { sum_c g[r,c], sum_c g[r,c] xhat[r,c] }
 *                        over the LOCAL columns; the caller gathers the
 *                        pairs of the P workers into part_sums[P, rows, 2]
 *   ddl_ln_bwd_input     dx[r,c] = rstd[r] * ( g[r,c] - weight * (S1[r] +
 *                        xhat[r,c] * S2[r]) ), S = sum over the P pairs,
 *                        weight = a
 *   ddl_ln_bwd_params    dgamma[c] = sum_r dy[r,c] xhat[r,c],
 *                        dbeta[c]  = sum_r dy[r,c]   (either may be NULL);
 *                        `workspace`: device memory for at least 2 * cols
 *                        floats (up to 512 * cols are used), contents on
 *                        entry do not matter.
 *
 * dy, x, gamma, dx, dgamma and dbeta are of `dtype` (DDL_DT_F32, DDL_DT_BF16 or
 * DDL_DT_F16: autograd hands gradients over in the type of the tensors); mean,
 * rstd, the sums and the workspace are fp32, as is all arithmetic, and results
 * are rounded once when stored.  The _f32 forms are the same calls with
 * dtype = DDL_DT_F32. */
int ddl_ln_bwd_partial(const void* dy, const void* x, int dtype, int64_t rows,
                       int64_t cols, int64_t ld_dy, int64_t ld_x,
                       const float* mean, const float* rstd,
                       const void* gamma, float* sums, void* stream);
int ddl_ln_bwd_input(const void* dy, const void* x, int dtype, int64_t rows,
                     int64_t cols, int64_t ld_dy, int64_t ld_x,
                     const float* mean, const float* rstd,
                     const void* gamma, const float* part_sums, int nparts,
                     float weight, void* dx, int64_t ld_dx, void* stream);
int ddl_ln_bwd_params(const void* dy, const void* x, int dtype, int64_t rows,
                      int64_t cols, int64_t ld_dy, int64_t ld_x,
                      const float* mean, const float* rstd, void* dgamma,
                      void* dbeta, float* workspace,
                      int64_t workspace_elems, void* stream);
int ddl_ln_bwd_partial_f32(const float* dy, const float* x, int64_t rows,
                           int64_t cols, int64_t ld_dy, int64_t ld_x,
                           const float* mean, const float* rstd,
                           const float* gamma, float* sums, void* stream);
int ddl_ln_bwd_input_f32(const float* dy, const float* x, int64_t rows,
                         int64_t cols, int64_t ld_dy, int64_t ld_x,
                         const float* mean, const float* rstd,
                         const float* gamma, const float* part_sums, int nparts,
                         float weight, float* dx, int64_t ld_dx, void* stream);
int ddl_ln_bwd_params_f32(const float* dy, const float* x, int64_t rows,
                          int64_t cols, int64_t ld_dy, int64_t ld_x,
                          const float* mean, const float* rstd, float* dgamma,
                          float* dbeta, float* workspace,
                          int64_t workspace_elems, void* stream);

/* The same three results in two launches instead of four, for a caller that
 * wants dx and the parameter gradients (rows of a few hundred elements are
 * launch-bound, so this halves the time):
 *
 *   ddl_ln_bwd_partial_params   sums[] as ddl_ln_bwd_partial, and in the
 *                               same pass over dy and x the row-split
 *                               partial column sums, left in `workspace`
 *   ddl_ln_bwd_input_params     dx as ddl_ln_bwd_input, and in the same
 *                               launch dgamma / dbeta (either may be NULL)
 *                               from the partial sums in `workspace`
 *
 * Both calls take the same rows, cols, workspace and workspace_elems (at least
 * 2 * cols floats, up to 512 * cols are used); the second must follow the first
 * on the same stream.  Element types as above; _f32 forms likewise. */
int ddl_ln_bwd_partial_params(const void* dy, const void* x, int dtype,
                              int64_t rows, int64_t cols, int64_t ld_dy,
                              int64_t ld_x, const float* mean,
                              const float* rstd, const void* gamma,
                              float* sums, float* workspace,
                              int64_t workspace_elems, void* stream);
int ddl_ln_bwd_input_params(const void* dy, const void* x, int dtype,
                            int64_t rows, int64_t cols, int64_t ld_dy,
                            int64_t ld_x, const float* mean, const float* rstd,
                            const void* gamma, const float* part_sums,
                            int nparts, float weight, void* dx, int64_t ld_dx,
                            const float* workspace, int64_t workspace_elems,
                            void* dgamma, void* dbeta, void* stream);
/* dx, the row sums and the parameter gradients with ONE pass over dy and x, for
 * a worker whose share of the row sums completes them: it holds its rows whole
 * (nparts = 1, part_sums may be NULL: the backward of the reference's
 * torch.nn.functional.layer_norm branch, nn/layernorm.py:310-319), or the
 * other workers' pairs are in part_sums[nparts][rows][2] before the launch
 * (slots p != my_part are read, slot my_part is written).  Results as
 * ddl_ln_bwd_partial_params followed by ddl_ln_bwd_input_params; the second
 * launch only adds up the partial column sums (none when dgamma and dbeta are
 * both NULL).  workspace as above.  Limits: nparts <= 64, rows of at most 1024
 * columns, columns and pitches multiples of 4, pointers aligned to 4 elements
 * (else DDL_E_UNSUPP: take the two calls). */
int ddl_ln_bwd_one_pass(const void* dy, const void* x, int dtype, int64_t rows,
                        int64_t cols, int64_t ld_dy, int64_t ld_x,
                        const float* mean, const float* rstd, const void* gamma,
                        float* part_sums, int nparts, int my_part, float weight,
                        void* dx, int64_t ld_dx, float* workspace,
                        int64_t workspace_elems, void* dgamma, void* dbeta,
                        void* stream);
int ddl_ln_bwd_partial_params_f32(const float* dy, const float* x, int64_t rows,
                                  int64_t cols, int64_t ld_dy, int64_t ld_x,
                                  const float* mean, const float* rstd,
                                  const float* gamma, float* sums,
                                  float* workspace, int64_t workspace_elems,
                                  void* stream);
int ddl_ln_bwd_input_params_f32(const float* dy, const float* x, int64_t rows,
                                int64_t cols, int64_t ld_dy, int64_t ld_x,
                                const float* mean, const float* rstd,
                                const float* gamma, const float* part_sums,
                                int nparts, float weight, float* dx,
                                int64_t ld_dx, const float* workspace,
                                int64_t workspace_elems, float* dgamma,
                                float* dbeta, void* stream);

/* ------------------------------------------------------------------------ *
 * DistributedEmbedding shard gather
 * ------------------------------------------------------------------------ */

/* out[t, :] = (lo <= ids[t] < hi) ? weight[ids[t] - lo, :] : 0   for t < n_ids.
 * `weight` is [hi-lo, dim] row-major with row stride `ldw`; rows are moved as
 * opaque bytes (elem_size 1, 2, 4 or 8).  ids are int64 (ids_is_i64 = 1) or
 * int32.  With lo = 0 and hi = num_embeddings this is
 *   torch.nn.functional.embedding(input, weight)   nn/embedding.py:244-246;
 * a narrower window is the vocabulary-sharded variant whose misses give zero
 * rows.  An id outside [0, num_embeddings) is a caller error the kernel does
 * not detect beyond the window test. */
int ddl_embedding_gather(const void* weight, int64_t dim, int64_t ldw,
                         int elem_size, const void* ids, int ids_is_i64,
                         int64_t n_ids, int64_t lo, int64_t hi,
                         void* out, void* stream);

/* The max_norm step of torch.nn.functional.embedding(input, weight, padding_idx,
 * max_norm, norm_type, ...) (nn/embedding.py:244-246), which runs before the
 * lookup and changes the table in place: every row that some id of the window
 * [lo, hi) names and whose `norm_type`-norm (1, 2, +inf or any p > 0; formed in
 * fp32) exceeds max_norm is multiplied by max_norm / (norm + 1e-7), once per
 * row however often it is named.  `weight` is [hi-lo, dim] of `dtype`
 * (DDL_DT_F32, DDL_DT_BF16 or DDL_DT_F16) with row stride `ldw`; `flags` is a
 * workspace of hi-lo int32.  ids as in ddl_embedding_gather. */
int ddl_embedding_renorm(void* weight, int dtype, int64_t dim, int64_t ldw,
                         const void* ids, int ids_is_i64, int64_t n_ids,
                         int64_t lo, int64_t hi, float max_norm,
                         float norm_type, int32_t* flags, void* stream);

/* Adjoint of ddl_embedding_gather with respect to the table:
 *   dweight[r, :] = sum over t with ids[t] - lo == r and ids[t] != padding_idx
 *                   of dy[t, :]                        for every r in [0, hi-lo)
 * (what autograd derives for torch.nn.functional.embedding,
 * nn/embedding.py:244-246; padding_idx < 0 = none).  dtype = DDL_DT_BF16,
 * DDL_DT_F16 or DDL_DT_F32 for dy and dweight alike; sums are accumulated in fp32 in
 * ascending token order whatever the length of a row's token list, so the
 * result is the same on every run.  With scale_grad_by_freq != 0 each row's
 * sum is divided by the number of tokens that contributed to it
 * (torch.nn.functional.embedding's option of that name, nn/embedding.py:244-246).
 * Every element of dweight is written, so it needs no clearing.  `workspace`:
 * device memory for at least 3 (hi-lo) + 1 + n_ids int32 (token counts, bucket
 * cursors and bucket starts of the rows, then the buckets), contents on entry
 * do not matter. */
int ddl_embedding_backward(const void* dy, int dtype, int64_t dim, int64_t ld_dy,
                           const void* ids, int ids_is_i64, int64_t n_ids,
                           int64_t lo, int64_t hi, int64_t padding_idx,
                           int scale_grad_by_freq,
                           void* dweight, int64_t ld_dw, int32_t* workspace,
                           int64_t workspace_elems, void* stream);

/* ddl_embedding_backward without the workspace argument, for callers that
 * cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation).  No counterpart in the reference.
 * The counters and buckets live in a 4 MiB device array built into the library
 * (one copy per GPU, held until the process ends); the call allocates nothing
 * and frees nothing.  It fails with DDL_E_UNSUPP when
 *   3 (hi - lo) + 1 + n_ids > DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS.
 * All calls on one GPU share that array: calls that overlap in time on one GPU
 * (different streams or threads) race; calls on one stream are safe.  The
 * array's device address is looked up the first time a GPU is used, so make
 * that first call outside any stream capture.  Results are those of
 * ddl_embedding_backward. */
#define DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS 1048576
int ddl_embedding_backward_static(const void* dy, int dtype, int64_t dim, int64_t ld_dy,
                                  const void* ids, int ids_is_i64, int64_t n_ids,
                                  int64_t lo, int64_t hi, int64_t padding_idx,
                                  int scale_grad_by_freq,
                                  void* dweight, int64_t ld_dw, void* stream);

/* ------------------------------------------------------------------------ *
 * DistributedLinear shard GEMM (fp32 accumulate; operands and result bf16,
 * fp16 or fp32)
 * ------------------------------------------------------------------------ */

/* y[M, N] = x[M, K] . w[N, K]^T + bias[N]   (bias may be NULL).
 * x, w, y row-major with leading dimensions ldx, ldw, ldy (elements), all of
 * `dtype` (DDL_DT_BF16, DDL_DT_F16 or DDL_DT_F32), accumulation in fp32.
 * Replaces  self.sublinear(x)  nn/linear.py:103  and
 *   torch.nn.functional.linear(input, weight, bias)  nn/linear_ag.py:486.
 * The 16-bit types run on the tuned MFMA kernel and need K, ldx, ldw multiples
 * of 8 and x, w aligned to 16 bytes (DDL_E_ALIGN otherwise); fp32, the default
 * dtype of the reference's layers and of its tests
 * (tests/layers/test_linear.py:48-305), takes any K and pitch. */
int ddl_linear(const void* x, const void* w, const void* bias, void* y, int dtype,
               int64_t M, int64_t N, int64_t K,
               int64_t ldx, int64_t ldw, int64_t ldy, void* stream);

/* ddl_linear with dtype = DDL_DT_BF16. */
int ddl_linear_bf16(const void* x, const void* w, const void* bias, void* y,
                    int64_t M, int64_t N, int64_t K,
                    int64_t ldx, int64_t ldw, int64_t ldy, void* stream);

/* The product with both operands addressed by two strides each (elements):
 *   y[m, n] = sum_k a[m a_row_stride + k a_k_stride] b[n b_row_stride + k b_k_stride] + bias[n]
 * so that the adjoint of the shard (what autograd runs for ddl_linear:
 * dx = dy . w, dw = dy^T . x, torch's linear backward behind nn/linear.py:103)
 * needs no transposed copies:
 *   dx[M,K] = gemm(a = dy (N, 1),  b = w (1, K))       reduction over N
 *   dw[N,K] = gemm(a = dy (1, N),  b = x (1, K))       reduction over M
 * a, b, bias and y are of `dtype`; y is row-major with pitch ldy.
 * fp32: any strides (products of at least 64 tiles of 256 x 256 whose operands
 * have a unit stride, 16-byte alignment and a pitch that is a multiple of 4 run
 * on the tiled MFMA kernel, everything else on a slower general one; the result
 * is the same up to the order of the fp32 sums).  bf16 / fp16 (the MFMA kernel of ddl_linear, which reads an
 * operand that is contiguous along its rows through transposing LDS reads): each
 * operand needs one stride equal to 1, the other (its pitch) a multiple of 8, and
 * 16-byte alignment; an operand contiguous along k needs K % 8 == 0, one
 * contiguous along its rows needs a row count (M for a, N for b) that is a
 * multiple of 8 (DDL_E_ALIGN otherwise) and (K + 64) * pitch < 2^30 elements
 * (DDL_E_UNSUPP otherwise: transpose it with ddl_transpose_2d instead).
 * ddl_gemm_f32 is the fp32 form. */
int ddl_gemm(const void* a, int64_t a_row_stride, int64_t a_k_stride,
             const void* b, int64_t b_row_stride, int64_t b_k_stride,
             const void* bias, void* y, int dtype, int64_t ldy,
             int64_t M, int64_t N, int64_t K, void* stream);
int ddl_gemm_f32(const float* a, int64_t a_row_stride, int64_t a_k_stride,
                 const float* b, int64_t b_row_stride, int64_t b_k_stride,
                 const float* bias, float* y, int64_t ldy,
                 int64_t M, int64_t N, int64_t K, void* stream);

/* dst[c, r] = src[r, c] for r < rows, c < cols; 2-byte elements only
 * (elem_size = 2); ld_src >= cols, ld_dst >= rows.  For the operands of the
 * adjoint that ddl_gemm cannot read where they lie (row counts that are not
 * multiples of 8): transposed into a buffer whose pitch is padded with zeros,
 * they go through ddl_linear,
 *   dx[M,K] = linear(dy[M,N],   wT[K,N])      dw[N,K] = linear(dyT[N,M], xT[K,M]). */
int ddl_transpose_2d(const void* src, void* dst, int64_t rows, int64_t cols,
                     int64_t ld_src, int64_t ld_dst, int elem_size, void* stream);

/* out[c] = sum over r < rows of a[r, c], fp32 accumulation, rounded once to
 * `dtype` (bf16, fp16 or fp32: the type of a and out), for the bias gradient.
 * `workspace` is device memory for at least `cols` floats (up to 64 * cols are
 * used: one row of partial sums per row split); its contents on entry do not
 * matter.  ddl_colsum_bf16 is the bf16 form. */
int ddl_colsum(const void* a, int dtype, int64_t rows, int64_t cols, int64_t ld,
               void* out, float* workspace, int64_t workspace_elems, void* stream);
int ddl_colsum_bf16(const void* a, int64_t rows, int64_t cols, int64_t ld,
                    void* out, float* workspace, int64_t workspace_elems,
                    void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DISTDL_HIP_H */
