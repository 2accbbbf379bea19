/*
 * tf24.h -- C ABI of lib2by4_gfx950.so: the 2:4 semi-structured sparse hot path of
 * huyz2023/2by4-pretrain, hand-written for MI355X (gfx950 / CDNA4).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer (HIP); the one exception is `rand` in mode
 *     TF24_PRUNE_MVUE_SEEDED, which points to {seed, offset} in host memory
 *     (TF24_PRUNE_MVUE_SEEDED_DEVICE takes the pair from device memory).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Nothing here
 *     allocates, frees or synchronises: the caller owns every buffer, work is only enqueued.
 *   - Return value: TF24_OK or a negative tf24_status; tf24_last_error() returns a
 *     thread-local human readable message for the last failure on the calling thread.
 *   - A logical [m,k] matrix is described by (layout, ld):
 *       TF24_ROW_MAJOR element (r,c) at r*ld + c,   TF24_COL_MAJOR element (r,c) at c*ld + r.
 *   - "group" = 4 consecutive elements along k.  In the canonical compressed form the values are
 *     row-major [m, k/2] and the metadata is the nibble stream: for each group
 *     pos0 | pos1<<2 (pos0 < pos1 = positions of the two kept elements), packed LSB-first
 *     into int16 [m, k/16] for 16-bit values or int32 [m, k/32] for 8-bit values.  One int16
 *     is exactly the index operand of one lane of V_SMFMAC_F32_16X16X64_{F16,BF16}; one int32
 *     that of V_SMFMAC_F32_16X16X128_FP8_FP8.
 *
 * Each entry point names the reference interface (huyz2023/2by4-pretrain) it replaces.
 */
#ifndef TF24_H
#define TF24_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  TF24_OK = 0,
  TF24_ERR_SHAPE = -1,   /* dimension not supported (multiples, minima) */
  TF24_ERR_DTYPE = -2,   /* dtype or dtype combination not supported */
  TF24_ERR_STRIDE = -3,  /* leading dimension / alignment not supported */
  TF24_ERR_LAUNCH = -4,  /* HIP reported an error at launch */
  TF24_ERR_ARG = -5      /* null pointer, bad enum, contradictory arguments */
} tf24_status;

typedef enum {
  TF24_F32 = 0,
  TF24_F16 = 1,
  TF24_BF16 = 2,
  TF24_E4M3 = 3, /* OCP float8 e4m3fn */
  TF24_E5M2 = 5, /* OCP float8 e5m2 (IEEE-like: infinities, NaN) */
  TF24_U8 = 4,   /* bytes: bool masks (nonzero = kept) */
  TF24_I8 = 6,   /* signed 8-bit integer values and operands (integer matmul, TF24_I32 results) */
  TF24_I32 = 7   /* 32-bit integer matmul results and bias */
} tf24_dtype;

typedef enum { TF24_ROW_MAJOR = 0, TF24_COL_MAJOR = 1 } tf24_layout;

typedef enum {
  TF24_PRUNE_MAGNITUDE = 0, /* keep the 2 largest |x| per group, ties -> larger index */
  TF24_PRUNE_MASK = 1,      /* keep what a supplied mask says */
  TF24_PRUNE_MVUE = 2,      /* MVUE24 sampling from a supplied U(0,1) tensor of the dense shape */
  TF24_PRUNE_MVUE_PACKED = 3, /* the same with only the uniforms that are used: a [m, k/2] tensor */
  TF24_PRUNE_MVUE_SEEDED = 4, /* MVUE24 with uniforms generated in the kernel: `rand` points to two uint64
                                 values {seed, offset} in HOST memory (read during the call).  The uniforms
                                 are exactly those tf24_mvue_uniforms writes for the same seed and offset. */
  TF24_PRUNE_MVUE_SEEDED_DEVICE = 5 /* the same with {seed, offset} in DEVICE memory (8-byte aligned), read by the
                                 kernel when it runs; behind the conversion the call enqueues offset += 4 on
                                 the same stream, as a host-side generator advances per sampling call.  A call
                                 recorded into a HIP graph therefore draws fresh uniforms on every replay
                                 (the host form would replay the values it read at capture). */
} tf24_prune_mode;

/* GELU is the exact (erf) form, torch.nn.functional.gelu's default; the reference's epilogues stop at SILU */
typedef enum { TF24_ACT_NONE = 0, TF24_ACT_RELU = 1, TF24_ACT_SILU = 2, TF24_ACT_GELU = 3 } tf24_activation;

/*
 * Storage of a compressed [m,k] matrix (values + metadata).
 *   CANONICAL  values [m, k/2] row-major, metadata [m, k/8 bytes] row-major (the interchange form).
 *   PANEL      the SMFMAC-native form the matmul streams.  Values: the k axis is cut into panels of
 *              KP = 128/sizeof(value) dense columns (64 for 16-bit values, 128 for 8-bit ones), i.e. the
 *              64 value bytes one row contributes to one LDS stage: [k/KP][m][64 bytes], the bytes of a
 *              row inside a panel being the canonical ones.  Metadata: the 4-byte word of 32 dense
 *              columns (8 nibbles, canonical order) of every row, column-block-major: [k/32][m][4 bytes].
 *              A 256-row tile of one stage is then one contiguous 16 KB run of values and 2 (4) contiguous
 *              1 KB runs of metadata, all copied to LDS with full-line GLOBAL_LOAD_LDS_DWORDX4, and the
 *              metadata lands in the order the matrix instructions' index operands are read in.
 *   CUTLASS    the form the reference stores and hands to its matmul binding: values as CANONICAL, metadata
 *              words (int16 for 16-bit values, int32 for 8-bit ones) permuted by CUTLASS's reorder_meta and
 *              stored ColumnMajorInterleaved<2> (sparse/csrc/mySparseSemiStructuredLinear_cuda.cu:826-851; the
 *              gather form of sparse/_semi_structured_conversions.py:178-213): canonical word (r, c) of the
 *              [m, k/16 | k/32] word matrix goes to row r/G*G + (r%8)*I + (r%G)/8 with (G, I) = (32, 4) for
 *              int16 and (16, 2) for int32 words, is swapped inside 2 x 2 blocks (even row, odd column <->
 *              odd row, even column), and lands at word (c'/2)*2m + 2r' + c'%2.  This is what
 *              SparseSemiStructuredTensor.indices() returns in the reference (sparse/semi_structured.py:536-546).
 *              Accepted as an input of tf24_repack_to, tf24_decompress and tf24_spmm (which then runs its
 *              general kernel: repack once to PANEL for speed) and produced by tf24_repack_to.
 */
typedef enum { TF24_COMPRESSED_CANONICAL = 0, TF24_COMPRESSED_PANEL = 1, TF24_COMPRESSED_CUTLASS = 2 } tf24_compressed_layout;

/* Library version string, e.g. "tf24 0.1.0 gfx950". Host only. */
const char* tf24_version(void);

/* Message of the last failing call on this thread ("" if none). Host only. */
const char* tf24_last_error(void);

/*
 * Dense -> 2:4 prune + compress.
 * Replaces sparse_semi_structured_from_dense_triton and its two Triton kernels
 * (sparse/_semi_structured_conversions.py:431-661, :664-1069, launcher :1072-1132),
 * called from SparseSemiStructuredTensor.__init__ (sparse/semi_structured.py:244-245).
 *   dense      [m,k] in_dtype (F32|F16|BF16), (layout, ld)
 *   mode       MAGNITUDE | MASK (mask required) | MVUE, MVUE_PACKED (rand required)
 *   mask       [m,k] mask_dtype (U8|F16|BF16|F32), nonzero = kept, same layout, leading dim mask_ld
 *   rand       [m,k] F32 uniforms in [0,1), same layout, leading dim rand_ld; group g of row r
 *              uses rand[r,4g] and rand[r,4g+1]; mode MVUE_PACKED: [m,k/2], group g uses
 *              rand[r,2g] and rand[r,2g+1] (half the bytes to generate and to read)
 *   values     m*k/2 elements of out_dtype (F16|BF16|E4M3|E5M2) in out_layout
 *   meta       m*k/8 bytes in out_layout (canonical: int16 [m,k/16] for 16-bit values, int32 [m,k/32] for E4M3|E5M2)
 * Shape rules (sparse/semi_structured.py:24-30,188-200): m % 32 == 0, k % 64 == 0 for 16-bit
 * values, k % 128 == 0 for 8-bit values.
 */
int tf24_prune_compress(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                        int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                        const float* rand, int64_t rand_ld,
                        void* values, int out_dtype, void* meta, int out_layout, void* stream);

/*
 * The packed uniforms [m, k/2] of TF24_PRUNE_MVUE_SEEDED as a tensor: Philox4x32-10 with key = seed and
 * counter = {row * (k/8) + c/4, offset} yields columns 4*(c/4) .. 4*(c/4)+3 of row `row`; each word gives
 * (word & 0xffffff) * 2^-24 in [0, 1).  The reference seeds an in-kernel Philox from Python's `random`
 * (sparse/_semi_structured_conversions.py:536-542, :1076), which is not reproducible; this one is, from
 * (seed, offset).  out: float32, TF24_ROW_MAJOR [m, k/2] with leading dimension ld >= k/2, or
 * TF24_COL_MAJOR (element (r, c) at c*ld + r, ld >= m).  k % 8 == 0.
 */
int tf24_mvue_uniforms(uint64_t seed, uint64_t offset, int64_t m, int64_t k, int layout, float* out, int64_t ld,
                       void* stream);

/*
 * tf24_prune_compress of a column-major matrix that also returns its row sums,
 *     rowsum[r] = sum_c dense[r, c]   (the unpruned input, added in float32, one rounding to rowsum_dtype).
 * Replaces the pair the training layer's backward issues on the same gradient (README.md:190-197):
 *     to_sparse_semi_structured(grad_output.t(), MVUE24=True)   and   grad_bias = grad_output.sum(0)
 * -- with dense = grad_output^T (column-major view) the row sums are the bias gradient, from the read
 * the compression makes anyway.  Arguments as tf24_prune_compress, plus
 *   rowsum     m elements of rowsum_dtype (F32|F16|BF16)
 *   workspace  tf24_prune_compress_rowsum_workspace_bytes(m, k) bytes of float32 scratch (one partial
 *              sum per row and block of 128 columns; added in a fixed order: deterministic)
 * layout must be TF24_COL_MAJOR (a row of a row-major matrix is contiguous and needs no fusion);
 * int8 input is not supported.
 */
int tf24_prune_compress_rowsum(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                               int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                               const float* rand, int64_t rand_ld,
                               void* values, int out_dtype, void* meta, int out_layout,
                               void* rowsum, int rowsum_dtype, void* workspace, int64_t workspace_bytes, void* stream);
int64_t tf24_prune_compress_rowsum_workspace_bytes(int64_t m, int64_t k);

/*
 * tf24_prune_compress_rowsum for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and so cannot bring a workspace.  No counterpart in
 * the reference.  Same arguments and bit-identical results; the partial row sums go to a fixed 4 MiB
 * array inside the library's device image instead (tf24_prune_compress_rowsum_static_max_bytes()), which
 * every GPU the library runs on holds until the process ends.  The call allocates and frees nothing.
 *   limit   tf24_prune_compress_rowsum_workspace_bytes(m, k) <= 4 MiB, i.e. m * ceil(k / 128) <= 2^20
 *           (config 4's 3072 x 12288 gradient needs 1.2 MiB); larger shapes return TF24_ERR_SHAPE.
 *   sharing every call on a GPU uses that GPU's one array: calls that overlap on one GPU (different
 *           streams, or threads on the same device) race on it and must be serialised by the caller.
 *           Nothing in the array has to start at zero: each call writes every partial sum it reads.
 */
int tf24_prune_compress_rowsum_static(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                      int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                                      const float* rand, int64_t rand_ld,
                                      void* values, int out_dtype, void* meta, int out_layout,
                                      void* rowsum, int rowsum_dtype, void* stream);
int64_t tf24_prune_compress_rowsum_static_max_bytes(void);

/*
 * Mask-driven 2:4 compression of W and of W^T from ONE read of W and of the mask:
 *   (values, meta)      = tf24_prune_compress(W   [m,k] row-major,          mode MASK, mask)
 *   (values_t, meta_t)  = tf24_prune_compress(W^T [k,m] (W read by columns), mode MASK, mask^T)
 * bit for bit.  Replaces the pair of conversions the training layer issues once per optimizer step,
 *   to_sparse_semi_structured(w, mask=w.mask) and to_sparse_semi_structured(w.T, mask=w.mask.T)
 * (README.md:165-166; each one the `PRUNE == 'mask'` branch of
 * sparse/_semi_structured_conversions.py:517-533), which read W and the mask twice.
 *   dense    [m,k] row-major, leading dimension ld; F32|F16|BF16
 *   mask     [m,k] row-major, leading dimension mask_ld; U8 (bool) or F32|F16|BF16, nonzero = keep.
 *            Any mask is accepted (groups with other than two kept elements follow the 16-row
 *            table in either direction); a transposable mask makes both results exact 2:4 copies.
 *   values, meta      m*k/2 elements of out_dtype and m*k/8 bytes: W compressed along k
 *   values_t, meta_t  the same sizes: W^T [k,m] compressed along m
 *   out_layout        TF24_COMPRESSED_CANONICAL or TF24_COMPRESSED_PANEL, for both results
 * Shape rules: both directions must satisfy tf24_prune_compress's, so m and k are multiples of 64
 * for 16-bit values and of 128 for 8-bit values.
 */
int tf24_prune_compress_dual(const void* dense, int in_dtype, int64_t ld, int64_t m, int64_t k,
                             const void* mask, int mask_dtype, int64_t mask_ld,
                             void* values, void* meta, void* values_t, void* meta_t,
                             int out_dtype, int out_layout, void* stream);
int tf24_prune_compress_dual_validate(int in_dtype, int64_t ld, int64_t m, int64_t k, int mask_dtype, int64_t mask_ld,
                                      int out_dtype, int out_layout);

/* The argument checks of tf24_prune_compress without touching the GPU (pointers are only
 * tested for NULL-ness through the has_* flags). Host only. */
int tf24_prune_compress_validate(int in_dtype, int layout, int64_t ld, int64_t m, int64_t k, int mode,
                                 int has_mask, int mask_dtype, int64_t mask_ld, int has_rand, int64_t rand_ld,
                                 int out_dtype);

/*
 * Compressed -> dense.  Replaces _sparse_semi_structured_to_dense_kernel
 * (sparse/_semi_structured_conversions.py:1163-1274) used by SparseSemiStructuredTensor.to_dense
 * (sparse/semi_structured.py:554-572).  values / meta in `layout` (any of the three; CUTLASS is the form
 * the reference's own decompression starts from, :217-290), dense_out [m,k] row-major contiguous of the
 * same dtype.
 */
int tf24_decompress(const void* values, int dtype, const void* meta, int layout, int64_t m, int64_t k,
                    void* dense_out, void* stream);

/*
 * Canonical <-> panel storage of a compressed operand (out of place).  The reference keeps one
 * storage form, the CUTLASS-reordered one made by _sparse_semi_structured_from_dense_triton
 * (sparse/_semi_structured_conversions.py:1072-1132); a caller holding canonical values and
 * metadata converts once to the panel form the tiled matmul streams.
 *   from_layout  the layout of values_in / meta_in; the outputs get the other one
 *   k % 64 == 0 (16-bit values) / k % 128 == 0 (8-bit)
 */
int tf24_repack(const void* values_in, const void* meta_in, int dtype, int64_t m, int64_t k, int from_layout,
                void* values_out, void* meta_out, void* stream);

/*
 * Storage conversion between any two of CANONICAL, PANEL and CUTLASS (out of place, from_layout != to_layout).
 * With from_layout CUTLASS this is the import of a compressed operand as the reference stores it -- the
 * (weight, meta) pair its matmul binding takes (sparse/sparse_semi_structured_linear.py:4-5) and
 * SparseSemiStructuredTensor.values() / indices() return (sparse/semi_structured.py:526-546); with to_layout
 * CUTLASS it is the reference's reordering step itself (sparse/_semi_structured_conversions.py:178-213,
 * Triton :639-661 and :1047-1069).  m % 32 == 0; k % 64 == 0 (16-bit values) / k % 128 == 0 (8-bit).
 * values_out NULL: only the metadata is converted (what indices() needs; the values of CANONICAL and CUTLASS are
 * the same bytes anyway).  meta_out NULL, between CANONICAL and PANEL: only the values (what values() needs).
 */
int tf24_repack_to(const void* values_in, const void* meta_in, int dtype, int64_t m, int64_t k, int from_layout,
                   int to_layout, void* values_out, void* meta_out, void* stream);

/*
 * Transposable 4x4 mask search over the 90 row-and-column 2:4 patterns.
 * Replaces _to_transposable_sparse_semi_structured_kernel and its launcher
 * (sparse/transposable_semi_structured.py:8-47, :50-94) behind TransposableSparse.forward (:198-200).
 *   dense [m,k] dtype (F32|F16|BF16), (layout, ld); m % 32 == 0, k % 64 == 0, ld % 8 == 0,
 *   16-byte aligned base
 *   sparse_out (may be NULL) dense*mask, same dtype/layout/ld;  mask_out bytes (0/1), same layout/ld
 */
int tf24_transposable_mask(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                           int use_abs, void* sparse_out, uint8_t* mask_out, void* stream);
int tf24_transposable_mask_validate(int dtype, int layout, int64_t ld, int64_t m, int64_t k);

/*
 * Dense-shaped 2:4 operators: outputs have the dense dtype/layout/ld and are written completely
 * (zeros at dropped positions).  k % 4 == 0 (row-major: k % 8 == 0 for 16-bit types).
 *   tf24_soft_threshold24  S-STE soft threshold, replaces _soft_threshold24_triton
 *                          (sparse/triton_ops.py:157-227, math sparse/utils.py:72-90)
 *   tf24_sparse24_dense    magnitude pruning, replaces _sparse24_triton (sparse/triton_ops.py:84-154)
 *   tf24_mvue24_dense      MVUE24 with supplied uniforms, replaces _MVUE24_approx_triton
 *                          (sparse/triton_ops.py:10-81); mask_out unused (pass NULL)
 */
int tf24_soft_threshold24(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                          void* sparse_out, void* mask_out, void* stream);
int tf24_sparse24_dense(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                        void* sparse_out, void* mask_out, void* stream);
int tf24_mvue24_dense(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                      const float* rand, int64_t rand_ld, void* sparse_out, void* stream);

/*
 * AdamW step with the masked decay folded in: one pass instead of masked_add_ followed by the
 * optimizer.  Follows the reference's optimizer (sparse/adamw.py:70-113: decoupled weight decay,
 * bias-corrected moments, no amsgrad) with the decay of sparse/decay.py:27-37 applied to the
 * gradient first, as the training loop of README.md:205-213 does; the gradient is only read.
 *   p, exp_avg, exp_avg_sq F32 in place; grad F32|F16|BF16; mask U8|F32|F16|BF16 or NULL (no decay)
 *   step = number of this update, starting at 1
 */
int tf24_adamw_masked_decay(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                            const void* mask, int mask_dtype, int64_t n, double lr, double beta1, double beta2,
                            double eps, double weight_decay, double decay_alpha, int64_t step, void* stream);
/*
 * The same update with the number of the update in device memory (int64, >= 1, advanced by the caller in
 * stream order before the call): the form a training step recorded into a HIP graph needs, where a host
 * number would be frozen at the recording -- what torch's optimizers call capturable; the reference's optimizer
 * (sparse/adamw.py:83-84) keeps the count as a host integer only.  The bias corrections 1 - beta^step are formed on
 * the device, in double like the host form's.
 */
int tf24_adamw_masked_decay_device_step(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                        const void* mask, int mask_dtype, int64_t n, double lr, double beta1,
                                        double beta2, double eps, double weight_decay, double decay_alpha,
                                        const int64_t* step, void* stream);

/*
 * The update of the STEP optimizer, one pass per tensor: replaces the body of AdamW_STEP.step
 * (sparse/adamw_step.py:84-148; the recipe is README.md:271-329).  Decoupled weight decay and the two
 * moments as in AdamW; then
 *   phase 1 (precond_variance == NULL): denom = sqrt(v) / sqrt(bc2) + eps, of max(max_exp_avg_sq, v)
 *            when max_exp_avg_sq is given (amsgrad; updated in place);
 *   phase 2 (precond_variance given: the variance frozen when the optimizer switched phases, :186-194):
 *            denom = sqrt(precond_variance) + eps^(3/4)                               (:131-135)
 *   p += -(lr / bc1) * exp_avg / denom.
 * z_option 1 | 2 with z_partial: the terms |v_t - v_{t-1}| (1) or log|v_t - v_{t-1}| (2) of the
 * variance-change statistic Z_t (:124-129, :152-158) are summed per block of 1024 elements into
 * z_partial[0 .. tf24_adamw_step_partials(n)); the caller adds the partial sums of all tracked
 * tensors and divides by their element count (option 2: then exponentiates).  z_option 0 and
 * z_partial NULL: no statistic.  p, moments, precond_variance float32; grad F32|F16|BF16; step >= 1.
 */
int tf24_adamw_step(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                    float* max_exp_avg_sq, const float* precond_variance, int64_t n,
                    double lr, double beta1, double beta2, double eps, double weight_decay, int64_t step,
                    float* z_partial, int z_option, void* stream);
int64_t tf24_adamw_step_partials(int64_t n);

/*
 * Masked decay, in place: grad[i] += alpha * p[i] where mask[i] == 0.
 * Replaces masked_add_kernel / masked_add_ (sparse/decay.py:7-37).  Flat over n elements
 * (the reference requires identical strides and indexes storage linearly).
 *   grad F32|F16|BF16, p F32|F16|BF16, mask U8|F32|F16|BF16
 */
int tf24_masked_add(void* grad, int grad_dtype, const void* p, int p_dtype, const void* mask, int mask_dtype,
                    int64_t n, float alpha, void* stream);

/*
 * 2:4 sparse x dense matmul on SMFMAC, float32 accumulation:
 *     C[i,j] = act( sum_k A[i,k] * B(k,j) + bias ),   A sparse [n_sparse, k], compressed.
 * Replaces sparse.cutlass.my_sparse_semi_structured_linear
 * (sparse/csrc/mySparseSemiStructuredLinear_cuda.cu:498-817, CUTLASS SparseGemm :61-76),
 * bound at sparse/sparse_semi_structured_linear.py:4-5.
 *   a_values, a_meta  the compressed operand in a_layout (PANEL: the fast kernels; CANONICAL and CUTLASS -- the
 *              reference's own storage, .cu:826-851 -- run the general kernel); dtype F16|BF16|E4M3|E5M2|I8 (B has the same dtype).
 *              I8 is the integer product of .cu:594-637: int32 accumulation, out_dtype and bias I32,
 *              activation none or ReLU, scale 1; every other dtype accumulates in float32 and takes
 *              out_dtype F16|BF16|F32 with a bias of that type
 *   b          dense operand, n_dense "columns" j: b_layout TF24_ROW_MAJOR means B is stored
 *              [n_dense, k] (k contiguous, element (k,j) at j*ldb + k: the X of X.W^T);
 *              TF24_COL_MAJOR means stored [k, n_dense] (element (k,j) at k*ldb + j)
 *   c          output; c_layout TF24_ROW_MAJOR stores C[i,j] at i*ldc + j ([n_sparse,n_dense]);
 *              TF24_COL_MAJOR stores it at j*ldc + i ([n_dense,n_sparse]: the Y of X.W^T)
 *   bias       NULL or [n_sparse] of out_dtype's float family (added per sparse row i)
 *   scale      multiplies the accumulator before bias (1.0 for 16-bit; scale_a*scale_b for fp8)
 *   workspace  NULL, or scratch of workspace_bytes for k-split partial tiles: products whose output
 *              tiles cannot fill the GPU (k-heavy shapes such as dW) are split along k and reduced in
 *              a second launch.  tf24_spmm_workspace_bytes() gives the size that enables every split
 *              the heuristic would take (0 = the shape is never split).  Deterministic either way.
 * Shape rules (.cu:101-109): n_sparse % 32 == 0, k % 64 == 0 (16-bit) / 128 (8-bit),
 * n_dense % 8 == 0 (16-bit) / 16 (8-bit).  Leading dimensions: ldb a multiple of 8 (16-bit) / 16 (8-bit)
 * elements and at most 16 MiB per row (a tile's rows are addressed by 32-bit offsets), ldc a multiple of 8 for
 * 16-bit outputs and of 4 for 32-bit ones (16-byte row segments); b, c, a_values 16-byte aligned, a_meta 16-byte
 * aligned in panel form (8 in canonical form, 4 in CUTLASS form).
 */
int tf24_spmm(const void* a_values, const void* a_meta, int a_layout, int dtype, int64_t n_sparse, int64_t k,
              const void* b, int b_layout, int64_t ldb, int64_t n_dense,
              void* c, int out_dtype, int c_layout, int64_t ldc,
              const void* bias, float scale, int activation, void* workspace, int64_t workspace_bytes, void* stream);
int64_t tf24_spmm_workspace_bytes(int dtype, int64_t n_sparse, int64_t k, int64_t n_dense);

/*
 * GELU-GLU: the last dimension of `in` [rows, cols] holds [x | gate] (cols/2 each);
 *     out[r, c] = x[r, c] * 0.5 * gate * (1 + tanh(sqrt(2/pi) * (gate + 0.044715 * gate^3))),  c < cols/2
 * and its backward pass
 *     grad_in[r, c]          = grad_out[r, c] * gelu_tanh(gate)
 *     grad_in[r, cols/2 + c] = grad_out[r, c] * x * d gelu_tanh(gate) / d gate.
 * Replaces the Triton kernels of sparse/GELUglu.py (forward :16-47 and :51-80, backward :83-153;
 * launchers :156-236).  Arithmetic is float32 with one rounding to `dtype` (F32|F16|BF16); the
 * reference computes in the storage type.
 *   layout  TF24_ROW_MAJOR: element (r, c) at r*ld + c (the reference's stride[-1] == 1 path);
 *           TF24_COL_MAJOR: at c*ld + r (its "fall back to 2D" path for transposed storage).
 *           `out` / `grad_out` are [rows, cols/2], `grad_in` is [rows, cols], in the same layout.
 * cols must be even.  16-byte accesses are used when the extents, leading dimensions and pointers
 * allow (multiples of 8 elements, 16-byte aligned); any other shape runs element-wise.
 */
int tf24_gelu_glu_forward(const void* in, int dtype, int layout, int64_t ld_in, int64_t rows, int64_t cols,
                          void* out, int64_t ld_out, void* stream);
int tf24_gelu_glu_backward(const void* grad_out, int64_t ld_grad_out, const void* in, int dtype, int layout,
                           int64_t ld_in, int64_t rows, int64_t cols, void* grad_in, int64_t ld_grad_in,
                           void* stream);

/*
 * out[c, r] = in[r, c] for 2-byte (F16|BF16) and 1-byte (E4M3|E5M2|U8) elements; in [rows, cols] with
 * leading dimension ld_in, out [cols, rows] with ld_out.  No counterpart in the reference (CUTLASS
 * reads either operand layout): it feeds tf24_spmm's fast kernel, which wants an 8-bit dense operand
 * with k contiguous, when `S @ dense` arrives with a row-major dense (16-bit operands are read
 * k-strided by the fast kernel itself and need no copy).
 * rows, cols and leading dimensions must be multiples of 16 bytes worth of elements.
 */
int tf24_transpose(const void* in, int dtype, int64_t ld_in, int64_t rows, int64_t cols, void* out, int64_t ld_out,
                   void* stream);
int tf24_spmm_validate(int dtype, int64_t n_sparse, int64_t k, int b_layout, int64_t ldb, int64_t n_dense,
                       int out_dtype, int c_layout, int64_t ldc, int activation);

#ifdef __cplusplus
}
#endif
#endif /* TF24_H */
