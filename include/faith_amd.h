/*
 * faith_amd.h -- C ABI of the MI355X (gfx950) forward bound-propagation kernels.
 *
 * Each entry point takes raw DEVICE pointers to contiguous fp32 arrays, plain
 * ints / floats, and a HIP stream handle passed as void* (NULL = the default
 * stream).  Launches are asynchronous on that stream.  Nothing is allocated or
 * freed; the caller owns every buffer, inputs and outputs alike (as in the
 * reference, Transformer_Verification_Code/Verifiers/Bounds.py:1270-1277).
 *
 * Return value: FAITH_OK (0) or a negative FAITH_ERR_* code.  Nothing aborts.
 * faith_last_error() returns a thread-local message for the last failure.
 *
 * Conventions shared by all entry points
 *   lw, uw   coefficient arrays; "natural" layout [rows, dim_in, dim_out]
 *            (Bounds.py:293-297) or "transposed" layout [rows, dim_out, dim_in]
 *            (what the reference's CUDA adapters pass, Bounds.py:1210-1211).
 *   lb, ub   constant terms [rows, dim_out].
 *   rows     batch * length; every op here is independent across rows.
 *   q        dual-norm selector FAITH_Q_*  (q = 1/(1-1/p), Bounds.py:277).
 *   words    number of equal blocks of dim_in that are normed separately and
 *            summed (perturbed_words, Bounds.py:319-326).
 */
#ifndef FAITH_AMD_H
#define FAITH_AMD_H

#ifdef __cplusplus
extern "C" {
#endif

#define FAITH_OK                0
#define FAITH_ERR_NULL         -1   /* a required pointer is NULL                    */
#define FAITH_ERR_SHAPE        -2   /* a dimension is non-positive or inconsistent   */
#define FAITH_ERR_UNSUPPORTED  -3   /* valid request this build has no kernel for    */
#define FAITH_ERR_ALIGN        -4   /* pointer not 4-byte aligned                    */
#define FAITH_ERR_LAUNCH       -5   /* HIP reported an error at launch               */

#define FAITH_Q_1    1   /* p = inf : sum of magnitudes  */
#define FAITH_Q_2    2   /* p = 2   : Euclidean norm     */
#define FAITH_Q_INF  0   /* p = 1   : largest magnitude  */
/* Any other p (the reference accepts every p, Bounds.py:277): pass the IEEE-754 bits of the dual
 * exponent q = 1 / (1 - 1/p), 1 < q < inf, in the int (e.g. memcpy from a float). */

#define FAITH_LAYOUT_NATURAL     0
#define FAITH_LAYOUT_TRANSPOSED  1

const char *faith_last_error(void);
/* Version of this interface; a binder compares it with the header it was built against.
 *   1: first interface.
 *   2: faith_dot_product_verification_QK and _V take `int layout` in front of `stream` (a caller built against
 *      version 1 would pass its stream where the layout goes). */
#define FAITH_ABI_VERSION 2
int faith_version(void);

/*
 * Kernel-variant selection for tuning runs (no counterpart in the reference, whose tile sizes
 * are compile-time: HandTunedKernels/matmul_config.h).  value 0 restores the built-in choice.
 * Kept per calling thread: a value set by one thread selects the variants of that thread's later calls only, so
 * threads that tune, or that apply a tuning table around their launches, do not disturb each other.  Every variant
 * of an operator meets the same tolerance; variants that sum in another order differ in the last bits.
 */
#define FAITH_TUNE_ACT_VARIANT   0   /* tile shape of the natural-layout relaxation kernels; 8 / 12 / 7 force the one-tile register-resident kernel with four wavefronts / sixteen wavefronts / sixteen wavefronts and non-temporal loads, 15 the persistent two-tile kernel; 0: eight wavefronts, two workgroups per CU (three for tanh), whole rows of the object dealt to the XCDs; 11 / 13 the four-wavefront shapes of concretize */
#define FAITH_TUNE_GEMM_VARIANT  1   /* macro-tile of the sign-split GEMM: 1 = 64x64, 2 = 128x128, 3 = 128x64, 4 = 64x128, 5 = 32x32 with K split over the wavefronts (dim_out % 32 == 0); 6 = faith_matmul_concretize_verification takes its one-launch kernel whenever the shape allows; 7 = it keeps layer and concretize apart; 8 = as 6, with 32x32 blocks also where the reduction is short enough for 16x16 blocks */
#define FAITH_TUNE_DOT_VARIANT   2   /* dot product: 1 = 128x64 persistent tiles with run-time extents (also where the straight-line instantiations for reductions of 32 / 64 / 128 would be taken), 2 = one 32x32 block per wavefront (short sequences only), 3 = transposed layout: the vector-ALU kernel also where the MFMA kernels apply; 4 = compact scores: the rows of the perturbed positions on the vector-ALU kernel also where the matrix-unit kernel takes them */
#define FAITH_TUNE_DOT_COORDS    3   /* dot product, 32x32 kernel: perturbation coordinates per wavefront, 1..16 */
#define FAITH_TUNE_CONV_VARIANT  4   /* convolution: 1 = the general kernel (run-time extents) for every layer; 2 = tiles in the plain order (not whole images per XCD); 3 = 2 x 2 blocks per wavefront also for short reductions */
#define FAITH_TUNE_COUNT         5
int faith_tune_set(int knob, int value);

/*
 * Plain device-to-device copy of n floats (n % 4 == 0, 16-byte aligned).  Measurement aid with no
 * counterpart in the reference: the yardstick for the HBM-bound kernels and the known-size
 * kernel that hardware byte counters are calibrated against.
 */
int faith_copy_f32(const float *src, float *dst, long long n, void *stream);

/*
 * Shader clock under matrix load, in MHz, one value per workgroup in mhz[0 .. workgroups-1]: every
 * workgroup issues 16 * iterations fp32 MFMAs per wavefront on all four SIMDs and divides the
 * shader-cycle counter by the constant 100 MHz counter.  Measurement aid with no counterpart in
 * the reference: the clock at which the MFMA peak has to be priced on the machine at hand.
 */
int faith_mfma_clock(float *mhz, int workgroups, int iterations, void *stream);

/*
 * Dual-norm concretization.  Replaces Bounds.concretize (Bounds.py:311-326) and the
 * CUDA `concretize` kernel (HandTunedKernels/dot_product_verification.cu:47-105).
 *   l[r,j] = lb[r,j] - eps * sum_w ||lw[r, block w, j]||_q
 *   u[r,j] = ub[r,j] + eps * sum_w ||uw[r, block w, j]||_q
 */
int faith_concretize(const float *lb, const float *ub, const float *lw, const float *uw,
                     float *l, float *u,
                     int rows, int dim_in, int dim_out,
                     float eps, int q, int words, int layout, void *stream);

/*
 * ReLU relaxation fused with concretization.  Replaces call_relu_verification
 * (HandTunedKernels/kernel.cpp:7-20, relu_verification.cu:134-147) with the arithmetic of
 * Bounds.ori_relu (Bounds.py:921-963).  `epsilon` is the perturbation radius, as in the
 * reference signature.  l_out / u_out may be NULL; when given they receive the concrete
 * pre-activation interval the relaxation was built from.
 */
int faith_relu_verification(const float *src_lb, const float *src_ub,
                            const float *src_lw, const float *src_uw,
                            float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                            float *l_out, float *u_out,
                            int length, int dim_in, int dim_out, float epsilon,
                            int q, int words, int layout, void *stream);

/*
 * tanh relaxation fused with concretization.  Replaces call_tanh_verification
 * (kernel.cpp:22-35, tanh_verification.cu:196-209) with the arithmetic of
 * Bounds.ori_tanh (Bounds.py:1027-1103): tangent / chord lines and two 10-step bisections.
 */
int faith_tanh_verification(const float *src_lb, const float *src_ub,
                            const float *src_lw, const float *src_uw,
                            float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                            float *l_out, float *u_out,
                            int length, int dim_in, int dim_out, float epsilon,
                            int q, int words, int layout, void *stream);

/*
 * Any unary relaxation, selected by `op`; same arguments as the two entries above.  The reference
 * has no CUDA entry for the last four: they replace the PyTorch methods Bounds.exp
 * (Bounds.py:970-1003), Bounds.reciprocal (:1136-1161), Bounds.sqr (:860-890) and Bounds.sqrt
 * (:892-919).  reciprocal and sqrt need strictly positive intervals (the reference asserts it);
 * here the caller checks l_out if it needs the guarantee.
 */
#define FAITH_OP_RELU        1
#define FAITH_OP_TANH        2
#define FAITH_OP_EXP         3
#define FAITH_OP_RECIPROCAL  4
#define FAITH_OP_SQR         5
#define FAITH_OP_SQRT        6
int faith_unary_verification(int op,
                             const float *src_lb, const float *src_ub,
                             const float *src_lw, const float *src_uw,
                             float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                             float *l_out, float *u_out,
                             int length, int dim_in, int dim_out, float epsilon,
                             int q, int words, int layout, void *stream);

/*
 * Product of two bound objects of one shape (McCormick planes).  No CUDA counterpart in the
 * reference: replaces the PyTorch method Bounds.multiply with a Bounds argument
 * (Bounds.py:608-651, planes from get_bounds_xy :666-688); Bounds.divide (:825-830) is this after
 * a reciprocal.  Natural layout, all twelve arrays shaped like x: [length, dim_in, dim_out] and
 * [length, dim_out].
 */
int faith_multiply_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                const float *y_lb, const float *y_ub, const float *y_lw, const float *y_uw,
                                float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                int length, int dim_in, int dim_out, float epsilon,
                                int q, int words, void *stream);

/*
 * The next three take a whole bound object -- rows_w coefficient rows (length * dim_in) and rows_b
 * constant rows (length), each dim_out long -- and handle all four tensors in one launch.  The
 * reference builds them from PyTorch expressions; there is no CUDA counterpart.  out may alias src (or the added
 * object).
 *
 * Scale, add, shift: Bounds.multiply with a float or a per-neuron tensor (Bounds.py:595-607,
 * :653-664) and Bounds.add with an object or a tensor (:383-395), alone or combined:
 *   out_l = src_l * s+ + src_u * s- (+ add_l) (+ shift on the constant rows only),  out_u mirrored,
 * with s = scale[h] when scale is given, else `scalar`;  s+ = s * (s > 0), s- = s - s+.
 * scale, shift and the added object may be NULL (the added object's four tensors together).
 */
int faith_affine_verification(const float *src_lb, const float *src_ub,
                              const float *src_lw, const float *src_uw,
                              const float *scale, float scalar,
                              const float *add_lb, const float *add_ub,
                              const float *add_lw, const float *add_uw,
                              const float *shift,
                              float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                              long long rows_w, long long rows_b, int dim_out, void *stream);

/*
 * out[r, :] = sum over h of src[r, h], written to every h: the sum / repeat pair of
 * Bounds.softmax (Bounds.py:1009-1012) without the intermediate.
 */
int faith_rowsum_verification(const float *src_lb, const float *src_ub,
                              const float *src_lw, const float *src_uw,
                              float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                              long long rows_w, long long rows_b, int dim_out, void *stream);

/*
 * Softmax over the last axis (Bounds.softmax, Bounds.py:1005-1014: exp, sum over dim_out repeated,
 * reciprocal, multiply -- PyTorch only in the reference) in one launch: a position's [dim_in, dim_out]
 * slab of coefficients stays in the registers of one workgroup through all four operators, each with
 * the arithmetic of its own entry point (faith_unary_verification, faith_rowsum_verification,
 * faith_multiply_verification) and every intermediate rounded to fp32 as those store it.  Natural
 * layout, shapes as faith_relu_verification.  sum_l (out, [length], may be NULL) receives the concrete
 * lower bound of the sum, which the reference asserts to be >= 1e-12 (Bounds.py:1140).  scale > 0 multiplies
 * the object first (the 1 / sqrt(head size) of the attention scores, VerifierForward.py:232-233; 1 for none),
 * rounded as faith_affine_verification would store it.  Outputs must
 * not alias inputs.  Returns FAITH_ERR_UNSUPPORTED when the slab does not fit (faith_softmax_fits
 * tells beforehand: dim_out <= 256, or <= 64 when it is no multiple of 4, and dim_in up to
 * 128 ... 8192 depending on dim_out); the caller then composes the four operators.
 */
int faith_softmax_verification(const float *src_lb, const float *src_ub,
                               const float *src_lw, const float *src_uw,
                               float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                               float *sum_l, float scale,
                               int length, int dim_in, int dim_out, float epsilon,
                               int q, int words, void *stream);
int faith_softmax_fits(int dim_in, int dim_out);

/*
 * out[r, :] = mean over h of src[r, h], written to every h: `matmul(w_avg)` with the dim_out x dim_out
 * matrix of 1 / dim_out that Bounds.layer_norm uses for the variance (Bounds.py:1116, :1123) -- all weights
 * positive, so lower stays lower -- without the GEMM.
 */
int faith_rowmean_verification(const float *src_lb, const float *src_ub,
                               const float *src_lw, const float *src_uw,
                               float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                               long long rows_w, long long rows_b, int dim_out, void *stream);

/*
 * Rows of an object that keeps the coefficients of n_positions positions per batch element only (the input object
 * of VerifierForward.py:127-156 has zeros everywhere else).  No counterpart in the reference, which writes the zeros
 * out; data movement only.  positions: int64 [batch, n_positions]; a position outside 0 .. length-1 names no row.
 * faith_rows_gather: out_a, out_b [batch, n_positions, dim_out] = the rows a, b [batch, length, dim_out] have at the
 * positions (zero for a position that names no row).  faith_rows_put: out_a, out_b [batch, length, dim_out] = a, b
 * with the rows at the positions replaced by rows_a, rows_b [batch, n_positions, dim_out].  Two tensors a launch:
 * the lower and the upper constants / intervals always travel together.  out_* must not overlap the inputs.
 * faith_rows_spread: out [batch, length, row_floats] = rows [batch, n_positions, row_floats] at the positions and
 * zero everywhere else -- the object with its zeros written out (row_floats = dim_in * dim_out for coefficient rows).
 */
int faith_rows_gather(const float *a, const float *b, const long long *positions, float *out_a, float *out_b,
                      int batch_size, int length, int n_positions, int dim_out, void *stream);
int faith_rows_put(const float *a, const float *b, const float *rows_a, const float *rows_b,
                   const long long *positions, float *out_a, float *out_b,
                   int batch_size, int length, int n_positions, int dim_out, void *stream);
int faith_rows_spread(const float *rows, const long long *positions, float *out,
                      int batch_size, int length, int n_positions, long long row_floats, void *stream);

/*
 * Concrete interval (Bounds.concretize, Bounds.py:311-326) of an object that keeps the coefficient rows of
 * n_positions positions per batch element only: lw, uw [batch, n_positions, dim_in, dim_out], lb, ub
 * [batch, length, dim_out], positions int64 [batch, n_positions] -> l, u [batch, length, dim_out]: the constants
 * where there are no coefficients, lb - eps * ||lw rows||_q and ub + eps * ||uw rows||_q at the positions (per word
 * block, as faith_concretize).  One launch where gathering the constants, faith_concretize on the rows and putting
 * the results back were three.  l, u must not overlap the inputs.
 */
int faith_concretize_rows(const float *lb, const float *ub, const float *lw, const float *uw,
                          const long long *positions, float *l, float *u, int batch_size, int length,
                          int n_positions, int dim_in, int dim_out, float eps, int q, int words, void *stream);

/*
 * The layer driver's own device work, one launch each where the reference evaluates three or four tensor
 * expressions; nothing here computes bounds.
 *
 * faith_input_coefficients: the coefficients of VerifierForward._bound_input (VerifierForward.py:127-156).
 * w [batch, rows, dim * words, dim] is written whole: word i of batch element b owns the block
 * [dim * i, dim * (i + 1)) x dim of one row -- row positions[b, i] (int64 [batch, words], device memory) of a
 * dense object (rows = sentence length; a position outside 0 .. rows-1 names no row), row i of a compact one
 * (compact != 0: rows == words, positions is not read and may be NULL) -- and that block is s * identity with
 * s = scales[b] (device memory, [batch]) or, scales NULL, `scale`; everything else is zero.
 *
 * faith_flag_below: the preconditions the reference asserts on the host (Bounds.py:892 `min(l) > 0` for sqrt:
 * strict != 0; :1147 `min(l) >= epsilon` for reciprocal: strict == 0), recorded per batch element instead:
 * flags[b] (bytes, device memory) is set to 1 if any of the per_batch values l[b, :] fails the comparison with
 * `bound` (a NaN fails it, as it fails the assert); flags are never cleared here.
 *
 * faith_verdict: VerifierForward._bound_classifier (:311-314) for every batch element:
 * safe[b] = (label == 0 ? l[b * stride] > 0 : u[b * stride] < 0) and not flags[b] (flags may be NULL).
 * safe: bytes, device memory or pinned host memory that the device can write.
 */
int faith_input_coefficients(float *w, const long long *positions, const float *scales, float scale,
                             int batch_size, int rows, int words, int dim, int compact, void *stream);
int faith_flag_below(const float *l, unsigned char *flags, int batch_size, long long per_batch, float bound,
                     int strict, void *stream);
int faith_verdict(const float *l, const float *u, const unsigned char *flags, unsigned char *safe,
                  int batch_size, long long stride, int label, void *stream);

/*
 * Layer normalisation without the variance (Bounds.layer_norm, Bounds.py:1111-1131, mode "no_var",
 * and the first step of mode "standard"): subtract the row mean -- the mean of the UPPER tensor
 * from the lower one and the reverse, as matmul(ones / H).multiply(-1.) gives it -- then scale by
 * weight[h] split by sign and add bias[h] to the constant rows.  weight and bias may be NULL
 * (NULL weight: mean subtraction only).  add_* (all four or none) is a second object of the same
 * shape added to src first: the residual connection in front of every normalisation
 * (`dense.add(x).layer_norm(...)`, VerifierForward.py:166, 181-189) without its own pass over memory;
 * the sum is rounded to fp32 as the separate Bounds.add rounds it.
 */
int faith_layer_norm_verification(const float *src_lb, const float *src_ub,
                                  const float *src_lw, const float *src_uw,
                                  const float *add_lb, const float *add_ub,
                                  const float *add_lw, const float *add_uw,
                                  const float *weight, const float *bias,
                                  float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                                  long long rows_w, long long rows_b, int dim_out, void *stream);

/*
 * Sign-split affine propagation  y = x @ W^T (+ bias).  Replaces the (commented-out)
 * call_matmul_verification (kernel.cpp:37-43, matmul_verification.cu:787-815) with the
 * arithmetic of Bounds.ori_matmul + add (Bounds.py:397-413, :383-395).
 *   x_lw, x_uw [batch*length, dim_in, dim_out]   natural layout
 *   x_lb, x_ub [batch*length, dim_out]
 *   W          [dim_y_out, dim_out]              nn.Linear layout
 *   bias       [dim_y_out] or NULL
 *   y_lw, y_uw [batch*length, dim_in, dim_y_out];  y_lb, y_ub [batch*length, dim_y_out]
 *
 * Arithmetic.  The reference forms W+ = W (W > 0), W- = W - W+ and four fp32 products per term,
 *   y_l = x_l W+ + x_u W-,   y_u = x_u W+ + x_l W-.
 * Since W+ + W- = W and W+ - W- = |W|, the same two results are  y_l = M - R,  y_u = M + R  with
 *   M = ((x_l + x_u) / 2) W      (centre),     R = ((x_u - x_l) / 2) |W|      (radius):
 * two products per term, which is what the kernels multiply (the sum and the difference of a coefficient pair
 * are rounded to fp32 once, by the thread that stages them; the halving is exact).  Consequences a binder can
 * rely on: (1) with x_u >= x_l element-wise R is a sum of non-negative products, so y_u >= y_l holds bit for
 * bit; (2) each result carries the rounding of BOTH operands' terms: its forward error is bounded by
 * (K + 2) u sum_k (|x_l| + |x_u|)_k |W|_k / 2 (u = 2^-24, K the reduction length) where the four-product form has
 * (K + 1) u sum_k |x_l|_k W+_k + |x_u|_k |W-|_k; measured against float64 on data shaped like the benchmark
 * configurations it is 1.3 - 1.9 times the four-product form's error and under 0.15 of rtol 1e-5 / atol 1e-6;
 * (3) the inputs must be finite (an infinite pair of opposite signs has no centre).  The constant terms
 * y_lb, y_ub are accumulated in double and rounded once.  Results are not bit-identical to the four-product form.
 */
int faith_matmul_verification(const float *x_lb, const float *x_ub,
                              const float *x_lw, const float *x_uw,
                              const float *W, const float *bias,
                              float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                              int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                              void *stream);

/*
 * Affine layer, residual connection and layer normalisation without the variance in one pass over the
 * coefficients: y = layer_norm(x @ W^T (+ bias) + res), i.e. `dense(x).add(res).layer_norm(normalizer, "no_var")`
 * of every encoder sub-block (VerifierForward.py:166, 181-189; Bounds.py:1016-1025, :397-413, :1111-1131).  The
 * reference has no fused counterpart.  x_* and y_* as faith_matmul_verification; res_lb, res_ub
 * [batch*length, dim_y_out]; res_lw, res_uw [batch*length*dim_in, dim_y_out] when res_positions is NULL (res_words 0),
 * else [batch, res_words, dim_in, dim_y_out]: the dim_in rows of the positions res_positions[batch, res_words]
 * (int64, as the compact attention entry points take them), every other row of the added object being zero (a position outside 0 .. length-1 names no row);
 * all four res_* NULL: no residual.  weight, norm_bias [dim_y_out] or NULL as faith_layer_norm_verification.
 * Shapes: dim_y_out 128 or 256, dim_out % 4 == 0, x_lw / x_uw / W 16-byte aligned, dim_in % 64 == 0 when
 * res_positions is given; faith_matmul_layer_norm_fits (rows = batch*length) answers 0 where the shape is not taken --
 * the entry point then returns FAITH_ERR_UNSUPPORTED with nothing written, and the caller runs
 * faith_matmul_verification and faith_layer_norm_verification --, 1 where it is taken but those two launches are
 * the faster choice (fewer than two 64-row tiles per compute unit), 2 where this entry point is.  The sum in front of the normalisation has the bits the separate launches
 * give it; the results differ from theirs by the order in which a row's mean is summed.  y_* must not overlap res_*.
 */
int faith_matmul_layer_norm_fits(long long rows, int dim_in, int dim_out, int dim_y_out, int res_words);
int faith_matmul_layer_norm_verification(const float *x_lb, const float *x_ub,
                                         const float *x_lw, const float *x_uw,
                                         const float *W, const float *bias,
                                         const float *res_lb, const float *res_ub,
                                         const float *res_lw, const float *res_uw,
                                         const long long *res_positions, int res_words,
                                         const float *weight, const float *norm_bias,
                                         float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                                         int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                                         void *stream);

/*
 * Affine layer and ReLU relaxation in one pass over the coefficients: y = relu(x @ W^T (+ bias)), i.e.
 * `dense(x).relu()` of the feed-forward block (VerifierForward.py:171-179; Bounds.py:1016-1025, :921-963).  The
 * reference has no fused counterpart.  Arguments as faith_matmul_verification, plus epsilon, q, words as
 * faith_relu_verification.  Shapes: dim_in 128 or 256 (a tile holds every coefficient row of a position), words 1,
 * dim_out % 4 == 0, x_lw / x_uw / W 16-byte aligned; faith_matmul_relu_fits (rows = batch*length) answers 0 / 1 / 2
 * as faith_matmul_layer_norm_fits does, and the entry point returns FAITH_ERR_UNSUPPORTED with nothing written
 * where the answer is 0.  The layer's result has the bits faith_matmul_verification gives it; each neuron's
 * interval is formed from column norms summed in the tile's order, so it may differ from faith_relu_verification's
 * in the last bit, and the slopes with it.
 */
int faith_matmul_relu_fits(long long rows, int dim_in, int dim_out, int dim_y_out, int words);
int faith_matmul_relu_verification(const float *x_lb, const float *x_ub,
                                   const float *x_lw, const float *x_uw,
                                   const float *W, const float *bias,
                                   float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                                   int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                                   float epsilon, int q, int words, void *stream);

/*
 * Affine layer followed by the concretization of its result: y = x @ W^T (+ bias), then
 * [l, u] of y.  Replaces Bounds.dense(...).concretize() (Bounds.py:1016-1025, :311-326) as the
 * classifier at the end of the verifier uses it (VerifierForward.py:300-314); the reference has
 * no fused counterpart (its tvm kernels keep matmul and concretize apart:
 * tvm_kernels/cuda_kernel/matmul.cu, concretize.cu).  ONE launch for problems of a single round
 * of tiles and a short reduction per position (ceil(dim_in / 128) * dim_out <= 128) with
 * dim_out % 8 == 0, dim_in % (32 words) == 0, words <= 8 and 16-byte aligned x_lw, x_uw, W;
 * otherwise faith_matmul_verification followed by faith_concretize on the same stream.  Arguments as faith_matmul_verification, plus l, u [batch*length, dim_y_out] and
 * epsilon, q, words as faith_concretize.
 */
int faith_matmul_concretize_verification(const float *x_lb, const float *x_ub,
                                         const float *x_lw, const float *x_uw,
                                         const float *W, const float *bias,
                                         float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                                         float *l, float *u,
                                         int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                                         float epsilon, int q, int words, void *stream);

/*
 * `groups` (1 ... 3) affine layers of one shape applied to the same bound object -- the query, key and value
 * layers of an attention block (VerifierForward.py:202-204, three `dense` calls in the reference) -- in one
 * launch where that pays (problems of a single round of small tiles, which would otherwise fill and drain
 * the machine three times), as `groups` calls of faith_matmul_verification otherwise.  W, bias, y_* are arrays
 * of `groups` pointers (host memory; bias or any of its entries may be NULL); results equal those of the
 * separate calls bit for bit.
 */
int faith_matmul_group_verification(const float *x_lb, const float *x_ub,
                                    const float *x_lw, const float *x_uw,
                                    int groups, const float *const *W, const float *const *bias,
                                    float *const *y_lb, float *const *y_ub,
                                    float *const *y_lw, float *const *y_uw,
                                    int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                                    void *stream);

/*
 * The two entry points above for an object whose coefficient rows and constant rows are counted
 * separately (as faith_layer_norm_verification counts them): x_lw, x_uw [rows_w, dim_out] -> y_lw, y_uw
 * [rows_w, dim_y_out]; x_lb, x_ub [rows_b, dim_out] -> y_lb, y_ub [rows_b, dim_y_out].  An ordinary
 * object has rows_w = rows_b * dim_in; one that keeps the coefficients of a few positions only
 * (VerifierForward.py:127-156 builds such an input: zero rows everywhere else) has fewer.
 * faith_matmul_rows_verification with rows_w = 0 multiplies the constant rows alone (x_lw, x_uw, y_lw, y_uw are
 * then not read and may be NULL): for a caller whose coefficient rows go through a kernel variant of its own
 * (faith_amd.autotune's generated variants).
 */
int faith_matmul_rows_verification(const float *x_lb, const float *x_ub,
                                   const float *x_lw, const float *x_uw,
                                   const float *W, const float *bias,
                                   float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                                   long long rows_w, long long rows_b, int dim_out, int dim_y_out,
                                   void *stream);
int faith_matmul_group_rows_verification(const float *x_lb, const float *x_ub,
                                         const float *x_lw, const float *x_uw, int groups,
                                         const float *const *W, const float *const *bias,
                                         float *const *y_lb, float *const *y_ub,
                                         float *const *y_lw, float *const *y_uw,
                                         long long rows_w, long long rows_b, int dim_out, int dim_y_out,
                                         void *stream);

/*
 * McCormick bounds of the attention scores  z[i,j] = sum_k x[i,k] * y[j,k].  Replaces
 * call_dot_product_verification_QK (kernel.cpp:45-51, dot_product_verification.cu:458-496)
 * with the arithmetic of Bounds.ori_dot_product (Bounds.py:710-823).
 * layout = FAITH_LAYOUT_NATURAL:
 *   x_lw, x_uw [batch, length_x, dim_in, dim_out];  y_lw, y_uw [batch, length_y, dim_in, dim_out]
 *   z_lw, z_uw [batch, length_x, dim_in, length_y]
 * layout = FAITH_LAYOUT_TRANSPOSED -- what the reference's adapter passes (Bounds.py:1279-1290,
 * kernel.cpp:133-186):
 *   x_lw, x_uw [batch, length_x, dim_out, dim_in];  y_lw, y_uw [batch, length_y, dim_out, dim_in]
 *   z_lw, z_uw [batch, length_x, length_y, dim_in]
 * Either way:
 *   x_lb, x_ub [batch, length_x, dim_out];  y_lb, y_ub [batch, length_y, dim_out]
 *   x_l, x_u   [batch, length_x, dim_out]  (out: concrete interval of x; caller's scratch)
 *   y_l, y_u   [batch, length_y, dim_out]  (out: concrete interval of y)
 * x_u may be NULL (here and in the three entry points below that take it): the planes take x from below on
 * both sides (Bounds.py:761-762), so nothing reads the upper interval of x -- the reference's adapter passes
 * it as scratch and drops it (Bounds.py:1274-1296); without it the upper coefficients of x are not read for
 * the concretization (natural layout), a quarter of that step's traffic.
 *   z_lb, z_ub [batch, length_x, length_y]
 * The reference entry has one `length`; here x and y may differ in length.  With dim_in == 1 the
 * result is the interval product of the constant terms (Bounds.py:711-721); x_l .. y_u are written
 * all the same.  words must divide dim_in.
  * Arithmetic: of the eight products per term that Bounds.ori_dot_product writes, the four y terms share their
 * multiplier b = x_l, and b+ + b- = b, b+ - b- = |b|, so they are computed as P + Q and P - Q with
 * P = sum (b / 2)(y_lw + y_uw), Q = sum (|b| / 2)(y_lw - y_uw): six products per term; y_lw +- y_uw are rounded to fp32
 * once.  The constant terms z_lb, z_ub are accumulated in double.  Not bit-identical to the eight-product form; within
 * rtol 1e-5 / atol 1e-6 of it on data shaped like the benchmark configurations.
 */
int faith_dot_product_verification_QK(float *x_l, float *y_l, float *x_u, float *y_u,
                                      const float *x_lb, const float *x_ub,
                                      const float *y_lb, const float *y_ub,
                                      const float *x_lw, const float *x_uw,
                                      const float *y_lw, const float *y_uw,
                                      float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                      int batch_size, int length_x, int length_y,
                                      int dim_out, int dim_in, float epsilon,
                                      int q, int words, int layout, void *stream);

/*
 * faith_dot_product_verification_QK for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments
 * and results, minus the four scratch arrays x_l, x_u, y_l, y_u: the concrete intervals (x_l, y_l, y_u;
 * the unused x_u is not computed) live in a device array inside the library, faith_static_scratch_bytes()
 * = 4 MiB per GPU, held until the process ends.  The call allocates and frees nothing.  Limit:
 * batch * (length_x + 2 * length_y) * dim_out floats (each of the three segments rounded up to 64 floats)
 * must fit the array, else FAITH_ERR_UNSUPPORTED (configuration-size attention, 4 heads x 128 x 64, needs
 * 0.4 MiB).  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU (two streams, two threads) race.
 */
long long faith_static_scratch_bytes(void);
int faith_dot_product_verification_QK_static(const float *x_lb, const float *x_ub,
                                             const float *y_lb, const float *y_ub,
                                             const float *x_lw, const float *x_uw,
                                             const float *y_lw, const float *y_uw,
                                             float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                             int batch_size, int length_x, int length_y,
                                             int dim_out, int dim_in, float epsilon,
                                             int q, int words, int layout, void *stream);

/*
 * McCormick bounds of the attention context  z[i,j] = sum_k x[i,k] * y[k,j]  (probabilities times
 * values).  Replaces call_dot_product_verification_V (kernel.cpp:53-60,
 * dot_product_verification.cu:498-535) with the arithmetic of Bounds.context -> ori_dot_product
 * (Bounds.py:843-850, :710-823).
 * layout = FAITH_LAYOUT_NATURAL: the value bounds are taken in their own natural layout; the transposed
 * views that Bounds.t() builds (Bounds.py:335-346) are never materialised.
 *   x_lw, x_uw [batch, length_x, dim_in, length_k];  x_lb, x_ub [batch, length_x, length_k]
 *   y_lw, y_uw [batch, length_k, dim_in, dim_out];   y_lb, y_ub [batch, length_k, dim_out]
 *   x_l, x_u   [batch, length_x, length_k];  y_l, y_u [batch, length_k, dim_out]   (out / scratch)
 *   z_lw, z_uw [batch, length_x, dim_in, dim_out];   z_lb, z_ub [batch, length_x, dim_out]
 * layout = FAITH_LAYOUT_TRANSPOSED -- what the reference's adapter passes (Bounds.py:1306-1329,
 * kernel.cpp:188-241): y is the value object after Bounds.t(), and every coefficient array has dim_in last.
 *   x_lw, x_uw [batch, length_x, length_k, dim_in];  x_lb, x_ub [batch, length_x, length_k]
 *   y_lw, y_uw [batch, dim_out, length_k, dim_in];   y_lb, y_ub [batch, dim_out, length_k]
 *   x_l, x_u   [batch, length_x, length_k];  y_l, y_u [batch, dim_out, length_k]   (out / scratch)
 *   z_lw, z_uw [batch, length_x, dim_out, dim_in];   z_lb, z_ub [batch, length_x, dim_out]
 */
int faith_dot_product_verification_V(float *x_l, float *y_l, float *x_u, float *y_u,
                                     const float *x_lb, const float *x_ub,
                                     const float *y_lb, const float *y_ub,
                                     const float *x_lw, const float *x_uw,
                                     const float *y_lw, const float *y_uw,
                                     float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                     int batch_size, int length_x, int length_k,
                                     int dim_out, int dim_in, float epsilon,
                                     int q, int words, int layout, void *stream);

/*
 * Interval bound propagation (the reference's method "ibp": the `if self.ibp` branches of
 * Bounds.py:863-866, :896-898, :924-926, :973-975, :1030-1032, :1139-1143 and :667-676).  The
 * coefficients are zero there, so an operator maps the concrete interval [l, u] of every neuron
 * (from faith_concretize) to the interval of its image; n elements.
 *   unary:   op = FAITH_OP_RELU / TANH / EXP / RECIPROCAL / SQR / SQRT
 *   product: the extreme of the four corner products of [x_l, x_u] and [y_l, y_u]
 */
int faith_interval_unary(int op, const float *l, const float *u, float *out_lb, float *out_ub,
                         long long n, void *stream);
int faith_interval_product(const float *x_l, const float *x_u, const float *y_l, const float *y_u,
                           float *z_lb, float *z_ub, long long n, void *stream);

/*
 * Attention scores with the heads taken where the dense layers leave them.  Replaces
 * transpose_for_scores on query and key (VerifierForward.py:208-229: four permuted copies per
 * object) followed by Bounds.dot_product (Bounds.py:833-841): the kernels address head h of
 *   x_lw, x_uw [batch, length_x, dim_in, heads * head_size];  x_lb, x_ub [batch, length_x, heads * head_size]
 *   y_lw, y_uw [batch, length_y, dim_in, heads * head_size];  y_lb, y_ub [batch, length_y, heads * head_size]
 * in place.  x_l, x_u / y_l, y_u (out, caller's scratch) have the layout of x_lb / y_lb.  The
 * scores come out with the heads stacked on the batch axis, as the softmax wants them:
 *   z_lw, z_uw [batch * heads, length_x, dim_in, length_y];  z_lb, z_ub [batch * heads, length_x, length_y]
 * (the reference verifies one input at a time, batch = 1; batch > 1 carries independent problems,
 * e.g. the perturbed positions of one sentence).
 */
int faith_attention_scores(float *x_l, float *y_l, float *x_u, float *y_u,
                           const float *x_lb, const float *x_ub,
                           const float *y_lb, const float *y_ub,
                           const float *x_lw, const float *x_uw,
                           const float *y_lw, const float *y_uw,
                           float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                           int batch_size, int heads, int length_x, int length_y,
                           int head_size, int dim_in, float epsilon,
                           int q, int words, void *stream);

/*
 * The same scores for a query and a key whose coefficients vanish outside n_positions positions of
 * every batch element, with only those rows in memory.  The input of a verification query has
 * coefficients at the perturbed position(s) alone (VerifierForward.py:127-156) and keeps that form
 * through layer norm and dense layers; in Bounds.dot_product (Bounds.py:761-818) the x terms of
 * z_lw[i, :, j] read x_lw[i] and the y terms y_lw[j], so z_lw[i, :, j] is zero unless i or j is one
 * of those positions, and 1 / length of the dense contraction is left:
 *   x_lw, x_uw, y_lw, y_uw [batch, n_positions, dim_in, heads * head_size]   coefficient rows of the positions
 *   positions              [batch, n_positions] int64 on the device, distinct within a batch element
 *                          (a value outside 0 ... length-1 means that the row is not there)
 *   x_lb, x_ub, y_lb, y_ub [batch, length, heads * head_size]                constants of every position
 *   x_l, y_l, y_u          [batch, length, heads * head_size]  IN: the concrete bounds (faith_concretize of the
 *                          rows that have coefficients, the constants themselves elsewhere)
 *   z_* as faith_attention_scores writes them, zeros included.
 * FAITH_ERR_UNSUPPORTED unless dim_in > 1, length % 4 == 0, head_size % 4 == 0, the tensors are 16-byte aligned
 * and 8 * n_positions * 128 + 16 * head_size * length <= 163840 (bytes of LDS): take the dense entry point then.
 */
int faith_attention_scores_compact(const float *x_l, const float *y_l, const float *y_u,
                                   const float *x_lb, const float *x_ub,
                                   const float *y_lb, const float *y_ub,
                                   const float *x_lw, const float *x_uw,
                                   const float *y_lw, const float *y_uw,
                                   const long long *positions,
                                   float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                   int batch_size, int heads, int length, int n_positions,
                                   int head_size, int dim_in, void *stream);

/*
 * Attention context with the values read, and the result written, where the dense layers want
 * them.  Replaces transpose_for_scores on the values, Bounds.context (Bounds.py:843-850) and
 * transpose_back (VerifierForward.py:253-263).
 *   x_lw, x_uw [batch * heads, length_x, dim_in, length_k];  x_lb, x_ub [batch * heads, length_x, length_k]   (probabilities)
 *   y_lw, y_uw [batch, length_k, dim_in, heads * head_size];  y_lb, y_ub [batch, length_k, heads * head_size]
 *   x_l, x_u like x_lb;  y_l, y_u like y_lb   (out / scratch)
 *   z_lw, z_uw [batch, length_x, dim_in, heads * head_size];  z_lb, z_ub [batch, length_x, heads * head_size]
 */
int faith_attention_context(float *x_l, float *y_l, float *x_u, float *y_u,
                            const float *x_lb, const float *x_ub,
                            const float *y_lb, const float *y_ub,
                            const float *x_lw, const float *x_uw,
                            const float *y_lw, const float *y_uw,
                            float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                            int batch_size, int heads, int length_x, int length_k,
                            int head_size, int dim_in, float epsilon,
                            int q, int words, void *stream);

/*
 * The same context for a value object whose coefficients vanish outside n_positions key positions of
 * every batch element (see faith_attention_scores_compact), with only those rows in memory:
 *   y_lw, y_uw [batch, n_positions, dim_in, heads * head_size];  positions [batch, n_positions] int64;
 *   y_lb, y_ub [batch, length_k, heads * head_size];  y_l, y_u (same shape) IN: its concrete bounds.
 * The y terms of Bounds.py:761-818, sums over the key positions of b(i, k) against y_lw / y_uw [k], then have one
 * addend per position that has coefficients; x (the probabilities), x_l, x_u and z are as for
 * faith_attention_context.  FAITH_ERR_UNSUPPORTED beyond 80 key positions, for a head size that is no multiple
 * of 4, dim_in == 1 or tensors that are not 16-byte aligned: take the dense entry point then.
 */
int faith_attention_context_compact(float *x_l, float *x_u, const float *y_l, const float *y_u,
                                    const float *x_lb, const float *x_ub,
                                    const float *y_lb, const float *y_ub,
                                    const float *x_lw, const float *x_uw,
                                    const float *y_lw, const float *y_uw,
                                    const long long *positions,
                                    float *z_lb, float *z_ub, float *z_lw, float *z_uw,
                                    int batch_size, int heads, int length_x, int length_k,
                                    int n_positions, int head_size, int dim_in, float epsilon,
                                    int q, int words, void *stream);

/*
 * Sign-split propagation through a 2-D convolution (NCHW).  Replaces the (commented-out)
 * call_convolution_verification (kernel.cpp:62-67, convolution_verification.cu:219-239).
 *   x_lw, x_uw [dim_in, CIN, Height, Width]   (dim_in plays the conv batch)
 *   x_lb, x_ub [batch_size, CIN, Height, Width]
 *   W          [COUT, CIN, K, K];  bias [COUT] or NULL (added to y_lb / y_ub only)
 *   y_lw, y_uw [dim_in, COUT, Ho, Wo];  y_lb, y_ub [batch_size, COUT, Ho, Wo]
 *   Ho = (Height + 2*padding_size - K) / Stride + 1, likewise Wo.
 * Arithmetic: as faith_matmul_verification -- y_l = M - R, y_u = M + R with M = conv((x_l + x_u) / 2, W) and
 * R = conv((x_u - x_l) / 2, |W|), two products per tap instead of the four of conv(x_l, W+) + conv(x_u, W-) and its
 * mirror; same consequences (y_u >= y_l bit for bit for ordered inputs, the error bound with K = CIN * K * K,
 * finite inputs); constant terms accumulated in double.
 */
int faith_convolution_verification(const float *x_lb, const float *x_ub,
                                   const float *x_lw, const float *x_uw,
                                   const float *W, const float *bias,
                                   float *y_lb, float *y_ub, float *y_lw, float *y_uw,
                                   int batch_size, int Height, int Width, int CIN, int COUT,
                                   int K, int Stride, int padding_size, int dim_in,
                                   void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FAITH_AMD_H */
