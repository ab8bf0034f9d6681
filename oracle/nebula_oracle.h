/* TEST INFRASTRUCTURE ONLY -- the CPU oracle for the Nebula forward path.
 *
 * A plain-C restatement of the reference's CPU (.cc) forward algorithm.  Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it; the product
 * libraries never do.  Every function names the reference lines it follows
 * (paths relative to the reference tree).
 *
 * Parity status (how each function is pinned is listed in tests/test_oracle_*.py):
 *   - every function below is checked bit-for-bit against the compiled, unmodified
 *     reference (oracle/_ref, CUSTOM_BLAS build) where that library exists, against the
 *     committed golden vectors in tests/golden/ (written from that same reference build),
 *     and against independent mathematics (double-precision direct convolution,
 *     torch.nn.functional on CPU, closed forms, brute force).
 *   - The reference's default BLAS is OpenBLAS (un-vendored, validated with 0.2 or later,
 *     README.md:34).  Its summation order is not pinned by anything in the reference, so
 *     GEMM-backed results are pinned through the reference's own CUSTOM_BLAS twin
 *     (common/gemm.h) exactly and through OpenBLAS only to 1e-5 relative.
 *   - PARITY UNPINNED: orc_resize_linear_u8 (the cv::resize step of the image driver's input
 *     contract).  OpenCV is not part of the reference tree and not installed; the function
 *     restates OpenCV's published 8-bit INTER_LINEAR arithmetic and is held only to
 *     mathematical checks (identity, constants, one grey level from exact bilinear).
 */
#ifndef NEBULA_ORACLE_H
#define NEBULA_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

/* activation_type_t values, common/def.h:62-78 */
enum {
    ORC_ACT_UNDEFINED = 0, ORC_ACT_ELU, ORC_ACT_HARDTAN, ORC_ACT_LEAKY, ORC_ACT_LHTAN, ORC_ACT_LINEAR,
    ORC_ACT_LOGGY, ORC_ACT_LOGISTIC, ORC_ACT_PLSE, ORC_ACT_RAMP, ORC_ACT_RELIE, ORC_ACT_RELU,
    ORC_ACT_STAIR, ORC_ACT_TANH, ORC_ACT_COUNT
};

/* Host threads used for the fan-out inside each primitive (network_t::num_threads). */
void orc_set_threads(unsigned n);
unsigned orc_get_threads(void);

/* GEMM backend.  0 = restatement of common/gemm.h (default, deterministic, equals the
 * reference's CUSTOM_BLAS build bit for bit).  orc_use_openblas() switches to a
 * cblas_sgemm found by dlopen/dlsym (the reference's default build links OpenBLAS);
 * returns 0 on success.  set_threads_sym may be NULL. */
int  orc_use_openblas(const char *so_path, const char *sgemm_sym, const char *set_threads_sym);
void orc_use_custom_gemm(void);
int  orc_gemm_backend(void);

/* common/utils.cc:81-119 */
void orc_im2col(const float *im, unsigned channel, unsigned height, unsigned width,
                unsigned ksize, unsigned stride, unsigned padding, float *col);
/* common/gemm.h:50-147 (row-major, C = beta*C + alpha*op(A)*op(B)) */
void orc_gemm(int ta, int tb, unsigned M, unsigned N, unsigned K, float alpha,
              const float *A, unsigned lda, const float *B, unsigned ldb,
              float beta, float *C, unsigned ldc);
/* common/utils.cc:162-179 */
void orc_forward_bias(float *out, const float *bias, unsigned channel, unsigned size, unsigned batch);
/* common/batchnorm.cc:58-97 */
void orc_batchnorm_normalize(float *out, const float *mean, const float *var,
                             unsigned channel, unsigned size, unsigned batch);
void orc_batchnorm_scale_down(float *out, const float *scale, unsigned channel, unsigned size, unsigned batch);
/* common/activations.cc:6-89 through models/layers/layer.cc:49-109; -1 for an id activate() rejects */
int  orc_activate(unsigned act, float *x, unsigned n);

/* output-size rules: models/layers/convolutional_layer.cc:146-147, pooling_layer.cc:48,60-61 */
unsigned orc_conv_out_dim(unsigned in, unsigned ksize, unsigned stride, unsigned padding);
unsigned orc_pool_out_dim(unsigned in, unsigned stride, unsigned padding);
unsigned orc_pool_default_padding(unsigned ksize);

/* models/layers/convolutional_layer.cc:365-409 (+ :502-536 when scale/mean/var are non-NULL).
 * workspace holds C*k*k*OH*OW floats. */
void orc_conv_forward(const float *x, const float *w, const float *bias,
                      const float *scale, const float *mean, const float *var,
                      float *y, float *workspace,
                      unsigned B, unsigned C, unsigned H, unsigned W,
                      unsigned F, unsigned ksize, unsigned stride, unsigned padding, unsigned act);
/* models/layers/connected_layer.cc:245-277 (+ :462-492) */
void orc_connected_forward(const float *x, const float *w, const float *bias,
                           const float *scale, const float *mean, const float *var,
                           float *y, unsigned B, unsigned I, unsigned O, unsigned act);
/* models/layers/pooling_layer.cc:109-182 */
void orc_maxpool_forward(const float *x, float *y, unsigned *index,
                         unsigned B, unsigned C, unsigned H, unsigned W,
                         unsigned ksize, unsigned stride, unsigned padding);
void orc_avgpool_forward(const float *x, float *y,
                         unsigned B, unsigned C, unsigned H, unsigned W,
                         unsigned ksize, unsigned stride, unsigned padding);
/* models/layers/shortcut_layer.cc:68-79 + common/utils.cc:28-60.
 * prev = output of the layer just before (shape out_*), conn = output `hops` layers back (shape in_*). */
void orc_shortcut_forward(const float *prev, const float *conn, float *out, unsigned B,
                          unsigned in_c, unsigned in_h, unsigned in_w,
                          unsigned out_c, unsigned out_h, unsigned out_w, unsigned act);
/* models/layers/softmax_layer.cc:85-106 */
void orc_softmax_forward(const float *x, float *y, unsigned rows, unsigned n);

/* rnn_layer_t::forward (models/layers/rnn_layer.cc:91-141).  weight/bias (and scale/mean/var or three
 * NULLs): 3 arrays in file order input gate [O][I], hidden gate [O][O], output gate [O][O].
 * x [T][B][I] -> y [T][B][O]. */
void orc_rnn_forward(const float *x, const float *const *weight, const float *const *bias,
                     const float *const *scale, const float *const *mean, const float *const *var,
                     float *y, unsigned T, unsigned B, unsigned I, unsigned O, unsigned act);

/* Top-k matches as convolutional_t::print_results() counts them (models/networks/convolutional.cc:428-447);
 * ties keep ascending class order (the reference's std::sort leaves them unspecified). */
unsigned orc_topk_matches(const float *probs, const unsigned *labels, unsigned rows, unsigned n, unsigned k);

/* recurrent_t::print_results() (models/networks/recurrent.cc:239-247): sum of label * output with one-hot
 * labels, and the "perplexity" figure the driver prints from it. */
float orc_target_prob_sum(const float *probs, const unsigned *targets, unsigned rows, unsigned n);
float orc_perplexity(float cumulative_cost, unsigned rows_seen);

/* convolutional_t::load_data (models/networks/convolutional.cc:384-412): 8-bit interleaved image ->
 * network input planes (resize if needed, / 255.0, planes 0 and 2 swapped).  The resize restates
 * OpenCV's 8-bit INTER_LINEAR and is PARITY UNPINNED (OpenCV is absent; see the .c file). */
void orc_resize_linear_u8(const unsigned char *src, unsigned src_h, unsigned src_w, unsigned ch,
                          unsigned char *dst, unsigned dst_h, unsigned dst_w);
void orc_image_to_input(const unsigned char *src, unsigned src_h, unsigned src_w, unsigned ch,
                        float *dst, unsigned dst_h, unsigned dst_w);

/* models/layers/lstm_layer.cc:233-346, first forward() on a fresh layer (zero h and c).
 * x is time-major [T][B][I]; y is [T][B][H].  The eight sub-layers come in *file* order
 * (lstm_layer.cc:194-206): iW, fW, oW, cW, iU, fU, oU, cU.  For sub-layer s:
 *   bias[s] -> [H], weight[s] -> [H][in] (in = H for W, I for U),
 *   scale/mean/var[s] -> [H] each, or the three arrays NULL when batch_normalize=0.
 * act = the [lstm] section's activation, applied inside every sub-layer
 * (connected_layer.cc:279-313).  cell (optional) receives c_t for all steps, [T][B][H]. */
void orc_lstm_forward(const float *x, const float *const *weight, const float *const *bias,
                      const float *const *scale, const float *const *mean, const float *const *var,
                      float *y, float *cell,
                      unsigned T, unsigned B, unsigned I, unsigned H, unsigned act);

#ifdef __cplusplus
}
#endif
#endif
