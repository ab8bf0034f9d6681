/*
 * nebula_hip.h -- C ABI of the MI355X (gfx950) forward path for Nebula's layer framework.
 *
 * One shared library (libnebula_hip.so) exports these entry points.  They take plain pointers and
 * sizes, return an int status (0 = NBL_OK) and never throw.  Every entry point names the interface
 * of the reference (yonseicasl/Nebula v1.4.1, paths relative to its tree) that it stands in for.
 *
 * Conventions (the reference's own, models/layers/layer.h:41-70):
 *   - tensors are fp32, NCHW, row-major, batch outermost; conv weights OIHW; FC weights [O][I];
 *     recurrent tensors are time-major [T][B][feature];
 *   - activation ids are the reference's activation_type_t values (common/def.h:62-78);
 *   - pointers named *_dev are device pointers valid on the context's GPU, pointers named *_host are
 *     host pointers; the caller owns every buffer it passes in;
 *   - all work is queued on the context's stream and is asynchronous; nbl_sync() waits for it.
 *     A context is not thread-safe.  Results follow the reference's CPU (.cc) path where its CPU
 *     and CUDA paths disagree.
 */
#ifndef NEBULA_HIP_H
#define NEBULA_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nbl_ctx nbl_ctx;
typedef struct nbl_conv_plan nbl_conv_plan;
typedef struct nbl_fc_plan nbl_fc_plan;
typedef struct nbl_lstm_plan nbl_lstm_plan;
typedef struct nbl_rnn_plan nbl_rnn_plan;

enum nbl_status {
    NBL_OK = 0,
    NBL_EINVAL = -1,        /* bad argument (null pointer, zero size, unknown id, shape mismatch) */
    NBL_EHIP = -2,          /* a HIP runtime call failed; nbl_last_error() has its text */
    NBL_ENOMEM = -3,        /* device allocation failed */
    NBL_EUNSUPPORTED = -4,  /* valid request outside what the kernels cover (e.g. > 2^31 elements) */
    NBL_ENODEVICE = -5      /* no usable gfx950 device */
};

/* activation_type_t, common/def.h:62-78 */
enum nbl_activation {
    NBL_ACT_UNDEFINED = 0, NBL_ACT_ELU, NBL_ACT_HARDTAN, NBL_ACT_LEAKY, NBL_ACT_LHTAN, NBL_ACT_LINEAR,
    NBL_ACT_LOGGY, NBL_ACT_LOGISTIC, NBL_ACT_PLSE, NBL_ACT_RAMP, NBL_ACT_RELIE, NBL_ACT_RELU,
    NBL_ACT_STAIR, NBL_ACT_TANH, NBL_ACT_COUNT
};

enum nbl_pool_mode { NBL_POOL_MAX = 0, NBL_POOL_AVG = 1 };

/* ---- context, memory, stream -------------------------------------------------------------------
 * Replaces network_t's constructor state: cudaSetDevice(0) + cublasCreate/cudnnCreate
 * (models/networks/network.cc:43-51) and the bare cudaMalloc/cudaMemcpy/cudaMemset calls spread over
 * every layer's init()/init_weight() (e.g. models/layers/convolutional_layer.cc:186-229,335-347). */
int nbl_ctx_create(int device, nbl_ctx **out);
/* Same, but queue all work on an existing hipStream_t (passed as void*); NULL = the null stream. */
int nbl_ctx_create_on_stream(int device, void *hip_stream, nbl_ctx **out);
int nbl_ctx_destroy(nbl_ctx *ctx);
/* Text of the last failure on this context ("" if none); with ctx == NULL, of the last failed
 * nbl_ctx_create*.  The string stays valid until the next failing call. */
const char *nbl_last_error(nbl_ctx *ctx);
void *nbl_ctx_stream(nbl_ctx *ctx);
int nbl_malloc(nbl_ctx *ctx, void **dev_ptr, size_t bytes);
int nbl_free(nbl_ctx *ctx, void *dev_ptr);
/* Page-locked host memory: nbl_h2d / nbl_d2h to and from it skip the driver's staging copy.  The
 * reference keeps its host-side layer outputs in plain new[] arrays (models/layers/softmax_layer.cc:34). */
int nbl_malloc_host(nbl_ctx *ctx, void **host_ptr, size_t bytes);
int nbl_free_host(nbl_ctx *ctx, void *host_ptr);
int nbl_h2d(nbl_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);   /* returns after the copy */
int nbl_d2h(nbl_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);   /* returns after the copy */
/* The same copy queued on the context's stream without waiting for it (dst_host should be page-locked, from
 * nbl_malloc_host; the data is there after the next nbl_sync).  This is the form a stream capture can record: the
 * reference's blocking cudaMemcpy of the softmax output (models/layers/softmax_layer.cu:38-39) becomes a copy node. */
int nbl_d2h_async(nbl_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
int nbl_fill_zero(nbl_ctx *ctx, void *dst_dev, size_t bytes);                   /* a fill kernel, capturable */
/* Device-to-device copy as a kernel on the context's stream (capturable; ranges must not overlap; both
 * pointers 16-byte aligned).  Replaces the reference's cudaMemcpy(..., cudaMemcpyDeviceToDevice) between
 * layer buffers (models/layers/lstm_layer.cu:41-55, models/layers/connected_layer.cu:244,282). */
int nbl_copy_d2d(nbl_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);
int nbl_sync(nbl_ctx *ctx);
/* Test support, no counterpart in the reference: overwrites the LDS of (in all likelihood) every CU with a 32-bit
 * pattern and waits.  LDS keeps what the previous kernel left there, so a kernel that reads LDS words it has not
 * written itself gives results that depend on its predecessor; running it behind a fill with a NaN pattern
 * (0x7fc00000, 0xffffffff) makes such a read show in the output. */
int nbl_lds_fill(nbl_ctx *ctx, unsigned pattern);

/* ---- convolution -------------------------------------------------------------------------------
 * nbl_conv2d_pack replaces convolutional_layer_t::init_weight()'s upload
 * (models/layers/convolutional_layer.cc:257-260,312-316,335-347): it takes the HOST arrays exactly as
 * they sit in the .wgh file (bias[F], weight[F][C][k][k], and scale/rolling_mean/rolling_variance[F]
 * or three NULLs when batch_normalize=0), re-lays the weights out for the implicit-GEMM kernel and
 * turns inference batchnorm + bias into one per-filter multiply-add
 *     y = act(conv * g + b),  g = scale / (sqrt(var) + 1e-5),  b = bias - mean * g
 * (the CPU form, common/batchnorm.cc:70: eps outside the root).
 *
 * nbl_conv2d_fwd replaces convolutional_layer_t::_forward_() (models/layers/convolutional_layer.cu:11-84;
 * CPU twin convolutional_layer.cc:365-409): per-image _im2col_ + cublasSgemm, _forward_batchnorm_,
 * _forward_bias_, _activate_ become one kernel.  x_dev [B][C][H][W] -> y_dev [B][F][OH][OW],
 * OH = (H + 2*pad - k)/stride + 1.  y_dev must not overlap x_dev (NBL_EINVAL). */
int nbl_conv2d_pack(nbl_ctx *ctx, const float *weight_host, const float *bias_host,
                    const float *scale_host, const float *mean_host, const float *var_host,
                    unsigned C, unsigned H, unsigned W, unsigned F,
                    unsigned ksize, unsigned stride, unsigned pad, int act, nbl_conv_plan **out);
int nbl_conv2d_fwd(nbl_ctx *ctx, const nbl_conv_plan *plan, const float *x_dev, float *y_dev, unsigned B);
/* Convolution with the following [shortcut] layer in its epilogue: y = post_act(act(conv(x)) + conn'),
 * conn' = conn cropped to the common channel/height/width box and sampled with stride
 * max(1, conn_w / OW), exactly what convolutional_layer_t::_forward_() followed by
 * shortcut_layer_t::_forward_() compute (models/layers/shortcut_layer.cu:27-52, common/utils.cc:28-60)
 * in the same float operations and order, without writing and re-reading the convolution's output.
 * conn_dev is [B][conn_c][conn_h][conn_w]; y_dev is [B][F][OH][OW].  y_dev may be conn_dev itself when conn has the
 * output's shape (the result then replaces the residual; every element is read and written by the same lane, and the
 * memory system sees one address stream: a 64x256x56x56 layer takes 84 instead of 106 us); any other overlap is an error.
 * An up-sampling shortcut (OW / conn_w > 1) is not fused: NBL_EUNSUPPORTED. */
int nbl_conv2d_shortcut_fwd(nbl_ctx *ctx, const nbl_conv_plan *plan, const float *x_dev, const float *conn_dev,
                            unsigned conn_c, unsigned conn_h, unsigned conn_w, float *y_dev, unsigned B, int post_act);
int nbl_conv2d_plan_destroy(nbl_ctx *ctx, nbl_conv_plan *plan);
/* Algorithmic FLOP of one forward at batch B (2*B*F*OH*OW*C*k*k) and the output dims. */
int nbl_conv2d_plan_info(const nbl_conv_plan *plan, unsigned *OH, unsigned *OW, double *flop_per_image);
/* Pick the tile shape by hand (tests / tuning); variant < 0 restores the built-in choice.
 * nbl_conv2d_num_variants() says how many exist.  Layers with at most 4 input channels and a filter larger than 1x1
 * (the first layer of an image network) have one more kernel, which builds the patch matrix from a strip of the
 * image staged in LDS: variant == nbl_conv2d_num_variants() names it (NBL_EINVAL for a plan that does not qualify;
 * it fuses no shortcut: nbl_conv2d_shortcut_fwd falls back to a tile shape). */
int nbl_conv2d_plan_set_variant(nbl_conv_plan *plan, int variant);
/* Name of a tile shape ("128x128", "64x64", ..., "strip" for index nbl_conv2d_num_variants()); NULL out of range. */
const char *nbl_conv2d_variant_name(int variant);
/* k-split of launches whose tile count leaves CUs idle in the last round: the tiles of that round are
 * cut into slices along C*k*k, one block each, and a second small kernel adds the slices in slice order
 * and applies the epilogue (the result does not depend on timing, but it differs in the last bits from
 * the unsplit sum order).  A plan keeps the scratch memory for this, so one plan must not run on two
 * streams at once.  mode -1 (default): measured
 * together with the tile shape on the first call at a batch size; 0: never; 1: wherever the built-in
 * cost model says so, with its slice count; 2..8: always, with that many slices (fewer where the patch
 * rows run out).  No counterpart in the reference, whose GEMM is cuBLAS's choice
 * (models/layers/convolutional_layer.cu:53-74). */
int nbl_conv2d_plan_set_split(nbl_conv_plan *plan, int mode);
/* Tile shape (index below nbl_conv2d_num_variants(), -1 before the first call) and number of k slices
 * (1 = unsplit) of the plan's most recent launch. */
int nbl_conv2d_plan_last_launch(const nbl_conv_plan *plan, int *variant, int *split_parts);
int nbl_conv2d_num_variants(void);

/* ---- launch table --------------------------------------------------------------------------------
 * The reference's forward is a fixed sequence of library calls (models/networks/network.cc:57-63); here the tile
 * shape and k-split of a convolution launch are a choice, and the choice is data: a process-wide table keyed by
 * the problem (C, H, W, F, filter, stride, padding, batch, and the residual a fused shortcut adds: its channels,
 * height, width and whether the result overwrites it).  On first use the table is read from the text file
 * <library directory>/../launch_tables/gfx950.txt (the environment variable NBL_LAUNCH_TABLE names another file,
 * "none" starts empty).  A launch whose plan has neither a pinned tile shape nor a split rule of its own looks
 * its problem up; a problem the table does not hold is measured on the device once (a few hundred trial launches
 * that write the real output) and entered, so every later plan of the same problem in the process launches the
 * same way.  With the search switched off (nbl_launch_table_set_search(0), or NBL_CONV_SEARCH=0 in the
 * environment) an unlisted problem takes the built-in cost model's choice instead and no launch ever depends on
 * timing.  Errors of these calls are reported through nbl_last_error(NULL). */
int nbl_launch_table_load(const char *path);      /* replaces the table with the file's entries (NULL: the default file); returns their number */
int nbl_launch_table_save(const char *path);      /* writes every entry, read or measured, in the format load reads; returns their number */
int nbl_launch_table_clear(void);
int nbl_launch_table_size(void);
int nbl_launch_table_set_search(int enabled);
/* Where the plan's most recent launch took its tile shape and k-split from. */
enum nbl_launch_source {
    NBL_LAUNCH_NONE = 0,      /* no launch yet */
    NBL_LAUNCH_PINNED = 1,    /* nbl_conv2d_plan_set_variant */
    NBL_LAUNCH_TABLE = 2,     /* an entry read from a table file */
    NBL_LAUNCH_SEARCHED = 3,  /* measured in this process (now, or earlier for an equal problem) */
    NBL_LAUNCH_MODEL = 4      /* the cost model: tiny problems, or the search switched off */
};
int nbl_conv2d_plan_launch_source(const nbl_conv_plan *plan);

/* Replaces _im2col_ (common/utils.h:48, utils.cu:34-74; CPU twin utils.cc:81-119).  The convolution
 * kernel never writes this buffer; the entry point exists so the gather it performs on the fly
 * (same device function, same index table) can be checked element for element.
 * x_dev [C][H][W] (one image) -> col_dev [C*k*k][OH*OW]. */
int nbl_im2col(nbl_ctx *ctx, const float *x_dev, unsigned C, unsigned H, unsigned W,
               unsigned ksize, unsigned stride, unsigned pad, float *col_dev);

/* ---- fully connected ---------------------------------------------------------------------------
 * nbl_fc_pack: connected_layer_t::init_weight() (models/layers/connected_layer.cc:186-206); HOST
 * arrays in .wgh order bias[O], weight[O][I], [scale, mean, var][O] or NULLs.
 * nbl_fc_fwd: connected_layer_t::_forward_() (models/layers/connected_layer.cu:19-53; CPU twin
 * connected_layer.cc:245-277): y[B][O] = act((x[B][I] . W^T) * g + b).  (The CUDA file adds bias[0]
 * to every output, connected_layer.cu:44; the CPU file is followed.)  A plan whose fan-in is a multiple
 * of 32 holds its weights three times on the device: row-major, as contiguous 16 KB tiles for the tiled kernels'
 * buffer loads, and (fan-in a multiple of 8) in operand-major order for the small-batch streaming kernel. */
int nbl_fc_pack(nbl_ctx *ctx, const float *weight_host, const float *bias_host,
                const float *scale_host, const float *mean_host, const float *var_host,
                unsigned I, unsigned O, int act, nbl_fc_plan **out);
int nbl_fc_fwd(nbl_ctx *ctx, const nbl_fc_plan *plan, const float *x_dev, float *y_dev, unsigned B);
/* Which product kernel nbl_fc_fwd runs (tests / tuning; no counterpart in the reference, whose product is cuBLAS's
 * choice, models/layers/connected_layer.cu:27-33).  0 (default): by shape -- up to 64 rows of batch over a matrix of 24 MB
 * or more take the weight-streaming kernel (weights from a third, operand-major copy straight into the matrix
 * cores' operand registers, activations through LDS; needs I % 8 == 0), everything else the LDS-tiled kernels;
 * 1: always the tiled kernels; 2: the streaming kernel wherever its shape limits allow. */
int nbl_fc_plan_set_kernel(nbl_fc_plan *plan, int kernel);
int nbl_fc_plan_destroy(nbl_ctx *ctx, nbl_fc_plan *plan);
/* nbl_fc_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels, same split of the
 * fan-in and therefore the same bits as nbl_fc_fwd, but the split-K partial sums go to a static device array of
 * NBL_FC_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends, and the call
 * never allocates or frees.  A product whose partial sums (splits x B x O floats; the split count is at most 64
 * and falls as B x O grows) exceed the array is refused with NBL_EUNSUPPORTED.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race. */
#define NBL_FC_NOALLOC_SCRATCH_BYTES (16u << 20)
int nbl_fc_fwd_noalloc(nbl_ctx *ctx, const nbl_fc_plan *plan, const float *x_dev, float *y_dev, unsigned B);

/* ---- LSTM --------------------------------------------------------------------------------------
 * nbl_lstm_pack: lstm_layer_t::init_weight() (models/layers/lstm_layer.cc:194-206).  The eight
 * sub-layers come as HOST arrays in FILE order iW, fW, oW, cW, iU, fU, oU, cU: weight_host[s] is
 * [H][H] for the W (hidden) four and [H][I] for the U (input) four, bias_host[s] is [H];
 * scale/mean/var_host are arrays of eight [H] vectors, or NULL when batch_normalize=0.
 * sub_act is the [lstm] section's activation, which the reference applies inside every sub-layer.
 * nbl_lstm_fwd: lstm_layer_t::_forward_() (models/layers/lstm_layer.cu:15-140; CPU twin
 * lstm_layer.cc:233-346) from zero hidden and cell state (or a kept one, below): x_dev [T][B][I] -> y_dev [T][B][H].
 * The per-step 8 GEMMs + 5 saxpy + 7 copies + 7 elementwise kernels become one input-side GEMM over
 * all steps and one fused recurrent kernel per step.  cell_dev (optional, may be NULL) receives the
 * final cell state [B][H]. */
int nbl_lstm_pack(nbl_ctx *ctx, const float *const *weight_host, const float *const *bias_host,
                  const float *const *scale_host, const float *const *mean_host, const float *const *var_host,
                  unsigned I, unsigned H, int sub_act, nbl_lstm_plan **out);
int nbl_lstm_fwd(nbl_ctx *ctx, nbl_lstm_plan *plan, const float *x_dev, float *y_dev, float *cell_dev,
                 unsigned T, unsigned B);
/* State kept between passes.  lstm_layer_t never clears hidden_state and cell_state between forward() calls
 * (lstm_layer.cu:15-140: the buffers are written in every step and read again by step 0 of the next call), which
 * is how the reference's recurrent driver runs one long token stream as consecutive batches of time_steps.  Its
 * two paths disagree on what exactly is kept (the .cu re-reads slot 0 of its per-step cell buffer, i.e. the cell
 * state after the FIRST step of the previous call, beside the last hidden state; the .cc does not rewind its
 * sub-layers at all), so this library offers the recurrence's own state and leaves the choice to the caller:
 * nbl_lstm_plan_carry_state(on = 1): from now on a pass starts from h_T and c_T of the previous pass of the same
 *   plan when that pass had the same B (otherwise, and always with on = 0, the default, from zero).  Passes of
 *   T1 and T2 steps then give what one pass of T1 + T2 steps gives (to rounding: the input-side product of a pass
 *   is one matrix product over all its steps, whose summation order may depend on their number).
 * nbl_lstm_plan_reset_state: the next pass starts from zero (a new sequence); carrying stays on.
 * nbl_lstm_plan_set_state: the next pass with this B starts from h_dev, c_dev ([B][H] each, copied on the
 *   context's stream); the plan must be carrying.  The state a pass ended with is its y[T-1] and cell_dev. */
int nbl_lstm_plan_carry_state(nbl_ctx *ctx, nbl_lstm_plan *plan, int on);
int nbl_lstm_plan_reset_state(nbl_ctx *ctx, nbl_lstm_plan *plan);
int nbl_lstm_plan_set_state(nbl_ctx *ctx, nbl_lstm_plan *plan, const float *h_dev, const float *c_dev, unsigned B);
/* The same layer fed by the recurrent driver's one-hot rows (models/networks/recurrent.cc:179-204, one 1.0
 * per row of input_size = vocabulary entries), given as the position of that 1: tokens_dev[T*B], time-major.
 * The input-side product  x . U^T  is then a gather of T*B columns of U (rows of a transposed copy the plan
 * builds on first use) instead of a [T*B x V].[V x 4H] GEMM; same values as nbl_lstm_fwd on the one-hot
 * matrix.  A token >= input_size stands for an all-zero row. */
int nbl_lstm_fwd_tokens(nbl_ctx *ctx, nbl_lstm_plan *plan, const unsigned *tokens_dev, float *y_dev, float *cell_dev,
                        unsigned T, unsigned B);
/* sum_dev[0] = sum over rows of probs[row][targets[row]]: the quantity recurrent_t::print_results()
 * accumulates into cumulative_cost with one-hot labels (models/networks/recurrent.cc:239-241); the driver's
 * "perplexity" is exp(-log2(cumulative_cost / rows_seen)) (:247).  Deterministic summation order. */
int nbl_target_prob_sum(nbl_ctx *ctx, const float *probs_dev, const unsigned *targets_dev, unsigned rows, unsigned n,
                        float *sum_dev);
int nbl_lstm_plan_destroy(nbl_ctx *ctx, nbl_lstm_plan *plan);

/* ---- RNN layer ---------------------------------------------------------------------------------
 * nbl_rnn_pack: rnn_layer_t::init_weight() (models/layers/rnn_layer.cc:73-77): three connected sub-layers as
 * HOST arrays in FILE order input gate [O][I], hidden gate [O][O], output gate [O][O] (bias [O] each;
 * scale/mean/var: three [O] vectors each, or NULL when batch_normalize=0); act is the [rnn] section's
 * activation, applied inside every sub-layer.
 * nbl_rnn_fwd: rnn_layer_t::forward() (rnn_layer.cc:91-141): x_dev [T][B][I] -> y_dev [T][B][O],
 *   in_t = input(x_t);  hid_t = hidden(t == 0 ? in_0 : state_{t-1});  state_t = in_t + hid_t;
 *   y_t = output(t == 0 ? hid_0 : state_t)
 * (step 0 reads the neighbouring sub-layers as the reference does).  The input gate of all steps is one
 * product, the recurrence one fused kernel per step, the output gate of steps 1..T-1 one product. */
int nbl_rnn_pack(nbl_ctx *ctx, const float *const *weight_host, const float *const *bias_host,
                 const float *const *scale_host, const float *const *mean_host, const float *const *var_host,
                 unsigned I, unsigned O, int act, nbl_rnn_plan **out);
int nbl_rnn_fwd(nbl_ctx *ctx, nbl_rnn_plan *plan, const float *x_dev, float *y_dev, unsigned T, unsigned B);
/* The same layer fed by the recurrent driver's one-hot rows (models/networks/recurrent.cc:179-204) given as the
 * position of their 1.0, tokens_dev[T*B] time-major, as nbl_lstm_fwd_tokens: the input gate's product becomes a
 * gather of rows of the transposed weights (built on first use), with the gate's own scale, bias and activation.
 * Same values as nbl_rnn_fwd on the one-hot matrix; a token >= I stands for an all-zero row. */
int nbl_rnn_fwd_tokens(nbl_ctx *ctx, nbl_rnn_plan *plan, const unsigned *tokens_dev, float *y_dev, unsigned T, unsigned B);
int nbl_rnn_plan_destroy(nbl_ctx *ctx, nbl_rnn_plan *plan);

/* count_dev[0] = number of rows whose label is among the k largest entries of probs[row][0..n): the
 * matches convolutional_t::print_results() counts (models/networks/convolutional.cc:428-447).  Equal
 * entries rank by ascending class index (the reference's std::sort leaves their order open). */
int nbl_topk_matches(nbl_ctx *ctx, const float *probs_dev, const unsigned *labels_dev, unsigned rows, unsigned n,
                     unsigned k, unsigned *count_dev);

/* ---- memory-bound layers -----------------------------------------------------------------------
 * nbl_pool_fwd: pooling_layer_t::_forward_() (models/layers/pooling_layer.cu:150-172; CPU twin
 * pooling_layer.cc:109-182).  Output size is the reference's rule OH = (H + 2*pad)/stride.
 * Max: first maximum in row-major window order wins, taps outside the image count as -1e8, index_dev
 * (may be NULL) receives the flat offset into the whole input tensor (0xffffffff if nothing beat the
 * sentinel).  Avg: sum of the in-image taps divided by k*k. */
int nbl_pool_fwd(nbl_ctx *ctx, const float *x_dev, float *y_dev, unsigned *index_dev,
                 unsigned B, unsigned C, unsigned H, unsigned W,
                 unsigned ksize, unsigned stride, unsigned pad, int mode);
unsigned nbl_pool_out_dim(unsigned in, unsigned stride, unsigned pad);
unsigned nbl_conv_out_dim(unsigned in, unsigned ksize, unsigned stride, unsigned pad);

/* shortcut_layer_t::_forward_() (models/layers/shortcut_layer.cu:27-52; CPU twin
 * shortcut_layer.cc:68-79 + common/utils.cc:28-60): y = act(prev + strided/cropped conn).
 * prev_dev and y_dev are [B][out_c][out_h][out_w] (y_dev may alias prev_dev); conn_dev is
 * [B][in_c][in_h][in_w]. */
int nbl_shortcut_fwd(nbl_ctx *ctx, const float *prev_dev, const float *conn_dev, float *y_dev, unsigned B,
                     unsigned in_c, unsigned in_h, unsigned in_w,
                     unsigned out_c, unsigned out_h, unsigned out_w, int act);

/* ---- image input contract ---------------------------------------------------------------------------
 * The preprocessing of convolutional_t::load_data (models/networks/convolutional.cc:384-412) on the
 * device, so that a batch travels over PCIe as bytes: `images` 8-bit interleaved images
 * [src_h][src_w][channels] (channel order as decoded, B G R) -> planes [images][channels][dst_h][dst_w]
 * of byte / 255.0 with planes 0 and 2 swapped; when the sizes differ the image is first resized as
 * cv::resize(..., cv::INTER_LINEAR) does for 8-bit data (OpenCV's fixed-point bilinear arithmetic,
 * restated from its published algorithm: OpenCV itself is not available to check against). */
int nbl_image_to_input(nbl_ctx *ctx, const unsigned char *src_dev, unsigned images, unsigned src_h, unsigned src_w,
                       unsigned channels, float *dst_dev, unsigned dst_h, unsigned dst_w);

/* softmax_layer_t::_forward_() (models/layers/softmax_layer.cu:30-41; CPU twin softmax_layer.cc:85-106). */
int nbl_softmax_fwd(nbl_ctx *ctx, const float *x_dev, float *y_dev, unsigned rows, unsigned n);

/* layer_t::_activate_() and the 13 _<name>_activation_ functions (models/layers/layer.cu:9-69,
 * common/activations.h:38-50; CPU twins common/activations.cc:6-89), in place. */
int nbl_activation_fwd(nbl_ctx *ctx, float *x_dev, size_t n, int act);

/* _forward_bias_ (common/utils.h:55; CPU twin utils.cc:162-179): y[b][c][s] += bias[c]. */
int nbl_forward_bias(nbl_ctx *ctx, float *y_dev, const float *bias_dev,
                     unsigned channel, unsigned size, unsigned batch);
/* _batchnorm_normalize_ + _batchnorm_scale_down_ (common/batchnorm.h:31-33; CPU twins
 * batchnorm.cc:58-97): y = (y - mean[c]) / (sqrt(var[c]) + 1e-5) * scale[c], in place. */
int nbl_batchnorm_inference(nbl_ctx *ctx, float *y_dev, const float *mean_dev, const float *var_dev,
                            const float *scale_dev, unsigned channel, unsigned size, unsigned batch);

/* ---- timing ------------------------------------------------------------------------------------
 * HIP-event timing on the context's own stream (torch.cuda.Event would watch torch's stream). */
int nbl_timer_start(nbl_ctx *ctx);
int nbl_timer_stop(nbl_ctx *ctx, float *elapsed_ms);   /* waits for the stop event */

const char *nbl_version(void);

#ifdef __cplusplus
}
#endif
#endif
