/* TEST INFRASTRUCTURE ONLY -- see nebula_oracle.h.  Plain-C restatement of the reference's
 * CPU forward path; never linked into the product. */
#define _GNU_SOURCE
#include "nebula_oracle.h"

#include <dlfcn.h>
#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------------------------
 * Host-thread fan-out.  The reference spawns num_threads std::threads inside every
 * primitive and splits an index range [tid*n/T, (tid+1)*n/T).  Each output element is
 * produced by exactly one thread, so the split never changes a result.
 * ------------------------------------------------------------------------------------- */
static unsigned g_threads = 1;

void orc_set_threads(unsigned n) { g_threads = n ? n : 1; }
unsigned orc_get_threads(void) { return g_threads; }

typedef void (*range_fn)(unsigned begin, unsigned end, void *arg);
typedef struct { range_fn fn; void *arg; unsigned begin, end; } range_job;

static void *range_tramp(void *p) {
    range_job *j = (range_job*)p;
    j->fn(j->begin, j->end, j->arg);
    return NULL;
}

static void fan_out(unsigned n, range_fn fn, void *arg) {
    unsigned T = g_threads;
    if(T > n) T = n ? n : 1;
    if(T <= 1) { fn(0, n, arg); return; }
    pthread_t *th = (pthread_t*)malloc(sizeof(pthread_t) * T);
    range_job *jobs = (range_job*)malloc(sizeof(range_job) * T);
    for(unsigned t = 0; t < T; t++) {
        jobs[t].fn = fn; jobs[t].arg = arg;
        jobs[t].begin = (unsigned)((unsigned long long)t * n / T);
        jobs[t].end = (unsigned)((unsigned long long)(t + 1) * n / T);
        pthread_create(&th[t], NULL, range_tramp, &jobs[t]);
    }
    for(unsigned t = 0; t < T; t++) pthread_join(th[t], NULL);
    free(jobs); free(th);
}

/* ---------------------------------------------------------------------------------------
 * GEMM.  Default: the four loop nests of common/gemm.h:50-106 with the beta pre-scale and
 * the row split of :108-147.  Float multiply then float add, no contraction.
 * ------------------------------------------------------------------------------------- */
typedef void (*cblas_sgemm_fn)(int order, int ta, int tb, int M, int N, int K, float alpha,
                               const float *A, int lda, const float *B, int ldb,
                               float beta, float *C, int ldc);
typedef void (*blas_threads_fn)(int);
static cblas_sgemm_fn g_sgemm = NULL;
static blas_threads_fn g_blas_threads = NULL;

int orc_use_openblas(const char *so_path, const char *sgemm_sym, const char *set_threads_sym) {
    void *h = dlopen(so_path, RTLD_NOW | RTLD_GLOBAL);
    if(!h) return -1;
    cblas_sgemm_fn f = (cblas_sgemm_fn)dlsym(h, sgemm_sym);
    if(!f) return -2;
    g_sgemm = f;
    g_blas_threads = set_threads_sym ? (blas_threads_fn)dlsym(h, set_threads_sym) : NULL;
    return 0;
}
void orc_use_custom_gemm(void) { g_sgemm = NULL; }
int orc_gemm_backend(void) { return g_sgemm ? 1 : 0; }

typedef struct {
    int ta, tb; unsigned N, K; float alpha;
    const float *A; unsigned lda; const float *B; unsigned ldb; float *C; unsigned ldc;
} gemm_args;

static void gemm_rows(unsigned begin, unsigned end, void *p) {
    const gemm_args *g = (const gemm_args*)p;
    const unsigned N = g->N, K = g->K, lda = g->lda, ldb = g->ldb, ldc = g->ldc;
    const float alpha = g->alpha, *A = g->A, *B = g->B; float *C = g->C;
    if(!g->tb) {
        /* nn (:50-62) and tn (:79-91): rank-1 style, C row updated K times */
        for(unsigned i = begin; i < end; i++)
            for(unsigned k = 0; k < K; k++) {
                const float a = alpha * (g->ta ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k]);
                const float *brow = B + (size_t)k * ldb;
                float *crow = C + (size_t)i * ldc;
                for(unsigned j = 0; j < N; j++) crow[j] += a * brow[j];
            }
    } else {
        /* nt (:64-77) and tt (:93-106): dot product in a float accumulator, added once */
        for(unsigned i = begin; i < end; i++)
            for(unsigned j = 0; j < N; j++) {
                float sum = 0;
                const float *brow = B + (size_t)j * ldb;
                for(unsigned k = 0; k < K; k++) {
                    const float a = g->ta ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k];
                    sum += alpha * a * brow[k];
                }
                C[(size_t)i * ldc + j] += sum;
            }
    }
}

void orc_gemm(int ta, int tb, unsigned M, unsigned N, unsigned K, float alpha,
              const float *A, unsigned lda, const float *B, unsigned ldb,
              float beta, float *C, unsigned ldc) {
    if(g_sgemm) {
        if(g_blas_threads) g_blas_threads((int)g_threads);
        /* CblasRowMajor=101, CblasNoTrans=111, CblasTrans=112 */
        g_sgemm(101, ta ? 112 : 111, tb ? 112 : 111, (int)M, (int)N, (int)K, alpha,
                A, (int)lda, B, (int)ldb, beta, C, (int)ldc);
        return;
    }
    for(unsigned i = 0; i < M; i++)
        for(unsigned j = 0; j < N; j++) C[(size_t)i * ldc + j] *= beta;
    gemm_args g = { ta, tb, N, K, alpha, A, lda, B, ldb, C, ldc };
    fan_out(M, gemm_rows, &g);
}

/* ---------------------------------------------------------------------------------------
 * im2col, common/utils.cc:81-119.  Row r of col = (channel c, tap i, tap j) with
 * r = (c*k + i)*k + j; the padding test is done in unsigned arithmetic, so a tap left of /
 * above the image wraps to a huge value and fails the `>= height/width` test.
 * ------------------------------------------------------------------------------------- */
typedef struct {
    const float *im; float *col;
    unsigned height, width, ksize, stride, padding, oh, ow;
} im2col_args;

static void im2col_rows(unsigned begin, unsigned end, void *p) {
    const im2col_args *a = (const im2col_args*)p;
    for(unsigned r = begin; r < end; r++) {
        const unsigned tj = r % a->ksize, ti = (r / a->ksize) % a->ksize, c = r / a->ksize / a->ksize;
        float *dst = a->col + (size_t)r * a->oh * a->ow;
        for(unsigned h = 0; h < a->oh; h++) {
            const unsigned row = ti + h * a->stride - a->padding;      /* may wrap */
            for(unsigned w = 0; w < a->ow; w++) {
                const unsigned colx = tj + w * a->stride - a->padding; /* may wrap */
                dst[h * a->ow + w] = (row >= a->height || colx >= a->width)
                    ? 0.0f : a->im[colx + a->width * (row + a->height * c)];
            }
        }
    }
}

void orc_im2col(const float *im, unsigned channel, unsigned height, unsigned width,
                unsigned ksize, unsigned stride, unsigned padding, float *col) {
    im2col_args a = { im, col, height, width, ksize, stride, padding,
                      orc_conv_out_dim(height, ksize, stride, padding),
                      orc_conv_out_dim(width, ksize, stride, padding) };
    fan_out(channel * ksize * ksize, im2col_rows, &a);
}

unsigned orc_conv_out_dim(unsigned in, unsigned ksize, unsigned stride, unsigned padding) {
    return (in + 2 * padding - ksize) / stride + 1;
}
unsigned orc_pool_out_dim(unsigned in, unsigned stride, unsigned padding) {
    return (in + 2 * padding) / stride;
}
unsigned orc_pool_default_padding(unsigned ksize) { return (ksize - 1) / 2; }

/* ---------------------------------------------------------------------------------------
 * Per-channel passes over [batch][channel][size], split over the batch.
 * ------------------------------------------------------------------------------------- */
typedef struct { float *out; const float *p0, *p1; unsigned channel, size; int op; } chan_args;

static void chan_pass(unsigned begin, unsigned end, void *p) {
    const chan_args *a = (const chan_args*)p;
    for(unsigned b = begin; b < end; b++)
        for(unsigned c = 0; c < a->channel; c++) {
            float *o = a->out + ((size_t)b * a->channel + c) * a->size;
            switch(a->op) {
                case 0: /* forward_bias, utils.cc:162-179 */
                    for(unsigned s = 0; s < a->size; s++) o[s] += a->p0[c];
                    break;
                case 1: /* batchnorm_normalize, batchnorm.cc:58-77: float subtract, then a double
                           divide by sqrt(var)+1e-5 (eps OUTSIDE the root), rounded to float */
                    for(unsigned s = 0; s < a->size; s++)
                        o[s] = (float)((double)(o[s] - a->p0[c]) / (sqrt((double)a->p1[c]) + 0.00001));
                    break;
                default: /* batchnorm_scale_down, batchnorm.cc:79-97 */
                    for(unsigned s = 0; s < a->size; s++) o[s] *= a->p0[c];
            }
        }
}

void orc_forward_bias(float *out, const float *bias, unsigned channel, unsigned size, unsigned batch) {
    chan_args a = { out, bias, NULL, channel, size, 0 };
    fan_out(batch, chan_pass, &a);
}
void orc_batchnorm_normalize(float *out, const float *mean, const float *var,
                             unsigned channel, unsigned size, unsigned batch) {
    chan_args a = { out, mean, var, channel, size, 1 };
    fan_out(batch, chan_pass, &a);
}
void orc_batchnorm_scale_down(float *out, const float *scale, unsigned channel, unsigned size, unsigned batch) {
    chan_args a = { out, scale, NULL, channel, size, 2 };
    fan_out(batch, chan_pass, &a);
}

/* ---------------------------------------------------------------------------------------
 * Activations, common/activations.cc:6-89.  The literals in the reference are doubles, so
 * every formula that touches one is evaluated in double and rounded to float on the store.
 * Three of them are not the textbook functions (elu squares positives; hardtan / lhtan
 * return 0/1 indicators) -- restated as written.
 * ------------------------------------------------------------------------------------- */
static float act_one(unsigned act, float x) {
    const double d = (double)x;
    switch(act) {
        case ORC_ACT_ELU:      return x > 0.0 ? (float)(double)(x * x) : (float)(d * (exp(d) - 1.0));
        case ORC_ACT_HARDTAN:  return (d < 1.0 && d > -1.0) ? 1.0f : 0.0f;
        case ORC_ACT_LEAKY:    return x > 0.0 ? x : (float)(0.1 * d);
        case ORC_ACT_LHTAN:    return (d > 0.0 && d < 1.0) ? 1.0f : 0.0f;
        case ORC_ACT_LOGGY:    return (float)(2.0 / (1.0 + exp(0.0 - d)) - 1.0);
        case ORC_ACT_LOGISTIC: return (float)(1.0 / (1.0 + exp(0.0 - d)));
        case ORC_ACT_PLSE:
            if(d < -4.0) return (float)(0.01 * (d + 4.0));
            if(d > 4.0)  return (float)(0.01 * (d - 4.0) + 1.0);
            return (float)(0.125 * d + 0.5);
        case ORC_ACT_RAMP:     return x > 0.0 ? (float)(d * (d + 0.01)) : (float)(0.01 * d);
        case ORC_ACT_RELIE:    return x > 0.0 ? x : (float)(0.01 * d);
        case ORC_ACT_RELU:     return x > 0.0 ? x : 0.0f;
        case ORC_ACT_STAIR: {
            const int n = (int)x, half = (int)(d / 2.0);
            return (n % 2) ? (x - (float)n) + (float)half : (float)half;
        }
        case ORC_ACT_TANH:     return (float)((exp(2.0 * d) - 1.0) / (exp(2.0 * d) + 1.0));
        default:               return x;
    }
}

typedef struct { unsigned act; float *x; } act_args;
static void act_range(unsigned begin, unsigned end, void *p) {
    const act_args *a = (const act_args*)p;
    for(unsigned i = begin; i < end; i++) a->x[i] = act_one(a->act, a->x[i]);
}

int orc_activate(unsigned act, float *x, unsigned n) {
    if(act == ORC_ACT_UNDEFINED || act >= ORC_ACT_COUNT) return -1;  /* layer.cc:102-107 */
    if(act == ORC_ACT_LINEAR) return 0;
    act_args a = { act, x };
    fan_out(n, act_range, &a);
    return 0;
}

/* ---------------------------------------------------------------------------------------
 * Inference batchnorm as the layers call it (convolutional_layer.cc:529-535,
 * connected_layer.cc:485-491): normalize with the rolling statistics, then scale.
 * ------------------------------------------------------------------------------------- */
static void bn_inference(float *y, const float *scale, const float *mean, const float *var,
                         unsigned channel, unsigned size, unsigned batch) {
    orc_batchnorm_normalize(y, mean, var, channel, size, batch);
    orc_batchnorm_scale_down(y, scale, channel, size, batch);
}

/* convolutional_layer.cc:365-409: zero y; per image im2col + GEMM(nn, alpha=beta=1);
 * [batchnorm]; bias; activation.  group is never read from the cfg (layer.cc:30) => 1. */
void orc_conv_forward(const float *x, const float *w, const float *bias,
                      const float *scale, const float *mean, const float *var,
                      float *y, float *workspace,
                      unsigned B, unsigned C, unsigned H, unsigned W,
                      unsigned F, unsigned ksize, unsigned stride, unsigned padding, unsigned act) {
    const unsigned oh = orc_conv_out_dim(H, ksize, stride, padding);
    const unsigned ow = orc_conv_out_dim(W, ksize, stride, padding);
    const unsigned patch = ksize * ksize * C, npatch = oh * ow;
    memset(y, 0, sizeof(float) * (size_t)B * F * npatch);
    for(unsigned b = 0; b < B; b++) {
        orc_im2col(x + (size_t)b * C * H * W, C, H, W, ksize, stride, padding, workspace);
        orc_gemm(0, 0, F, npatch, patch, 1.0f, w, patch, workspace, npatch, 1.0f,
                 y + (size_t)b * F * npatch, npatch);
    }
    if(scale) bn_inference(y, scale, mean, var, F, npatch, B);
    orc_forward_bias(y, bias, F, npatch, B);
    orc_activate(act, y, B * F * npatch);
}

/* connected_layer.cc:245-277: zero y; GEMM(nt); [batchnorm with size=1]; bias; activation. */
void orc_connected_forward(const float *x, const float *w, const float *bias,
                           const float *scale, const float *mean, const float *var,
                           float *y, unsigned B, unsigned I, unsigned O, unsigned act) {
    memset(y, 0, sizeof(float) * (size_t)B * O);
    orc_gemm(0, 1, B, O, I, 1.0f, x, I, w, I, 1.0f, y, O);
    if(scale) bn_inference(y, scale, mean, var, O, 1, B);
    orc_forward_bias(y, bias, O, 1, B);
    orc_activate(act, y, B * O);
}

/* ---------------------------------------------------------------------------------------
 * Pooling, pooling_layer.cc:109-182.  Window scanned i-major / j-minor; taps outside the
 * image (unsigned wrap again) read as -1e8 for max and 0 for avg; strict '>' keeps the
 * first maximum; the stored index is the flat offset into the whole [B][C][H][W] input,
 * -1 (0xffffffff) when nothing beat the sentinel.  Average divides by k*k always.
 * ------------------------------------------------------------------------------------- */
typedef struct {
    const float *x; float *y; unsigned *index;
    unsigned C, H, W, ksize, stride, padding, oh, ow; int is_max;
} pool_args;

static void pool_images(unsigned begin, unsigned end, void *p) {
    const pool_args *a = (const pool_args*)p;
    for(unsigned b = begin; b < end; b++)
    for(unsigned c = 0; c < a->C; c++)
    for(unsigned h = 0; h < a->oh; h++)
    for(unsigned w = 0; w < a->ow; w++) {
        const unsigned o = w + a->ow * (h + a->oh * (c + a->C * b));
        float best = -1e8f, acc = 0.0f;
        int best_at = -1;
        for(unsigned i = 0; i < a->ksize; i++)
        for(unsigned j = 0; j < a->ksize; j++) {
            const unsigned row = h * a->stride + i - a->padding;
            const unsigned col = w * a->stride + j - a->padding;
            const unsigned at = col + a->W * (row + a->H * (c + b * a->C));
            const int valid = row < a->H && col < a->W;
            if(a->is_max) {
                const float v = valid ? a->x[at] : -1e8f;
                if(v > best) { best = v; best_at = (int)at; }
            } else {
                acc += valid ? a->x[at] : 0.0f;
            }
        }
        if(a->is_max) { a->y[o] = best; a->index[o] = (unsigned)best_at; }
        else a->y[o] = acc / (float)(a->ksize * a->ksize);
    }
}

void orc_maxpool_forward(const float *x, float *y, unsigned *index,
                         unsigned B, unsigned C, unsigned H, unsigned W,
                         unsigned ksize, unsigned stride, unsigned padding) {
    pool_args a = { x, y, index, C, H, W, ksize, stride, padding,
                    orc_pool_out_dim(H, stride, padding), orc_pool_out_dim(W, stride, padding), 1 };
    fan_out(B, pool_images, &a);
}
void orc_avgpool_forward(const float *x, float *y,
                         unsigned B, unsigned C, unsigned H, unsigned W,
                         unsigned ksize, unsigned stride, unsigned padding) {
    pool_args a = { x, y, NULL, C, H, W, ksize, stride, padding,
                    orc_pool_out_dim(H, stride, padding), orc_pool_out_dim(W, stride, padding), 0 };
    fan_out(B, pool_images, &a);
}

/* ---------------------------------------------------------------------------------------
 * Shortcut, shortcut_layer.cc:68-79 + utils.cc:28-60: out = prev; then over the common
 * (min) channel/height/width box, out[.., h*sample, w*sample] += conn[.., h*stride, w*stride]
 * with stride = max(1, in_w/out_w), sample = max(1, out_w/in_w) (integer division); then activate.
 * ------------------------------------------------------------------------------------- */
void orc_shortcut_forward(const float *prev, const float *conn, float *out, unsigned B,
                          unsigned in_c, unsigned in_h, unsigned in_w,
                          unsigned out_c, unsigned out_h, unsigned out_w, unsigned act) {
    const size_t n = (size_t)B * out_c * out_h * out_w;
    memcpy(out, prev, sizeof(float) * n);
    const unsigned stride = in_w / out_w > 1 ? in_w / out_w : 1;
    const unsigned sample = out_w / in_w > 1 ? out_w / in_w : 1;
    const unsigned w_n = in_w < out_w ? in_w : out_w;
    const unsigned h_n = in_h < out_h ? in_h : out_h;
    const unsigned c_n = in_c < out_c ? in_c : out_c;
    for(unsigned b = 0; b < B; b++)
    for(unsigned c = 0; c < c_n; c++)
    for(unsigned h = 0; h < h_n; h++)
    for(unsigned w = 0; w < w_n; w++) {
        const unsigned o = w * sample + out_w * (h * sample + out_h * (c + out_c * b));
        const unsigned i = w * stride + in_w * (h * stride + in_h * (c + in_c * b));
        out[o] += conn[i];
    }
    orc_activate(act, out, (unsigned)n);
}

/* softmax_layer.cc:85-106: max from -FLT_MAX, e = exp(x - max) (float subtract), sequential
 * float sum, float divide. */
void orc_softmax_forward(const float *x, float *y, unsigned rows, unsigned n) {
    for(unsigned r = 0; r < rows; r++) {
        const float *in = x + (size_t)r * n; float *out = y + (size_t)r * n;
        float sum = 0.0f, mx = (float)(0.0 - FLT_MAX);
        for(unsigned j = 0; j < n; j++) if(in[j] > mx) mx = in[j];
        for(unsigned j = 0; j < n; j++) {
            const float e = (float)exp((double)(in[j] - mx));
            sum += e; out[j] = e;
        }
        for(unsigned j = 0; j < n; j++) out[j] /= sum;
    }
}

/* ---------------------------------------------------------------------------------------
 * Input contract of the image driver, convolutional_t::load_data
 * (models/networks/convolutional.cc:384-412): an 8-bit interleaved image (rows of
 * width*channels bytes, channel order as decoded: B, G, R) is resized with
 * cv::resize(..., cv::INTER_LINEAR) when its size differs from the network's, turned into
 * planes  data[c][h][w] = byte / 255.0  (double division, rounded to float), and planes 0 and
 * 2 are swapped.
 *
 * PARITY UNPINNED for the resize: cv::resize lives in OpenCV, which is neither vendored in
 * the reference nor installed here, and the reference holds no image fixtures.  What
 * follows restates the published 8-bit INTER_LINEAR algorithm of OpenCV's imgproc module
 * (resize.cpp: pixel-centre mapping fx = (dx + 0.5) * scale - 0.5; horizontal and vertical
 * weights as shorts scaled by 2048 with round-half-even; horizontal pass in int; vertical
 * pass ((b0 * (S0 >> 4)) >> 16) + ((b1 * (S1 >> 4)) >> 16) + 2) >> 2).  Pinned only by
 * mathematics (tests/test_oracle_math.py): identity at equal size, constants stay constant,
 * within one grey level of exact bilinear interpolation; tap tables equal to their rational
 * closed form (source index and 11-bit weight of every destination pixel, from exact
 * fractions); exact halving equal to the rounded 2x2 box mean that OpenCV itself substitutes
 * for that ratio (INTER_AREA, same result by construction); exact doubling equal to the
 * 1/4 : 3/4 stencil on ramps (no rounding occurs) and impulses.  The byte -> float planes
 * and the plane swap are pinned bit for bit by their closed form.
 * ------------------------------------------------------------------------------------- */
static int orc_round_half_even(double v) { return (int)nearbyint(v); }   /* default rounding mode */

/* Exported so that the tests can hold the table against its rational closed form. */
void orc_linear_taps(unsigned dst_n, unsigned src_n, int clamp_weight, int *ofs, short *w) {
    const double scale = (double)src_n / (double)dst_n;
    for(unsigned d = 0; d < dst_n; d++) {
        float f = (float)((d + 0.5) * scale - 0.5);
        int s = (int)floor((double)f);
        f -= (float)s;
        if(clamp_weight) {          /* horizontal taps: weight forced to 0 at the borders */
            if(s < 0) { f = 0.0f; s = 0; }
            if(s >= (int)src_n - 1) { f = 0.0f; s = (int)src_n - 1; }
        }
        ofs[d] = s;
        w[2 * d] = (short)orc_round_half_even((double)((1.0f - f) * 2048.0f));
        w[2 * d + 1] = (short)orc_round_half_even((double)(f * 2048.0f));
    }
}

void orc_resize_linear_u8(const unsigned char *src, unsigned src_h, unsigned src_w, unsigned ch,
                          unsigned char *dst, unsigned dst_h, unsigned dst_w) {
    int *xofs = (int*)malloc(sizeof(int) * dst_w), *yofs = (int*)malloc(sizeof(int) * dst_h);
    short *alpha = (short*)malloc(sizeof(short) * 2 * dst_w), *beta = (short*)malloc(sizeof(short) * 2 * dst_h);
    orc_linear_taps(dst_w, src_w, 1, xofs, alpha);
    orc_linear_taps(dst_h, src_h, 0, yofs, beta);
    for(unsigned dy = 0; dy < dst_h; dy++) {
        /* vertical taps: the two source rows are clipped into the image, the weights are not touched */
        int r0 = yofs[dy], r1 = yofs[dy] + 1;
        if(r0 < 0) r0 = 0; if(r0 > (int)src_h - 1) r0 = (int)src_h - 1;
        if(r1 < 0) r1 = 0; if(r1 > (int)src_h - 1) r1 = (int)src_h - 1;
        const int b0 = beta[2 * dy], b1 = beta[2 * dy + 1];
        for(unsigned dx = 0; dx < dst_w; dx++) {
            const int sx = xofs[dx], sx1 = sx + 1 < (int)src_w ? sx + 1 : sx;   /* weight is 0 where sx + 1 is outside */
            const int a0 = alpha[2 * dx], a1 = alpha[2 * dx + 1];
            for(unsigned c = 0; c < ch; c++) {
                const int S0 = src[((size_t)r0 * src_w + sx) * ch + c] * a0 + src[((size_t)r0 * src_w + sx1) * ch + c] * a1;
                const int S1 = src[((size_t)r1 * src_w + sx) * ch + c] * a0 + src[((size_t)r1 * src_w + sx1) * ch + c] * a1;
                const int v = (((b0 * (S0 >> 4)) >> 16) + ((b1 * (S1 >> 4)) >> 16) + 2) >> 2;
                dst[((size_t)dy * dst_w + dx) * ch + c] = (unsigned char)(v < 0 ? 0 : v > 255 ? 255 : v);
            }
        }
    }
    free(xofs); free(yofs); free(alpha); free(beta);
}

void orc_image_to_input(const unsigned char *src, unsigned src_h, unsigned src_w, unsigned ch,
                        float *dst, unsigned dst_h, unsigned dst_w) {
    const unsigned char *img = src;
    unsigned char *tmp = NULL;
    if(src_h != dst_h || src_w != dst_w) {
        tmp = (unsigned char*)malloc((size_t)dst_h * dst_w * ch);
        orc_resize_linear_u8(src, src_h, src_w, ch, tmp, dst_h, dst_w);
        img = tmp;
    }
    const size_t plane = (size_t)dst_h * dst_w;
    for(unsigned h = 0; h < dst_h; h++)
        for(unsigned c = 0; c < ch; c++)
            for(unsigned w = 0; w < dst_w; w++)
                dst[c * plane + (size_t)h * dst_w + w] = (float)(img[((size_t)h * dst_w + w) * ch + c] / 255.0);
    if(ch >= 3)     /* convolutional.cc:403-405 swaps plane 0 and plane 2 */
        for(size_t i = 0; i < plane; i++) { const float t = dst[i]; dst[i] = dst[i + 2 * plane]; dst[i + 2 * plane] = t; }
    free(tmp);
}

/* recurrent_t::print_results(), test branch (models/networks/recurrent.cc:239-247) with the one-hot labels
 * of load_data (:193-197): cumulative_cost += label[i] * output[i] over every element in order (float;
 * the zero labels add +0), then the printed figure exp(-log2(cumulative_cost / rows_seen)), evaluated in
 * float as the C++ overloads do for float arguments. */
float orc_target_prob_sum(const float *probs, const unsigned *targets, unsigned rows, unsigned n) {
    float cum = 0.0f;
    for(unsigned r = 0; r < rows; r++)
        for(unsigned j = 0; j < n; j++) cum += (targets[r] == j ? 1.0f : 0.0f) * probs[(size_t)r * n + j];
    return cum;
}

float orc_perplexity(float cumulative_cost, unsigned rows_seen) {
    return expf(-1.0f * log2f(cumulative_cost / (float)rows_seen));
}

/* ---------------------------------------------------------------------------------------
 * RNN layer, rnn_layer.cc:91-141.  Three connected sub-layers in file order input, hidden,
 * output (rnn_layer.cc:73-77), all initialised from the same section (same output size,
 * activation and batch_normalize).  Per time step, on the B rows of that step:
 *   in_t  = input_gate(x_t)
 *   hid_t = hidden_gate(t == 0 ? in_0 : state_{t-1})     (:103-104: without an argument the
 *           sub-layer reads its prev_layer, which is the input gate)
 *   state = 0; state += in_t; state += hid_t              (:108-115, two axpy with alpha 1)
 *   out_t = output_gate(t == 0 ? hid_0 : state)           (:116-117: prev_layer is the hidden gate)
 * The layer's output is the output gate's [T][B][O].  Every sub-layer call is a full
 * connected forward (GEMM nt, [BN], bias, activation).
 * ------------------------------------------------------------------------------------- */
void orc_rnn_forward(const float *x, const float *const *weight, const float *const *bias,
                     const float *const *scale, const float *const *mean, const float *const *var,
                     float *y, unsigned T, unsigned B, unsigned I, unsigned O, unsigned act) {
    const size_t n = (size_t)B * O;
    float *in = (float*)malloc(sizeof(float) * n), *hid = (float*)malloc(sizeof(float) * n);
    float *state = (float*)calloc(n, sizeof(float));
    for(unsigned t = 0; t < T; t++) {
        orc_connected_forward(x + (size_t)t * B * I, weight[0], bias[0], scale ? scale[0] : NULL,
                              mean ? mean[0] : NULL, var ? var[0] : NULL, in, B, I, O, act);
        orc_connected_forward(t ? state : in, weight[1], bias[1], scale ? scale[1] : NULL,
                              mean ? mean[1] : NULL, var ? var[1] : NULL, hid, B, O, O, act);
        for(size_t e = 0; e < n; e++) { float s = 0.0f; s += 1.0f * in[e]; s += 1.0f * hid[e]; state[e] = s; }
        orc_connected_forward(t ? state : hid, weight[2], bias[2], scale ? scale[2] : NULL,
                              mean ? mean[2] : NULL, var ? var[2] : NULL, y + (size_t)t * n, B, O, O, act);
    }
    free(in); free(hid); free(state);
}

/* convolutional_t::print_results(), test branch (models/networks/convolutional.cc:428-447): per row the
 * class indices are sorted by descending output and the label counts as a match when it is among the first
 * top_k.  The reference sorts with std::sort, whose order among equal outputs is unspecified; here equal
 * outputs keep ascending index order (a stable sort), which is what decides a tie at the k-th place. */
unsigned orc_topk_matches(const float *probs, const unsigned *labels, unsigned rows, unsigned n, unsigned k) {
    unsigned matches = 0;
    for(unsigned r = 0; r < rows; r++) {
        const float *p = probs + (size_t)r * n;
        const unsigned l = labels[r];
        if(l >= n) continue;
        unsigned before = 0;
        for(unsigned j = 0; j < n; j++) if(p[j] > p[l] || (p[j] == p[l] && j < l)) before++;
        if(before < k) matches++;
    }
    return matches;
}

/* ---------------------------------------------------------------------------------------
 * LSTM, lstm_layer.cc:233-346.  Sub-layer slots in file order (lstm_layer.cc:194-206):
 *   0 iW  1 fW  2 oW  3 cW  4 iU  5 fU  6 oU  7 cU
 * Per step: every sub-layer runs a full connected forward (GEMM nt, [BN], bias, the section's
 * activation); gate = U-part + W-part (float add); i,f,o = logistic, g = tanh;
 * i *= g;  c_t = c_{t-1};  c_t *= f;  c_t += i;  h = tanh(c_t);  h *= o;  y[t] = h.
 * ------------------------------------------------------------------------------------- */
void orc_lstm_forward(const float *x, const float *const *weight, const float *const *bias,
                      const float *const *scale, const float *const *mean, const float *const *var,
                      float *y, float *cell,
                      unsigned T, unsigned B, unsigned I, unsigned H, unsigned act) {
    const size_t n = (size_t)B * H;
    float *sub[8];
    for(int s = 0; s < 8; s++) sub[s] = (float*)malloc(sizeof(float) * n);
    float *hid = (float*)calloc(n, sizeof(float));
    float *c_prev = (float*)calloc(n, sizeof(float));
    float *c_now = (float*)malloc(sizeof(float) * n);
    enum { iW, fW, oW, cW, iU, fU, oU, cU };
    for(unsigned t = 0; t < T; t++) {
        const float *xt = x + (size_t)t * B * I;
        for(int s = 0; s < 8; s++) {
            const int from_hidden = s < 4;
            orc_connected_forward(from_hidden ? hid : xt, weight[s], bias[s],
                                  scale ? scale[s] : NULL, mean ? mean[s] : NULL, var ? var[s] : NULL,
                                  sub[s], B, from_hidden ? H : I, H, act);
        }
        float *gi = sub[iU], *gf = sub[fU], *go = sub[oU], *gc = sub[cU];
        for(size_t e = 0; e < n; e++) {
            gi[e] += 1.0f * sub[iW][e]; gf[e] += 1.0f * sub[fW][e];
            gc[e] += 1.0f * sub[cW][e]; go[e] += 1.0f * sub[oW][e];
        }
        orc_activate(ORC_ACT_LOGISTIC, gi, (unsigned)n);
        orc_activate(ORC_ACT_LOGISTIC, gf, (unsigned)n);
        orc_activate(ORC_ACT_LOGISTIC, go, (unsigned)n);
        orc_activate(ORC_ACT_TANH, gc, (unsigned)n);
        for(size_t e = 0; e < n; e++) {
            gi[e] *= 1.0f * gc[e];
            float c = c_prev[e];
            c *= 1.0f * gf[e];
            c += 1.0f * gi[e];
            c_now[e] = c;
        }
        memcpy(hid, c_now, sizeof(float) * n);
        orc_activate(ORC_ACT_TANH, hid, (unsigned)n);
        for(size_t e = 0; e < n; e++) hid[e] *= 1.0f * go[e];
        memcpy(y + (size_t)t * n, hid, sizeof(float) * n);
        if(cell) memcpy(cell + (size_t)t * n, c_now, sizeof(float) * n);
        float *tmp = c_prev; c_prev = c_now; c_now = tmp;
    }
    for(int s = 0; s < 8; s++) free(sub[s]);
    free(hid); free(c_prev); free(c_now);
}
