/* Sanitizer driver for the CPU oracle (oracle/nebula_oracle.c), built by tests/test_sanitizers.py with
 * -fsanitize=address,undefined.  Calls every oracle function on small awkward shapes (odd sizes, padding larger
 * than one, strides that do not divide, one and three host threads) so that an out-of-bounds access or undefined
 * arithmetic in the restatement shows up; results are compared elsewhere (tests/test_oracle_*.py). */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nebula_oracle.h"

static unsigned long long state = 88172645463325252ull;
static float rnd(void) {                /* xorshift, uniform in [-1, 1) */
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;
    return (float)((double)(state >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}
static float *randv(size_t n) {
    float *p = (float*)malloc((n ? n : 1) * sizeof(float));
    for(size_t i = 0; i < n; i++) p[i] = rnd();
    return p;
}
static float *posv(size_t n) {          /* variances */
    float *p = randv(n);
    for(size_t i = 0; i < n; i++) p[i] = 0.5f + fabsf(p[i]);
    return p;
}
static int finite_all(const float *p, size_t n) {
    for(size_t i = 0; i < n; i++) if(!isfinite(p[i])) return 0;
    return 1;
}

int main(void) {
    for(unsigned threads = 1; threads <= 3; threads += 2) {
        orc_set_threads(threads);
        /* convolution geometries: B, C, H, W, F, k, stride, pad */
        const unsigned conv[][8] = { {2, 3, 9, 7, 5, 3, 1, 1}, {1, 2, 11, 11, 4, 5, 2, 2}, {3, 1, 6, 8, 2, 1, 1, 0},
                                     {2, 3, 13, 13, 3, 7, 2, 3}, {1, 4, 5, 5, 6, 5, 1, 0}, {2, 2, 8, 8, 3, 3, 3, 2} };
        for(size_t g = 0; g < sizeof(conv) / sizeof(conv[0]); g++) {
            const unsigned B = conv[g][0], C = conv[g][1], H = conv[g][2], W = conv[g][3], F = conv[g][4], k = conv[g][5],
                           s = conv[g][6], p = conv[g][7];
            const unsigned OH = orc_conv_out_dim(H, k, s, p), OW = orc_conv_out_dim(W, k, s, p);
            float *x = randv((size_t)B * C * H * W), *w = randv((size_t)F * C * k * k), *b = randv(F);
            float *sc = randv(F), *mu = randv(F), *var = posv(F);
            float *y = randv((size_t)B * F * OH * OW), *ws = randv((size_t)C * k * k * OH * OW);
            float *col = randv((size_t)C * k * k * OH * OW);
            orc_im2col(x, C, H, W, k, s, p, col);
            orc_conv_forward(x, w, b, NULL, NULL, NULL, y, ws, B, C, H, W, F, k, s, p, ORC_ACT_RELU);
            orc_conv_forward(x, w, b, sc, mu, var, y, ws, B, C, H, W, F, k, s, p, ORC_ACT_LEAKY);
            if(!finite_all(y, (size_t)B * F * OH * OW)) { fprintf(stderr, "conv %zu not finite\n", g); return 1; }
            /* pooling on the same input, with the default padding and with none */
            for(unsigned pad = 0; pad <= orc_pool_default_padding(k); pad += (orc_pool_default_padding(k) ? orc_pool_default_padding(k) : 1)) {
                const unsigned PH = orc_pool_out_dim(H, s, pad), PW = orc_pool_out_dim(W, s, pad);
                float *py = randv((size_t)B * C * PH * PW);
                unsigned *idx = (unsigned*)malloc(((size_t)B * C * PH * PW + 1) * sizeof(unsigned));
                orc_maxpool_forward(x, py, idx, B, C, H, W, k, s, pad);
                orc_avgpool_forward(x, py, B, C, H, W, k, s, pad);
                free(py); free(idx);
            }
            free(x); free(w); free(b); free(sc); free(mu); free(var); free(y); free(ws); free(col);
        }
        /* shortcut shape pairs: conn (c,h,w) -> out (c,h,w) */
        const unsigned sh[][6] = { {4, 8, 8, 4, 8, 8}, {2, 8, 8, 6, 4, 4}, {6, 4, 4, 2, 8, 8}, {3, 19, 19, 5, 10, 10}, {5, 7, 9, 5, 7, 9} };
        for(size_t g = 0; g < sizeof(sh) / sizeof(sh[0]); g++) {
            const unsigned B = 2;
            float *conn = randv((size_t)B * sh[g][0] * sh[g][1] * sh[g][2]);
            float *prev = randv((size_t)B * sh[g][3] * sh[g][4] * sh[g][5]);
            float *out = randv((size_t)B * sh[g][3] * sh[g][4] * sh[g][5]);
            orc_shortcut_forward(prev, conn, out, B, sh[g][0], sh[g][1], sh[g][2], sh[g][3], sh[g][4], sh[g][5], ORC_ACT_LEAKY);
            free(conn); free(prev); free(out);
        }
        /* connected, softmax, the four GEMM forms, primitives, activations */
        {
            const unsigned B = 5, I = 37, O = 11;
            float *x = randv(B * I), *w = randv(O * I), *b = randv(O), *sc = randv(O), *mu = randv(O), *var = posv(O), *y = randv(B * O);
            orc_connected_forward(x, w, b, NULL, NULL, NULL, y, B, I, O, ORC_ACT_LOGISTIC);
            orc_connected_forward(x, w, b, sc, mu, var, y, B, I, O, ORC_ACT_TANH);
            float *p = randv(B * O);
            orc_softmax_forward(y, p, B, O);
            unsigned labels[5] = { 0, 3, 10, 7, 2 };
            (void)orc_topk_matches(p, labels, B, O, 1); (void)orc_topk_matches(p, labels, B, O, 5); (void)orc_topk_matches(p, labels, B, O, O);
            (void)orc_perplexity(orc_target_prob_sum(p, labels, B, O), B);
            orc_forward_bias(y, b, O, 1, B);
            orc_batchnorm_normalize(y, mu, var, O, 1, B);
            orc_batchnorm_scale_down(y, sc, O, 1, B);
            for(unsigned a = 0; a <= ORC_ACT_COUNT; a++) {
                float *t = randv(33);
                t[0] = 0.0f; t[1] = -0.0f; t[2] = 80.0f; t[3] = -80.0f; t[4] = 3.5f; t[5] = -3.5f;
                const int rc = orc_activate(a, t, 33);
                if((rc == 0) != (a > ORC_ACT_UNDEFINED && a < ORC_ACT_COUNT)) { fprintf(stderr, "activation id %u: rc %d\n", a, rc); return 1; }
                free(t);
            }
            for(int ta = 0; ta < 2; ta++) for(int tb = 0; tb < 2; tb++) {
                const unsigned M = 7, N = 9, K = 13;
                float *A = randv(M * K), *Bm = randv(K * N), *Cm = randv(M * N);
                orc_gemm(ta, tb, M, N, K, 0.75f, A, ta ? M : K, Bm, tb ? K : N, 0.5f, Cm, N);
                free(A); free(Bm); free(Cm);
            }
            free(x); free(w); free(b); free(sc); free(mu); free(var); free(y); free(p);
        }
        /* LSTM and RNN, with and without sub-layer batch normalisation */
        {
            const unsigned T = 3, B = 2, I = 5, H = 6;
            const float *w[8], *b[8], *sc[8], *mu[8], *var[8];
            for(int s = 0; s < 8; s++) {
                w[s] = randv((size_t)H * (s < 4 ? H : I)); b[s] = randv(H); sc[s] = randv(H); mu[s] = randv(H); var[s] = posv(H);
            }
            float *x = randv(T * B * I), *y = randv(T * B * H), *cell = randv(T * B * H);
            orc_lstm_forward(x, w, b, NULL, NULL, NULL, y, cell, T, B, I, H, ORC_ACT_LINEAR);
            orc_lstm_forward(x, w, b, sc, mu, var, y, NULL, T, B, I, H, ORC_ACT_TANH);
            if(!finite_all(y, T * B * H)) { fprintf(stderr, "lstm not finite\n"); return 1; }
            const float *rw[3] = { w[4], w[0], w[1] }, *rb[3] = { b[0], b[1], b[2] };
            const float *rsc[3] = { sc[0], sc[1], sc[2] }, *rmu[3] = { mu[0], mu[1], mu[2] }, *rvar[3] = { var[0], var[1], var[2] };
            orc_rnn_forward(x, rw, rb, NULL, NULL, NULL, y, T, B, I, H, ORC_ACT_RELU);
            orc_rnn_forward(x, rw, rb, rsc, rmu, rvar, y, T, B, I, H, ORC_ACT_LEAKY);
            for(int s = 0; s < 8; s++) { free((void*)w[s]); free((void*)b[s]); free((void*)sc[s]); free((void*)mu[s]); free((void*)var[s]); }
            free(x); free(y); free(cell);
        }
        /* image input contract: up, down, identity, exact halving */
        {
            const unsigned geo[][4] = { {7, 9, 7, 9}, {7, 9, 12, 5}, {16, 12, 8, 6}, {5, 5, 11, 11}, {1, 1, 3, 3} };
            for(size_t g = 0; g < sizeof(geo) / sizeof(geo[0]); g++) {
                const unsigned sh_ = geo[g][0], sw = geo[g][1], dh = geo[g][2], dw = geo[g][3], ch = 3;
                unsigned char *src = (unsigned char*)malloc((size_t)sh_ * sw * ch), *dst = (unsigned char*)malloc((size_t)dh * dw * ch);
                for(size_t i = 0; i < (size_t)sh_ * sw * ch; i++) src[i] = (unsigned char)(rnd() * 127.0f + 128.0f);
                float *planes = randv((size_t)dh * dw * ch);
                orc_resize_linear_u8(src, sh_, sw, ch, dst, dh, dw);
                orc_image_to_input(src, sh_, sw, ch, planes, dh, dw);
                free(src); free(dst); free(planes);
            }
        }
    }
    printf("ok\n");
    return 0;
}
