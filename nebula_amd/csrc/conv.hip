// Convolution forward as an implicit GEMM on the fp32 matrix cores of gfx950.
//
//   Y[f][n] = sum_kk  Wp[kk][f] * patch(kk, n)        f < F,  n = (b, oh, ow),  kk = (c, i, j)
//
// The patch matrix (what im2col would write, common/utils.cc:81-119) is never stored: each block
// gathers its BK x BN slice straight from the NCHW input into LDS.  The gather is driven by a small
// per-layer table, one entry per kk, holding the input offset c*H*W + i*W + j and the tap (i, j);
// a pixel column n contributes its base offset and its top-left input coordinate.  The same device
// function feeds nbl_im2col, so the index map can be compared element for element with the CPU one.
//
// Tiling: a block of 64*WAVES_M*WAVES_N threads owns a BM x BN tile of Y; each wave owns
// (MT*32) x (NT*32) of it as MT*NT accumulators of v_mfma_f32_32x32x2_f32.  Filters are the MFMA
// rows and pixels the MFMA columns, so that the 32 lanes holding one accumulator row write 32
// consecutive pixels of one output plane.  Both operands sit in LDS k-major ([k][m] and [k][n]):
// lanes 0-31 read 32 consecutive floats of row k, lanes 32-63 of row k+1 (one ds_read_b32 per
// operand per MFMA, which the 64-cycle fp32 MFMA hides easily).  Weights are re-laid out once, at
// pack time, to [Kp][Mp] so their tile loads are contiguous float4s.  LDS is double buffered with
// register staging: the loads of tile t+1 are issued before the MFMAs of tile t.
#include "nbl_internal.h"

#include <vector>

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int CONV_BK = 16;          // k-tile depth (8 MFMA k-steps)
constexpr int CONV_MP_ALIGN = 384;   // lcm of the BM values below
constexpr int KTAB_PAD_TAP = 0x4000; // tap row of a padded table entry: always outside the image

struct ConvArgs {
    const float *x; const float *wp; const int2 *ktab; const float *g; const float *b; float *y;
    int H, W, F, OW, OHW, CHW, stride, pad;
    int N;        // B * OH * OW
    int Kp, Mp;
    int act, has_scale;
    int tiles_m, tiles_n;
};

struct PixelCoord { int xbase; int ih0; int iw0; };

// Pixel column n -> input base offset and top-left tap coordinate.  n >= N gives a coordinate
// that fails every bounds test.
__device__ __forceinline__ PixelCoord conv_pixel(int n, int N, int OHW, int OW, int stride, int pad,
                                                 int CHW, int W) {
    PixelCoord p;
    if(n < N) {
        const int b = n / OHW, pix = n - b * OHW;
        const int oh = pix / OW, ow = pix - oh * OW;
        p.ih0 = oh * stride - pad;
        p.iw0 = ow * stride - pad;
        p.xbase = b * CHW + p.ih0 * W + p.iw0;
    } else {
        p.ih0 = -(1 << 30); p.iw0 = 0; p.xbase = 0;
    }
    return p;
}

// One element of the patch matrix: the reference's padding rule (taps outside the image read 0).
__device__ __forceinline__ float conv_gather(const float *__restrict__ x, const PixelCoord &p, int2 ke,
                                             int H, int W) {
    const int ih = p.ih0 + (ke.y >> 16), iw = p.iw0 + (ke.y & 0xffff);
    const bool inside = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
    return inside ? x[p.xbase + ke.x] : 0.0f;
}

template<int MT, int NT, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N)
void conv_igemm_kernel(const ConvArgs a) {
    constexpr int BK = CONV_BK;
    constexpr int NTHREADS = 64 * WAVES_M * WAVES_N;
    constexpr int BM = MT * 32 * WAVES_M, BN = NT * 32 * WAVES_N;
    constexpr int LDA = BM + 32, LDB = BN + 32;        // rows k and k+1 land in different bank halves
    static_assert(NTHREADS % BN == 0 || BN % NTHREADS == 0, "pixel columns must split evenly over threads");
    constexpr int COLS_PER_THREAD = BN > NTHREADS ? BN / NTHREADS : 1;
    constexpr int KSTEP = BN >= NTHREADS ? 1 : NTHREADS / BN;   // k rows covered per pass
    constexpr int RB = BK / KSTEP;                              // passes over the k-tile
    constexpr int A_VEC = BK * BM / 4;                          // float4s in a weight tile
    constexpr int RA = (A_VEC + NTHREADS - 1) / NTHREADS;

    __shared__ float As[2][BK][LDA];
    __shared__ float Bs[2][BK][LDB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int half = lane >> 5, l32 = lane & 31;

    // m-tile fastest: the blocks that share one pixel tile run next to each other.
    const int tile = blockIdx.x;
    const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const float *__restrict__ x = a.x;
    const int k_first = (BN >= NTHREADS) ? 0 : tid / BN;
    PixelCoord px[COLS_PER_THREAD];
    #pragma unroll
    for(int c = 0; c < COLS_PER_THREAD; c++)
        px[c] = conv_pixel(n0 + (tid % BN) + c * NTHREADS, a.N, a.OHW, a.OW, a.stride, a.pad, a.CHW, a.W);

    float breg[COLS_PER_THREAD][RB];
    float4 areg[RA];

    auto load_tile = [&](int kt) {
        const int kbase = kt * BK;
        #pragma unroll
        for(int r = 0; r < RB; r++) {
            // uniform over the wave: the table entry comes through scalar registers
            const int kk = __builtin_amdgcn_readfirstlane(kbase + k_first + r * KSTEP);
            const int2 ke = a.ktab[kk];
            #pragma unroll
            for(int c = 0; c < COLS_PER_THREAD; c++) breg[c][r] = conv_gather(x, px[c], ke, a.H, a.W);
        }
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int v = tid + r * NTHREADS;
            if(A_VEC % NTHREADS == 0 || v < A_VEC) {
                const int row = v / (BM / 4), col4 = v % (BM / 4);
                areg[r] = *reinterpret_cast<const float4*>(a.wp + (size_t)(kbase + row) * a.Mp + m0 + col4 * 4);
            }
        }
    };
    auto store_tile = [&](int buf) {
        #pragma unroll
        for(int r = 0; r < RB; r++)
            #pragma unroll
            for(int c = 0; c < COLS_PER_THREAD; c++)
                Bs[buf][k_first + r * KSTEP][(tid % BN) + c * NTHREADS] = breg[c][r];
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int v = tid + r * NTHREADS;
            if(A_VEC % NTHREADS == 0 || v < A_VEC) {
                const int row = v / (BM / 4), col4 = v % (BM / 4);
                *reinterpret_cast<float4*>(&As[buf][row][col4 * 4]) = areg[r];
            }
        }
    };

    floatx16 acc[MT][NT];
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int j = 0; j < NT; j++)
            #pragma unroll
            for(int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int nkt = a.Kp / BK;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    for(int kt = 0; kt < nkt; kt++) {
        const int buf = kt & 1;
        if(kt + 1 < nkt) load_tile(kt + 1);
        #pragma unroll
        for(int ks = 0; ks < BK / 2; ks++) {
            const int kk = 2 * ks + half;
            float av[MT], bv[NT];
            #pragma unroll
            for(int i = 0; i < MT; i++) av[i] = As[buf][kk][(wm * MT + i) * 32 + l32];
            #pragma unroll
            for(int j = 0; j < NT; j++) bv[j] = Bs[buf][kk][(wn * NT + j) * 32 + l32];
            #pragma unroll
            for(int i = 0; i < MT; i++)
                #pragma unroll
                for(int j = 0; j < NT; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        if(kt + 1 < nkt) store_tile(buf ^ 1);
        __syncthreads();
    }

    // Epilogue: y = act(acc * g[f] + b[f]).  Accumulator register r of a 32x32 tile holds row
    // 8*(r/4) + 4*(lane/32) + r%4 and column lane%32.
    #pragma unroll
    for(int j = 0; j < NT; j++) {
        const int n = n0 + (wn * NT + j) * 32 + l32;
        if(n >= a.N) continue;
        const int b = n / a.OHW, pix = n - b * a.OHW;
        float *__restrict__ yb = a.y + (size_t)b * a.F * a.OHW + pix;
        #pragma unroll
        for(int i = 0; i < MT; i++) {
            #pragma unroll
            for(int r = 0; r < 16; r++) {
                const int f = m0 + (wm * MT + i) * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
                if(f < a.F) {
                    float v = acc[i][j][r];
                    v = a.has_scale ? v * a.g[f] + a.b[f] : v + a.b[f];
                    yb[(size_t)f * a.OHW] = nbl_act_apply(a.act, v);
                }
            }
        }
    }
}

__global__ void im2col_kernel(const float *__restrict__ x, const int2 *__restrict__ ktab, float *__restrict__ col,
                              int K, int H, int W, int OW, int OHW, int stride, int pad) {
    const int pix = blockIdx.x * blockDim.x + threadIdx.x;
    const int kk = blockIdx.y;
    if(pix >= OHW || kk >= K) return;
    const PixelCoord p = conv_pixel(pix, OHW, OHW, OW, stride, pad, 0, W);
    col[(size_t)kk * OHW + pix] = conv_gather(x, p, ktab[kk], H, W);
}

// One entry per kk = (c*k + i)*k + j (the row order of the reference's col matrix).
std::vector<int2> build_ktab(unsigned C, unsigned H, unsigned W, unsigned k, unsigned Kp) {
    std::vector<int2> tab(Kp);
    const unsigned K = C * k * k;
    for(unsigned kk = 0; kk < Kp; kk++) {
        if(kk < K) {
            const unsigned j = kk % k, i = (kk / k) % k, c = kk / k / k;
            tab[kk].x = (int)(c * H * W + i * W + j);
            tab[kk].y = (int)((i << 16) | j);
        } else {
            tab[kk].x = 0;
            tab[kk].y = KTAB_PAD_TAP << 16;
        }
    }
    return tab;
}

struct Variant { int bm, bn, threads; void (*kernel)(const ConvArgs); const char *name; };

const Variant VARIANTS[] = {
    { 128, 128, 256, conv_igemm_kernel<2, 2, 2, 2>, "128x128" },
    {  64, 256, 256, conv_igemm_kernel<2, 2, 1, 4>, "64x256" },
    {  96, 256, 256, conv_igemm_kernel<3, 2, 1, 4>, "96x256" },
    {  64, 128, 256, conv_igemm_kernel<1, 2, 2, 2>, "64x128" },
    {  64,  64, 256, conv_igemm_kernel<1, 1, 2, 2>, "64x64" },
    { 128,  64, 256, conv_igemm_kernel<2, 1, 2, 2>, "128x64" },
};
constexpr int NUM_VARIANTS = sizeof(VARIANTS) / sizeof(VARIANTS[0]);

}  // namespace

struct nbl_conv_plan {
    unsigned C, H, W, F, k, stride, pad, OH, OW, K, Kp, Mp;
    int act; bool has_scale;
    float *wp_dev; int2 *ktab_dev; float *g_dev; float *b_dev;
    int variant;   // < 0: chosen per call
};

namespace {

// Tile choice: the largest tile whose grid still covers the chip about twice; wasted rows in the
// last m-tile count against a shape.
int choose_variant(const nbl_conv_plan *p, unsigned N, int num_cu) {
    int best = 0; double best_cost = 1e300;
    for(int v = 0; v < NUM_VARIANTS; v++) {
        const double tm = nbl_div_up(p->F, VARIANTS[v].bm), tn = nbl_div_up(N, VARIANTS[v].bn);
        const double blocks = tm * tn;
        const double slots = 2.0 * num_cu;                       // two blocks per CU resident
        const double rounds = std::ceil(blocks / slots);
        const double tile_work = (double)VARIANTS[v].bm * VARIANTS[v].bn;
        // smaller tiles pay more LDS traffic and launch overhead per flop
        const double eff = tile_work >= 128 * 128 ? 1.0 : tile_work >= 64 * 128 ? 0.92 : 0.8;
        const double cost = rounds * tile_work / eff;
        if(cost < best_cost) { best_cost = cost; best = v; }
    }
    return best;
}

}  // namespace

extern "C" {

int nbl_conv2d_num_variants(void) { return NUM_VARIANTS; }

int nbl_conv2d_pack(nbl_ctx *ctx, const float *weight_host, const float *bias_host,
                    const float *scale_host, const float *mean_host, const float *var_host,
                    unsigned C, unsigned H, unsigned W, unsigned F,
                    unsigned ksize, unsigned stride, unsigned pad, int act, nbl_conv_plan **out) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, out != NULL, "nbl_conv2d_pack: out is NULL");
    *out = NULL;
    NBL_REQUIRE(ctx, weight_host && bias_host, "nbl_conv2d_pack: weight/bias is NULL");
    NBL_REQUIRE(ctx, (scale_host != NULL) == (mean_host != NULL) && (scale_host != NULL) == (var_host != NULL),
                "nbl_conv2d_pack: scale, mean and var must be given together");
    NBL_REQUIRE(ctx, C && H && W && F && ksize && stride, "nbl_conv2d_pack: zero dimension");
    NBL_REQUIRE(ctx, nbl_act_valid(act), "nbl_conv2d_pack: undefined activation type %d", act);
    NBL_REQUIRE(ctx, H + 2 * pad >= ksize && W + 2 * pad >= ksize, "nbl_conv2d_pack: filter larger than padded input");
    if(H >= KTAB_PAD_TAP - pad || W >= 0xffff || ksize >= 0x4000)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_pack: image or filter too large for the tap table");

    nbl_conv_plan *p = new nbl_conv_plan();
    p->C = C; p->H = H; p->W = W; p->F = F; p->k = ksize; p->stride = stride; p->pad = pad;
    p->OH = nbl_conv_out_dim(H, ksize, stride, pad);
    p->OW = nbl_conv_out_dim(W, ksize, stride, pad);
    p->K = C * ksize * ksize;
    p->Kp = nbl_div_up(p->K, CONV_BK) * CONV_BK;
    p->Mp = nbl_div_up(F, CONV_MP_ALIGN) * CONV_MP_ALIGN;
    p->act = act; p->has_scale = scale_host != NULL; p->variant = -1;
    p->wp_dev = NULL; p->ktab_dev = NULL; p->g_dev = NULL; p->b_dev = NULL;

    // [F][K] -> [Kp][Mp], zero padded
    std::vector<float> wp((size_t)p->Kp * p->Mp, 0.0f);
    for(unsigned f = 0; f < F; f++)
        for(unsigned kk = 0; kk < p->K; kk++) wp[(size_t)kk * p->Mp + f] = weight_host[(size_t)f * p->K + kk];
    std::vector<float> g(p->Mp, 0.0f), b(p->Mp, 0.0f);
    nbl_fold_batchnorm(bias_host, scale_host, mean_host, var_host, F, g.data(), b.data());
    std::vector<int2> tab = build_ktab(C, H, W, ksize, p->Kp);

    int rc;
    if((rc = nbl_malloc(ctx, (void**)&p->wp_dev, wp.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->ktab_dev, tab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->g_dev, g.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->b_dev, b.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->wp_dev, wp.data(), wp.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->ktab_dev, tab.data(), tab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->g_dev, g.data(), g.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->b_dev, b.data(), b.size() * sizeof(float))) != NBL_OK) {
        nbl_conv2d_plan_destroy(ctx, p);
        return rc;
    }
    *out = p;
    return NBL_OK;
}

int nbl_conv2d_plan_destroy(nbl_ctx *ctx, nbl_conv_plan *p) {
    if(!ctx || !p) return NBL_EINVAL;
    nbl_free(ctx, p->wp_dev); nbl_free(ctx, p->ktab_dev); nbl_free(ctx, p->g_dev); nbl_free(ctx, p->b_dev);
    delete p;
    return NBL_OK;
}

int nbl_conv2d_plan_info(const nbl_conv_plan *p, unsigned *OH, unsigned *OW, double *flop_per_image) {
    if(!p) return NBL_EINVAL;
    if(OH) *OH = p->OH;
    if(OW) *OW = p->OW;
    if(flop_per_image) *flop_per_image = 2.0 * p->F * p->OH * p->OW * p->K;
    return NBL_OK;
}

int nbl_conv2d_plan_set_variant(nbl_conv_plan *p, int variant) {
    if(!p || variant >= NUM_VARIANTS) return NBL_EINVAL;
    p->variant = variant < 0 ? -1 : variant;
    return NBL_OK;
}

int nbl_conv2d_fwd(nbl_ctx *ctx, const nbl_conv_plan *p, const float *x_dev, float *y_dev, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && x_dev && y_dev, "nbl_conv2d_fwd: NULL argument");
    if(B == 0) return NBL_OK;
    const size_t in_elems = (size_t)B * p->C * p->H * p->W, out_elems = (size_t)B * p->F * p->OH * p->OW;
    const size_t npix = (size_t)B * p->OH * p->OW;
    if(in_elems >= (1ull << 31) || out_elems >= (1ull << 31) || npix >= (1ull << 31) - 512)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: tensors of 2^31 elements or more are not supported");
    const int v = p->variant >= 0 ? p->variant : choose_variant(p, (unsigned)npix, ctx->num_cu);
    const Variant &var = VARIANTS[v];
    ConvArgs a;
    a.x = x_dev; a.wp = p->wp_dev; a.ktab = p->ktab_dev; a.g = p->g_dev; a.b = p->b_dev; a.y = y_dev;
    a.H = p->H; a.W = p->W; a.F = p->F; a.OW = p->OW; a.OHW = p->OH * p->OW; a.CHW = p->C * p->H * p->W;
    a.stride = p->stride; a.pad = p->pad; a.N = (int)npix; a.Kp = p->Kp; a.Mp = p->Mp;
    a.act = p->act; a.has_scale = p->has_scale ? 1 : 0;
    a.tiles_m = nbl_div_up(p->F, var.bm);
    a.tiles_n = nbl_div_up((unsigned)npix, var.bn);
    // the last m-tile may read weight columns past F: they must exist (zero padded) in the packed matrix
    if((unsigned)a.tiles_m * var.bm > p->Mp)
        return nbl_fail(ctx, NBL_EINVAL, "nbl_conv2d_fwd: internal: tile %s overruns the packed weights", var.name);
    const size_t blocks = (size_t)a.tiles_m * a.tiles_n;
    if(blocks >= (1ull << 31)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: grid too large");
    hipLaunchKernelGGL(var.kernel, dim3((unsigned)blocks), dim3(var.threads), 0, ctx->stream, a);
    NBL_LAUNCH_CHECK(ctx, "conv_igemm_kernel");
    return NBL_OK;
}

int nbl_im2col(nbl_ctx *ctx, const float *x_dev, unsigned C, unsigned H, unsigned W,
               unsigned ksize, unsigned stride, unsigned pad, float *col_dev) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, x_dev && col_dev, "nbl_im2col: NULL pointer");
    NBL_REQUIRE(ctx, C && H && W && ksize && stride, "nbl_im2col: zero dimension");
    NBL_REQUIRE(ctx, H + 2 * pad >= ksize && W + 2 * pad >= ksize, "nbl_im2col: filter larger than padded input");
    if(H >= KTAB_PAD_TAP - pad || W >= 0xffff || ksize >= 0x4000)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_im2col: image or filter too large for the tap table");
    const unsigned OH = nbl_conv_out_dim(H, ksize, stride, pad), OW = nbl_conv_out_dim(W, ksize, stride, pad);
    const unsigned K = C * ksize * ksize;
    if(K > 65535) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_im2col: more than 65535 patch rows");
    std::vector<int2> tab = build_ktab(C, H, W, ksize, K);
    int2 *tab_dev = NULL;
    int rc = nbl_malloc(ctx, (void**)&tab_dev, tab.size() * sizeof(int2));
    if(rc != NBL_OK) return rc;
    if((rc = nbl_h2d(ctx, tab_dev, tab.data(), tab.size() * sizeof(int2))) != NBL_OK) { nbl_free(ctx, tab_dev); return rc; }
    hipLaunchKernelGGL(im2col_kernel, dim3(nbl_div_up(OH * OW, 256), K), dim3(256), 0, ctx->stream,
                       x_dev, tab_dev, col_dev, (int)K, (int)H, (int)W, (int)OW, (int)(OH * OW), (int)stride, (int)pad);
    hipError_t e = hipGetLastError();
    rc = nbl_free(ctx, tab_dev);   // waits for the kernel
    if(e != hipSuccess) return nbl_fail(ctx, NBL_EHIP, "launch of im2col_kernel failed: %s", hipGetErrorString(e));
    return rc;
}

}  // extern "C"
