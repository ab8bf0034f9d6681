// Convolution forward for layers with very few input channels (ResNet's 7x7/2 stem, AlexNet's 11x11/4 first layer,
// VGG's first 3x3: C = 3).  Same product as conv_igemm_kernel,
//
//   Y[f][n] = sum_kk  W[kk][f] * patch(kk, n),      kk = (c*k + i)*k + j   (the row order of common/utils.cc:81-119),
//
// but the patch matrix is built from LDS instead of from global memory: the BN = 128 pixels of a block's tile lie in
// a few output rows of ONE image, so all their patches come from a strip of (rows - 1)*stride + k input rows.  The
// block copies that strip (all C channels, zero padding included) into LDS once; afterwards patch element (kk, n) is
// strip[otab[kk] + base(n)], one LDS read at an address that costs one integer add.  With few channels every gathered
// element would otherwise cost an address, two bounds tests and a select per 4-byte global load, and those ordinary
// vector instructions do not overlap with the matrix pipe: the table gather of conv_igemm_kernel runs the stem at
// 56-58 % of the fp32 MFMA peak with 5.9 of them per MFMA.
//
// Weights are read straight from global memory (L1/L2 hits: every wave of a block, and every block, reads the same
// few tens of KB) in the packed layout [Kp / 4][Mp][4]: one 16-byte load gives a lane the four k-steps of its half
// (lanes 0-31 feed the even quads of k to the MFMAs, lanes 32-63 the odd quads; both operands use the same pairing).
// Nothing is staged per k-tile, so the k loop has no barrier at all.
//
// Tiles never straddle images (an image's last tile may be partly empty), so that one strip serves a tile.
#include "nbl_internal.h"

#include <type_traits>
#include <vector>

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float vec4f __attribute__((ext_vector_type(4)));
typedef int vec4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int STRIP_BN = 128;        // pixels per block tile: 4 waves x 32
constexpr size_t STRIP_LDS_LIMIT = 80 * 1024;     // two blocks per CU (160 KB of LDS)

struct StripArgs {
    const float *x; const float *wq; const float *g; const float *b; float *y; const int *otab;
    int C, H, W, F, OW, OHW, stride, pad;
    int K, Kp, Mp, tiles_m, tiles_per_image;
    int rows, pitch;
    int act;
    int runs;               // pixel tiles of the launch (tiles_per_image * batch)
    FastDiv div_tiles_m, div_tiles_per_image, div_ow;      // the block's set-up divides by these three
    FastDiv div_rows;       // staging: line -> channel
};

// (MT = 2: five blocks per CU fit its LDS use when the registers allow it too -- 6272 tiles of the 7x7 stem at batch 64
// are then 4.9 rounds of resident blocks instead of 6.1)
template<int MT, bool FAST_ACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MT == 2 ? 5 : 2, MT == 2 ? 5 : MT == 3 ? 3 : 2)))
void conv_strip_kernel(const StripArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int strip_elems = a.C * a.rows * a.pitch;
    float *strip = lds;                                     // [C][rows][pitch]
    int *otab = reinterpret_cast<int*>(lds + ((strip_elems + 3) & ~3));         // [Kp], 16-byte aligned

    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // uniform, and known to be: per-row buffer descriptors are built from it
    // Workgroups go to the 8 XCDs round robin by index and each XCD has its own L2: eight consecutive pixel tiles
    // (whose strips overlap in all but a row or two) share an XCD, groups of eight are dealt round robin.
    int tm, tn;
    {
        const unsigned xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, run_local = a.div_tiles_m.div(slot),
                       within = slot - run_local * (unsigned)a.tiles_m;
        const unsigned run = ((run_local >> 3) * 8u + xcd) * 8u + (run_local & 7u);
        if(run >= (unsigned)a.runs) return;             // the grid is padded to whole rounds of groups
        tm = (int)within; tn = (int)run;
    }
    const int img = (int)a.div_tiles_per_image.div((unsigned)tn), p0 = (tn - img * a.tiles_per_image) * STRIP_BN;
    const int m0 = tm * MT * 32;
    const int oh0 = (int)a.div_ow.div((unsigned)p0), ih0 = oh0 * a.stride - a.pad;

    // ---- stage the strip: rows ih0 .. ih0 + rows - 1, columns -pad .. W + pad - 1 of every channel ----
    // The strip's (channel, row) lines are dealt to the four waves in turn, lanes along the line, through a buffer descriptor that covers
    // exactly that image row: a column left or right of the image is an out-of-range offset and reads 0, a row
    // above or below the image gets an empty descriptor.  Per element that leaves one load, one LDS write and the
    // add for its LDS address -- ordinary vector instructions are paid for in matrix-pipe time.  STAGE_LINES lines
    // are requested before the first is written, so a block waits for memory a few times, not once per line.
    {
        constexpr int STAGE_LINES = 8, STAGE_J = 4;          // lines in flight per wave; 64-lane pieces of a line
        const float *__restrict__ xim = a.x + (size_t)img * a.C * a.H * a.W;
        const int nlines = a.C * a.rows;                     // line l = (channel l / rows, row l % rows); wave w takes lines w, w + 4, ...
        for(int w0 = 0; w0 < a.pitch; w0 += 64 * STAGE_J) {                                     // (one pass unless a row has more than 256 columns)
            unsigned voff[STAGE_J];                          // the range check looks at this per-lane offset only
            #pragma unroll
            for(int j = 0; j < STAGE_J; j++) voff[j] = (unsigned)(w0 + lane + 64 * j - a.pad) * 4u;   // wraps (out of range) left of the image
            for(int l0 = wave; l0 < nlines; l0 += 4 * STAGE_LINES) {
                float v[STAGE_LINES][STAGE_J];
                #pragma unroll
                for(int u = 0; u < STAGE_LINES; u++) {
                    const int l = l0 + 4 * u;                                                   // uniform
                    const int c = (int)a.div_rows.div((unsigned)l), ih = ih0 + l - c * a.rows;
                    const bool row_inside = l < nlines && (unsigned)ih < (unsigned)a.H;
                    const __amdgpu_buffer_rsrc_t row = __builtin_amdgcn_make_buffer_rsrc(
                        const_cast<float*>(xim + (row_inside ? (size_t)c * a.H + ih : 0) * a.W), 0, row_inside ? a.W * 4 : 0, 0x00020000);
                    #pragma unroll
                    for(int j = 0; j < STAGE_J; j++)
                        v[u][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(row, (int)voff[j], 0, 0));
                }
                #pragma unroll
                for(int u = 0; u < STAGE_LINES; u++) {
                    const int l = l0 + 4 * u;
                    if(l < nlines) {
                        float *dst = strip + l * a.pitch + w0 + lane;
                        #pragma unroll
                        for(int j = 0; j < STAGE_J; j++) if(w0 + lane + 64 * j < a.pitch) dst[64 * j] = v[u][j];
                    }
                }
            }
        }
        for(int e = tid; e < a.Kp; e += 256) otab[e] = a.otab[e];
    }
    __syncthreads();

    // this lane's pixel (one per lane: 32 MFMA columns per wave)
    const int pl = p0 + wave * 32 + l32;
    const bool live = pl < a.OHW;
    const int oh = live ? (int)a.div_ow.div((unsigned)pl) : oh0, ow = live ? pl - oh * a.OW : 0;
    const int pixbase = (oh - oh0) * a.stride * a.pitch + ow * a.stride;

    // weights: lane (half, l32) reads quad 2*s + half of filters m0 + l32*MT + i as 16-byte buffer loads whose
    // per-lane offset is constant; the step's offset is uniform and rides in the scalar offset
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.wq), 0, (int)((unsigned)a.Kp * (unsigned)a.Mp * 4u), 0x00020000);
    const unsigned w_lane = (unsigned)(half * a.Mp + m0 + l32 * MT) * 16u;
    const unsigned w_step = (unsigned)a.Mp * 32u;           // two quads of k per step
    // steps of 8 patch rows; the packed weights are zero from row K to row Kp, and the table sends those rows to strip
    // offset 0, so that they read the pixel's own first tap (initialised image data) against the zero weight and never
    // a word of LDS this block has not written
    const int nsteps = (a.K + 7) / 8;
    auto load_a = [&](vec4f (&dst)[MT], int s) {
        #pragma unroll
        for(int i = 0; i < MT; i++)
            dst[i] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(wres, (int)(w_lane + 16u * i), (int)((unsigned)s * w_step), 0));
    };
    const vec4i *tab4 = reinterpret_cast<const vec4i*>(otab) + half;
    auto load_b = [&](float (&dst)[4], vec4i o) {
        #pragma unroll
        for(int e = 0; e < 4; e++) dst[e] = strip[o[e] + pixbase];
    };

    floatx16 acc[MT];
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    // Software pipeline, written out over four steps so that every stage lives in registers of its own and nothing
    // is moved: the weights of step s+3 and the strip offsets of step s+2 are requested at the start of step s, the
    // strip values of step s+1 are read (with the offsets requested a step earlier) before the MFMAs of step s issue.
    // Requests past the end repeat the last step; the steps of the last round past the end are skipped (uniform test).
    vec4f wa[4][MT];
    vec4i off[4];
    float bv[2][4];
    const int last = nsteps - 1;
    load_a(wa[0], 0);
    load_a(wa[1], min(1, last));
    load_a(wa[2], min(2, last));
    off[0] = tab4[0];
    off[1] = tab4[2 * min(1, last)];
    load_b(bv[0], off[0]);
#define NBL_STRIP_STEP(U)                                                                                   \
    if(U == 0 || s + U < nsteps) {                                                                          \
        load_a(wa[(U + 3) & 3], min(s + U + 3, last));                                                      \
        off[(U + 2) & 3] = tab4[2 * min(s + U + 2, last)];                                                  \
        load_b(bv[(U + 1) & 1], off[(U + 1) & 3]);                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                  \
        _Pragma("unroll") for(int e = 0; e < 4; e++)                                                        \
            _Pragma("unroll") for(int i = 0; i < MT; i++)                                                   \
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[U & 3][i][e], bv[U & 1][e], acc[i], 0, 0, 0); \
        __builtin_amdgcn_sched_barrier(0);                                                                  \
    }
    for(int s = 0; s < nsteps; s += 4) {
        NBL_STRIP_STEP(0)
        NBL_STRIP_STEP(1)
        NBL_STRIP_STEP(2)
        NBL_STRIP_STEP(3)
    }
#undef NBL_STRIP_STEP

    // ---- epilogue: y = act(acc * g[f] + b[f]) ----
    // Accumulator register r = 4*q + rr of tile i is filter f = m0 + (8*q + 4*half + rr)*MT + i at this lane's pixel:
    // for one q a lane owns 4*MT consecutive filters, whose constants are vector loads from the zero-padded g and b.
    // Stores are buffer stores: the lane's part of the address (its pixel, its half's filters) is a constant vector
    // offset, the filter's row is uniform and rides in the scalar offset -- no address arithmetic per element.
    if(!live) return;
    const __amdgpu_buffer_rsrc_t yres = __builtin_amdgcn_make_buffer_rsrc(a.y + (size_t)img * a.F * a.OHW, 0, (int)((unsigned)a.F * (unsigned)a.OHW * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t gres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.g), 0, a.Mp * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.b), 0, a.Mp * 4, 0x00020000);
    const unsigned y_lane = ((unsigned)(half * 4 * MT) * (unsigned)a.OHW + (unsigned)pl) * 4u;
    const unsigned c_lane = (unsigned)(half * 4 * MT) * 4u;
    const unsigned row_bytes = (unsigned)a.OHW * 4u;
    const bool whole = m0 + MT * 32 <= a.F;                 // uniform: every filter row of the tile exists
    // MODE 0: relu or linear (one max or nothing); 1: leaky / relie (their double-precision product); 2: any activation.
    // WHOLE: no filter row of the tile lies past F.  All three are uniform, so the element loop holds no test of them.
    auto finish = [&](auto mode_, auto whole_) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode_)::value;
        constexpr bool WHOLE = decltype(whole_)::value;
        const bool relu = a.act == NBL_ACT_RELU;
        const double slope = a.act == NBL_ACT_RELIE ? 0.01 : 0.1;
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            const unsigned fq = (unsigned)(m0 + 8 * q * MT);    // uniform; this lane's filters start 4*half*MT further on
            vec4f gq[MT], bq[MT];
            #pragma unroll
            for(int u = 0; u < MT; u++) {
                gq[u] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(gres, (int)(c_lane + 16u * u), (int)(fq * 4u), 0));
                bq[u] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(bres, (int)(c_lane + 16u * u), (int)(fq * 4u), 0));
            }
            #pragma unroll
            for(int e = 0; e < 4 * MT; e++) {
                const int rr = e / MT, i = e % MT;
                float t = __builtin_fmaf(acc[i][q * 4 + rr], gq[e / 4][e % 4], bq[e / 4][e % 4]);
                if(MODE == 0) t = relu ? (t > 0.0f ? t : 0.0f) : t;
                else if(MODE == 1) t = t > 0.0f ? t : (float)(slope * (double)t);
                else t = nbl_act_apply(a.act, t);
                // a filter row past F must not be written (it would land in the next image): its lane offset is pushed out of range
                const unsigned voff = WHOLE || (int)(fq + 4 * half * MT + e) < a.F ? y_lane : 0x80000000u;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, t), yres, (int)voff, (int)((fq + e) * row_bytes), 0);
            }
        }
    };
    typedef std::integral_constant<int, 0> plain; typedef std::integral_constant<int, 1> sloped; typedef std::integral_constant<int, 2> any;
    if(!FAST_ACT) { if(whole) finish(any(), std::true_type()); else finish(any(), std::false_type()); }
    else if(a.act == NBL_ACT_RELU || a.act == NBL_ACT_LINEAR) { if(whole) finish(plain(), std::true_type()); else finish(plain(), std::false_type()); }
    else { if(whole) finish(sloped(), std::true_type()); else finish(sloped(), std::false_type()); }
}

}  // namespace

int nbl_conv_strip_pack(nbl_ctx *ctx, nbl_strip_plan *sp) {
    sp->eligible = false; sp->otab_dev = NULL;
    if(sp->C > 4 || sp->k < 2 || sp->Kp % 32 != 0) return NBL_OK;
    const int OHW = sp->OH * sp->OW;
    int rows_out = (STRIP_BN - 2) / sp->OW + 2;            // output rows 128 consecutive pixels can touch
    if(rows_out > sp->OH) rows_out = sp->OH;
    (void)OHW;
    sp->rows = (rows_out - 1) * sp->stride + sp->k;
    sp->pitch = sp->W + 2 * sp->pad;
    const size_t strip_elems = (size_t)sp->C * sp->rows * sp->pitch;
    sp->lds_bytes = ((strip_elems + 3) & ~(size_t)3) * sizeof(float) + (size_t)sp->Kp * sizeof(int);
    if(sp->lds_bytes > STRIP_LDS_LIMIT) return NBL_OK;
    sp->mt = sp->F <= 64 ? 2 : sp->F <= 96 ? 3 : 4;
    if((unsigned)(nbl_div_up(sp->F, sp->mt * 32) * sp->mt * 32) > (unsigned)sp->Mp) return NBL_OK;   // the last filter tile must exist in the packed weights
    // padding rows (K .. Kp) get offset 0: added to a pixel's base that is the pixel's first tap of channel 0, a word the
    // block has staged; its product with the zero weight of a padding row is 0 (or NaN exactly where the real
    // patch holds a NaN or Inf in that tap, which makes the sum NaN already)
    std::vector<int> otab(sp->Kp, 0);
    for(int c = 0; c < sp->C; c++)
        for(int i = 0; i < sp->k; i++)
            for(int j = 0; j < sp->k; j++)
                otab[(c * sp->k + i) * sp->k + j] = (c * sp->rows + i) * sp->pitch + j;
    int rc;
    if((rc = nbl_malloc(ctx, (void**)&sp->otab_dev, otab.size() * sizeof(int))) != NBL_OK ||
       (rc = nbl_h2d(ctx, sp->otab_dev, otab.data(), otab.size() * sizeof(int))) != NBL_OK) {
        nbl_free(ctx, sp->otab_dev); sp->otab_dev = NULL;
        return rc;
    }
    sp->eligible = true;
    return NBL_OK;
}

void nbl_conv_strip_destroy(nbl_ctx *ctx, nbl_strip_plan *sp) {
    if(sp->otab_dev) nbl_free(ctx, sp->otab_dev);
    sp->otab_dev = NULL; sp->eligible = false;
}

int nbl_conv_strip_forward(nbl_ctx *ctx, const nbl_strip_plan *sp, const float *x_dev, float *y_dev, unsigned B) {
    if(!sp->eligible) return nbl_fail(ctx, NBL_EINVAL, "nbl_conv2d_fwd: internal: layer does not qualify for the strip kernel");
    StripArgs a;
    a.x = x_dev; a.wq = sp->wq_dev; a.g = sp->g_dev; a.b = sp->b_dev; a.y = y_dev; a.otab = sp->otab_dev;
    a.C = sp->C; a.H = sp->H; a.W = sp->W; a.F = sp->F; a.OW = sp->OW; a.OHW = sp->OH * sp->OW; a.stride = sp->stride; a.pad = sp->pad;
    a.K = sp->K; a.Kp = sp->Kp; a.Mp = sp->Mp; a.tiles_m = (int)nbl_div_up(sp->F, sp->mt * 32);
    a.tiles_per_image = (int)nbl_div_up(a.OHW, STRIP_BN);
    a.rows = sp->rows; a.pitch = sp->pitch; a.act = sp->act;
    a.runs = a.tiles_per_image * (int)B;
    a.div_tiles_m = make_fastdiv((unsigned)a.tiles_m); a.div_tiles_per_image = make_fastdiv((unsigned)a.tiles_per_image);
    a.div_ow = make_fastdiv((unsigned)a.OW); a.div_rows = make_fastdiv((unsigned)a.rows);
    const size_t grid = nbl_div_up_sz((size_t)a.runs, 64) * 64 * a.tiles_m;
    if(grid >= (1ull << 31)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: grid too large");
    const bool fast = sp->act == NBL_ACT_RELU || sp->act == NBL_ACT_LINEAR || sp->act == NBL_ACT_LEAKY || sp->act == NBL_ACT_RELIE;
    // more than 64 KB of dynamic LDS has to be asked for, once per kernel and device
#define NBL_STRIP_LAUNCH(MT, FA) \
    do { static nbl_lds_limit_raised raised; \
         NBL_HIP(ctx, raised.ensure(conv_strip_kernel<MT, FA>, ctx->device, (int)STRIP_LDS_LIMIT)); \
         hipLaunchKernelGGL((conv_strip_kernel<MT, FA>), dim3((unsigned)grid), dim3(256), sp->lds_bytes, ctx->stream, a); } while(0)
    if(sp->mt == 2)      { if(fast) NBL_STRIP_LAUNCH(2, true); else NBL_STRIP_LAUNCH(2, false); }
    else if(sp->mt == 3) { if(fast) NBL_STRIP_LAUNCH(3, true); else NBL_STRIP_LAUNCH(3, false); }
    else                 { if(fast) NBL_STRIP_LAUNCH(4, true); else NBL_STRIP_LAUNCH(4, false); }
#undef NBL_STRIP_LAUNCH
    NBL_LAUNCH_CHECK(ctx, "conv_strip_kernel");
    return NBL_OK;
}
