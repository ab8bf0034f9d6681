// Convolution forward as an implicit GEMM on the fp32 matrix cores of gfx950.
//
//   Y[f][n] = sum_kk  Wp[kk][f] * patch(kk, n)        f < F,  n = (b, oh, ow),  kk = a (c, i, j)
//
// The patch matrix (what im2col would write, common/utils.cc:81-119) is never stored: each block
// gathers its BK x BN slice straight from the NCHW input into LDS.  The gather is driven by small
// per-layer tables: one entry per patch row holding the input offset c*H*W + i*W + j and the tap
// (i, j), or, for layers whose rows are packed tap-major, one entry per k-tile; a pixel column n
// contributes its base offset and its top-left input coordinate.  The same device function feeds
// nbl_im2col, so the index map can be compared element for element with the CPU one.
//
// Tiling: a block of 64*WAVES_M*WAVES_N threads owns a BM x BN tile of Y; each wave owns
// (MT*32) x (NT*32) of it as MT*NT accumulators of v_mfma_f32_32x32x2_f32.  Filters are the MFMA
// rows and pixels the MFMA columns, so that the 32 lanes holding one accumulator row write 32*NT
// consecutive pixels of one output plane.  Both operands sit in LDS k-major ([k][m] and [k][n]):
// lanes 0-31 read row k, lanes 32-63 row k+1, each lane its MT (NT) adjacent values in one read.
// Weights are re-laid out once, at pack time, to [Kp][Mp] so their tile loads are contiguous
// float4s.  LDS is double buffered and fed through two register stages: the global loads of
// k-tile t+2 are issued before the MFMAs of k-tile t.
//
// Work distribution: one block per output tile, except that the tiles of an under-filled last round
// may be cut into slices along k (one block per slice, raw sums to scratch, a finishing kernel adds
// them in order and applies the epilogue); block indices are renumbered so that the filter tiles of
// one pixel tile share an XCD.  The tile shape and the k-split of a (layer geometry, batch, residual) come
// from a launch table: a text file shipped next to the library holds the choices measured for the benchmarked
// networks, a geometry it does not list is measured on first use (conv_tune) and added to the table in memory,
// so equal problems launch equally for the life of the process.
#include "nbl_internal.h"

#include <dlfcn.h>

#include <array>
#include <cmath>
#include <cstdlib>
#include <type_traits>
#include <algorithm>
#include <map>
#include <mutex>
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
    int K, Kp, Mp;
    unsigned x_bytes;
    int act, has_scale;
    int tiles_m, tiles_n;
    // optional fused shortcut: y = post_act(act(conv) + res'), res' = res cropped/strided as common/utils.cc:28-60
    const float *res; int res_c, res_hw, res_w, res_stride, res_box_h, res_box_w, post_act;
    // output (and residual, when there is one and it has the output's shape) addressable with 32-bit byte
    // offsets and a cheap activation on both sides: full tiles may take the short epilogue
    int short_epilogue;   // 0: no, 1: relu/linear only, 2: leaky or relie somewhere
    // split along k: blocks [0, whole_tiles) compute one whole tile each; after them every remaining tile
    // is shared by `split` blocks, block part p accumulating its slice of the k-tiles and writing raw sums
    // to ws[p][f][n - n_start]; conv_split_finish_kernel adds the parts and applies the epilogue
    int whole_tiles, split, n_start, n_tail;
    int units;     // whole_tiles + (tiles - whole_tiles) * split: work units of the launch
    int xcd_group_log2; // log2 of the consecutive pixel tiles that share an XCD (see the block index mapping in the kernel)
    FastDiv div_tiles_m, div_ohw, div_ow, div_split;
    float *ws;
    // tap-major layers: one entry per k-tile, {byte offset of the tile's tap in channel c0's plane +
    // c0*H*W*4, 31 - tap index (the left shift that brings the tap's bit of a pixel's outside mask to
    // bit 31), or 0 for an all-padding tile}
    const int2 *ttab; int ksize; unsigned plane_bytes;
};

// Activation of the short epilogue, written as selects on uniform flags so that the epilogue stays one
// straight line of code the scheduler can interleave with its loads.  SLOPED = false knows relu and
// linear; SLOPED = true adds leaky and relie with the predicate and double-precision product of
// nbl_act_apply.
template<bool SLOPED>
__device__ __forceinline__ float conv_cheap_activation(float t, int act) {
    const bool linear = act == NBL_ACT_LINEAR;
    float neg = 0.0f;
    if(SLOPED) {
        const double slope = act == NBL_ACT_RELIE ? 0.01 : 0.1;
        neg = act == NBL_ACT_RELU ? 0.0f : (float)(slope * (double)t);
    }
    const float r = t > 0.0f ? t : neg;
    return linear ? t : r;
}

struct PixelCoord { int xbase; int ih0; int iw0; };

// Pixel column n -> input base offset and top-left tap coordinate.  n >= N gives a coordinate
// that fails every bounds test.
__device__ __forceinline__ PixelCoord conv_pixel(int n, int N, int OHW, int OW, int stride, int pad,
                                                 int CHW, int W, const FastDiv &dohw, const FastDiv &dow) {
    PixelCoord p;
    if(n < N) {
        const int b = (int)dohw.div((unsigned)n), pix = n - b * OHW;
        const int oh = (int)dow.div((unsigned)pix), ow = pix - oh * OW;
        p.ih0 = oh * stride - pad;
        p.iw0 = ow * stride - pad;
        p.xbase = b * CHW + p.ih0 * W + p.iw0;
    } else {
        p.ih0 = -(1 << 30); p.iw0 = 0; p.xbase = 0;
    }
    return p;
}

// True when tap (i, j) of table entry ke falls inside the image for pixel p (the reference's padding
// rule: taps outside read 0).
__device__ __forceinline__ bool conv_tap_inside(const PixelCoord &p, int2 ke, int H, int W) {
    const int ih = p.ih0 + (ke.y >> 16), iw = p.iw0 + (ke.y & 0xffff);
    return (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
}

// One element of the patch matrix.
__device__ __forceinline__ float conv_gather(const float *__restrict__ x, const PixelCoord &p, int2 ke,
                                             int H, int W) {
    return conv_tap_inside(p, ke, H, W) ? x[p.xbase + ke.x] : 0.0f;
}

// Input reads go through a raw buffer descriptor: an offset at or past the end of the tensor returns 0
// in hardware, so "outside the image", "past the last pixel column" and "past the last patch row" all
// become one out-of-range offset and the loads need neither a branch nor a select on their result
// (either would have to wait for the load before the MFMAs of the current tile could start).
constexpr unsigned OOB_OFFSET = 0x80000000u;     // tensors are limited to < 2^31 bytes

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float *p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}
// The range check looks at the per-lane offset only; the scalar offset is added afterwards.  A lane
// whose offset is out of range therefore reads 0 whatever the scalar part is.
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, unsigned byte_off, unsigned uniform_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, (int)uniform_off, 0));
}
__device__ __forceinline__ auto buf_load4(__amdgpu_buffer_rsrc_t r, unsigned byte_off, unsigned uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, (int)uniform_off, 0);
}
// Native 4-float vector: staged tiles move as values (a struct float4 copy can become a memcpy through a
// private-memory slot that is never promoted to registers).
typedef float vec4f __attribute__((ext_vector_type(4)));

// How a block gathers its slice of the patch matrix.
enum { GATHER_PADDED = 0,   // any geometry: every tap is bounds-checked
       GATHER_NOPAD = 1,    // padding = 0: every tap of a real pixel is inside the image
       GATHER_1X1_VEC4 = 2, // 1x1, stride 1, padding 0, OH*OW % 4 == 0, C % 32 == 0: four pixels per 16-byte load
       // Patch rows ordered (c / 16, i, j, c % 16) with C a multiple of the k-tile depth: a k-tile is 16
       // channels of ONE tap, so whether the tap is inside the image is decided once per pixel and k-tile (a bit of a mask
       // computed at block start), and the 16 rows differ by a uniform plane offset that travels in the
       // load's scalar offset.  Per gathered element no address or bounds arithmetic is left.
       GATHER_TAP_MAJOR = 3
};

// OCC = blocks the register budget must leave room for on a CU (the persistent grid is sized with it)
template<int MT, int NT, int WAVES_M, int WAVES_N, int OCC, int GATHER, bool FAST_ACT>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, OCC) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void conv_igemm_kernel(const ConvArgs a) {
    constexpr int BK = CONV_BK;
    constexpr int NTHREADS = 64 * WAVES_M * WAVES_N;
    constexpr int BM = MT * 32 * WAVES_M, BN = NT * 32 * WAVES_N;
    constexpr int LDA = BM + 32, LDB = BN + 32;        // rows k and k+1 land in different bank halves
    constexpr bool VEC4 = GATHER == GATHER_1X1_VEC4, TAPM = GATHER == GATHER_TAP_MAJOR;
    constexpr int NCOLS = VEC4 ? BN / 4 : BN;          // column groups a k row is split into
    static_assert(NTHREADS % NCOLS == 0, "pixel columns must split evenly over threads");
    constexpr int KGROUPS = NTHREADS / NCOLS;          // thread groups along k
    static_assert(BK % KGROUPS == 0, "k rows must split evenly over thread groups");
    constexpr int RB = BK / KGROUPS;                   // k rows gathered per thread
    constexpr int A_VEC = BK * BM / 4;                 // float4s in a weight tile
    constexpr int RA = (A_VEC + NTHREADS - 1) / NTHREADS;
    static_assert(RA <= 2, "weight tile needs at most two float4 per thread");
    // LDS layout of a k-tile.  The table-driven gathers give a thread RB consecutive patch rows of ONE pixel, so their
    // tiles are kept as quads of k: [k / 4][column][k % 4] -- a thread's four rows are one 16-byte LDS write (four
    // 4-byte writes cost the matrix pipe about 4 % in a stand-alone copy of this loop), and a lane fetches its operands
    // of four k-steps with one 16-byte read.  Lanes 0-31 then feed the k of the even quads and lanes 32-63 the k of the
    // odd quads to the MFMAs; any pairing of k is legal as long as both operands use the same one, and the packed
    // weights are laid out to match ([Kp / 4][Mp][4]).  The 1x1 gather loads four PIXELS of one row per thread and
    // keeps k-major rows ([k][column], rows k and k+1 in different bank halves through the +32).
    constexpr bool KQ = !VEC4;
    constexpr int PADQ = 8;                            // quad layout: row pitch (BM + 8) * 16 bytes puts consecutive quads half the banks apart
    static_assert(VEC4 || RB % 4 == 0, "a thread's patch rows must be whole quads");

    __shared__ __attribute__((aligned(16))) float As[KQ ? 2 * (BK / 4) * (BM + PADQ) * 4 : 2 * BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[KQ ? 2 * (BK / 4) * (BN + PADQ) * 4 : 2 * BK * LDB];
    constexpr int A_BUF = KQ ? (BK / 4) * (BM + PADQ) * 4 : BK * LDA;      // floats per buffer
    constexpr int B_BUF = KQ ? (BK / 4) * (BN + PADQ) * 4 : BK * LDB;
    constexpr int A_QROW = (BM + PADQ) * 4, B_QROW = (BN + PADQ) * 4;       // floats between quads (quad layout)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int half = lane >> 5, l32 = lane & 31;

    // which output tile, and which slice of its k-tiles, this block computes (all uniform)
    const int nkt = a.Kp / BK;        // even: Kp is a multiple of 2*BK
    // Workgroups are dealt to the 8 XCDs round robin by index, and each XCD has its own L2.  The work
    // units are therefore renumbered so that a run of tiles_m consecutive units (the filter tiles of one
    // pixel tile, which read the same input) lands on one XCD, and so do xcd_group consecutive runs: neighbouring
    // pixel tiles of a 3x3 layer read each other's rows (every input row of a 56-wide plane is needed by three
    // 64-pixel tiles), and with neighbours on different XCDs each of them fetched those rows from memory again.
    // Groups of runs are dealt round robin in turn.
    int tile;
    {
        const unsigned xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, run_local = a.div_tiles_m.div(slot),
                       within = slot - run_local * (unsigned)a.tiles_m;
        const unsigned gl = (unsigned)a.xcd_group_log2, group_local = run_local >> gl, j = run_local & ((1u << gl) - 1u);
        const unsigned unit = ((((group_local << 3) + xcd) << gl) + j) * (unsigned)a.tiles_m + within;
        if(unit >= (unsigned)a.units) return;         // the grid is padded to whole rounds of groups
        tile = (int)unit;
    }
    const int unit = tile;
    int part = 0, kt_begin = 0, kt_end = nkt;
    if(tile >= a.whole_tiles) {
        const int u = tile - a.whole_tiles, pairs = nkt / 2;
        const int ut = (int)a.div_split.div((unsigned)u);
        tile = a.whole_tiles + ut;
        part = u - ut * a.split;
        kt_begin = 2 * (int)a.div_split.div((unsigned)(part * pairs));
        kt_end = 2 * (int)a.div_split.div((unsigned)((part + 1) * pairs));
    }
    const bool split_block = unit >= a.whole_tiles;

    const __amdgpu_buffer_rsrc_t xres = make_rsrc(a.x, a.x_bytes);
    const int ncol = tid % NCOLS;
    // Scalar modes: one pixel column per thread, RB consecutive k rows, and the k rows of a wave are
    // uniform (NCOLS is a multiple of 64), so the table entries travel through scalar registers.
    // VEC4 mode: four pixel columns per thread, k rows strided by KGROUPS, no table (offset = k * H*W).
    const int kgroup = VEC4 ? tid / NCOLS : __builtin_amdgcn_readfirstlane(tid / NCOLS);
    const int krow0 = VEC4 ? kgroup : kgroup * RB;

    // ---- load side state: the k-tile the next global loads belong to ----
    int ld_kt = kt_begin;
    const int tile_n = (int)a.div_tiles_m.div((unsigned)tile), tile_m = tile - tile_n * a.tiles_m;
    const int ld_m0 = tile_m * BM;
    PixelCoord px;
    unsigned xoff;
    {
        const int n0 = tile_n * BN;
        // VEC4 reads with plain 16-byte global loads, so its addresses must be real: a column group past
        // the last pixel re-reads the last group (its results are never stored), a row past the last patch
        // row re-reads the last row and is zeroed when the tile is written to LDS.
        const int ncol_first = VEC4 ? min(n0 + ncol * 4, a.N - 4) : n0 + ncol;
        px = conv_pixel(ncol_first, a.N, a.OHW, a.OW, a.stride, a.pad, a.CHW, a.W, a.div_ohw, a.div_ow);
        // byte offset of the pixel's top-left tap; a column past the last pixel is out of range for every k
        xoff = px.ih0 > -(1 << 29) ? (unsigned)px.xbase * 4u : OOB_OFFSET;
    }
    // byte offsets of this thread's loads inside one k-tile's slice of the input (1x1 vector mode) and of the
    // packed weights; the k-tile's own offset is uniform and goes into the scalar offset of the buffer loads.
    // (A load through a 64-bit per-lane pointer costs matrix-pipe time for its address arithmetic and issue;
    // a buffer load with a constant vector offset and a scalar k offset costs none.)
    unsigned vec_off[VEC4 ? RB : 1];
    if(VEC4) {
        #pragma unroll
        for(int r = 0; r < RB; r++) vec_off[r] = (unsigned)(px.xbase + (krow0 + r * KGROUPS) * a.OHW) * 4u;
    }
    const __amdgpu_buffer_rsrc_t wres = make_rsrc(a.wp, (unsigned)a.Kp * (unsigned)a.Mp * 4u);
    // weight tile: k-major rows [16][BM] read as float4s along the filters, or quads [4][BM][4] read as one float4 per
    // (quad, filter); either way a thread's piece sits at a constant offset from the k-tile's start
    const unsigned w_off0 = A_VEC >= NTHREADS || tid < A_VEC
        ? (KQ ? (unsigned)((tid / BM) * a.Mp + tid % BM + ld_m0) * 16u
              : (unsigned)((tid / (BM / 4)) * a.Mp + (tid % (BM / 4)) * 4 + ld_m0) * 4u) : OOB_OFFSET;
    const unsigned w_off1 = RA > 1 && (A_VEC >= 2 * NTHREADS || tid + NTHREADS < A_VEC)
        ? (KQ ? (unsigned)(((tid + NTHREADS) / BM) * a.Mp + (tid + NTHREADS) % BM + ld_m0) * 16u
              : (unsigned)(((tid + NTHREADS) / (BM / 4)) * a.Mp + ((tid + NTHREADS) % (BM / 4)) * 4 + ld_m0) * 4u) : OOB_OFFSET;
    // tap-major: bit i*ksize+j is set when that tap of this thread's pixel is OUTSIDE the image; bit 31 is always
    // set and stands for the padding k-tiles behind the last patch row
    unsigned outmask = 0x80000000u;
    if(TAPM) {
        int t = 0;
        for(int i = 0; i < a.ksize; i++)
            for(int j = 0; j < a.ksize; j++, t++)
                if(!((unsigned)(px.ih0 + i) < (unsigned)a.H && (unsigned)(px.iw0 + j) < (unsigned)a.W)) outmask |= 1u << t;
    }

    // Two register stages: the loads of k-tile t+2 are issued while k-tile t is multiplied and t+1 is
    // still in flight, so every global load has two k-tiles of MFMA time to arrive.
    struct Stage {
        float b[VEC4 ? 1 : RB];
        vec4f b4[VEC4 ? RB : 1];
        vec4f a0, a1;
    };
    Stage st0, st1;
    int2 ke[VEC4 || TAPM ? 1 : RB];  // table entries of the next k-tile to gather (tap-major: the k-tile's one entry)

    auto load_ktab = [&](int kt) {
        if(TAPM) {
            ke[0] = a.ttab[kt];
        } else if(!VEC4) {
            const int2 *__restrict__ tp = a.ktab + kt * BK + krow0;
            #pragma unroll
            for(int r = 0; r < RB; r++) ke[r] = tp[r];
        }
    };
    auto load_tile = [&](Stage &st, int kt) {
        if(VEC4) {
            // 1x1: input plane = output plane, patch row k = channel k, and C is a multiple of 32 (no padding
            // rows).  The k-tile's offset is uniform and travels in the scalar offset of the buffer load, the
            // thread's own offset is constant: no vector arithmetic per load.
            const unsigned xk = (unsigned)kt * (unsigned)(BK * sizeof(float)) * (unsigned)a.OHW;
            #pragma unroll
            for(int r = 0; r < RB; r++) st.b4[r] = __builtin_bit_cast(vec4f, buf_load4(xres, vec_off[r], xk));
        } else if(TAPM) {
            // the tap's bit of the outside mask, moved to bit 31, pushes the offset out of range (the pixel's own
            // offset plus the tap's is below 2^31, or already out of range for a column past the last pixel)
            const unsigned off = (xoff + (unsigned)ke[0].x) | ((outmask << (ke[0].y & 31)) & 0x80000000u);
            #pragma unroll
            for(int r = 0; r < RB; r++) st.b[r] = buf_load(xres, off, (unsigned)(krow0 + r) * a.plane_bytes);
        } else {
            #pragma unroll
            for(int r = 0; r < RB; r++) {
                unsigned off = xoff + (unsigned)ke[r].x * 4u;     // stays out of range when xoff is (tables hold < 2^29)
                if(GATHER == GATHER_PADDED) off = conv_tap_inside(px, ke[r], a.H, a.W) ? off : OOB_OFFSET;
                else if(ke[r].y < 0) off = OOB_OFFSET;            // uniform: padding row of the table
                st.b[r] = buf_load(xres, off);
            }
        }
        // weights: the k-tile's uniform offset in the scalar offset, the thread's constant offset in the vector
        // offset (out of range for a thread with nothing to load, which then reads zeros)
        const unsigned wk = (unsigned)kt * (unsigned)(BK * sizeof(float)) * (unsigned)a.Mp;
        st.a0 = __builtin_bit_cast(vec4f, buf_load4(wres, w_off0, wk));
        if(RA > 1) st.a1 = __builtin_bit_cast(vec4f, buf_load4(wres, w_off1, wk));
    };
    // issue the loads of the next k-tile; the table entries of the k-tile after it follow (the tables end
    // in all-padding tiles, so the entry after the last k-tile exists)
    auto ld_next = [&](Stage &st) {
        load_tile(st, ld_kt);
        ++ld_kt;
        load_ktab(ld_kt);
    };
    auto store_tile = [&](const Stage &st, int buf) {
        if(VEC4) {
            #pragma unroll
            for(int r = 0; r < RB; r++) *reinterpret_cast<vec4f*>(&Bs[buf * B_BUF + (krow0 + r * KGROUPS) * LDB + ncol * 4]) = st.b4[r];
        } else {
            #pragma unroll
            for(int q = 0; q < RB / 4; q++)
                *reinterpret_cast<vec4f*>(&Bs[buf * B_BUF + (krow0 / 4 + q) * B_QROW + ncol * 4]) =
                    vec4f{st.b[4 * q], st.b[4 * q + 1], st.b[4 * q + 2], st.b[4 * q + 3]};
        }
        #pragma unroll
        for(int u = 0; u < RA; u++) {
            const int v = tid + u * NTHREADS;
            float *dst = KQ ? &As[buf * A_BUF + (v / BM) * A_QROW + (v % BM) * 4]
                            : &As[buf * A_BUF + (v / (BM / 4)) * LDA + (v % (BM / 4)) * 4];
            if(A_VEC >= (u + 1) * NTHREADS || v < A_VEC) *reinterpret_cast<vec4f*>(dst) = u == 0 ? st.a0 : st.a1;
        }
    };

    floatx16 acc[MT][NT];

    // Rows and columns are dealt to the MFMA tiles of a wave interleaved: tile i of the wave holds rows
    // l*MT + i (l = 0..31) and tile j holds columns l*NT + j.  A lane therefore finds the MT (NT)
    // operand values of one k in adjacent LDS words, and in the epilogue it owns NT adjacent pixels of each of its rows.
    //
    // ALL operands of a k-tile are fetched into registers (8 k-steps x (MT + NT) values): once every wave holds
    // its copy, the tile's LDS buffer is free, so the one barrier per k-tile can sit in the MIDDLE of the tile's
    // MFMAs instead of at their end -- the operands of the next tile are then read from LDS behind the second half of
    // this tile's MFMAs, and no wave starts a tile by waiting for LDS.  (In a stand-alone copy of this loop, 64x64
    // tile, 6 blocks per CU: 81 % of the matrix peak with the barrier at the end of the tile, 88-89 % here.)
    // Operand registers: quad layout -- opa[h][i] holds k-steps 4h..4h+3 of row tile i; k-major layout -- element j
    // of opa[h][i] is k-step 4h + j all the same, fetched with 4-byte reads.
    struct Operands { vec4f a[2][MT]; vec4f b[2][NT]; };
    const int a_lane = KQ ? half * A_QROW + (wm * MT * 32 + l32 * MT) * 4 : half * LDA + wm * MT * 32 + l32 * MT;
    const int b_lane = KQ ? half * B_QROW + (wn * NT * 32 + l32 * NT) * 4 : half * LDB + wn * NT * 32 + l32 * NT;
    // the operands of k-steps 4h..4h+3 of the tile in LDS buffer `buf`
    auto read_half = [&](int buf, int h, vec4f (&oa)[MT], vec4f (&ob)[NT]) {
        if(KQ) {
            const float *ap = &As[buf * A_BUF + a_lane + 2 * h * A_QROW], *bp = &Bs[buf * B_BUF + b_lane + 2 * h * B_QROW];
            #pragma unroll
            for(int i = 0; i < MT; i++) oa[i] = *reinterpret_cast<const vec4f*>(ap + 4 * i);
            #pragma unroll
            for(int j = 0; j < NT; j++) ob[j] = *reinterpret_cast<const vec4f*>(bp + 4 * j);
        } else {
            const float *ap = &As[buf * A_BUF + a_lane + 8 * h * LDA], *bp = &Bs[buf * B_BUF + b_lane + 8 * h * LDB];
            #pragma unroll
            for(int e = 0; e < 4; e++) {
                #pragma unroll
                for(int i = 0; i < MT; i++) oa[i][e] = ap[e * 2 * LDA + i];
                #pragma unroll
                for(int j = 0; j < NT; j++) ob[j][e] = bp[e * 2 * LDB + j];
            }
        }
    };
    // MFMAs of k-steps [s0, s1) of the tile whose operands are in `o`
    auto mfma_steps = [&](const Operands &o, auto s0_, auto s1_) {
        constexpr int s0 = decltype(s0_)::value, s1 = decltype(s1_)::value;
        #pragma unroll
        for(int ks = s0; ks < s1; ks++)
            #pragma unroll
            for(int i = 0; i < MT; i++)
                #pragma unroll
                for(int j = 0; j < NT; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(o.a[ks / 4][i][ks % 4], o.b[ks / 4][j][ks % 4], acc[i][j], 0, 0, 0);
    };
    constexpr int KS_BEFORE = MT * NT >= 2 ? 1 : 2;       // k-steps multiplied before the barrier
    typedef std::integral_constant<int, 0> ks_first;
    typedef std::integral_constant<int, KS_BEFORE> ks_split;
    typedef std::integral_constant<int, BK / 2> ks_last;
    Operands cur;
    // One k-tile: `cur` holds its operands; `st` holds the next k-tile, which goes to LDS buffer `buf`.
    auto tile_step = [&](const Stage &st, int buf) {
        mfma_steps(cur, ks_first(), ks_split());
        __builtin_amdgcn_sched_barrier(0);
        store_tile(st, buf);
        __syncthreads();
        vec4f na[MT], nb[NT];
        read_half(buf, 0, na, nb);                  // next tile's first half, in flight behind the MFMAs below
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(cur, ks_split(), ks_last());
        __builtin_amdgcn_sched_barrier(0);
        #pragma unroll
        for(int i = 0; i < MT; i++) cur.a[0][i] = na[i];
        #pragma unroll
        for(int j = 0; j < NT; j++) cur.b[0][j] = nb[j];
        read_half(buf, 1, cur.a[1], cur.b[1]);      // needed four k-steps into the next tile
    };

    // Short epilogue of a full tile whose rows are reached as base pointer + 32-bit byte offset: per row
    // one integer add besides the arithmetic.  An instruction spent here is an instruction the matrix
    // pipe waits for, which is most of what a layer with few patch rows does.  The per-filter scale is
    // always applied (it is 1.0 where the layer has no batch normalisation, and acc * 1 + b rounds as
    // acc + b does).
    // (forced inline: called from four places, and as a real call it would take the accumulators through memory)
    typedef float __attribute__((ext_vector_type(NT))) pixvec;
    // Tiles of up to 64 accumulator registers per lane request their residual rows before the last two k-tiles
    // (prefetch_residual) and hand them to the epilogue in registers; larger tiles have no registers to spare for that
    // (they spill) and load them in the epilogue, one group of rows ahead.
    constexpr bool PREFETCH_RES = MT * NT <= 2;
    constexpr int NPRE = PREFETCH_RES ? 16 * MT : 1;
    auto short_epilogue = [&](auto sloped, auto with_residual, int f_lane, unsigned yoff, unsigned roff, unsigned res_pitch,
                              const pixvec (&rpre)[NPRE], int act, int post_act) __attribute__((always_inline)) {
        // sloped: 0 relu / linear through selects on uniform flags, 1 leaky / relie as well, 2 the ReLU network's two
        //         cases resolved at compile time: relu without a residual, or linear + residual + relu (one max each)
        // with_residual: 0 none, 1 rows res_pitch bytes apart from byte offset roff (in rpre already when PREFETCH_RES)
        constexpr bool SLOPED = decltype(sloped)::value == 1, RELU_NET = decltype(sloped)::value == 2,
                       RES = decltype(with_residual)::value != 0;
        const unsigned row_bytes = (unsigned)a.OHW * 4u;
        const __amdgpu_buffer_rsrc_t rres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(RES ? a.res : a.y), 0, (int)0xffffffffu, 0x00020000);
        // Output rows (and residual rows) go through buffer descriptors: the lane's own offset is a constant vector
        // offset, the row's offset is uniform and rides in the scalar offset -- no address arithmetic per row.  (Both
        // tensors are below 4 GiB here, which is what selects this epilogue.)
        const __amdgpu_buffer_rsrc_t yres = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, (int)0xffffffffu, 0x00020000);
        // per-filter constants one group of rows ahead of their use
        vec4f gv[2][MT], bv[2][MT];
        auto load_constants = [&](int q) {
            #pragma unroll
            for(int u = 0; u < MT; u++) {
                gv[q & 1][u] = *reinterpret_cast<const vec4f*>(a.g + f_lane + q * 8 * MT + 4 * u);
                bv[q & 1][u] = *reinterpret_cast<const vec4f*>(a.b + f_lane + q * 8 * MT + 4 * u);
            }
        };
        load_constants(0);
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            if(q + 1 < 4) load_constants(q + 1);
            pixvec rv[4 * MT];
            if(RES) {
                #pragma unroll
                for(int e = 0; e < 4 * MT; e++) {
                    if constexpr(PREFETCH_RES) {
                        rv[e] = rpre[q * 4 * MT + e];
                    } else {
                        const unsigned row = (unsigned)(q * 8 * MT + e) * res_pitch;       // uniform
                        if constexpr(NT == 1) rv[e][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rres, (int)roff, (int)row, 0));
                        else rv[e] = __builtin_bit_cast(pixvec, __builtin_amdgcn_raw_buffer_load_b64(rres, (int)roff, (int)row, 0));
                    }
                }
            }
            #pragma unroll
            for(int e = 0; e < 4 * MT; e++) {
                const int rr = e / MT, i = e % MT;
                const float ge = gv[q & 1][e / 4][e % 4], be = bv[q & 1][e / 4][e % 4];
                pixvec o;
                #pragma unroll
                for(int j = 0; j < NT; j++) {
                    const float t = __builtin_fmaf(acc[i][j][q * 4 + rr], ge, be);
                    if(RELU_NET) {
                        const float u = RES ? __fadd_rn(t, rv[e][j]) : t;
                        o[j] = u > 0.0f ? u : 0.0f;
                    } else {
                        o[j] = conv_cheap_activation<SLOPED>(t, act);
                        if(RES) o[j] = conv_cheap_activation<SLOPED>(__fadd_rn(o[j], rv[e][j]), post_act);
                    }
                }
                const unsigned row = (unsigned)(q * 8 * MT + e) * row_bytes;       // uniform
                typedef int __attribute__((ext_vector_type(2))) int2v;
                if constexpr(NT == 1) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, o[0]), yres, (int)yoff, (int)row, 0);
                else __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(int2v, o), yres, (int)yoff, (int)row, 0);
            }
        }
    };

    // Where a finished tile goes, decided before the last two k-tiles are multiplied so that the residual rows of a
    // fused shortcut can be requested then and arrive under that work instead of after it.
    // Short epilogue: every filter row of the tile exists, the lane's NT pixels are one aligned
    // vector (OH*OW even keeps pairs inside one image), and rows are reached as base pointer +
    // 32-bit offset, so a row costs one integer add besides its arithmetic.  An instruction spent
    // here is an instruction the matrix pipe waits for, which is what layers with few patch rows
    // are made of.
    // A fused shortcut with fewer channels than filters gives a tile's rows a residual either all or not at
    // all (mixed tiles take the general path); a tile without one applies the two activations in a row, which
    // is one activation when either is linear.  A strided or larger connection is read at its own row pitch;
    // pairs of pixels (NT = 2) are one vector of it only at stride 1 and equal width.
    struct EpiloguePlan {
        bool lane_live, use_short, tile_res;
        int f_lane, act, post_act;
        unsigned yoff, roff, res_pitch;       // byte offsets of the lane's first row; bytes between residual rows
    };
    auto plan_epilogue = [&]() {
        EpiloguePlan p;
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        const int nbase = n0 + wn * NT * 32 + l32 * NT;
        p.lane_live = nbase < a.N;
        const int nb = p.lane_live ? nbase : 0;
        const int b0 = (int)a.div_ohw.div((unsigned)nb), pix0 = nb - b0 * a.OHW;
        p.tile_res = a.res != NULL && m0 + BM <= a.res_c;
        const bool tile_plain = a.res == NULL || m0 >= a.res_c;
        p.use_short = FAST_ACT && a.short_epilogue && m0 + BM <= a.F && (NT == 1 || (a.OHW & 1) == 0) && (p.tile_res || tile_plain) &&
                      (!p.tile_res || NT == 1 || (a.res_stride == 1 && a.res_hw == a.OHW)) &&
                      (!tile_plain || a.res == NULL || a.act == NBL_ACT_LINEAR || a.post_act == NBL_ACT_LINEAR);
        p.f_lane = m0 + wm * MT * 32 + half * 4 * MT;
        p.yoff = ((unsigned)(b0 * a.F + p.f_lane) * (unsigned)a.OHW + (unsigned)pix0) * 4u;
        p.roff = p.yoff;
        p.res_pitch = (unsigned)a.OHW * 4u;
        p.act = a.act; p.post_act = a.post_act;
        if(p.tile_res) {
            const bool res_same_shape = a.res_c == a.F && a.res_hw == a.OHW && a.res_stride == 1;   // uniform
            if(!res_same_shape) {
                unsigned rpix = (unsigned)pix0;
                if(a.res_hw != a.OHW || a.res_stride != 1) {
                    const int h = (int)a.div_ow.div((unsigned)pix0), w = pix0 - h * a.OW;
                    rpix = (unsigned)(h * a.res_stride * a.res_w + w * a.res_stride);
                }
                p.roff = ((unsigned)(b0 * a.res_c + p.f_lane) * (unsigned)a.res_hw + rpix) * 4u;
                p.res_pitch = (unsigned)a.res_hw * 4u;
            }
        } else if(a.res != NULL) {
            p.act = a.act == NBL_ACT_LINEAR ? a.post_act : a.act;
            p.post_act = NBL_ACT_LINEAR;
        }
        return p;
    };
    // The 16 * MT residual rows of this lane (row q * 8 * MT + e of the lane's filters sits in entry q * 4 * MT + e).
    // A block reads only the residual of the tile it writes itself, so an output written over the connection is safe.
    auto prefetch_residual = [&](const EpiloguePlan &p, pixvec (&rpre)[NPRE]) {
        if(!PREFETCH_RES || !(p.lane_live && p.use_short && p.tile_res)) return;
        const __amdgpu_buffer_rsrc_t rres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.res), 0, (int)0xffffffffu, 0x00020000);
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            #pragma unroll
            for(int e = 0; e < 4 * MT; e++) {
                const unsigned row = (unsigned)(q * 8 * MT + e) * p.res_pitch;       // uniform
                constexpr int at = PREFETCH_RES ? 4 * MT : 0;       // (keeps the index inside the one-entry array of the other case)
                if constexpr(NT == 1) rpre[q * at + (PREFETCH_RES ? e : 0)][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rres, (int)p.roff, (int)row, 0));
                else rpre[q * at + (PREFETCH_RES ? e : 0)] = __builtin_bit_cast(pixvec, __builtin_amdgcn_raw_buffer_load_b64(rres, (int)p.roff, (int)row, 0));
            }
        }
    };

    // Epilogue of one finished output tile: y = act(acc * g[f] + b[f]) (+ fused shortcut).
    // Accumulator register r of a 32x32 MFMA tile holds tile row 8*(r/4) + 4*(lane/32) + r%4 and tile
    // column lane%32; with the interleaving above that is filter row*MT + i and pixel (lane%32)*NT + j
    // of the wave's sub-tile.
    auto epilogue = [&](const EpiloguePlan &p, const pixvec (&rpre)[NPRE]) {
        if(!p.lane_live) return;
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        const int nbase = n0 + wn * NT * 32 + l32 * NT;
        const int b0 = (int)a.div_ohw.div((unsigned)nbase), pix0 = nbase - b0 * a.OHW;
        if constexpr(FAST_ACT) if(p.use_short) {       // (the host selects the short epilogue for the cheap activations only)
            typedef std::integral_constant<int, 0> no_res;
            typedef std::integral_constant<int, 1> with_res;
            typedef std::integral_constant<int, 0> flags; typedef std::integral_constant<int, 1> slopes; typedef std::integral_constant<int, 2> relu_net;
            // (uniform) the two forms a ReLU network's layers take: relu alone, or linear + residual + relu
            const bool is_relu_net = a.short_epilogue == 1 && (p.tile_res ? p.act == NBL_ACT_LINEAR && p.post_act == NBL_ACT_RELU
                                                                          : p.act == NBL_ACT_RELU && p.post_act == NBL_ACT_LINEAR);
            if(is_relu_net) {
                if(!p.tile_res) short_epilogue(relu_net(), no_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
                else short_epilogue(relu_net(), with_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
            } else if(a.short_epilogue == 1) {
                if(!p.tile_res) short_epilogue(flags(), no_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
                else short_epilogue(flags(), with_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
            } else {
                if(!p.tile_res) short_epilogue(slopes(), no_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
                else short_epilogue(slopes(), with_res(), p.f_lane, p.yoff, p.roff, p.res_pitch, rpre, p.act, p.post_act);
            }
            return;
        }
        // the NT pixels of this lane are contiguous in memory when they sit in one image; then (and when
        // the address is 8-byte aligned) a pair is written as one 64-bit store
        const bool pair_ok = NT == 2 && pix0 + 1 < a.OHW && ((pix0 | a.OHW) & 1) == 0;
        float *__restrict__ ybase = a.y + (size_t)b0 * a.F * a.OHW + pix0;
        // fused shortcut: per pixel of this lane, where its residual sits and whether it has one
        int roff[NT]; bool rok[NT];
        #pragma unroll
        for(int j = 0; j < NT; j++) { roff[j] = 0; rok[j] = false; }
        if(a.res) {
            #pragma unroll
            for(int j = 0; j < NT; j++) {
                const int n = nbase + j;
                if(n < a.N) {
                    const int b = n / a.OHW, pix = n - b * a.OHW;
                    const int h = pix / a.OW, w = pix - h * a.OW;
                    rok[j] = h < a.res_box_h && w < a.res_box_w;
                    roff[j] = b * a.res_c * a.res_hw + h * a.res_stride * a.res_w + w * a.res_stride;
                }
            }
        }
        const float *__restrict__ res = a.res;
        // residuals of a lane's NT pixels are adjacent when the shortcut keeps the spatial size: one 64-bit load
        const bool res_pair = res && pair_ok && rok[0] && rok[NT - 1] && roff[NT - 1] == roff[0] + 1 &&
                              ((roff[0] | a.res_hw) & 1) == 0;
        // One group of four accumulator registers (4*MT consecutive filters of this lane) at a time, so the
        // epilogue's temporaries stay few next to the load stages that are live across it.  The group's
        // per-filter constants are 4*MT consecutive entries of the zero-padded g and b vectors; the
        // residuals of group q+1 are requested before group q is combined and stored, so residual reads
        // and output writes overlap.
        float rv[2][4 * MT][NT];
        auto load_residuals = [&](int q, int slot) {
            const int fq = m0 + wm * MT * 32 + (q * 8 + half * 4) * MT;
            #pragma unroll
            for(int e = 0; e < 4 * MT; e++) {
                const int f = fq + e;
                #pragma unroll
                for(int j = 0; j < NT; j++) rv[slot][e][j] = 0.0f;
                if(f < a.F && f < a.res_c) {
                    if(res_pair) {
                        const float2 t = *reinterpret_cast<const float2*>(res + roff[0] + f * a.res_hw);
                        rv[slot][e][0] = t.x; rv[slot][e][NT - 1] = t.y;
                    } else {
                        #pragma unroll
                        for(int j = 0; j < NT; j++) if(rok[j]) rv[slot][e][j] = res[roff[j] + f * a.res_hw];
                    }
                }
            }
        };
        if(res) load_residuals(0, 0);
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            const int fq = m0 + wm * MT * 32 + (q * 8 + half * 4) * MT;
            const int slot = q & 1;
            if(res && q + 1 < 4) load_residuals(q + 1, slot ^ 1);
            if(fq >= a.F) continue;
            float gq[4 * MT], bq[4 * MT];
            #pragma unroll
            for(int v = 0; v < MT; v++) {
                const float4 bb = *reinterpret_cast<const float4*>(a.b + fq + 4 * v);
                bq[4 * v] = bb.x; bq[4 * v + 1] = bb.y; bq[4 * v + 2] = bb.z; bq[4 * v + 3] = bb.w;
                if(a.has_scale) {
                    const float4 gg = *reinterpret_cast<const float4*>(a.g + fq + 4 * v);
                    gq[4 * v] = gg.x; gq[4 * v + 1] = gg.y; gq[4 * v + 2] = gg.z; gq[4 * v + 3] = gg.w;
                }
            }
            #pragma unroll
            for(int rr = 0; rr < 4; rr++) {
                #pragma unroll
                for(int i = 0; i < MT; i++) {
                    const int e = rr * MT + i, r = q * 4 + rr;
                    const int f = fq + e;
                    if(f >= a.F) continue;
                    const float bf = bq[e], gf = a.has_scale ? gq[e] : 1.0f;
                    float v[NT];
                    #pragma unroll
                    for(int j = 0; j < NT; j++) {
                        float t = acc[i][j][r];
                        t = __builtin_fmaf(t, gf, bf);   // gf = 1: rounds as t + bf
                        if(FAST_ACT) {
                            // relu / linear / leaky / relie: no transcendental, same predicates as nbl_act_apply
                            if(a.act == NBL_ACT_RELU) t = t > 0.0f ? t : 0.0f;
                            else if(a.act == NBL_ACT_LEAKY) t = t > 0.0f ? t : (float)(0.1 * (double)t);
                            else if(a.act == NBL_ACT_RELIE) t = t > 0.0f ? t : (float)(0.01 * (double)t);
                        } else {
                            t = nbl_act_apply(a.act, t);
                        }
                        v[j] = t;
                    }
                    if(res) {
                        #pragma unroll
                        for(int j = 0; j < NT; j++) {
                            // an element without a residual keeps its value: adding a 0.0f placeholder would turn -0 into +0
                            float t = (f < a.res_c && rok[j]) ? __fadd_rn(v[j], rv[slot][e][j]) : v[j];
                            if(FAST_ACT) {
                                if(a.post_act == NBL_ACT_RELU) t = t > 0.0f ? t : 0.0f;
                                else if(a.post_act == NBL_ACT_LEAKY) t = t > 0.0f ? t : (float)(0.1 * (double)t);
                                else if(a.post_act == NBL_ACT_RELIE) t = t > 0.0f ? t : (float)(0.01 * (double)t);
                            } else {
                                t = nbl_act_apply(a.post_act, t);
                            }
                            v[j] = t;
                        }
                    }
                    if(pair_ok) {
                        *reinterpret_cast<float2*>(ybase + (size_t)f * a.OHW) = make_float2(v[0], v[NT - 1]);
                    } else {
                        #pragma unroll
                        for(int j = 0; j < NT; j++) {
                            const int n = nbase + j;
                            if(n < a.N) {
                                const int b = n / a.OHW, pix = n - b * a.OHW;
                                a.y[((size_t)b * a.F + f) * a.OHW + pix] = v[j];
                            }
                        }
                    }
                }
            }
        }
    };

    // Raw sums of a split block: ws[part][f][n - n_start], the lane's NT pixels as one vector where aligned.
    auto store_partial = [&]() {
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        const int nbase = n0 + wn * NT * 32 + l32 * NT;
        if(nbase >= a.N) return;
        float *__restrict__ wsp = a.ws + (size_t)part * a.F * a.n_tail + (nbase - a.n_start);
        const bool vec_ok = NT == 2 && nbase + 1 < a.N && (a.n_tail & 1) == 0;
        #pragma unroll
        for(int r = 0; r < 16; r++) {
            #pragma unroll
            for(int i = 0; i < MT; i++) {
                const int f = m0 + wm * MT * 32 + (8 * (r / 4) + 4 * half + r % 4) * MT + i;
                if(f >= a.F) continue;
                float *dst = wsp + (size_t)f * a.n_tail;
                if(vec_ok) {
                    *reinterpret_cast<float2*>(dst) = make_float2(acc[i][0][r], acc[i][NT - 1][r]);
                } else {
                    #pragma unroll
                    for(int j = 0; j < NT; j++) if(nbase + j < a.N) dst[j] = acc[i][j][r];
                }
            }
        }
    };

    // ---- pipeline start: the block's first two k-tiles ----
    st0.a0 = st0.a1 = st1.a0 = st1.a1 = vec4f{0.f, 0.f, 0.f, 0.f};
    load_ktab(kt_begin);
    ld_next(st0);
    ld_next(st1);
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int j = 0; j < NT; j++)
            #pragma unroll
            for(int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    store_tile(st0, 0);
    __syncthreads();
    read_half(0, 0, cur.a[0], cur.b[0]);
    read_half(0, 1, cur.a[1], cur.b[1]);

    for(int kt = kt_begin; kt < kt_end - 2; kt += 2) {
        // operands of k-tile kt are in registers, kt+1 is in flight in stage 1
        ld_next(st0);
        tile_step(st1, 1);
        // operands of k-tile kt+1 are in registers, kt+2 is in flight in stage 0
        ld_next(st1);
        tile_step(st0, 0);
    }
    // last pair: nothing left to load but the residual rows the epilogue will add
    pixvec rpre[NPRE];
    EpiloguePlan plan;
    if(!split_block) {
        plan = plan_epilogue();
        prefetch_residual(plan, rpre);
    }
    tile_step(st1, 1);
    mfma_steps(cur, ks_first(), ks_last());
    if(split_block) store_partial();
    else epilogue(plan, rpre);
}

// Second half of a k-split convolution: adds the parts in order and applies the epilogue the whole-tile
// blocks apply themselves.  One thread per filter and VEC adjacent pixel columns of the split region (VEC = 4
// needs the region's width to be a multiple of 4).  All parts are requested before the first is added -- there are
// at most 8, and a part index past the count re-reads the last part instead of branching -- so the kernel is one
// memory round trip, not one per part.  VSTORE: the thread's pixels are one aligned vector of one output plane
// (OH*OW % 4 == 0); otherwise each pixel finds its own place.
template<int VEC, bool VSTORE>
__global__ void conv_split_finish_kernel(const ConvArgs a) {
    typedef float __attribute__((ext_vector_type(VEC))) vec;
    const int nloc = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    const int f = blockIdx.y;
    if(nloc >= a.n_tail) return;
    const size_t part_elems = (size_t)a.F * a.n_tail, at = (size_t)f * a.n_tail + nloc;
    vec part[8];
    #pragma unroll
    for(int p = 0; p < 8; p++) part[p] = *reinterpret_cast<const vec*>(a.ws + (size_t)min(p, a.split - 1) * part_elems + at);
    vec t = part[0];
    #pragma unroll
    for(int p = 1; p < 8; p++) {
        if(p < a.split) {
            #pragma unroll
            for(int e = 0; e < VEC; e++) t[e] = __fadd_rn(t[e], part[p][e]);
        }
    }
    const float g = a.g[f], bias = a.b[f];
    const int n0 = a.n_start + nloc;
    int b = n0 / a.OHW, pix = n0 - b * a.OHW;
    #pragma unroll
    for(int e = 0; e < VEC; e++) {
        float v = nbl_act_apply(a.act, __builtin_fmaf(t[e], g, bias));
        if(a.res) {
            const int h = pix / a.OW, w = pix - h * a.OW;
            if(f < a.res_c && h < a.res_box_h && w < a.res_box_w)
                v = __fadd_rn(v, a.res[((size_t)b * a.res_c + f) * a.res_hw + h * a.res_stride * a.res_w + w * a.res_stride]);
            v = nbl_act_apply(a.post_act, v);
        }
        if(VSTORE) t[e] = v;
        else a.y[((size_t)b * a.F + f) * a.OHW + pix] = v;
        if(++pix == a.OHW) { pix = 0; ++b; }       // the next pixel may belong to the next image
    }
    if(VSTORE) {
        b = n0 / a.OHW; pix = n0 - b * a.OHW;
        *reinterpret_cast<vec*>(a.y + ((size_t)b * a.F + f) * a.OHW + pix) = t;
    }
}

__global__ void im2col_kernel(const float *__restrict__ x, const int2 *__restrict__ ktab, float *__restrict__ col,
                              int K, int H, int W, int OW, int OHW, int stride, int pad, FastDiv dohw, FastDiv dow) {
    const int pix = blockIdx.x * blockDim.x + threadIdx.x;
    const int kk = blockIdx.y;
    if(pix >= OHW || kk >= K) return;
    const PixelCoord p = conv_pixel(pix, OHW, OHW, OW, stride, pad, 0, W, dohw, dow);
    col[(size_t)kk * OHW + pix] = conv_gather(x, p, ktab[kk], H, W);
}

// Row of the packed patch matrix that holds channel c, tap t = i*k + j.  Reference order (the row
// order of the reference's col matrix): (c*k + i)*k + j.  Tap-major order: channels in groups of the
// k-tile depth, within a group the taps, within a tap the group's channels, so that a k-tile is 16
// channels of one tap and the k-tiles that follow revisit the same 16 input planes for the other taps
// while they are still in cache.
inline unsigned patch_row(unsigned c, unsigned t, unsigned taps, bool tap_major) {
    return tap_major ? (c / CONV_BK) * (taps * CONV_BK) + t * CONV_BK + c % CONV_BK : c * taps + t;
}

// One entry per patch row, in packed order.
std::vector<int2> build_ktab(unsigned C, unsigned H, unsigned W, unsigned k, unsigned Kp, bool tap_major = false) {
    std::vector<int2> tab(Kp);
    for(unsigned kk = 0; kk < Kp; kk++) {
        tab[kk].x = 0;
        tab[kk].y = (int)0x80000000u | (KTAB_PAD_TAP << 16);   // sign bit: padding row
    }
    for(unsigned c = 0; c < C; c++)
        for(unsigned i = 0; i < k; i++)
            for(unsigned j = 0; j < k; j++) {
                const unsigned kk = patch_row(c, i * k + j, k * k, tap_major);
                tab[kk].x = (int)(c * H * W + i * W + j);
                tab[kk].y = (int)((i << 16) | j);
            }
    return tab;
}

// Tap-major layers: one entry per k-tile (see ConvArgs::ttab).
std::vector<int2> build_ttab(unsigned C, unsigned H, unsigned W, unsigned k, unsigned tiles) {
    std::vector<int2> tab(tiles);
    const unsigned taps = k * k, K = C * taps;
    for(unsigned kt = 0; kt < tiles; kt++) {
        if(kt * CONV_BK < K) {
            const unsigned t = kt % taps, c0 = kt / taps * CONV_BK, i = t / k, j = t % k;
            tab[kt].x = (int)((c0 * H * W + i * W + j) * 4);
            tab[kt].y = (int)(31 - t);      // shift that brings the tap's bit of the outside mask to bit 31
        } else {
            tab[kt].x = 0; tab[kt].y = 0;   // padding tile: bit 31 of the mask, which is always set
        }
    }
    return tab;
}

typedef void (*ConvKernel)(const ConvArgs);
// kernel[gather mode][any activation ? 1 : 0]
struct Variant { int bm, bn, threads, blocks_per_cu; ConvKernel kernel[4][2]; const char *name; };

// blocks_per_cu: resident blocks per CU (register- and LDS-limited), the size of the persistent grid
#define NBL_CONV_VARIANT(MT, NT, WM, WN, OCC, NAME) \
    { MT * 32 * WM, NT * 32 * WN, 64 * WM * WN, OCC, \
      { { conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_PADDED, true>, conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_PADDED, false> }, \
        { conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_NOPAD, true>, conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_NOPAD, false> }, \
        { conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_1X1_VEC4, true>, conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_1X1_VEC4, false> }, \
        { conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_TAP_MAJOR, true>, conv_igemm_kernel<MT, NT, WM, WN, OCC, GATHER_TAP_MAJOR, false> } }, \
      NAME }

const Variant VARIANTS[] = {
    NBL_CONV_VARIANT(2, 2, 2, 2, 3, "128x128"),
    NBL_CONV_VARIANT(2, 2, 1, 4, 2, "64x256"),
    NBL_CONV_VARIANT(3, 2, 1, 4, 2, "96x256"),
    NBL_CONV_VARIANT(1, 2, 2, 2, 4, "64x128"),
    NBL_CONV_VARIANT(1, 1, 2, 2, 6, "64x64"),
    NBL_CONV_VARIANT(2, 1, 2, 2, 4, "128x64"),
};
constexpr int NUM_VARIANTS = sizeof(VARIANTS) / sizeof(VARIANTS[0]);

}  // namespace

struct nbl_conv_plan {
    unsigned C, H, W, F, k, stride, pad, OH, OW, K, Kp, Mp;
    int act; bool has_scale;
    float *wp_dev;      // packed weights as quads of patch rows, [Kp / 4][Mp][4] (every gather but the 1x1 vector gather)
    float *wp_rows_dev; // the same as k-major rows [Kp][Mp], kept only for layers the 1x1 vector gather can take
    int2 *ktab_dev; float *g_dev; float *b_dev;
    bool tap_major; int2 *ttab_dev;   // patch rows in (c / 16, i, j, c % 16) order, with a per-k-tile table (C % 16 == 0, 1 < k*k <= 31)
    int variant;   // < 0: chosen per call
    unsigned tuned_batch; int tuned_variant;   // the launch chosen for the last (batch, residual) seen: from the table or the tile search
    std::array<unsigned, 4> tuned_res;         // ... the residual it was chosen for: {channels, height, width, written in place}, zeros without one
    int launch_source;                         // NBL_LAUNCH_* of the most recent launch
    int split_mode;             // k-split of under-filled launches: -1 measured with the tile search, 0 never, 1 whenever the model below says so, 2..8 always with that many slices
    int tuned_slices;           // 0 = unsplit, 1 = the cost model's slice count, 2..8 = that many
    float *ws_dev; size_t ws_bytes;   // partial sums of split launches (grown on demand)
    int last_variant, last_split;     // what the most recent launch used
    nbl_strip_plan strip;             // layers with very few input channels: the kernel of conv_strip.hip, variant index NUM_VARIANTS
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

// Which tiles of a launch are split along k, and into how many parts.  Blocks are dealt to CUs round
// robin, so a launch takes as long as the CU with the most tiles: ceil(tiles / CUs) tile times, however
// few tiles the last round holds.  The tiles of that last round (whole pixel-tile columns, so that the
// split region is one range of pixel columns) are cut into `split` k-slices each so that they spread
// over the idle CUs; the price is writing and re-reading the partial sums and one more small launch.
struct SplitPlan { int whole_tiles, split; };

// forced: 0 = the cost model chooses the slice count, 2..8 = that many slices (fewer if the patch rows run out)
SplitPlan plan_split(int tiles_m, int tiles_n, int bm, int bn, unsigned Kp, unsigned F, unsigned N, int num_cu, int forced = 0) {
    const int tiles = tiles_m * tiles_n, pairs = (int)(Kp / (2 * CONV_BK));
    SplitPlan none = { tiles, 1 };
    int whole = tiles / num_cu * num_cu;
    whole -= whole % tiles_m;
    const int left = tiles - whole;
    if(left == 0 || pairs < 2) return none;
    const double tile_us = 2.0 * bm * bn * Kp / (100e12 / num_cu) * 1e6;     // one CU, one tile, at a realistic rate
    double best_us = std::ceil((double)left / num_cu) * tile_us;
    int best = 1;
    const size_t n_tail = N - (size_t)(whole / tiles_m) * bn;
    for(int g = 2; g <= 8 && g <= pairs; g++) {
        const size_t ws_bytes = (size_t)g * F * n_tail * sizeof(float);
        if(ws_bytes > ((size_t)1 << 30)) break;
        const double us = std::ceil((double)left * g / num_cu) / g * tile_us + 2.0 * ws_bytes / 4e12 * 1e6 + 5.0;
        if(us < best_us) { best_us = us; best = g; }
    }
    if(forced >= 2) {
        best = forced < pairs ? forced : pairs;
        if((size_t)best * F * n_tail * sizeof(float) > ((size_t)1 << 30)) return none;
    }
    if(best == 1) return none;
    SplitPlan sp = { whole, best };
    return sp;
}


// ---- launch table --------------------------------------------------------------------------------------------------
// Which tile shape and how many k slices a convolution launches with is a property of the problem -- geometry, batch,
// and the residual a fused shortcut adds -- so it is kept in a process-wide table keyed by exactly that.  The table
// starts from a text file (one line per problem, written by nbl_launch_table_save after a run that measured them);
// a problem the file does not list is measured once (conv_tune) and entered, so that every later plan of the same
// problem launches the same way, and nbl_launch_table_save can write the grown table out for the next process.
//   line:  conv C H W F k stride pad batch res_c res_h res_w in_place tile slices [us]
//   tile = a name nbl_conv2d_variant_name returns; slices = 0 (unsplit) or 2..8; us = the time measured when the
//   entry was made (information only).  '#' starts a comment.
typedef std::array<unsigned, 12> LaunchKey;     // C H W F k stride pad batch res_c res_h res_w in_place
struct LaunchChoice { int variant; int slices; float us; bool from_file; };

std::mutex g_table_lock;
std::map<LaunchKey, LaunchChoice> g_table;
bool g_table_initialised = false;       // the default file has been looked for
bool g_search_enabled = true;           // problems the table does not list are measured (false: cost model only)

int variant_by_name(const char *name) {
    for(int v = 0; v < NUM_VARIANTS; v++) if(strcmp(VARIANTS[v].name, name) == 0) return v;
    return strcmp(name, "strip") == 0 ? NUM_VARIANTS : -1;
}

// <directory of this shared library>/../launch_tables/gfx950.txt
std::string default_table_path() {
    Dl_info info;
    if(!dladdr((const void*)&variant_by_name, &info) || !info.dli_fname) return std::string();
    std::string lib(info.dli_fname);
    const size_t slash = lib.rfind('/');
    const std::string dir = slash == std::string::npos ? std::string(".") : lib.substr(0, slash);
    return dir + "/../launch_tables/gfx950.txt";
}

// Reads a table file into `out`; returns the number of entries or -1 when the file cannot be opened or a line
// is malformed (`bad_line` then holds its number).
int read_table_file(const char *path, std::map<LaunchKey, LaunchChoice> &out, int *bad_line) {
    FILE *f = fopen(path, "r");
    *bad_line = 0;
    if(!f) return -1;
    char line[512];
    int n = 0, lineno = 0;
    while(fgets(line, sizeof(line), f)) {
        lineno++;
        char *hash = strchr(line, '#');
        if(hash) *hash = 0;
        char *q = line;
        while(*q == ' ' || *q == '\t' || *q == '\n' || *q == '\r') q++;
        if(!*q) continue;
        LaunchKey key; char tile[32]; int slices = 0; float us = 0.0f;
        const int got = sscanf(q, "conv %u %u %u %u %u %u %u %u %u %u %u %u %31s %d %f", &key[0], &key[1], &key[2], &key[3], &key[4],
                               &key[5], &key[6], &key[7], &key[8], &key[9], &key[10], &key[11], tile, &slices, &us);
        const int v = got >= 14 ? variant_by_name(tile) : -1;
        if(got < 14 || v < 0 || slices < 0 || slices == 1 || slices > 8) { *bad_line = lineno; fclose(f); return -1; }
        LaunchChoice c = { v, slices, got >= 15 ? us : 0.0f, true };
        out[key] = c;
        n++;
    }
    fclose(f);
    return n;
}

// First use: the file NBL_LAUNCH_TABLE names ("none": no file), else the one shipped next to the library.  A file
// that is missing or malformed leaves the table empty -- every problem is then measured -- and is not an error.
void table_initialise_locked() {
    if(g_table_initialised) return;
    g_table_initialised = true;
    const char *search = getenv("NBL_CONV_SEARCH");
    if(search && strcmp(search, "0") == 0) g_search_enabled = false;
    const char *env = getenv("NBL_LAUNCH_TABLE");
    if(env && strcmp(env, "none") == 0) return;
    const std::string path = env && *env ? std::string(env) : default_table_path();
    if(path.empty()) return;
    std::map<LaunchKey, LaunchChoice> t;
    int bad = 0;
    if(read_table_file(path.c_str(), t, &bad) >= 0) g_table.swap(t);
}

bool table_lookup(const LaunchKey &key, LaunchChoice *out) {
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    const auto it = g_table.find(key);
    if(it == g_table.end()) return false;
    *out = it->second;
    return true;
}

void table_enter(const LaunchKey &key, const LaunchChoice &c) {
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    g_table[key] = c;
}

bool search_enabled() {
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    return g_search_enabled;
}

}  // namespace

extern "C" {

int nbl_conv2d_num_variants(void) { return NUM_VARIANTS; }

int nbl_launch_table_load(const char *path) {
    const std::string file = path && *path ? std::string(path) : default_table_path();
    std::map<LaunchKey, LaunchChoice> t;
    int bad = 0;
    const int n = file.empty() ? -1 : read_table_file(file.c_str(), t, &bad);
    if(n < 0) {
        if(bad) return nbl_fail(NULL, NBL_EINVAL, "nbl_launch_table_load: %s, line %d: not a launch table line", file.c_str(), bad);
        return nbl_fail(NULL, NBL_EINVAL, "nbl_launch_table_load: cannot open %s", file.empty() ? "(no default path)" : file.c_str());
    }
    std::lock_guard<std::mutex> hold(g_table_lock);
    g_table_initialised = true;
    g_table.swap(t);
    return n;
}

int nbl_launch_table_clear(void) {
    std::lock_guard<std::mutex> hold(g_table_lock);
    g_table_initialised = true;
    g_table.clear();
    return NBL_OK;
}

int nbl_launch_table_size(void) {
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    return (int)g_table.size();
}

int nbl_launch_table_save(const char *path) {
    if(!path || !*path) return nbl_fail(NULL, NBL_EINVAL, "nbl_launch_table_save: no path");
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    FILE *f = fopen(path, "w");
    if(!f) return nbl_fail(NULL, NBL_EINVAL, "nbl_launch_table_save: cannot write %s", path);
    fprintf(f, "# gfx950 convolution launch table: tile shape and k slices per problem, as measured on the device\n"
               "# conv C H W F k stride pad batch res_c res_h res_w in_place tile slices us\n");
    for(const auto &e : g_table) {
        fprintf(f, "conv");
        for(unsigned v : e.first) fprintf(f, " %u", v);
        fprintf(f, " %s %d %.1f\n", e.second.variant == NUM_VARIANTS ? "strip" : VARIANTS[e.second.variant].name, e.second.slices, e.second.us);
    }
    const bool ok = fclose(f) == 0;
    return ok ? (int)g_table.size() : nbl_fail(NULL, NBL_EINVAL, "nbl_launch_table_save: writing %s failed", path);
}

int nbl_launch_table_set_search(int enabled) {
    std::lock_guard<std::mutex> hold(g_table_lock);
    table_initialise_locked();
    g_search_enabled = enabled != 0;
    return NBL_OK;
}

int nbl_conv2d_plan_launch_source(const nbl_conv_plan *p) { return p ? p->launch_source : NBL_EINVAL; }

const char *nbl_conv2d_variant_name(int variant) {
    return variant == NUM_VARIANTS ? "strip" : variant >= 0 && variant < NUM_VARIANTS ? VARIANTS[variant].name : NULL;
}

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
    p->Kp = nbl_div_up(p->K, 2 * CONV_BK) * 2 * CONV_BK;   // the k loop consumes tiles in pairs
    p->Mp = nbl_div_up(F, CONV_MP_ALIGN) * CONV_MP_ALIGN;
    p->act = act; p->has_scale = scale_host != NULL; p->variant = -1;
    p->split_mode = -1; p->tuned_slices = 0; p->ws_dev = NULL; p->ws_bytes = 0; p->last_variant = -1; p->last_split = 1;
    p->tuned_batch = 0; p->tuned_variant = -1; p->tuned_res = { 0u, 0u, 0u, 0u }; p->launch_source = NBL_LAUNCH_NONE;
    p->strip.eligible = false; p->strip.otab_dev = NULL;
    p->wp_dev = NULL; p->wp_rows_dev = NULL; p->ktab_dev = NULL; p->g_dev = NULL; p->b_dev = NULL; p->ttab_dev = NULL;
    p->tap_major = ksize > 1 && ksize * ksize <= 31 && C % CONV_BK == 0;

    // [F][K] -> quads of patch rows [Kp / 4][Mp][4], zero padded; layers the 1x1 vector gather can take (decided per
    // call: it also needs a 16-byte aligned input) keep k-major rows [Kp][Mp] as well
    const bool vec4_geometry = ksize == 1 && stride == 1 && pad == 0 && (p->OH * p->OW) % 4 == 0 && p->K == p->Kp;
    std::vector<float> wp((size_t)p->Kp * p->Mp, 0.0f), wrows(vec4_geometry ? (size_t)p->Kp * p->Mp : 0, 0.0f);
    const unsigned taps = ksize * ksize;
    for(unsigned f = 0; f < F; f++)
        for(unsigned kk = 0; kk < p->K; kk++) {
            const unsigned row = patch_row(kk / taps, kk % taps, taps, p->tap_major);    // kk = c*taps + t in the file
            const float v = weight_host[(size_t)f * p->K + kk];
            wp[((size_t)(row / 4) * p->Mp + f) * 4 + row % 4] = v;
            if(vec4_geometry) wrows[(size_t)row * p->Mp + f] = v;
        }
    std::vector<float> g(p->Mp, 0.0f), b(p->Mp, 0.0f);
    nbl_fold_batchnorm(bias_host, scale_host, mean_host, var_host, F, g.data(), b.data());
    std::vector<int2> tab = build_ktab(C, H, W, ksize, p->Kp + 4 * CONV_BK, p->tap_major);   // + all-padding tiles behind the last k-tile
    std::vector<int2> ttab = build_ttab(C, H, W, ksize, p->Kp / CONV_BK + 4);

    int rc;
    if((rc = nbl_malloc(ctx, (void**)&p->wp_dev, wp.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->ktab_dev, tab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->ttab_dev, ttab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->ttab_dev, ttab.data(), ttab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->g_dev, g.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->b_dev, b.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->wp_dev, wp.data(), wp.size() * sizeof(float))) != NBL_OK ||
       (vec4_geometry && ((rc = nbl_malloc(ctx, (void**)&p->wp_rows_dev, wrows.size() * sizeof(float))) != NBL_OK ||
                          (rc = nbl_h2d(ctx, p->wp_rows_dev, wrows.data(), wrows.size() * sizeof(float))) != NBL_OK)) ||
       (rc = nbl_h2d(ctx, p->ktab_dev, tab.data(), tab.size() * sizeof(int2))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->g_dev, g.data(), g.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->b_dev, b.data(), b.size() * sizeof(float))) != NBL_OK) {
        nbl_conv2d_plan_destroy(ctx, p);
        return rc;
    }
    nbl_strip_plan &sp = p->strip;
    sp.C = (int)C; sp.H = (int)H; sp.W = (int)W; sp.F = (int)F; sp.k = (int)ksize; sp.stride = (int)stride; sp.pad = (int)pad;
    sp.OH = (int)p->OH; sp.OW = (int)p->OW; sp.K = (int)p->K; sp.Kp = (int)p->Kp; sp.Mp = (int)p->Mp; sp.act = act;
    sp.wq_dev = p->wp_dev; sp.g_dev = p->g_dev; sp.b_dev = p->b_dev;
    if(!p->tap_major && (rc = nbl_conv_strip_pack(ctx, &sp)) != NBL_OK) {      // (its table follows the reference row order)
        nbl_conv2d_plan_destroy(ctx, p);
        return rc;
    }
    *out = p;
    return NBL_OK;
}

int nbl_conv2d_plan_destroy(nbl_ctx *ctx, nbl_conv_plan *p) {
    if(!ctx || !p) return NBL_EINVAL;
    nbl_conv_strip_destroy(ctx, &p->strip);
    nbl_free(ctx, p->ttab_dev);
    nbl_free(ctx, p->wp_dev); nbl_free(ctx, p->wp_rows_dev); nbl_free(ctx, p->ktab_dev); nbl_free(ctx, p->g_dev); nbl_free(ctx, p->b_dev);
    nbl_free(ctx, p->ws_dev);
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
    // index NUM_VARIANTS names the strip kernel of layers with very few input channels (only where the plan qualifies)
    if(!p || variant > NUM_VARIANTS || (variant == NUM_VARIANTS && !p->strip.eligible)) return NBL_EINVAL;
    p->variant = variant < 0 ? -1 : variant;
    p->tuned_batch = 0;
    return NBL_OK;
}

int nbl_conv2d_plan_set_split(nbl_conv_plan *p, int mode) {
    if(!p || mode < -1 || mode > 8) return NBL_EINVAL;
    p->split_mode = mode;
    p->tuned_batch = 0;     // the next call searches again under the new rule
    return NBL_OK;
}

int nbl_conv2d_plan_last_launch(const nbl_conv_plan *p, int *variant, int *split_parts) {
    if(!p) return NBL_EINVAL;
    if(variant) *variant = p->last_variant;
    if(split_parts) *split_parts = p->last_split;
    return NBL_OK;
}

struct ConvResidual { const float *res; unsigned c, h, w; int post_act; };

// slices: 0 = unsplit, 1 = k-split with the cost model's slice count, 2..8 = k-split with that many slices
static int conv_launch(nbl_ctx *ctx, nbl_conv_plan *p, const float *x_dev, float *y_dev, unsigned B, int v,
                       int slices, const ConvResidual *rs) {
    if(v == NUM_VARIANTS) {           // strip kernel: whole tiles only, no fused shortcut
        if(rs || !p->strip.eligible) return nbl_fail(ctx, NBL_EINVAL, "nbl_conv2d_fwd: internal: strip kernel asked for a layer it does not take");
        const int rc = nbl_conv_strip_forward(ctx, &p->strip, x_dev, y_dev, B);
        if(rc == NBL_OK) { p->last_variant = v; p->last_split = 1; }
        return rc;
    }
    const size_t in_elems = (size_t)B * p->C * p->H * p->W;
    const size_t npix = (size_t)B * p->OH * p->OW;
    const Variant &var = VARIANTS[v];
    ConvArgs a;
    a.x = x_dev; a.wp = p->wp_dev; a.ktab = p->ktab_dev; a.g = p->g_dev; a.b = p->b_dev; a.y = y_dev;
    a.H = p->H; a.W = p->W; a.F = p->F; a.OW = p->OW; a.OHW = p->OH * p->OW; a.CHW = p->C * p->H * p->W;
    a.stride = p->stride; a.pad = p->pad; a.N = (int)npix; a.K = p->K; a.Kp = p->Kp; a.Mp = p->Mp;
    a.x_bytes = (unsigned)(in_elems * sizeof(float));
    a.act = p->act; a.has_scale = p->has_scale ? 1 : 0;
    a.tiles_m = nbl_div_up(p->F, var.bm);
    a.tiles_n = nbl_div_up((unsigned)npix, var.bn);
    // the last m-tile may read weight columns past F: they must exist (zero padded) in the packed matrix
    if((unsigned)a.tiles_m * var.bm > p->Mp)
        return nbl_fail(ctx, NBL_EINVAL, "nbl_conv2d_fwd: internal: tile %s overruns the packed weights", var.name);
    const size_t blocks = (size_t)a.tiles_m * a.tiles_n;
    if(blocks >= (1ull << 31)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: grid too large");
    bool fast_act = p->act == NBL_ACT_RELU || p->act == NBL_ACT_LINEAR || p->act == NBL_ACT_LEAKY ||
                    p->act == NBL_ACT_RELIE;
    a.res = NULL; a.res_c = a.res_hw = a.res_w = a.res_stride = a.res_box_h = a.res_box_w = 0; a.post_act = NBL_ACT_LINEAR;
    if(rs) {
        // stride / crop rule of the shortcut layer (common/utils.cc:32-40); up-sampling is not fused
        a.res = rs->res; a.res_c = (int)rs->c; a.res_hw = (int)(rs->h * rs->w); a.res_w = (int)rs->w;
        a.res_stride = rs->w / p->OW > 1 ? (int)(rs->w / p->OW) : 1;
        a.res_box_h = (int)(rs->h < p->OH ? rs->h : p->OH);
        a.res_box_w = (int)(rs->w < p->OW ? rs->w : p->OW);
        a.post_act = rs->post_act;
        fast_act = fast_act && (rs->post_act == NBL_ACT_RELU || rs->post_act == NBL_ACT_LINEAR ||
                                rs->post_act == NBL_ACT_LEAKY || rs->post_act == NBL_ACT_RELIE);
    }
    const size_t out_bytes = (size_t)npix * p->F * sizeof(float);
    // the short epilogue reads a residual whose box covers the whole output plane (same size, or sub-sampled by the
    // shortcut's stride) and that has no more channels than there are filters; residual tensor below 4 GiB
    const bool res_plain_box = rs && rs->c <= p->F && a.res_box_h == (int)p->OH && a.res_box_w == (int)p->OW &&
                               (size_t)B * rs->c * rs->h * rs->w * sizeof(float) < (1ull << 32);
    const bool sloped = p->act == NBL_ACT_LEAKY || p->act == NBL_ACT_RELIE ||
                        (rs && (rs->post_act == NBL_ACT_LEAKY || rs->post_act == NBL_ACT_RELIE));
    a.short_epilogue = !(fast_act && out_bytes < (1ull << 32) && (!rs || res_plain_box) &&
                         ((size_t)y_dev & 7) == 0 && (!rs || ((size_t)rs->res & 7) == 0)) ? 0 : sloped ? 2 : 1;
    a.ttab = p->ttab_dev; a.ksize = (int)p->k; a.plane_bytes = p->H * p->W * 4u;
    int gather = p->pad == 0 ? GATHER_NOPAD : GATHER_PADDED;
    if(p->tap_major) gather = GATHER_TAP_MAJOR;
    if(p->wp_rows_dev && ((size_t)x_dev & 15) == 0) { gather = GATHER_1X1_VEC4; a.wp = p->wp_rows_dev; }
    a.whole_tiles = (int)blocks; a.split = 1; a.n_start = 0; a.n_tail = 0; a.ws = NULL;
    size_t grid = blocks;
    if(slices && p->F <= 65535) {     // the finishing kernel's grid has one row per filter
        const SplitPlan sp = plan_split(a.tiles_m, a.tiles_n, var.bm, var.bn, p->Kp, p->F, (unsigned)npix, ctx->num_cu,
                                        slices >= 2 ? slices : 0);
        if(sp.split > 1) {
            a.whole_tiles = sp.whole_tiles; a.split = sp.split;
            a.n_start = sp.whole_tiles / a.tiles_m * var.bn;
            a.n_tail = (int)npix - a.n_start;
            const size_t need = (size_t)sp.split * p->F * a.n_tail * sizeof(float);
            if(need > p->ws_bytes) {
                int rc = nbl_free(ctx, p->ws_dev);      // waits for launches that may still use it
                p->ws_dev = NULL; p->ws_bytes = 0;
                if(rc != NBL_OK || (rc = nbl_malloc(ctx, (void**)&p->ws_dev, need)) != NBL_OK) return rc;
                p->ws_bytes = need;
            }
            a.ws = p->ws_dev;
            grid = (size_t)sp.whole_tiles + (blocks - sp.whole_tiles) * sp.split;
        }
    }
    a.units = (int)grid;
    {
        const size_t runs = nbl_div_up_sz(grid, (size_t)a.tiles_m);
        a.xcd_group_log2 = runs >= 128 ? 3 : runs >= 64 ? 2 : runs >= 32 ? 1 : 0;       // every XCD still gets at least two groups
    }
    a.div_split = make_fastdiv((unsigned)a.split); a.div_tiles_m = make_fastdiv((unsigned)a.tiles_m); a.div_ohw = make_fastdiv((unsigned)a.OHW); a.div_ow = make_fastdiv((unsigned)a.OW);
    const size_t round = (8u << a.xcd_group_log2) * (size_t)a.tiles_m;
    grid = nbl_div_up_sz(grid, round) * round;
    if(grid >= (1ull << 31)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: grid too large");
    hipLaunchKernelGGL(var.kernel[gather][fast_act ? 0 : 1], dim3((unsigned)grid), dim3(var.threads), 0,
                       ctx->stream, a);
    NBL_LAUNCH_CHECK(ctx, "conv_igemm_kernel");
    p->last_variant = v; p->last_split = a.split;
    if(a.split > 1) {
        if(a.OHW % 4 == 0 && a.n_tail % 4 == 0 && ((size_t)y_dev & 15) == 0)
            hipLaunchKernelGGL((conv_split_finish_kernel<4, true>), dim3(nbl_div_up((unsigned)a.n_tail / 4, 256), p->F), dim3(256), 0,
                               ctx->stream, a);
        else if(a.n_tail % 4 == 0)
            hipLaunchKernelGGL((conv_split_finish_kernel<4, false>), dim3(nbl_div_up((unsigned)a.n_tail / 4, 256), p->F), dim3(256), 0,
                               ctx->stream, a);
        else
            hipLaunchKernelGGL((conv_split_finish_kernel<1, false>), dim3(nbl_div_up((unsigned)a.n_tail, 256), p->F), dim3(256), 0,
                               ctx->stream, a);
        NBL_LAUNCH_CHECK(ctx, "conv_split_finish_kernel");
    }
    return NBL_OK;
}

// Tile search on the device: every tile shape, with and without the k-split of the last round, runs the
// real problem and the fastest wins.  Block-count quantisation against the number of resident blocks
// decides more than any static rule predicts, so the shapes are measured once per (layer, batch) and the
// result is kept in the plan.  The first pass splits with the cost model's slice count; the second also tries
// the other slice counts on the three best tile shapes (the model is off by up to 15 % on some layers: AlexNet's
// 256 -> 384 3x3 layer at batch 128 takes 351 us with its choice and 300 us with three slices of 128x64 tiles).
static int conv_tune(nbl_ctx *ctx, nbl_conv_plan *p, const float *x_dev, float *y_dev, unsigned B,
                     const ConvResidual *rs, float *winner_us) {
    *winner_us = 0.0f;
    struct Candidate { int variant; int slices; float ms; };
    std::vector<Candidate> cand;
    for(int v = 0; v < NUM_VARIANTS; v++) {
        if(nbl_div_up(p->F, VARIANTS[v].bm) * VARIANTS[v].bm > p->Mp) continue;
        if(p->split_mode <= 0) cand.push_back({ v, 0, 0.0f });
        if(p->split_mode != 0) {
            const int slices = p->split_mode >= 2 ? p->split_mode : 1;
            const SplitPlan sp = plan_split(nbl_div_up(p->F, VARIANTS[v].bm), nbl_div_up(B * p->OH * p->OW, VARIANTS[v].bn),
                                            VARIANTS[v].bm, VARIANTS[v].bn, p->Kp, p->F, B * p->OH * p->OW, ctx->num_cu,
                                            slices >= 2 ? slices : 0);
            // nothing to measure where nothing is split (but a launch must exist when the caller insists on splitting)
            if(sp.split > 1 || p->split_mode > 0) cand.push_back({ v, slices, 0.0f });
        }
    }
    if(p->strip.eligible && !rs) cand.push_back({ NUM_VARIANTS, 0, 0.0f });
    const int fallback = choose_variant(p, B * p->OH * p->OW, ctx->num_cu);
    if(cand.empty()) { p->tuned_batch = B; p->tuned_variant = fallback; p->tuned_slices = p->split_mode > 0 ? p->split_mode : 0; return NBL_OK; }

    // A pass queues every candidate back to back, `reps` launches each between two events, and waits once at
    // the end: the device never idles between candidates, so all of them are measured at the same (ramped-up)
    // clock and with the launch gaps of steady use.  Pass 1 ranks all candidates, pass 2 repeats the best four
    // with more launches and decides.
    std::vector<hipEvent_t> ev(cand.size() + 1);
    size_t made = 0;
    int rc = NBL_OK;
    for(; made < ev.size(); made++)
        if(hipEventCreate(&ev[made]) != hipSuccess) { rc = nbl_fail(ctx, NBL_EHIP, "hipEventCreate failed"); break; }
    auto pass = [&](std::vector<Candidate> &c, int reps) -> int {
        int r = NBL_OK;
        // clock ramp and cache warm-up, not timed
        for(int i = 0; i < 2 * reps && r == NBL_OK; i++) r = conv_launch(ctx, p, x_dev, y_dev, B, c[0].variant, c[0].slices, rs);
        for(size_t i = 0; i < c.size() && r == NBL_OK; i++) {
            if(hipEventRecord(ev[i], ctx->stream) != hipSuccess) return nbl_fail(ctx, NBL_EHIP, "hipEventRecord failed");
            for(int k = 0; k < reps && r == NBL_OK; k++) r = conv_launch(ctx, p, x_dev, y_dev, B, c[i].variant, c[i].slices, rs);
        }
        if(r != NBL_OK) return r;
        if(hipEventRecord(ev[c.size()], ctx->stream) != hipSuccess || hipEventSynchronize(ev[c.size()]) != hipSuccess)
            return nbl_fail(ctx, NBL_EHIP, "event timing failed");
        for(size_t i = 0; i < c.size(); i++)
            if(hipEventElapsedTime(&c[i].ms, ev[i], ev[i + 1]) != hipSuccess) return nbl_fail(ctx, NBL_EHIP, "hipEventElapsedTime failed");
        return NBL_OK;
    };
    if(rc == NBL_OK) rc = pass(cand, 5);
    size_t ranked = cand.size();          // candidates of the second pass that come from the first
    if(rc == NBL_OK) {
        std::sort(cand.begin(), cand.end(), [](const Candidate &l, const Candidate &r) { return l.ms < r.ms; });
        if(cand.size() > 4) cand.resize(4);
        ranked = cand.size();
        if(p->split_mode < 0) {
            // other slice counts on the best three tile shapes
            std::vector<int> shapes;
            for(size_t i = 0; i < cand.size() && shapes.size() < 3; i++)
                if(cand[i].variant < NUM_VARIANTS && std::find(shapes.begin(), shapes.end(), cand[i].variant) == shapes.end())
                    shapes.push_back(cand[i].variant);
            ranked = cand.size();
            for(int v : shapes) {
                const Variant &var = VARIANTS[v];
                const unsigned npix = B * p->OH * p->OW;
                const int model = plan_split(nbl_div_up(p->F, var.bm), nbl_div_up(npix, var.bn), var.bm, var.bn, p->Kp, p->F, npix, ctx->num_cu, 0).split;
                for(int g : { 2, 3, 4, 5, 6, 8 }) {
                    const SplitPlan sp = plan_split(nbl_div_up(p->F, var.bm), nbl_div_up(npix, var.bn), var.bm, var.bn, p->Kp, p->F, npix, ctx->num_cu, g);
                    if(sp.split != g || g == model) continue;          // fewer patch rows than slices, nothing to split, or measured already
                    bool have = false;
                    for(size_t i = 0; i < ranked; i++) have = have || (cand[i].variant == v && cand[i].slices == g);
                    if(!have) cand.push_back({ v, g, 0.0f });
                }
            }
            ev.resize(cand.size() + 1);
            for(; made < ev.size(); made++)
                if(hipEventCreate(&ev[made]) != hipSuccess) { rc = nbl_fail(ctx, NBL_EHIP, "hipEventCreate failed"); break; }
        }
        if(rc == NBL_OK) rc = pass(cand, 15);
    }
    for(size_t i = 0; i < made; i++) (void)hipEventDestroy(ev[i]);
    if(rc != NBL_OK) return rc;
    // A slice count the model did not choose has to win by 3 %: with this many candidates the fastest of a pass is
    // partly the luckiest, and back-to-back launches of one layer are not quite the layer inside its network.
    size_t best = 0, other = ranked;
    for(size_t i = 1; i < cand.size() && i < ranked; i++) if(cand[i].ms < cand[best].ms) best = i;
    for(size_t i = ranked + 1; i < cand.size(); i++) if(cand[i].ms < cand[other].ms) other = i;
    if(other < cand.size() && cand[other].ms < 0.97f * cand[best].ms) best = other;
    p->tuned_batch = B; p->tuned_variant = cand[best].variant; p->tuned_slices = cand[best].slices;
    *winner_us = cand[best].ms * 1000.0f / 15.0f;
    return NBL_OK;
}

// The search's own measurement of one problem (see conv_tune); y_dev may be the residual itself (in place).
static int conv_search(nbl_ctx *ctx, nbl_conv_plan *p, const float *x_dev, float *y_dev, unsigned B,
                       const ConvResidual *rs, float *winner_us) {
    if(!(rs && rs->res == y_dev)) return conv_tune(ctx, p, x_dev, y_dev, B, rs, winner_us);
    // in place: the search's many launches must not feed on their own output, so they write to a buffer of their
    // own (the residual is only read) and the caller's launch is the one that writes y.  This is the one place
    // where a forward call holds a second output-sized tensor for a moment; a problem the launch table lists never
    // comes here.
    const size_t out_bytes = (size_t)B * p->F * p->OH * p->OW * sizeof(float);
    float *tmp = NULL;
    int rc = nbl_malloc(ctx, (void**)&tmp, out_bytes);
    if(rc != NBL_OK) {
        const std::string why(ctx->err);
        return nbl_fail(ctx, rc, "nbl_conv2d_shortcut_fwd: the tile search of an in-place launch needs %zu bytes for its trial outputs (%s); "
                        "list the problem in the launch table or pin the launch to avoid the search", out_bytes, why.c_str());
    }
    rc = conv_tune(ctx, p, x_dev, tmp, B, rs, winner_us);
    const int rc_free = nbl_free(ctx, tmp);       // waits for the search's launches
    return rc != NBL_OK ? rc : rc_free;
}

// One launch (plus the finishing kernel of a k-split one) over B images that fit the kernel's 32-bit offsets.
static int conv_forward_chunk(nbl_ctx *ctx, nbl_conv_plan *p, const float *x_dev, float *y_dev, unsigned B,
                              const ConvResidual *rs) {
    const size_t npix = (size_t)B * p->OH * p->OW;
    int v = p->variant;
    int slices = p->split_mode > 0 ? p->split_mode : 0;
    if(v >= 0) p->launch_source = NBL_LAUNCH_PINNED;
    else {
        const std::array<unsigned, 4> res_sig = rs ? std::array<unsigned, 4>{ rs->c, rs->h, rs->w, rs->res == y_dev ? 1u : 0u }
                                                   : std::array<unsigned, 4>{ 0u, 0u, 0u, 0u };
        if(p->tuned_batch != B || p->tuned_res != res_sig) {
            const LaunchKey key = { p->C, p->H, p->W, p->F, p->k, p->stride, p->pad, B, res_sig[0], res_sig[1], res_sig[2], res_sig[3] };
            LaunchChoice c;
            // the table holds choices made with everything open; a caller's own split rule is searched under that rule
            const bool open_split = p->split_mode < 0;
            const auto usable = [&](const LaunchChoice &lc) {
                if(lc.variant == NUM_VARIANTS) return p->strip.eligible && !rs;
                return lc.variant >= 0 && lc.variant < NUM_VARIANTS && nbl_div_up(p->F, VARIANTS[lc.variant].bm) * VARIANTS[lc.variant].bm <= p->Mp;
            };
            if(open_split && table_lookup(key, &c) && usable(c)) {
                p->tuned_variant = c.variant; p->tuned_slices = c.slices;
                p->launch_source = c.from_file ? NBL_LAUNCH_TABLE : NBL_LAUNCH_SEARCHED;
            } else if(2.0 * p->F * p->K * (double)npix < 5e7 || !search_enabled()) {
                // the search overwrites y with correct results several times; tiny problems are not worth it
                p->tuned_variant = choose_variant(p, (unsigned)npix, ctx->num_cu);
                p->tuned_slices = p->split_mode > 0 ? p->split_mode : p->split_mode < 0 && 2.0 * p->F * p->K * (double)npix >= 5e7 ? 1 : 0;
                p->launch_source = NBL_LAUNCH_MODEL;
            } else {
                float us = 0.0f;
                const int rc = conv_search(ctx, p, x_dev, y_dev, B, rs, &us);
                if(rc != NBL_OK) return rc;
                p->launch_source = NBL_LAUNCH_SEARCHED;
                if(open_split) {
                    // entered with the slice count written out (1 stands for "what the cost model says")
                    int written = p->tuned_slices;
                    if(written == 1 && p->tuned_variant < NUM_VARIANTS) {
                        const Variant &var = VARIANTS[p->tuned_variant];
                        const int model = plan_split(nbl_div_up(p->F, var.bm), nbl_div_up((unsigned)npix, var.bn), var.bm, var.bn,
                                                     p->Kp, p->F, (unsigned)npix, ctx->num_cu, 0).split;
                        written = model > 1 ? model : 0;
                    }
                    const LaunchChoice found = { p->tuned_variant, written, us, false };
                    table_enter(key, found);
                    p->tuned_slices = written;
                }
            }
            p->tuned_batch = B; p->tuned_res = res_sig;
        }
        v = p->tuned_variant;
        slices = p->tuned_slices;
    }
    if(v == NUM_VARIANTS && rs) { v = choose_variant(p, (unsigned)npix, ctx->num_cu); slices = 0; }     // the strip kernel fuses no shortcut
    return conv_launch(ctx, p, x_dev, y_dev, B, v, slices, rs);
}

// Images per launch: the kernels address the input with 32-bit byte offsets (below 2^31, the top bit marks an
// out-of-range lane), the output and the residual with 32-bit element counts.  A larger batch runs as consecutive
// slices of whole images, each its own launch with its own table entry -- images are independent, as in the
// reference's per-image loop (models/layers/convolutional_layer.cc:374-399).
static unsigned conv_images_per_launch(const nbl_conv_plan *p, const ConvResidual *rs) {
    const size_t in_image = (size_t)p->C * p->H * p->W, out_image = (size_t)p->F * p->OH * p->OW;
    const size_t res_image = rs ? (size_t)rs->c * rs->h * rs->w : 0;
    size_t n = (((size_t)1 << 29) - 1) / in_image;
    n = std::min<size_t>(n, (((size_t)1 << 31) - 1) / out_image);
    n = std::min<size_t>(n, (((size_t)1 << 31) - 1024) / ((size_t)p->OH * p->OW));
    if(res_image) n = std::min<size_t>(n, (((size_t)1 << 31) - 1) / res_image);
    return (unsigned)std::min<size_t>(n, 0xffffffffu);
}

static int conv_forward(nbl_ctx *ctx, const nbl_conv_plan *plan, const float *x_dev, float *y_dev, unsigned B,
                        const ConvResidual *rs) {
    nbl_conv_plan *p = const_cast<nbl_conv_plan*>(plan);      // the chosen launch is a cache
    const unsigned per_launch = conv_images_per_launch(p, rs);
    if(per_launch == 0)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_fwd: one image of this layer has 2^29 input or 2^31 output elements or more");
    if(B <= per_launch) return conv_forward_chunk(ctx, p, x_dev, y_dev, B, rs);
    // equal slices rather than full ones and a remainder: at most two batch sizes, hence two table entries, ever occur
    const unsigned launches = nbl_div_up(B, per_launch), base = B / launches, extra = B % launches;
    const size_t in_image = (size_t)p->C * p->H * p->W, out_image = (size_t)p->F * p->OH * p->OW;
    unsigned done = 0;
    for(unsigned i = 0; i < launches; i++) {
        const unsigned nb = base + (i < extra ? 1u : 0u);
        ConvResidual part;
        if(rs) { part = *rs; part.res = rs->res + (size_t)done * rs->c * rs->h * rs->w; }
        const int rc = conv_forward_chunk(ctx, p, x_dev + (size_t)done * in_image, y_dev + (size_t)done * out_image, nb, rs ? &part : NULL);
        if(rc != NBL_OK) return rc;
        done += nb;
    }
    return NBL_OK;
}

// [a, a + a_bytes) and [b, b + b_bytes) share a byte
static bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes) {
    const size_t pa = (size_t)a, pb = (size_t)b;
    return pa < pb + b_bytes && pb < pa + a_bytes;
}

int nbl_conv2d_fwd(nbl_ctx *ctx, const nbl_conv_plan *plan, const float *x_dev, float *y_dev, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, plan && x_dev && y_dev, "nbl_conv2d_fwd: NULL argument");
    if(B == 0) return NBL_OK;
    // blocks read whole neighbourhoods of x while others write y
    NBL_REQUIRE(ctx, !ranges_overlap(x_dev, (size_t)B * plan->C * plan->H * plan->W * sizeof(float),
                                     y_dev, (size_t)B * plan->F * plan->OH * plan->OW * sizeof(float)),
                "nbl_conv2d_fwd: y must not overlap x");
    return conv_forward(ctx, plan, x_dev, y_dev, B, NULL);
}

int nbl_conv2d_shortcut_fwd(nbl_ctx *ctx, const nbl_conv_plan *plan, const float *x_dev, const float *conn_dev,
                            unsigned conn_c, unsigned conn_h, unsigned conn_w, float *y_dev, unsigned B, int post_act) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, plan && x_dev && y_dev && conn_dev, "nbl_conv2d_shortcut_fwd: NULL argument");
    NBL_REQUIRE(ctx, conn_c && conn_h && conn_w, "nbl_conv2d_shortcut_fwd: zero dimension");
    NBL_REQUIRE(ctx, nbl_act_valid(post_act), "nbl_conv2d_shortcut_fwd: undefined activation type %d", post_act);
    // Writing the result over the residual is sound when the two have the same shape: every element is then read and
    // written by the same lane (also in the finishing kernel of a k-split launch), and nothing else reads conn.
    const size_t y_bytes = (size_t)B * plan->F * plan->OH * plan->OW * sizeof(float);
    if(y_dev == conn_dev)
        NBL_REQUIRE(ctx, conn_c == plan->F && conn_h == plan->OH && conn_w == plan->OW,
                    "nbl_conv2d_shortcut_fwd: y may alias conn only when conn has the output's shape");
    else
        NBL_REQUIRE(ctx, !ranges_overlap(conn_dev, (size_t)B * conn_c * conn_h * conn_w * sizeof(float), y_dev, y_bytes),
                    "nbl_conv2d_shortcut_fwd: y may alias conn only as a whole (same address, same shape)");
    NBL_REQUIRE(ctx, !ranges_overlap(x_dev, (size_t)B * plan->C * plan->H * plan->W * sizeof(float), y_dev, y_bytes),
                "nbl_conv2d_shortcut_fwd: y must not overlap x");
    if(plan->OW / conn_w > 1)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_conv2d_shortcut_fwd: an up-sampling shortcut cannot be fused");
    if(B == 0) return NBL_OK;
    ConvResidual rs = { conn_dev, conn_c, conn_h, conn_w, post_act };
    return conv_forward(ctx, plan, x_dev, y_dev, B, &rs);
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
                       x_dev, tab_dev, col_dev, (int)K, (int)H, (int)W, (int)OW, (int)(OH * OW), (int)stride, (int)pad,
                       make_fastdiv(OH * OW), make_fastdiv(OW));
    hipError_t e = hipGetLastError();
    rc = nbl_free(ctx, tab_dev);   // waits for the kernel
    if(e != hipSuccess) return nbl_fail(ctx, NBL_EHIP, "launch of im2col_kernel failed: %s", hipGetErrorString(e));
    return rc;
}

}  // extern "C"
