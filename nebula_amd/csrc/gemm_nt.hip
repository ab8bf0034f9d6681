// C[m][n] = sum_k A[m][k] * Bw[n][k]  ("NT": both operands k-contiguous) on the fp32 matrix cores,
// with the epilogues of the fully-connected layer and of the LSTM cell.
//
// Fully connected (models/layers/connected_layer.cc:245-277): A = activations [B][I], Bw = the weight
// matrix exactly as the .wgh file holds it, [O][I].  Batch rows are the MFMA rows and output neurons
// the MFMA columns, so one accumulator row is written as 32 consecutive floats of y[b][:].
//
// LSTM (models/layers/lstm_layer.cc:233-346): the input half  U.x  is hoisted out of the time loop
// (one GEMM over all T*B rows) and the recurrent half  W.h  runs once per step with the gate
// non-linearities and the cell update fused behind it.  The four gate matrices are interleaved at
// pack time (8 hidden units wide when H % 128 == 0: lstm_step_kernel, one launch per step; 32 wide
// otherwise), so that the i, f, g, o pre-activations of one (batch row, hidden unit) sit in one MFMA
// tile or in the four tiles of one wave.
//
// LDS layout: [row][BK + 4] floats per operand.  A k-tile of 32 is consumed by 16 MFMAs; lanes 0-31
// feed k = 0..15 and lanes 32-63 feed k = 16..31 (any pairing of k values is legal as long as both
// operands use the same one), so every lane fetches its 16 values as four 16-byte LDS reads.
#include "nbl_internal.h"

#include <cmath>
#include <cstdlib>
#include <mutex>
#include <vector>

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int GEMM_BK = 32;
constexpr int GEMM_LD = GEMM_BK + 4;

enum { EPI_DIRECT = 0, EPI_PARTIAL = 1, EPI_LSTM = 2 };

typedef float vec4f __attribute__((ext_vector_type(4)));

struct GemmArgs {
    const float *A; const float *Bw; float *C;
    int M, N, K, lda, ldb, ldc;
    int vec_ok;               // rows 16-byte aligned and K % 4 == 0: float4 global loads are legal
    int b_tiled;              // Bw is stored as contiguous [128 rows][32 k] tiles, tile (n / 128, k / 32) at ((n/128) * K/32 + k/32) * 4096 floats
    int k_chunk;              // k range per blockIdx.z (multiple of GEMM_BK)
    // EPI_DIRECT: C = act((acc * g[n]) + b[n])
    const float *g; const float *b; int act, has_scale;
    // EPI_LSTM: N = 4*Hp in interleaved order; gx [M][N] input-side pre-activations (already activated by
    // sub_act), b = recurrent-side bias, act = sub_act; c [M][H] cell state (in place), C = h out [M][H]
    const float *gx; float *c; int H;
};

// Gate non-linearities of the LSTM cell in single precision (the layer's tolerance is 1e-4 relative;
// expf is good to an ulp or two).  tanh follows the reference's (e^{2x} - 1) / (e^{2x} + 1) with the
// argument clamped where that quotient has long rounded to +-1, so it cannot overflow.
__device__ __forceinline__ float lstm_logistic(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float lstm_tanh(float x) {
    const float e = expf(2.0f * fminf(fmaxf(x, -15.0f), 15.0f));
    return (e - 1.0f) / (e + 1.0f);
}

__device__ __forceinline__ float4 load_row4(const float *__restrict__ base, int row, int rows, int ld,
                                            int k, int K, int vec_ok) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if(row < rows) {
        const float *p = base + (size_t)row * ld + k;
        if(vec_ok && k + 3 < K) {
            v = *reinterpret_cast<const float4*>(p);
        } else {
            if(k < K) v.x = p[0];
            if(k + 1 < K) v.y = p[1];
            if(k + 2 < K) v.z = p[2];
            if(k + 3 < K) v.w = p[3];
        }
    }
    return v;
}

template<int MT, int NT, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N)
void gemm_nt_kernel(const GemmArgs a) {
    constexpr int BK = GEMM_BK, LD = GEMM_LD;
    constexpr int NTHREADS = 64 * WAVES_M * WAVES_N;
    constexpr int BM = MT * 32 * WAVES_M, BN = NT * 32 * WAVES_N;
    constexpr int RA = (BM * 8 + NTHREADS - 1) / NTHREADS, RB = (BN * 8 + NTHREADS - 1) / NTHREADS;

    __shared__ __attribute__((aligned(16))) float As[2][BM][LD];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int half = lane >> 5, l32 = lane & 31;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int k_begin = blockIdx.z * a.k_chunk;
    const int k_end = min(a.K, k_begin + a.k_chunk);
    const int nkt = (k_end - k_begin + BK - 1) / BK;

    float4 areg[RA], breg[RB];
    auto load_tile = [&](int kt) {
        const int k0 = k_begin + kt * BK;
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int v = tid + r * NTHREADS;
            if((BM * 8) % NTHREADS == 0 || v < BM * 8)
                areg[r] = load_row4(a.A, m0 + (v >> 3), a.M, a.lda, k0 + (v & 7) * 4, k_end, a.vec_ok);
        }
        #pragma unroll
        for(int r = 0; r < RB; r++) {
            const int v = tid + r * NTHREADS;
            if((BN * 8) % NTHREADS == 0 || v < BN * 8)
                breg[r] = load_row4(a.Bw, n0 + (v >> 3), a.N, a.ldb, k0 + (v & 7) * 4, k_end, a.vec_ok);
        }
    };
    auto store_tile = [&](int buf) {
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int v = tid + r * NTHREADS;
            if((BM * 8) % NTHREADS == 0 || v < BM * 8)
                *reinterpret_cast<float4*>(&As[buf][v >> 3][(v & 7) * 4]) = areg[r];
        }
        #pragma unroll
        for(int r = 0; r < RB; r++) {
            const int v = tid + r * NTHREADS;
            if((BN * 8) % NTHREADS == 0 || v < BN * 8)
                *reinterpret_cast<float4*>(&Bs[buf][v >> 3][(v & 7) * 4]) = breg[r];
        }
    };

    floatx16 acc[MT][NT];
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int j = 0; j < NT; j++)
            #pragma unroll
            for(int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    if(nkt > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();
    for(int kt = 0; kt < nkt; kt++) {
        const int buf = kt & 1;
        if(kt + 1 < nkt) load_tile(kt + 1);
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            float4 av[MT], bv[NT];
            #pragma unroll
            for(int i = 0; i < MT; i++)
                av[i] = *reinterpret_cast<const float4*>(&As[buf][(wm * MT + i) * 32 + l32][half * 16 + q * 4]);
            #pragma unroll
            for(int j = 0; j < NT; j++)
                bv[j] = *reinterpret_cast<const float4*>(&Bs[buf][(wn * NT + j) * 32 + l32][half * 16 + q * 4]);
            #pragma unroll
            for(int i = 0; i < MT; i++)
                #pragma unroll
                for(int j = 0; j < NT; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].x, bv[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].y, bv[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].z, bv[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].w, bv[j].w, acc[i][j], 0, 0, 0);
                }
        }
        if(kt + 1 < nkt) store_tile(buf ^ 1);
        __syncthreads();
    }

    // accumulator register r of a 32x32 tile: row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
    if(EPI == EPI_LSTM) {
        // wave tile columns: tile j = gate j (i, f, g, o) of hidden unit hb*32 + lane%32
        const int hb = blockIdx.x * WAVES_N + wn;
        const int h = hb * 32 + l32;
        if(h < a.H) {
            #pragma unroll
            for(int i = 0; i < MT; i++)
                #pragma unroll
                for(int r = 0; r < 16; r++) {
                    const int m = m0 + (wm * MT + i) * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
                    if(m >= a.M) continue;
                    float pre[4];
                    #pragma unroll
                    for(int gate = 0; gate < 4; gate++) {
                        const int n = hb * 128 + gate * 32 + l32;
                        pre[gate] = nbl_act_apply(a.act, acc[i][gate % NT][r] + a.b[n]) + a.gx[(size_t)m * a.ldc + n];
                    }
                    const float gi = lstm_logistic(pre[0]);
                    const float gf = lstm_logistic(pre[1]);
                    const float gg = lstm_tanh(pre[2]);
                    const float go = lstm_logistic(pre[3]);
                    // c_t = c_{t-1}*f + i*g with each product rounded, as the reference's separate passes do
                    const size_t e = (size_t)m * a.H + h;
                    const float ig = __fmul_rn(gi, gg);
                    const float cf = __fmul_rn(a.c[e], gf);
                    const float ct = __fadd_rn(cf, ig);
                    a.c[e] = ct;
                    a.C[e] = __fmul_rn(lstm_tanh(ct), go);
                }
        }
        return;
    }
    float *__restrict__ Cout = a.C + (EPI == EPI_PARTIAL ? (size_t)blockIdx.z * a.M * a.ldc : 0);
    #pragma unroll
    for(int j = 0; j < NT; j++) {
        const int n = n0 + (wn * NT + j) * 32 + l32;
        if(n >= a.N) continue;
        float gn = 1.0f, bn = 0.0f;
        if(EPI == EPI_DIRECT) { bn = a.b[n]; if(a.has_scale) gn = a.g[n]; }
        #pragma unroll
        for(int i = 0; i < MT; i++)
            #pragma unroll
            for(int r = 0; r < 16; r++) {
                const int m = m0 + (wm * MT + i) * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
                if(m >= a.M) continue;
                float v = acc[i][j][r];
                if(EPI == EPI_DIRECT) {
                    v = a.has_scale ? v * gn + bn : v + bn;
                    v = nbl_act_apply(a.act, v);
                }
                Cout[(size_t)m * a.ldc + n] = v;
            }
    }
}

// The same product for operands whose rows are 16-byte aligned with K % 4 == 0 (every layer of the
// shipped networks): identical tiling and LDS layout as gemm_nt_kernel, but
//  - every global load is an unconditional 16-byte load (a row past the matrix repeats the last row and its
//    products are never stored; a k past the chunk re-reads the chunk's last four values and is replaced by
//    zeros when the stage is written to LDS), so no branch makes the compiler wait for all loads at once;
//  - the loads run through a ring of DEPTH register stages: while k-tile t is multiplied, tiles t+2 ..
//    t+DEPTH are on their way.  At small batch (M <= 64, DEPTH = 4) the layer is a stream of the [N][K]
//    weight matrix and the bytes in flight per CU decide its rate (one stage covers about a quarter of the
//    HBM latency and held the stream to 3.2 TB/s); large tiles take DEPTH = 2.
// Output: raw partial sums part[blockIdx.z][M][N] (EPI_PARTIAL) or act(sum * g + b) (EPI_DIRECT).
template<int MT, int NT, int WAVES_M, int WAVES_N, int DEPTH, int EPI, bool BUF>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N)
void gemm_nt_stream_kernel(const GemmArgs a) {
    constexpr int BK = GEMM_BK, LD = GEMM_LD, NTHREADS = 64 * WAVES_M * WAVES_N;
    constexpr int BM = MT * 32 * WAVES_M, BN = NT * 32 * WAVES_N;
    static_assert((BM * 8) % NTHREADS == 0 && (BN * 8) % NTHREADS == 0, "tiles must split evenly over the threads");
    static_assert(DEPTH == 2 || DEPTH == 4, "the ring below is written out for two or four stages");
    constexpr int RA = BM * 8 / NTHREADS, RB = BN * 8 / NTHREADS;
    __shared__ __attribute__((aligned(16))) float As[2][BM][LD];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int half = lane >> 5, l32 = lane & 31;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int k_begin = blockIdx.z * a.k_chunk;
    const int k_end = min(a.K, k_begin + a.k_chunk);
    const int nkt = (k_end - k_begin + BK - 1) / BK;
    if(nkt <= 0) return;

    struct Stage { vec4f a[RA], b[RB]; bool valid; };
    Stage st0, st1, st2, st3;           // named, not an array: an indexed array of stages ends up in scratch memory
    const int acol = (tid & 7) * 4;
    const float *__restrict__ arow[RA];
    const float *__restrict__ brow[RB];
    // BUF (every k-tile whole, operands below 2 GiB): buffer loads whose vector offset is the thread's constant
    // (row, column) offset -- out of range for a row past the matrix, which then reads zeros -- and whose scalar
    // offset is the k-tile's: no vector arithmetic per load and nothing to zero afterwards.
    unsigned aoff[RA], boff[RB];
    __amdgpu_buffer_rsrc_t ares, bres;
    if(BUF) {
        ares = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.A), 0, (int)((unsigned)a.M * (unsigned)a.lda * 4u), 0x00020000);
        bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.Bw), 0,
                                                 (int)((unsigned)(a.b_tiled ? (a.N + 127) / 128 * 128 : a.N) * (unsigned)a.ldb * 4u), 0x00020000);
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int row = m0 + ((tid + r * NTHREADS) >> 3);
            aoff[r] = row < a.M ? ((unsigned)row * (unsigned)a.lda + (unsigned)acol) * 4u : 0x80000000u;
        }
        #pragma unroll
        for(int r = 0; r < RB; r++) {
            const int row = n0 + ((tid + r * NTHREADS) >> 3);
            // tiled weights: the thread's piece of the 16 KB tile (rows past N are zeros in the tiled copy)
            boff[r] = a.b_tiled ? (unsigned)(tid + r * NTHREADS) * 16u
                                : row < a.N ? ((unsigned)row * (unsigned)a.ldb + (unsigned)acol) * 4u : 0x80000000u;
        }
    } else {
        #pragma unroll
        for(int r = 0; r < RA; r++) arow[r] = a.A + (size_t)min(m0 + ((tid + r * NTHREADS) >> 3), a.M - 1) * a.lda;
        #pragma unroll
        for(int r = 0; r < RB; r++) brow[r] = a.Bw + (size_t)min(n0 + ((tid + r * NTHREADS) >> 3), a.N - 1) * a.ldb;
    }
    auto load_tile = [&](Stage &s, int kt) {
        if(BUF) {
            const unsigned ko = (unsigned)(k_begin + min(kt, nkt - 1) * BK) * 4u;     // uniform
            // tiled weights: tile (blockIdx.x, k / 32), 16 KB each, one row of tiles per 128 output rows
            const unsigned kob = a.b_tiled ? ((unsigned)blockIdx.x * (unsigned)(a.K / BK) + (unsigned)(k_begin / BK + min(kt, nkt - 1))) * 16384u : ko;
            s.valid = true;
            #pragma unroll
            for(int r = 0; r < RA; r++) s.a[r] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(ares, (int)aoff[r], (int)ko, 0));
            #pragma unroll
            for(int r = 0; r < RB; r++) s.b[r] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(bres, (int)boff[r], (int)kob, 0));
            return;
        }
        const int k = k_begin + min(kt, nkt - 1) * BK + acol;
        const bool valid = k < k_end;
        const int kk = valid ? k : k_end - 4;
        s.valid = valid;            // the zeroing happens when the stage is written to LDS: touching the values
                                    // here would make the loads wait for themselves
        #pragma unroll
        for(int r = 0; r < RA; r++) s.a[r] = *reinterpret_cast<const vec4f*>(arow[r] + kk);
        #pragma unroll
        for(int r = 0; r < RB; r++) s.b[r] = *reinterpret_cast<const vec4f*>(brow[r] + kk);
    };
    auto store_tile = [&](const Stage &s, int buf) {
        #pragma unroll
        for(int r = 0; r < RA; r++) {
            const int v = tid + r * NTHREADS;
            const vec4f t = s.a[r];
            *reinterpret_cast<vec4f*>(&As[buf][v >> 3][(v & 7) * 4]) =
                BUF ? t : vec4f{s.valid ? t.x : 0.f, s.valid ? t.y : 0.f, s.valid ? t.z : 0.f, s.valid ? t.w : 0.f};
        }
        #pragma unroll
        for(int r = 0; r < RB; r++) {
            const int v = tid + r * NTHREADS;
            const vec4f t = s.b[r];
            *reinterpret_cast<vec4f*>(&Bs[buf][v >> 3][(v & 7) * 4]) =
                BUF ? t : vec4f{s.valid ? t.x : 0.f, s.valid ? t.y : 0.f, s.valid ? t.z : 0.f, s.valid ? t.w : 0.f};
        }
    };
    floatx16 acc[MT][NT];
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int j = 0; j < NT; j++)
            #pragma unroll
            for(int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    auto compute_tile = [&](int buf) {
        #pragma unroll
        for(int q = 0; q < 4; q++) {
            float4 av[MT], bv[NT];
            #pragma unroll
            for(int i = 0; i < MT; i++)
                av[i] = *reinterpret_cast<const float4*>(&As[buf][(wm * MT + i) * 32 + l32][half * 16 + q * 4]);
            #pragma unroll
            for(int j = 0; j < NT; j++)
                bv[j] = *reinterpret_cast<const float4*>(&Bs[buf][(wn * NT + j) * 32 + l32][half * 16 + q * 4]);
            #pragma unroll
            for(int i = 0; i < MT; i++)
                #pragma unroll
                for(int j = 0; j < NT; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].x, bv[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].y, bv[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].z, bv[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i].w, bv[j].w, acc[i][j], 0, 0, 0);
                }
        }
    };

    // k-tile t travels through stage t % DEPTH into LDS buffer t % 2.  One step: refill the stage that was
    // written to LDS one step ago with tile t+DEPTH, multiply tile t, write tile t+1 (past the end: a repeat of
    // the last tile, never multiplied) into the other buffer.
    #define NBL_GEMM_STEP(U, CUR, NEXT)                                 \
        {                                                               \
            load_tile(CUR, kt + U + DEPTH);                             \
            compute_tile(U & 1);                                        \
            store_tile(NEXT, (U + 1) & 1);                              \
            __syncthreads();                                            \
        }
    load_tile(st0, 0); load_tile(st1, 1);
    if(DEPTH == 4) { load_tile(st2, 2); load_tile(st3, 3); }
    store_tile(st0, 0);
    __syncthreads();
    // whole rounds of the ring run without a condition inside (a conditional step makes the compiler wait for
    // nearly every outstanding load where the paths join); the last nkt % DEPTH tiles follow one by one
    int kt = 0;
    for(; kt + DEPTH <= nkt; kt += DEPTH) {
        if(DEPTH == 4) {
            NBL_GEMM_STEP(0, st0, st1)
            NBL_GEMM_STEP(1, st1, st2)
            NBL_GEMM_STEP(2, st2, st3)
            NBL_GEMM_STEP(3, st3, st0)
        } else {
            NBL_GEMM_STEP(0, st0, st1)
            NBL_GEMM_STEP(1, st1, st0)
        }
    }
    if(kt < nkt) NBL_GEMM_STEP(0, st0, st1)
    if(DEPTH == 4) {
        if(kt + 1 < nkt) NBL_GEMM_STEP(1, st1, st2)
        if(kt + 2 < nkt) NBL_GEMM_STEP(2, st2, st3)
    }
    #undef NBL_GEMM_STEP

    // accumulator register r of a 32x32 tile: row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
    float *__restrict__ Cout = a.C + (EPI == EPI_PARTIAL ? (size_t)blockIdx.z * a.M * a.ldc : 0);
    #pragma unroll
    for(int j = 0; j < NT; j++) {
        const int n = n0 + (wn * NT + j) * 32 + l32;
        if(n >= a.N) continue;
        float gn = 1.0f, bn = 0.0f;
        if(EPI == EPI_DIRECT) { bn = a.b[n]; if(a.has_scale) gn = a.g[n]; }
        #pragma unroll
        for(int i = 0; i < MT; i++)
            #pragma unroll
            for(int r = 0; r < 16; r++) {
                const int m = m0 + (wm * MT + i) * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
                if(m >= a.M) continue;
                float v = acc[i][j][r];
                if(EPI == EPI_DIRECT) {
                    v = a.has_scale ? v * gn + bn : v + bn;
                    v = nbl_act_apply(a.act, v);
                }
                Cout[(size_t)m * a.ldc + n] = v;
            }
    }
}

// ---- weight streaming for small batches ---------------------------------------------------------------------------
// At up to 64 rows of batch a connected layer is one pass over its [N][K] weight matrix: 415 MB for 6.6 GFLOP in
// VGG-16's first connected layer, so the layer lasts as long as memory takes to deliver the weights, provided nothing
// else stands in their way.  Here the weights never touch LDS: they are stored once more in operand-major order
// (opmajor_offset: the 64 16-byte pieces a wave's load instruction fetches for one 8-wide k block of one 32-row tile
// are one contiguous KiB, and a tile's k blocks follow each other, so a wave reads its tile as ONE contiguous
// stream), every lane loads its own MFMA operands straight into registers through a ring of loads per tile,
// and no barrier sits between a weight load and its use.  Only the activations X[M][K] -- small, and shared by every
// wave of a block -- go through LDS, a chunk of 256 k at a time, double buffered, one barrier per chunk.
// Work split: a block is 4 waves x NT tiles of 32 neurons and one k range (blockIdx.y), FC_RING weight loads in flight
// per tile and wave; raw sums of a split go to
// part[blockIdx.y][M][N] for splitk_reduce_kernel, an unsplit launch applies the epilogue itself.
constexpr int FC_KALIGN = 32;              // k ranges of blocks and the padded k extent of w_op are multiples of this many k blocks
constexpr int FC_CHUNK_KB = 32;            // k blocks of X per LDS buffer (256 k)
constexpr int FC_X_PITCH = FC_CHUNK_KB * 8 + 4;      // floats between rows of a chunk in LDS

struct FcStreamArgs {
    const float *x; const float *w_op; float *out;
    const float *g; const float *b; int act, has_scale;
    int M, N, K;
    int K8p;                // k blocks per row tile in w_op (K / 8 rounded up to a multiple of FC_KALIGN; the padding holds zeros)
    int ntiles;             // row tiles of 32 neurons in w_op
    int kb_per_split;       // k blocks per blockIdx.y (a multiple of FC_KALIGN)
    int direct;             // gridDim.y == 1: out is y and the epilogue is applied here; else out is the partial-sum workspace
};

template<int MT, int NT, int FC_RING>
__global__ __launch_bounds__(256) void fc_stream_kernel(const FcStreamArgs a) {
    static_assert(FC_KALIGN % FC_RING == 0 && FC_CHUNK_KB % FC_RING == 0, "groups of ring refills must tile a chunk");
    extern __shared__ __attribute__((aligned(16))) float xs[];        // [2][32 * MT][FC_X_PITCH]
    constexpr int ROWS = 32 * MT, XBUF = ROWS * FC_X_PITCH;
    constexpr int XLOADS = ROWS * (FC_CHUNK_KB * 2) / 256;            // 16-byte pieces of a chunk per thread
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, r = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb_begin = blockIdx.y * a.kb_per_split;
    const int nkb = min(a.kb_per_split, a.K8p - kb_begin);            // > 0 and a multiple of FC_KALIGN by construction
    const int nchunks = (nkb + FC_CHUNK_KB - 1) / FC_CHUNK_KB;

    // weights: tile rt of this wave starts at byte (rt * K8p + kb_begin) * 1024; the lane's piece at + lane * 16
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.w_op), 0,
                                                                          (int)((unsigned)a.ntiles * (unsigned)a.K8p * 1024u), 0x00020000);
    int rt[NT]; unsigned wlane[NT], wbase[NT];
    #pragma unroll
    for(int j = 0; j < NT; j++) {
        rt[j] = (blockIdx.x * 4 + wave) * NT + j;
        wlane[j] = rt[j] < a.ntiles ? (unsigned)lane * 16u : 0x80000000u;       // a tile past the matrix loads zeros and no memory
        wbase[j] = (unsigned)(rt[j] < a.ntiles ? rt[j] : 0) * (unsigned)a.K8p * 1024u + (unsigned)kb_begin * 1024u;
    }
    vec4f ring[NT][FC_RING];
    auto load_w = [&](int j, int slot, int kbl) {
        // past the block's last k block the last one is read again (never multiplied): no branch, no new memory traffic
        const unsigned so = wbase[j] + (unsigned)min(kbl, nkb - 1) * 1024u;
        ring[j][slot] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(wres, (int)wlane[j], (int)so, 0));
    };
    #pragma unroll
    for(int u = 0; u < FC_RING; u++)
        #pragma unroll
        for(int j = 0; j < NT; j++) load_w(j, u, u);

    // activations: thread t stages the 16-byte pieces (row = t / 64 + 4 * i, column piece t % 64) of a chunk
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.x), 0,
                                                                          (int)((unsigned)a.M * (unsigned)a.K * 4u), 0x00020000);
    const int xcol = tid & 63, xrow0 = tid >> 6;
    vec4f xstage[XLOADS];
    auto stage_load = [&](int c) {
        const int k = (kb_begin + c * FC_CHUNK_KB) * 8 + xcol * 4;
        const bool k_ok = k < a.K && k < (kb_begin + nkb) * 8;          // K is a multiple of 4: a piece is inside or outside as a whole
        #pragma unroll
        for(int i = 0; i < XLOADS; i++) {
            const int row = xrow0 + 4 * i;
            const unsigned off = k_ok && row < a.M ? ((unsigned)row * (unsigned)a.K + (unsigned)k) * 4u : 0x80000000u;
            xstage[i] = __builtin_bit_cast(vec4f, __builtin_amdgcn_raw_buffer_load_b128(xres, (int)off, 0, 0));
        }
    };
    auto stage_store = [&](int buf) {
        #pragma unroll
        for(int i = 0; i < XLOADS; i++)
            *reinterpret_cast<vec4f*>(&xs[buf * XBUF + (xrow0 + 4 * i) * FC_X_PITCH + xcol * 4]) = xstage[i];
    };

    floatx16 acc[MT][NT];
    #pragma unroll
    for(int i = 0; i < MT; i++)
        #pragma unroll
        for(int j = 0; j < NT; j++)
            #pragma unroll
            for(int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    stage_load(0);
    stage_store(0);
    const int xlane = r * FC_X_PITCH + half * 4;           // this lane's operand piece of k block 0 of a chunk
    int kbl = 0;                                            // k block of the block's range the next MFMAs consume
    // One group of FC_RING k blocks from the chunk in LDS at xb: the group's activations first (LDS answers in order,
    // so the first step waits for its own piece only), then per k block its MFMAs and at once the refill of the ring
    // slots they have just read, so that a weight load is always FC_RING k blocks ahead of its use.  (Left to itself
    // the scheduler moves all refills behind the group's last MFMA, where the next group's first MFMA waits for them.)
    auto group = [&](const float *xb, int gi) __attribute__((always_inline)) {
        #pragma unroll
        for(int u0 = 0; u0 < FC_RING; u0 += 8) {
            vec4f xv[8][MT];
            #pragma unroll
            for(int u = 0; u < 8; u++)
                #pragma unroll
                for(int i = 0; i < MT; i++) xv[u][i] = *reinterpret_cast<const vec4f*>(xb + i * 32 * FC_X_PITCH + (gi * FC_RING + u0 + u) * 8);
            #pragma unroll
            for(int u = 0; u < 8; u++) {
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for(int j = 0; j < NT; j++) {
                    const vec4f w = ring[j][u0 + u];
                    #pragma unroll
                    for(int e = 0; e < 4; e++)
                        #pragma unroll
                        for(int i = 0; i < MT; i++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u][i][e], w[e], acc[i][j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                #pragma unroll
                for(int j = 0; j < NT; j++) load_w(j, u0 + u, kbl + u0 + u + FC_RING);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        kbl += FC_RING;
    };
    for(int c = 0; c < nchunks; c++) {
        __syncthreads();        // chunk c is in LDS; every wave has finished reading the other buffer (chunk c - 1)
        const float *xb = xs + (c & 1) * XBUF + xlane;
        const int groups = min(FC_CHUNK_KB, nkb - c * FC_CHUNK_KB) / FC_RING;
        for(int gi = 0; gi + 1 < groups; gi++) group(xb, gi);
        // The next chunk's activations are requested before the chunk's LAST group and written to LDS behind it: the
        // memory counter retires loads in issue order, so waiting for these loads means waiting for every older one --
        // requested here, only the last group's refills are younger and the weight ring stays full across the wait.
        if(c + 1 < nchunks) stage_load(c + 1);
        __builtin_amdgcn_sched_barrier(0);
        group(xb, groups - 1);
        if(c + 1 < nchunks) stage_store((c + 1) & 1);
    }

    // accumulator register e of a 32x32 tile: row (batch) 8*(e/4) + 4*(lane/32) + e%4, column (neuron) lane%32
    float *__restrict__ out = a.out + (a.direct ? (size_t)0 : (size_t)blockIdx.y * a.M * a.N);
    #pragma unroll
    for(int j = 0; j < NT; j++) {
        const int n = rt[j] * 32 + r;
        if(n >= a.N) continue;
        float gn = 1.0f, bn = 0.0f;
        if(a.direct) { bn = a.b[n]; if(a.has_scale) gn = a.g[n]; }
        #pragma unroll
        for(int i = 0; i < MT; i++)
            #pragma unroll
            for(int e = 0; e < 16; e++) {
                const int m = i * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
                if(m >= a.M) continue;
                float v = acc[i][j][e];
                if(a.direct) {
                    v = a.has_scale ? v * gn + bn : v + bn;
                    v = nbl_act_apply(a.act, v);
                }
                out[(size_t)m * a.N + n] = v;
            }
    }
}

// y[m][n] = act((sum_z part[z][m][n]) * g[n] + b[n]), the parts added in ascending z.  VEC adjacent n per thread
// (VEC = 4 needs N % 4 == 0 and 16-byte aligned buffers); eight parts are requested before the first is added, so
// the kernel is one memory round trip per eight parts instead of one per part.
template<int VEC>
__global__ void splitk_reduce_kernel(const float *__restrict__ part, float *__restrict__ y,
                                     const float *__restrict__ g, const float *__restrict__ b,
                                     int M, int N, int S, int act, int has_scale) {
    typedef float __attribute__((ext_vector_type(VEC))) vec;
    const size_t e = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    const size_t total = (size_t)M * N;
    if(e >= total) return;
    const int n = (int)(e % N);
    vec v = 0.0f;
    int z = 0;
    for(; z + 8 <= S; z += 8) {
        vec t[8];
        #pragma unroll
        for(int u = 0; u < 8; u++) t[u] = *reinterpret_cast<const vec*>(part + (size_t)(z + u) * total + e);
        #pragma unroll
        for(int u = 0; u < 8; u++)
            #pragma unroll
            for(int c = 0; c < VEC; c++) v[c] = __fadd_rn(v[c], t[u][c]);
    }
    for(; z < S; z++) {
        const vec t = *reinterpret_cast<const vec*>(part + (size_t)z * total + e);
        #pragma unroll
        for(int c = 0; c < VEC; c++) v[c] = __fadd_rn(v[c], t[c]);
    }
    vec o;
    #pragma unroll
    for(int c = 0; c < VEC; c++) {
        const float s = has_scale ? v[c] * g[n + c] + b[n + c] : v[c] + b[n + c];
        o[c] = nbl_act_apply(act, s);
    }
    *reinterpret_cast<vec*>(y + e) = o;
}

// A wave's share of a skinny product: acc0 + acc1 = sum over `kw` consecutive k of A[row][k] * B[col][k]
// as one 32x32 MFMA tile, with both operands read STRAIGHT from global memory: ap / bp point at the
// lane's row (lane % 32) of each operand, advanced by 4 floats for lanes 32-63, so that per 8 k the
// lanes 0-31 supply k+0..3 and lanes 32-63 k+4..7 of both operands (a legal pairing).  Loads run one
// batch of U steps ahead; two accumulators take turns because with one wave per SIMD nothing else
// hides the latency between two MFMAs on the same registers.  kw must be a multiple of 32.
// astep / bstep: floats between a lane's pieces of consecutive 8-wide k blocks: 8 in a row-major matrix; 256 in the
// operand-major layout below, where the 64 pieces one load instruction fetches are one contiguous KiB.
__device__ __forceinline__ void wave_tile_from_global(const float *__restrict__ ap, const float *__restrict__ bp, int kw,
                                                      floatx16 &acc0, floatx16 &acc1, int astep = 8, int bstep = 8) {
    constexpr int U = 4;                    // 8-wide k steps per batch of loads
    const int nb = kw / (8 * U);
    float4 av[2][U], bv[2][U];
    auto load = [&](int buf, int b) {
        #pragma unroll
        for(int u = 0; u < U; u++) {
            av[buf][u] = *reinterpret_cast<const float4*>(ap + (size_t)(b * U + u) * astep);
            bv[buf][u] = *reinterpret_cast<const float4*>(bp + (size_t)(b * U + u) * bstep);
        }
    };
    #pragma unroll
    for(int i = 0; i < 16; i++) { acc0[i] = 0.0f; acc1[i] = 0.0f; }
    auto compute = [&](int buf) {
        #pragma unroll
        for(int u = 0; u < U; u++) {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf][u].x, bv[buf][u].x, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf][u].y, bv[buf][u].y, acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf][u].z, bv[buf][u].z, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf][u].w, bv[buf][u].w, acc1, 0, 0, 0);
        }
    };
    if(nb == 8) {
        // the common width (k range of 256 per wave): loads run two batches ahead through three register sets
        // (three ahead through four sets is slower again),
        // which covers more of the memory latency than one batch of MFMAs (0.44 us) does
        float4 aw[3][U], bw[3][U];
        auto load3 = [&](int buf, int bb) {
            #pragma unroll
            for(int u = 0; u < U; u++) {
                aw[buf][u] = *reinterpret_cast<const float4*>(ap + (size_t)(bb * U + u) * astep);
                bw[buf][u] = *reinterpret_cast<const float4*>(bp + (size_t)(bb * U + u) * bstep);
            }
        };
        load3(0, 0);
        load3(1, 1);
        #pragma unroll
        for(int bb = 0; bb < 8; bb++) {
            if(bb + 2 < 8) load3((bb + 2) % 3, bb + 2);
            __builtin_amdgcn_sched_barrier(0);
            #pragma unroll
            for(int u = 0; u < U; u++) {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[bb % 3][u].x, bw[bb % 3][u].x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[bb % 3][u].y, bw[bb % 3][u].y, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[bb % 3][u].z, bw[bb % 3][u].z, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[bb % 3][u].w, bw[bb % 3][u].w, acc1, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }
    load(0, 0);
    int b = 0;
    for(; b + 2 <= nb; b += 2) {
        load(1, b + 1);
        compute(0);
        if(b + 2 < nb) load(0, b + 2);
        compute(1);
    }
    if(b < nb) compute(0);
}

// One LSTM time step in one launch, for layers packed with gate interleave 8 (row of gate g, hidden unit
// h: (h/8)*32 + g*8 + h%8), so that ONE 32x32 MFMA tile holds the four gate pre-activations of 8 hidden
// units for 32 batch rows.  A step is latency, not throughput ([B x H].[H x 4H] is 3.4 us of MFMA time
// on the whole chip), so the work is cut for many small independent pieces: a block owns one such
// tile, its four waves each take a quarter of the k range and read their MFMA operands STRAIGHT from
// global memory (each lane one 16-byte piece of its row per 8 k: lanes 0-31 supply k+0..3, lanes
// 32-63 k+4..7 of both operands, which is a legal pairing), several loads in flight per lane and no
// barrier until the four partial tiles meet in LDS.  Then each thread owns one (batch row, hidden
// unit): sum of the four partial tiles for each gate, bias, input-side pre-activation, the cell update
// (lstm_layer.cc:264-312, each product rounded on its own) and h_t written into y[t], which is the
// next step's operand.  Needs H % 128 == 0 and 16-byte aligned rows.
// Operand-major layout of a [rows][K] matrix (rows and K padded to 32 and 8): the 16-byte piece lane (half, r) of
// a wave feeds to the MFMAs of the 8-wide k block kb of row tile rt -- elements k = 8*kb + 4*half .. +3 of row
// 32*rt + r -- sits at float offset ((rt * K/8 + kb) * 64 + half*32 + r) * 4.  A wave's load instruction then
// reads one contiguous KiB (8 cache lines) where the row-major matrix makes it touch 32 lines for the same bytes;
// with row-major operands the step kernels kept the CU's address unit busy for 6 of their 9 us.
__host__ __device__ inline size_t opmajor_offset(unsigned row, unsigned k, unsigned K) {
    return (((size_t)(row / 32) * (K / 8) + k / 8) * 64 + ((k % 8) / 4) * 32 + row % 32) * 4 + k % 4;
}

struct LstmStepArgs {
    const float *hprev_op;      // h_{t-1}, operand-major [ceil(B/32)*32][H]
    const float *w_op;          // recurrent weights, operand-major [Np][H]
    const float *gx; const float *bw; float *c; float *hout;
    float *hnext_op;            // h_t in operand-major layout for the next step
    int B, H, Np, sub_act;
};

__global__ __launch_bounds__(256)
void lstm_step_kernel(const LstmStepArgs a) {
    __shared__ float red[4][32][33];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int kw = a.H >> 2;                // k range of one wave
    // what the cell update needs besides the products is requested first and arrives behind the k loop
    const int ml = tid >> 3, hh = tid & 7;
    const int m = m0 + ml, h = blockIdx.x * 8 + hh;
    const bool live = m < a.B;
    const size_t e = (size_t)(live ? m : 0) * a.H + h;
    float gxv[4], bwv[4];
    #pragma unroll
    for(int gate = 0; gate < 4; gate++) {
        gxv[gate] = a.gx[(size_t)(live ? m : 0) * a.Np + n0 + gate * 8 + hh];
        bwv[gate] = a.bw[n0 + gate * 8 + hh];
    }
    const float cprev = a.c[e];
    floatx16 acc0, acc1;                    // (rows past the batch hold zeros in the operand-major h; their sums are dropped)
    wave_tile_from_global(a.hprev_op + opmajor_offset(m0 + r, wave * kw + half * 4, a.H),
                          a.w_op + opmajor_offset(n0 + r, wave * kw + half * 4, a.H), kw, acc0, acc1, 256, 256);

    // accumulator register i of a 32x32 tile: row 8*(i/4) + 4*(lane/32) + i%4 (batch), column lane%32 (gate column)
    #pragma unroll
    for(int i = 0; i < 16; i++) red[wave][8 * (i >> 2) + 4 * half + (i & 3)][r] = acc0[i] + acc1[i];
    __syncthreads();
    if(!live) return;
    float pre[4];
    #pragma unroll
    for(int gate = 0; gate < 4; gate++) {
        const int col = gate * 8 + hh;
        const float t = ((red[0][ml][col] + red[1][ml][col]) + (red[2][ml][col] + red[3][ml][col])) + bwv[gate];
        pre[gate] = (a.sub_act == NBL_ACT_LINEAR ? t : nbl_act_apply(a.sub_act, t)) + gxv[gate];
    }
    const float gi = lstm_logistic(pre[0]);
    const float gf = lstm_logistic(pre[1]);
    const float gg = lstm_tanh(pre[2]);
    const float go = lstm_logistic(pre[3]);
    const float ig = __fmul_rn(gi, gg);
    const float cf = __fmul_rn(cprev, gf);
    const float ct = __fadd_rn(cf, ig);
    a.c[e] = ct;
    const float ht = __fmul_rn(lstm_tanh(ct), go);
    a.hout[e] = ht;
    a.hnext_op[opmajor_offset(m, h, a.H)] = ht;
}

// One step of the RNN layer's recurrence (rnn_layer.cc:100-115) in one launch, same work split as
// lstm_step_kernel: hid = act((prev . Wh^T) * g + b), state = in_t + hid; a block owns a 32x32 tile of
// the [B x O] step.  hid is also stored where the caller wants it (step 0's output gate reads it).
struct RnnStepArgs {
    const float *prev;               // row-major [B][H] (step 0: the input gate's output) or operand-major
    int prev_opmajor;
    const float *w_op;               // hidden gate's weights, operand-major [H][H]
    const float *g; const float *b; const float *in_t;
    float *state; float *hid;        // hid may be NULL
    float *state_op;                 // the new state once more, operand-major, for the next step
    int B, H, act;                   // H = layer width (rows of Wh and its fan-in)
};

__global__ __launch_bounds__(256)
void rnn_step_kernel(const RnnStepArgs a) {
    __shared__ float red[4][32][33];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int kw = a.H >> 2;
    const int arow = min(m0 + r, a.B - 1);  // row-major operand: rows past the batch repeat the last one; their sums are dropped
    // what follows the products is requested first and arrives behind the k loop
    const int ml = tid >> 3, c4 = (tid & 7) * 4;
    const int m = m0 + ml;
    const bool live = m < a.B;
    const size_t e = (size_t)(live ? m : 0) * a.H + n0 + c4;
    const float4 in = *reinterpret_cast<const float4*>(a.in_t + e);
    const float4 gq = *reinterpret_cast<const float4*>(a.g + n0 + c4), bq = *reinterpret_cast<const float4*>(a.b + n0 + c4);
    floatx16 acc0, acc1;
    wave_tile_from_global(a.prev_opmajor ? a.prev + opmajor_offset(m0 + r, wave * kw + half * 4, a.H)
                                         : a.prev + (size_t)arow * a.H + wave * kw + half * 4,
                          a.w_op + opmajor_offset(n0 + r, wave * kw + half * 4, a.H), kw, acc0, acc1,
                          a.prev_opmajor ? 256 : 8, 256);
    #pragma unroll
    for(int i = 0; i < 16; i++) red[wave][8 * (i >> 2) + 4 * half + (i & 3)][r] = acc0[i] + acc1[i];
    __syncthreads();
    // thread -> 4 adjacent columns of one row
    if(!live) return;
    const float gs[4] = { gq.x, gq.y, gq.z, gq.w }, bs[4] = { bq.x, bq.y, bq.z, bq.w };
    float v[4];
    #pragma unroll
    for(int j = 0; j < 4; j++) {
        const int col = c4 + j;
        const float sum = (red[0][ml][col] + red[1][ml][col]) + (red[2][ml][col] + red[3][ml][col]);
        v[j] = nbl_act_apply(a.act, __builtin_fmaf(sum, gs[j], bs[j]));
    }
    if(a.hid) *reinterpret_cast<float4*>(a.hid + e) = make_float4(v[0], v[1], v[2], v[3]);
    const float4 st = make_float4(__fadd_rn(in.x, v[0]), __fadd_rn(in.y, v[1]), __fadd_rn(in.z, v[2]), __fadd_rn(in.w, v[3]));
    *reinterpret_cast<float4*>(a.state + e) = st;
    *reinterpret_cast<float4*>(a.state_op + opmajor_offset(m, n0 + c4, a.H)) = st;     // four adjacent k: one piece
}

// state = a + b elementwise (the two axpy of rnn_layer.cc:108-115 on a zeroed state)
__global__ void add_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(i < n) out[i] = __fadd_rn(a[i], b[i]);
}

// LSTM cell for one time step from split-K partial sums of the recurrent GEMM:
//   pre[gate] = sub_act(sum_z part[z][m][n] + bw[n]) + gx[m][n],  n = (h/32)*128 + gate*32 + h%32
//   i, f, o = logistic(pre), g = tanh(pre);  c = c*f + i*g;  h_out = tanh(c)*o
// (lstm_layer.cc:264-312: each product is rounded on its own, as the separate CPU passes do).
__global__ void lstm_cell_kernel(const float *__restrict__ part, const float *__restrict__ gx,
                                 const float *__restrict__ bw, float *__restrict__ c, float *__restrict__ h_out,
                                 int M, int H, int Np, int S, int sub_act) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if(e >= M * H) return;
    const int m = e / H, h = e - m * H;
    const int nbase = (h >> 5) * 128 + (h & 31);
    const size_t plane = (size_t)M * Np;
    const float *__restrict__ p0 = part + (size_t)m * Np + nbase;
    float acc[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
    #pragma unroll 8
    for(int z = 0; z < S; z++) {
        #pragma unroll
        for(int gate = 0; gate < 4; gate++) acc[gate] += p0[(size_t)z * plane + gate * 32];
    }
    float pre[4];
    #pragma unroll
    for(int gate = 0; gate < 4; gate++) {
        const float t = acc[gate] + bw[nbase + gate * 32];
        pre[gate] = (sub_act == NBL_ACT_LINEAR ? t : nbl_act_apply(sub_act, t)) + gx[(size_t)m * Np + nbase + gate * 32];
    }
    const float gi = lstm_logistic(pre[0]);
    const float gf = lstm_logistic(pre[1]);
    const float gg = lstm_tanh(pre[2]);
    const float go = lstm_logistic(pre[3]);
    const float ig = __fmul_rn(gi, gg);
    const float cf = __fmul_rn(c[e], gf);
    const float ct = __fadd_rn(cf, ig);
    c[e] = ct;
    h_out[e] = __fmul_rn(lstm_tanh(ct), go);
}

// dst[c][r] = src[r][c] through a 32x33 LDS tile (both sides coalesced).
__global__ void transpose_kernel(const float *__restrict__ src, float *__restrict__ dst, unsigned rows, unsigned cols) {
    __shared__ float tile[32][33];
    const unsigned c0 = blockIdx.x * 32, r0 = blockIdx.y * 32, tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for(unsigned j = ty; j < 32; j += 8)
        if(r0 + j < rows && c0 + tx < cols) tile[j][tx] = src[(size_t)(r0 + j) * cols + c0 + tx];
    __syncthreads();
    for(unsigned j = ty; j < 32; j += 8)
        if(c0 + j < cols && r0 + tx < rows) dst[(size_t)(c0 + j) * rows + r0 + tx] = tile[tx][j];
}

// Input half of an LSTM whose input rows are one-hot (the recurrent driver's encoding,
// models/networks/recurrent.cc:179-204): x . Ucat^T is then column token[row] of Ucat, i.e. row
// token[row] of its transpose, so the [T*B x V].[V x 4H] product becomes a gather of T*B rows:
//   gx[row][n] = sub_act(UcatT[token[row]][n] + bu[n])
// (the same single float add the GEMM epilogue performs on a sum whose other terms are zero).
__global__ void token_gather_kernel(const float *__restrict__ w_t, const unsigned *__restrict__ tokens,
                                    const float *__restrict__ scale, const float *__restrict__ bias,
                                    float *__restrict__ out_rows, unsigned Np, unsigned vocab, int act) {
    // scale: per-column factor of a sub-layer with folded batch normalisation (the epilogue form of the products:
    // v * g + b), or NULL (v + b)
    const unsigned row = blockIdx.x, tok = tokens[row];
    const float *__restrict__ src = w_t + (size_t)tok * Np;
    float *__restrict__ out = out_rows + (size_t)row * Np;
    if((Np & 3u) == 0) {
        for(unsigned i = threadIdx.x; i < Np / 4; i += blockDim.x) {
            // a token outside the vocabulary is an all-zero row
            const float4 q = tok < vocab ? reinterpret_cast<const float4*>(src)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 b = reinterpret_cast<const float4*>(bias)[i];
            float v[4] = { q.x, q.y, q.z, q.w };
            const float bb[4] = { b.x, b.y, b.z, b.w };
            float gg[4] = { 1.f, 1.f, 1.f, 1.f };
            if(scale) { const float4 g = reinterpret_cast<const float4*>(scale)[i]; gg[0] = g.x; gg[1] = g.y; gg[2] = g.z; gg[3] = g.w; }
            #pragma unroll
            for(int c = 0; c < 4; c++) v[c] = nbl_act_apply(act, scale ? v[c] * gg[c] + bb[c] : v[c] + bb[c]);
            reinterpret_cast<float4*>(out)[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
    } else {
        for(unsigned i = threadIdx.x; i < Np; i += blockDim.x) {
            const float v = tok < vocab ? src[i] : 0.0f;
            out[i] = nbl_act_apply(act, scale ? v * scale[i] + bias[i] : v + bias[i]);
        }
    }
}

bool aligned16(const void *p) { return ((size_t)p & 15) == 0; }

}  // namespace

struct nbl_fc_plan {
    unsigned I, O; int act; bool has_scale;
    float *w_dev, *g_dev, *b_dev;
    float *w_tiled_dev;         // the weights once more as contiguous 16 KB [128 rows][32 k] tiles (I % 32 == 0), or NULL
    float *w_op_dev; unsigned K8p;      // ... and in operand-major order for fc_stream_kernel (I % 8 == 0), K8p k blocks per row tile, or NULL
    int kernel;                 // 0: chosen per call; 1: the LDS-tiled kernels; 2: the weight-streaming kernel wherever it applies
    float *ws_dev; size_t ws_bytes;     // split-K partial sums, grown on demand
};

struct nbl_lstm_plan {
    unsigned I, H, Hp;                  // Hp = H rounded up to 32
    int sub_act;
    float *ucat_dev;                    // [4*Hp][I]  input-side weights, interleaved gate order, BN scale folded in
    float *wcat_dev;                    // [4*Hp][H]  recurrent-side weights, same order
    float *wcat_op_dev;                 // the same matrix in operand-major layout (gate interleave 8 only)
    float *hop_dev[2]; size_t hop_bytes; // h_{t-1} / h_t in operand-major layout, [ceil(B/32)*32][H] each
    float *bu_dev, *bw_dev;             // [4*Hp] biases (BN shift folded in); for a linear sub_act bw is folded into bu
    float *gx_dev; float *h0_dev; float *c_dev; size_t gx_bytes, state_bytes;
    float *part_dev; size_t part_bytes;   // split-K partial sums of one recurrent step
    float *ucat_t_dev;                    // [I][4*Hp] transpose of ucat_dev, built on the first token-input forward
    unsigned G;                           // gate interleave: row of (gate, h) = (h/G)*4G + gate*G + h%G; 8 = single-launch steps
    // hidden and cell state kept between forward passes (hidden_state / cell_state of lstm_layer_t, which its forward
    // never clears): carry != 0 starts a pass from the state the previous pass of the same batch size ended with
    int carry; unsigned state_B;          // state_B: batch size the kept state belongs to, 0 = none (start from zero)
};

// rnn_layer_t: three connected sub-layers (input, hidden, output gate) and the per-forward buffers
struct nbl_rnn_plan {
    unsigned I, O;
    nbl_fc_plan *gate[3];
    float *in_all, *states, *hid0, *tmp;     // [T*B][O], [T*B][O], [B][O], [B][O]
    float *wh_op;                            // hidden gate's weights in operand-major layout (O % 128 == 0)
    float *sop[2]; size_t sop_bytes;         // state of the previous / this step in operand-major layout
    float *wi_t;                             // input gate's weights transposed to [I][O], built on the first token-fed pass
    size_t rows_alloc, seqs_alloc;
};

namespace {

// Grows the plan's split-K workspace to `need` bytes (or checks the fixed one) and returns where the parts go.
int splitk_workspace(nbl_ctx *ctx, size_t need, int S, int M, int N, float **ws, size_t *ws_bytes,
                     float *fixed_ws, size_t fixed_cap, float **part) {
    if(fixed_ws) {
        if(need > fixed_cap)
            return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_fc_fwd_noalloc: the %d partial sums of this %d x %d product need %zu bytes, "
                            "the static scratch holds %zu", S, M, N, need, fixed_cap);
        *part = fixed_ws;
        return NBL_OK;
    }
    if(*ws_bytes < need) {
        int rc = nbl_free(ctx, *ws);
        *ws = NULL; *ws_bytes = 0;
        if(rc != NBL_OK) return rc;
        if((rc = nbl_malloc(ctx, (void**)ws, need)) != NBL_OK) return rc;
        *ws_bytes = need;
    }
    *part = *ws;
    return NBL_OK;
}

int launch_splitk_reduce(nbl_ctx *ctx, const float *part, float *C, const float *g, const float *b, int M, int N, int S,
                         int act, int has_scale) {
    const size_t total = (size_t)M * N;
    if(N % 4 == 0 && aligned16(part) && aligned16(C))
        hipLaunchKernelGGL(splitk_reduce_kernel<4>, dim3((unsigned)nbl_div_up_sz(total / 4, 256)), dim3(256), 0, ctx->stream,
                           part, C, g, b, M, N, S, act, has_scale);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel<1>, dim3((unsigned)nbl_div_up_sz(total, 256)), dim3(256), 0, ctx->stream,
                           part, C, g, b, M, N, S, act, has_scale);
    NBL_LAUNCH_CHECK(ctx, "splitk_reduce_kernel");
    return NBL_OK;
}

template<int MT, int NT, int RING>
int launch_fc_stream_kernel(nbl_ctx *ctx, const FcStreamArgs &a, dim3 grid) {
    const size_t lds = (size_t)2 * 32 * MT * FC_X_PITCH * sizeof(float);
    static nbl_lds_limit_raised raised;         // more than 64 KB of dynamic LDS has to be asked for, once per kernel and device
    if(lds > 64 * 1024) NBL_HIP(ctx, raised.ensure(fc_stream_kernel<MT, NT, RING>, ctx->device, (int)lds));
    hipLaunchKernelGGL((fc_stream_kernel<MT, NT, RING>), grid, dim3(256), lds, ctx->stream, a);
    NBL_LAUNCH_CHECK(ctx, "fc_stream_kernel");
    return NBL_OK;
}

// The weight-streaming kernel over operand-major weights.  Returns 1 (and launches nothing) for a shape it does not take.
int launch_fc_stream(nbl_ctx *ctx, const float *A, const float *Bw_op, unsigned K8p, float *C, int M, int N, int K,
                     const float *g, const float *b, int act, int has_scale, float **ws, size_t *ws_bytes,
                     float *fixed_ws, size_t fixed_cap) {
    const unsigned ntiles = nbl_div_up(N, 32);
    if(M > 64 || K % 8 != 0 || (size_t)ntiles * K8p * 1024 >= (1ull << 32) || (size_t)M * K * 4 >= (1ull << 31))
        return 1;
    // One tile of 32 neurons per wave and 16 loads in flight: measured against two tiles per wave and rings of 8 and 32
    // on VGG-16's connected layers at batch 32 (80.2 us against 84.0 / 82.1 / 81.7 for the 415 MB layer, 18.3 against
    // 20.1 / 22.0 / 20.9 for the 68 MB one): the finer blocks halve the partial sums a split launch writes.
    constexpr int NT = 1, RING = 16;
    const int MT = M <= 32 ? 1 : 2;
    const unsigned groups = nbl_div_up(ntiles, 4 * NT);
    // Split of the k range: blocks are dealt to the CUs evenly, so the launch lasts as long as the CU with the most
    // work.  In bytes a CU has to pull: its blocks' weights, a fixed cost per block (start-up: the first chunk of
    // activations, the ring's first loads), and its share of the partial sums written and read back.
    int best_s = 1; double best_cost = 0.0;
    for(int s = 1; s <= 64; s++) {
        const unsigned kbps = nbl_div_up(nbl_div_up(K8p, s), FC_KALIGN) * FC_KALIGN, s_eff = nbl_div_up(K8p, kbps);
        if((int)s_eff != s) continue;
        const double rounds = (double)nbl_div_up_sz((size_t)groups * s, ctx->num_cu);
        const double cost = rounds * ((double)kbps * 4 * NT * 1024 + 48.0 * 1024) +
                            (s > 1 ? 2.0 * s * M * N * 4 / ctx->num_cu + 64.0 * 1024 : 0.0);
        if(s == 1 || cost < best_cost) { best_cost = cost; best_s = s; }
    }
    FcStreamArgs a;
    a.x = A; a.w_op = Bw_op; a.g = g; a.b = b; a.act = act; a.has_scale = has_scale;
    a.M = M; a.N = N; a.K = K; a.K8p = (int)K8p; a.ntiles = (int)ntiles;
    a.kb_per_split = (int)(nbl_div_up(nbl_div_up(K8p, best_s), FC_KALIGN) * FC_KALIGN);
    const int S = (int)nbl_div_up(K8p, a.kb_per_split);
    a.direct = S == 1;
    float *part = C;
    if(S > 1) {
        const int rc = splitk_workspace(ctx, (size_t)S * M * N * sizeof(float), S, M, N, ws, ws_bytes, fixed_ws, fixed_cap, &part);
        if(rc != NBL_OK) return rc;
    }
    a.out = part;
    const dim3 grid(groups, S);
    const int rc = MT == 1 ? launch_fc_stream_kernel<1, NT, RING>(ctx, a, grid) : launch_fc_stream_kernel<2, NT, RING>(ctx, a, grid);
    if(rc != NBL_OK) return rc;
    if(S > 1) return launch_splitk_reduce(ctx, part, C, g, b, M, N, S, act, has_scale);
    return NBL_OK;
}

// Bw_tiled: the same weights as 16 KB tiles (see GemmArgs::b_tiled), or NULL; used whenever the buffer-load kernel runs
// ws / ws_bytes: the plan's split-K workspace, grown here on demand (NULL: never split).  With fixed_ws the partial
// sums go to that buffer of fixed_cap bytes instead and nothing is allocated or freed: a product whose split
// needs more than fixed_cap is refused.
// Bw_op / K8p: the weights in operand-major order (nbl_fc_pack), or NULL; kernel: nbl_fc_plan::kernel
int launch_fc(nbl_ctx *ctx, const float *A, const float *Bw, float *C, int M, int N, int K,
              const float *g, const float *b, int act, int has_scale, float **ws, size_t *ws_bytes,
              const float *Bw_tiled = NULL, float *fixed_ws = NULL, size_t fixed_cap = 0,
              const float *Bw_op = NULL, unsigned K8p = 0, int kernel = 0) {
    // Small batches over a large matrix: the weight-streaming kernel.  (Below some tens of MB a layer is a few
    // microseconds either way and the tiled kernel's finer k-split fills the chip better; so it does for a short
    // fan-in, which leaves a streaming block two or three chunks of activations to walk: the 1024 -> 10000
    // projection behind an LSTM at batch 64 takes 23.5 us tiled and 26.1 us streamed, a fan-in of 4096 ties.)
    if(Bw_op && M <= 64 && kernel != 1 && aligned16(A) && (ws || fixed_ws) &&
       (kernel == 2 || ((size_t)N * K * sizeof(float) >= ((size_t)24 << 20) && K >= 4096))) {
        const int rc = launch_fc_stream(ctx, A, Bw_op, K8p, C, M, N, K, g, b, act, has_scale, ws, ws_bytes, fixed_ws, fixed_cap);
        if(rc != 1) return rc;       // (a shape it does not take falls through to the tiled kernels)
    }
    GemmArgs a;
    memset(&a, 0, sizeof(a));
    a.A = A; a.Bw = Bw; a.C = C; a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = K; a.ldc = N;
    a.vec_ok = (K % 4 == 0) && aligned16(A) && aligned16(Bw);
    a.g = g; a.b = b; a.act = act; a.has_scale = has_scale;
    // tile: 32*MT rows of batch per wave row
    const bool small_m = M <= 32;
    // Large batches: 128x128 tiles hold two blocks of four waves per CU, whose stalls (tile hand-over: LDS writes, barrier,
    // first LDS reads) tend to fall together; 64x64 tiles hold four blocks per CU and keep the matrix pipe busier
    // wherever they alone fill the chip at least twice over without a k-split: the LSTM's input product over all
    // time steps ([4096 x 1024].[1024 x 4096]) 277 -> 253 us.  Launches that need a k-split to fill the chip keep
    // the large tile (AlexNet's 9216 -> 4096 layer at batch 128: 85.1 us against 86.7).
    const bool t64 = M > 64 && a.vec_ok && K % GEMM_BK == 0 && (size_t)M * K * 4 < (1ull << 31) &&
                     (size_t)nbl_div_up(N, 128) * 128 * K * 4 < (1ull << 31) &&
                     (size_t)nbl_div_up(M, 64) * nbl_div_up(N, 64) >= 2 * (size_t)ctx->num_cu;
    const int BM = t64 ? 64 : small_m ? 32 : (M <= 64 ? 64 : 128);
    const int BN = t64 ? 64 : 128;
    const unsigned gm = nbl_div_up(M, BM), gn = nbl_div_up(N, BN);
    // Split K so that every CU walks about the same number of k-tiles: blocks are dealt to the CUs round robin, so a
    // launch lasts as long as the CU with the most blocks, ceil(blocks / CUs) chunks of k-tiles plus a partial tile
    // written (and read again by the reduction) per block.  The chunk count need not be a power of two: 640 blocks on
    // 256 CUs (three on some, two on others) stream a 492 MB matrix 7 % slower than 500.
    int S = 1;
    const int ktiles = nbl_div_up(K, GEMM_BK);
    if(ws || fixed_ws) {
        double best = 0.0;
        for(int s = 1; s <= 64 && ktiles / s >= 2; s++) {
            const int chunk = nbl_div_up(ktiles, s), s_eff = nbl_div_up(ktiles, chunk);
            if(s_eff != s) continue;
            const size_t blocks = (size_t)gm * gn * s;
            const double rounds = (double)nbl_div_up_sz(blocks, ctx->num_cu);
            const double cost = rounds * ((double)chunk * (BM + BN) * GEMM_BK + (s > 1 ? 2.0 * BM * BN : 0.0));
            if(s == 1 || cost < best) { best = cost; S = s; }
        }
    }
    a.k_chunk = nbl_div_up(ktiles, S) * GEMM_BK;
    S = nbl_div_up(K, a.k_chunk);
    dim3 grid(gn, gm, S), block(256);
    // every k-tile whole and both operands addressable by 31-bit byte offsets: the buffer-load variant
    const bool buf_ok = a.vec_ok && K % GEMM_BK == 0 && (size_t)M * K * 4 < (1ull << 31) &&
                        (size_t)nbl_div_up(N, 128) * 128 * K * 4 < (1ull << 31);
    if(buf_ok && Bw_tiled && !t64) { a.Bw = Bw_tiled; a.b_tiled = 1; }
    if(S > 1) {
        float *part = NULL;
        const int rc_ws = splitk_workspace(ctx, (size_t)S * M * N * sizeof(float), S, M, N, ws, ws_bytes, fixed_ws, fixed_cap, &part);
        if(rc_ws != NBL_OK) return rc_ws;
        a.C = part;
        if(t64)                        hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 2, 2, 4, EPI_PARTIAL, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 32 && buf_ok)    hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 1, 4, 4, EPI_PARTIAL, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 64 && buf_ok)    hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 1, 1, 4, 4, EPI_PARTIAL, true>), grid, block, 0, ctx->stream, a);
        else if(buf_ok)                hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 2, 2, 2, 2, EPI_PARTIAL, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 32 && a.vec_ok)  hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 1, 4, 4, EPI_PARTIAL, false>), grid, block, 0, ctx->stream, a);
        else if(BM == 64 && a.vec_ok)  hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 1, 1, 4, 4, EPI_PARTIAL, false>), grid, block, 0, ctx->stream, a);
        else if(a.vec_ok)              hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 2, 2, 2, 2, EPI_PARTIAL, false>), grid, block, 0, ctx->stream, a);
        else if(BM == 32)  hipLaunchKernelGGL((gemm_nt_kernel<1, 1, 1, 4, EPI_PARTIAL>), grid, block, 0, ctx->stream, a);
        else if(BM == 64)  hipLaunchKernelGGL((gemm_nt_kernel<1, 2, 2, 2, EPI_PARTIAL>), grid, block, 0, ctx->stream, a);
        else               hipLaunchKernelGGL((gemm_nt_kernel<2, 2, 2, 2, EPI_PARTIAL>), grid, block, 0, ctx->stream, a);
        NBL_LAUNCH_CHECK(ctx, "gemm_nt_kernel(split-k)");
        const int rc_red = launch_splitk_reduce(ctx, part, C, g, b, M, N, S, act, has_scale);
        if(rc_red != NBL_OK) return rc_red;
    } else {
        if(t64)                        hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 2, 2, 4, EPI_DIRECT, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 32 && buf_ok)    hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 1, 4, 4, EPI_DIRECT, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 64 && buf_ok)    hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 1, 1, 4, 4, EPI_DIRECT, true>), grid, block, 0, ctx->stream, a);
        else if(buf_ok)                hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 2, 2, 2, 2, EPI_DIRECT, true>), grid, block, 0, ctx->stream, a);
        else if(BM == 32 && a.vec_ok)  hipLaunchKernelGGL((gemm_nt_stream_kernel<1, 1, 1, 4, 4, EPI_DIRECT, false>), grid, block, 0, ctx->stream, a);
        else if(BM == 64 && a.vec_ok)  hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 1, 1, 4, 4, EPI_DIRECT, false>), grid, block, 0, ctx->stream, a);
        else if(a.vec_ok)              hipLaunchKernelGGL((gemm_nt_stream_kernel<2, 2, 2, 2, 2, EPI_DIRECT, false>), grid, block, 0, ctx->stream, a);
        else if(BM == 32)  hipLaunchKernelGGL((gemm_nt_kernel<1, 1, 1, 4, EPI_DIRECT>), grid, block, 0, ctx->stream, a);
        else if(BM == 64)  hipLaunchKernelGGL((gemm_nt_kernel<1, 2, 2, 2, EPI_DIRECT>), grid, block, 0, ctx->stream, a);
        else               hipLaunchKernelGGL((gemm_nt_kernel<2, 2, 2, 2, EPI_DIRECT>), grid, block, 0, ctx->stream, a);
        NBL_LAUNCH_CHECK(ctx, "gemm_nt_kernel");
    }
    return NBL_OK;
}

}  // namespace

extern "C" {

int nbl_fc_pack(nbl_ctx *ctx, const float *weight_host, const float *bias_host,
                const float *scale_host, const float *mean_host, const float *var_host,
                unsigned I, unsigned O, int act, nbl_fc_plan **out) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, out != NULL, "nbl_fc_pack: out is NULL");
    *out = NULL;
    NBL_REQUIRE(ctx, weight_host && bias_host, "nbl_fc_pack: weight/bias is NULL");
    NBL_REQUIRE(ctx, (scale_host != NULL) == (mean_host != NULL) && (scale_host != NULL) == (var_host != NULL),
                "nbl_fc_pack: scale, mean and var must be given together");
    NBL_REQUIRE(ctx, I && O, "nbl_fc_pack: zero dimension");
    NBL_REQUIRE(ctx, nbl_act_valid(act), "nbl_fc_pack: undefined activation type %d", act);
    if((size_t)I * O >= (1ull << 31)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_fc_pack: weight matrix too large");
    nbl_fc_plan *p = new nbl_fc_plan();
    p->I = I; p->O = O; p->act = act; p->has_scale = scale_host != NULL;
    p->w_dev = p->g_dev = p->b_dev = p->ws_dev = p->w_tiled_dev = p->w_op_dev = NULL; p->ws_bytes = 0; p->K8p = 0; p->kernel = 0;
    std::vector<float> g(O), b(O);
    nbl_fold_batchnorm(bias_host, scale_host, mean_host, var_host, O, g.data(), b.data());
    int rc;
    if((rc = nbl_malloc(ctx, (void**)&p->w_dev, (size_t)I * O * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->g_dev, O * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->b_dev, O * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->w_dev, weight_host, (size_t)I * O * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->g_dev, g.data(), O * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->b_dev, b.data(), O * sizeof(float))) != NBL_OK) {
        nbl_fc_plan_destroy(ctx, p);
        return rc;
    }
    // Streaming layout: every block of the product walks its own contiguous run of 16 KB tiles, where the row-major
    // matrix gives it 128 B from each of 128 rows per k-tile (a plain read of the two layouts: 6.0 vs 5.3 TB/s).
    const size_t tiled_elems = (size_t)nbl_div_up(O, 128) * 128 * I;
    if(I % GEMM_BK == 0 && tiled_elems * sizeof(float) < (1ull << 31)) {
        std::vector<float> tiled(tiled_elems, 0.0f);
        const unsigned ktiles = I / GEMM_BK;
        for(unsigned n = 0; n < O; n++) {
            const float *src = weight_host + (size_t)n * I;
            for(unsigned kt = 0; kt < ktiles; kt++) {
                float *dst = tiled.data() + (((size_t)(n / 128) * ktiles + kt) * 128 + n % 128) * GEMM_BK;
                memcpy(dst, src + (size_t)kt * GEMM_BK, GEMM_BK * sizeof(float));
            }
        }
        if((rc = nbl_malloc(ctx, (void**)&p->w_tiled_dev, tiled_elems * sizeof(float))) != NBL_OK ||
           (rc = nbl_h2d(ctx, p->w_tiled_dev, tiled.data(), tiled_elems * sizeof(float))) != NBL_OK) {
            nbl_fc_plan_destroy(ctx, p);
            return rc;
        }
    }
    // Operand-major copy for the weight-streaming kernel (small batches): row tiles of 32 neurons, K8p k blocks of 8
    // each (the k range padded with zeros to whole rings of loads), the 64 pieces of a k block contiguous.
    const unsigned K8p = nbl_div_up(nbl_div_up(I, 8), FC_KALIGN) * FC_KALIGN, ntiles = nbl_div_up(O, 32);
    if(I % 8 == 0 && (size_t)ntiles * K8p * 1024 < (1ull << 32)) {
        std::vector<float> wop((size_t)ntiles * K8p * 256, 0.0f);
        for(unsigned n = 0; n < O; n++) {
            const float *src = weight_host + (size_t)n * I;
            float *tile = wop.data() + (size_t)(n / 32) * K8p * 256 + (n % 32) * 4;
            for(unsigned k = 0; k < I; k += 4)      // the piece of lane (half = k / 4 % 2, r = n % 32) of k block k / 8
                memcpy(tile + (size_t)(k / 8) * 256 + ((k / 4) % 2) * 128, src + k, 4 * sizeof(float));
        }
        if((rc = nbl_malloc(ctx, (void**)&p->w_op_dev, wop.size() * sizeof(float))) != NBL_OK ||
           (rc = nbl_h2d(ctx, p->w_op_dev, wop.data(), wop.size() * sizeof(float))) != NBL_OK) {
            nbl_fc_plan_destroy(ctx, p);
            return rc;
        }
        p->K8p = K8p;
    }
    *out = p;
    return NBL_OK;
}

int nbl_fc_plan_set_kernel(nbl_fc_plan *p, int kernel) {
    if(!p || kernel < 0 || kernel > 2) return NBL_EINVAL;
    p->kernel = kernel;
    return NBL_OK;
}

int nbl_fc_plan_destroy(nbl_ctx *ctx, nbl_fc_plan *p) {
    if(!ctx || !p) return NBL_EINVAL;
    nbl_free(ctx, p->w_dev); nbl_free(ctx, p->g_dev); nbl_free(ctx, p->b_dev); nbl_free(ctx, p->ws_dev);
    nbl_free(ctx, p->w_tiled_dev); nbl_free(ctx, p->w_op_dev);
    delete p;
    return NBL_OK;
}

int nbl_fc_fwd(nbl_ctx *ctx, const nbl_fc_plan *plan, const float *x_dev, float *y_dev, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, plan && x_dev && y_dev, "nbl_fc_fwd: NULL argument");
    if(B == 0) return NBL_OK;
    if((size_t)B * plan->I >= (1ull << 31) || (size_t)B * plan->O >= (1ull << 31))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_fc_fwd: tensors of 2^31 elements or more are not supported");
    nbl_fc_plan *p = const_cast<nbl_fc_plan*>(plan);   // the split-K workspace is a cache
    return launch_fc(ctx, x_dev, p->w_dev, y_dev, (int)B, (int)p->O, (int)p->I, p->g_dev, p->b_dev,
                     p->act, p->has_scale ? 1 : 0, &p->ws_dev, &p->ws_bytes, p->w_tiled_dev, NULL, 0, p->w_op_dev, p->K8p, p->kernel);
}

// ---- fully connected without allocation ----------------------------------------------------------
// Split-K partial sums of nbl_fc_fwd_noalloc live in a file-scope device array, one copy per GPU for the life of
// the process.  On the host the array's NAME is only a handle: the address kernels can use comes from
// hipGetSymbolAddress, asked once per device with that device current (at context creation), and is kept per device.
}  // extern "C"

namespace {

constexpr size_t FC_SCRATCH_BYTES = (size_t)NBL_FC_NOALLOC_SCRATCH_BYTES;
constexpr int FC_SCRATCH_MAX_DEVICES = 64;
static __device__ __align__(256) float fc_noalloc_scratch[FC_SCRATCH_BYTES / sizeof(float)];
float *g_fc_scratch_ptr[FC_SCRATCH_MAX_DEVICES];
std::mutex g_fc_scratch_lock;

}  // namespace

// Device address of this GPU's copy of the scratch array, looked up once per device (with that device current) when
// the device's first context is created, so that nbl_fc_fwd_noalloc itself only launches kernels -- nothing in it
// loads a code object or touches the current device, which a stream capture around it could not record.
int nbl_fc_scratch_resolve(nbl_ctx *ctx) {
    ctx->fc_scratch = NULL;
    if(ctx->device < 0 || ctx->device >= FC_SCRATCH_MAX_DEVICES) return NBL_OK;      // nbl_fc_fwd_noalloc refuses such a context
    std::lock_guard<std::mutex> hold(g_fc_scratch_lock);
    if(!g_fc_scratch_ptr[ctx->device]) {
        NBL_HIP(ctx, hipSetDevice(ctx->device));
        void *p = NULL;
        NBL_HIP(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(fc_noalloc_scratch)));
        if(!p || ((size_t)p & 255) != 0)
            return nbl_fail(ctx, NBL_EHIP, "hipGetSymbolAddress returned an unusable address %p for the static scratch array", p);
        g_fc_scratch_ptr[ctx->device] = (float*)p;
    }
    ctx->fc_scratch = g_fc_scratch_ptr[ctx->device];
    return NBL_OK;
}

extern "C" {

int nbl_fc_fwd_noalloc(nbl_ctx *ctx, const nbl_fc_plan *plan, const float *x_dev, float *y_dev, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, plan && x_dev && y_dev, "nbl_fc_fwd_noalloc: NULL argument");
    if(B == 0) return NBL_OK;
    if((size_t)B * plan->I >= (1ull << 31) || (size_t)B * plan->O >= (1ull << 31))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_fc_fwd_noalloc: tensors of 2^31 elements or more are not supported");
    float *scratch = ctx->fc_scratch;
    if(!scratch)
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_fc_fwd_noalloc: no static scratch on device %d (index beyond %d)", ctx->device, FC_SCRATCH_MAX_DEVICES);
    // every partial sum the reduction reads is written by this call's product kernel first, so the contents a
    // previous call left behind never show
    return launch_fc(ctx, x_dev, plan->w_dev, y_dev, (int)B, (int)plan->O, (int)plan->I, plan->g_dev, plan->b_dev,
                     plan->act, plan->has_scale ? 1 : 0, NULL, NULL, plan->w_tiled_dev, scratch, FC_SCRATCH_BYTES,
                     plan->w_op_dev, plan->K8p, plan->kernel);
}

// ---- LSTM ----------------------------------------------------------------------------------------
// file order of the eight sub-layers (lstm_layer.cc:194-206) and the gate each one feeds;
// compute order of the gates inside a wave tile is i, f, g (cell candidate), o.
int nbl_lstm_pack(nbl_ctx *ctx, const float *const *weight_host, const float *const *bias_host,
                  const float *const *scale_host, const float *const *mean_host, const float *const *var_host,
                  unsigned I, unsigned H, int sub_act, nbl_lstm_plan **out) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, out != NULL, "nbl_lstm_pack: out is NULL");
    *out = NULL;
    NBL_REQUIRE(ctx, weight_host && bias_host, "nbl_lstm_pack: weight/bias is NULL");
    NBL_REQUIRE(ctx, (scale_host != NULL) == (mean_host != NULL) && (scale_host != NULL) == (var_host != NULL),
                "nbl_lstm_pack: scale, mean and var must be given together");
    NBL_REQUIRE(ctx, I && H, "nbl_lstm_pack: zero dimension");
    NBL_REQUIRE(ctx, nbl_act_valid(sub_act), "nbl_lstm_pack: undefined activation type %d", sub_act);
    for(int s = 0; s < 8; s++) {
        NBL_REQUIRE(ctx, weight_host[s] && bias_host[s], "nbl_lstm_pack: sub-layer %d has a NULL array", s);
        if(scale_host) NBL_REQUIRE(ctx, scale_host[s] && mean_host[s] && var_host[s],
                                   "nbl_lstm_pack: sub-layer %d has a NULL batchnorm array", s);
    }
    // file slot of (side, gate): W side = 0..3, U side = 4..7; within a side the file order is i, f, o, c
    static const int slot_of_gate[4] = { 0, 1, 3, 2 };   // gate i, f, g(c), o -> offset inside the side
    nbl_lstm_plan *p = new nbl_lstm_plan();
    memset(p, 0, sizeof(*p));
    p->I = I; p->H = H; p->Hp = nbl_div_up(H, 32) * 32; p->sub_act = sub_act;
    p->G = H % 128 == 0 ? 8 : 32;
    const unsigned Np = 4 * p->Hp;
    std::vector<float> ucat((size_t)Np * I, 0.0f), wcat((size_t)Np * H, 0.0f), bu(Np, 0.0f), bw(Np, 0.0f);
    std::vector<float> g(H), b(H);
    for(int side = 0; side < 2; side++) {         // 0 = W (hidden), 1 = U (input)
        const unsigned fan_in = side == 0 ? H : I;
        std::vector<float> &cat = side == 0 ? wcat : ucat;
        std::vector<float> &bias = side == 0 ? bw : bu;
        for(int gate = 0; gate < 4; gate++) {
            const int s = side * 4 + slot_of_gate[gate];
            nbl_fold_batchnorm(bias_host[s], scale_host ? scale_host[s] : NULL, mean_host ? mean_host[s] : NULL,
                               var_host ? var_host[s] : NULL, H, g.data(), b.data());
            for(unsigned h = 0; h < H; h++) {
                const size_t row = (size_t)(h / p->G) * (4 * p->G) + gate * p->G + (h % p->G);
                const float *src = weight_host[s] + (size_t)h * fan_in;
                float *dst = cat.data() + row * fan_in;
                // batchnorm scale folded into the row (1 when batch_normalize=0)
                for(unsigned k = 0; k < fan_in; k++) dst[k] = scale_host ? (float)((double)src[k] * (double)g[h]) : src[k];
                bias[row] = b[h];
            }
        }
    }
    // gate pre-activation = sub_act(U.x + bu) + sub_act(W.h + bw); for a linear sub_act the two biases merge
    if(sub_act == NBL_ACT_LINEAR)
        for(unsigned n = 0; n < Np; n++) { bu[n] = bu[n] + bw[n]; bw[n] = 0.0f; }
    int rc;
    if(p->G == 8) {        // the per-step kernel reads the recurrent weights in operand-major order (H % 128 == 0 here)
        std::vector<float> wop((size_t)Np * H);
        for(unsigned n = 0; n < Np; n++)
            for(unsigned k = 0; k < H; k++) wop[opmajor_offset(n, k, H)] = wcat[(size_t)n * H + k];
        if((rc = nbl_malloc(ctx, (void**)&p->wcat_op_dev, wop.size() * sizeof(float))) != NBL_OK ||
           (rc = nbl_h2d(ctx, p->wcat_op_dev, wop.data(), wop.size() * sizeof(float))) != NBL_OK) {
            nbl_lstm_plan_destroy(ctx, p);
            return rc;
        }
    }
    if((rc = nbl_malloc(ctx, (void**)&p->ucat_dev, ucat.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->wcat_dev, wcat.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->bu_dev, Np * sizeof(float))) != NBL_OK ||
       (rc = nbl_malloc(ctx, (void**)&p->bw_dev, Np * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->ucat_dev, ucat.data(), ucat.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->wcat_dev, wcat.data(), wcat.size() * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->bu_dev, bu.data(), Np * sizeof(float))) != NBL_OK ||
       (rc = nbl_h2d(ctx, p->bw_dev, bw.data(), Np * sizeof(float))) != NBL_OK) {
        nbl_lstm_plan_destroy(ctx, p);
        return rc;
    }
    *out = p;
    return NBL_OK;
}

int nbl_lstm_plan_destroy(nbl_ctx *ctx, nbl_lstm_plan *p) {
    if(!ctx || !p) return NBL_EINVAL;
    nbl_free(ctx, p->ucat_dev); nbl_free(ctx, p->wcat_dev); nbl_free(ctx, p->bu_dev); nbl_free(ctx, p->bw_dev);
    nbl_free(ctx, p->gx_dev); nbl_free(ctx, p->h0_dev); nbl_free(ctx, p->c_dev); nbl_free(ctx, p->part_dev);
    nbl_free(ctx, p->ucat_t_dev); nbl_free(ctx, p->wcat_op_dev); nbl_free(ctx, p->hop_dev[0]); nbl_free(ctx, p->hop_dev[1]);
    delete p;
    return NBL_OK;
}

// h [B][H] row-major -> the operand-major copy lstm_step_kernel reads (rows past B stay as they are)
__global__ __launch_bounds__(256)
void lstm_state_to_opmajor_kernel(const float *__restrict__ h, float *__restrict__ hop, unsigned B, unsigned H) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= (size_t)B * H) return;
    const unsigned m = (unsigned)(i / H), k = (unsigned)(i % H);
    hop[opmajor_offset(m, k, H)] = h[i];
}

// Buffers of the running state for batch size B (grown on demand; growing drops a kept state).
static int lstm_state_buffers(nbl_ctx *ctx, nbl_lstm_plan *p, unsigned B) {
    int rc;
    const size_t st_need = (size_t)B * p->H * sizeof(float);
    if(p->state_bytes < st_need) {
        if((rc = nbl_free(ctx, p->h0_dev)) != NBL_OK || (rc = nbl_free(ctx, p->c_dev)) != NBL_OK) return rc;
        p->h0_dev = p->c_dev = NULL; p->state_bytes = 0; p->state_B = 0;
        if((rc = nbl_malloc(ctx, (void**)&p->h0_dev, st_need)) != NBL_OK ||
           (rc = nbl_malloc(ctx, (void**)&p->c_dev, st_need)) != NBL_OK) return rc;
        p->state_bytes = st_need;
    }
    const size_t hop_need = (size_t)nbl_div_up(B, 32) * 32 * p->H * sizeof(float);
    if(p->G == 8 && p->hop_bytes < hop_need) {
        if((rc = nbl_free(ctx, p->hop_dev[0])) != NBL_OK || (rc = nbl_free(ctx, p->hop_dev[1])) != NBL_OK) return rc;
        p->hop_dev[0] = p->hop_dev[1] = NULL; p->hop_bytes = 0; p->state_B = 0;
        if((rc = nbl_malloc(ctx, (void**)&p->hop_dev[0], hop_need)) != NBL_OK ||
           (rc = nbl_malloc(ctx, (void**)&p->hop_dev[1], hop_need)) != NBL_OK) return rc;
        p->hop_bytes = hop_need;
        // rows past the batch are read (their sums are dropped) and must hold numbers; the step kernel writes
        // real rows only, so zeroing once is enough
        if((rc = nbl_fill_zero(ctx, p->hop_dev[0], hop_need)) != NBL_OK ||
           (rc = nbl_fill_zero(ctx, p->hop_dev[1], hop_need)) != NBL_OK) return rc;
    }
    return NBL_OK;
}

// x_dev: dense input rows, or NULL with tokens_dev: one token per row (one-hot input)
static int lstm_forward(nbl_ctx *ctx, nbl_lstm_plan *p, const float *x_dev, const unsigned *tokens_dev, float *y_dev,
                        float *cell_dev, unsigned T, unsigned B) {
    if(T == 0 || B == 0) return NBL_OK;
    const unsigned Np = 4 * p->Hp;
    if((size_t)T * B * Np >= (1ull << 31) || (x_dev && (size_t)T * B * p->I >= (1ull << 31)))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_lstm_fwd: tensors of 2^31 elements or more are not supported");
    int rc;
    const size_t gx_need = (size_t)T * B * Np * sizeof(float), st_need = (size_t)B * p->H * sizeof(float);
    if(p->gx_bytes < gx_need) {
        if((rc = nbl_free(ctx, p->gx_dev)) != NBL_OK) return rc;
        p->gx_dev = NULL; p->gx_bytes = 0;
        if((rc = nbl_malloc(ctx, (void**)&p->gx_dev, gx_need)) != NBL_OK) return rc;
        p->gx_bytes = gx_need;
    }
    if((rc = lstm_state_buffers(ctx, p, B)) != NBL_OK) return rc;
    const size_t hop_need = (size_t)nbl_div_up(B, 32) * 32 * p->H * sizeof(float);
    // Initial state: zero (the first forward() of a fresh reference layer), or -- when the plan carries its state and
    // holds one for this batch size -- h and c as the previous pass (or nbl_lstm_plan_set_state) left them:
    // c in c_dev, h in hop_dev[0] (operand-major) or h0_dev.
    if(!(p->carry && p->state_B == B)) {
        if((rc = nbl_fill_zero(ctx, p->c_dev, st_need)) != NBL_OK) return rc;
        if(p->G == 8) { if((rc = nbl_fill_zero(ctx, p->hop_dev[0], hop_need)) != NBL_OK) return rc; }
        else if((rc = nbl_fill_zero(ctx, p->h0_dev, st_need)) != NBL_OK) return rc;
    }
    p->state_B = 0;       // (set again once this pass has been queued completely)
    // input half for every step at once: gx[T*B][Np] = sub_act(x . Ucat^T + bu)
    if(tokens_dev) {
        if(!p->ucat_t_dev) {
            if((rc = nbl_malloc(ctx, (void**)&p->ucat_t_dev, (size_t)Np * p->I * sizeof(float))) != NBL_OK) return rc;
            hipLaunchKernelGGL(transpose_kernel, dim3(nbl_div_up(p->I, 32), nbl_div_up(Np, 32)), dim3(256), 0, ctx->stream,
                               p->ucat_dev, p->ucat_t_dev, Np, p->I);
            NBL_LAUNCH_CHECK(ctx, "transpose_kernel");
        }
        hipLaunchKernelGGL(token_gather_kernel, dim3(T * B), dim3(256), 0, ctx->stream,
                           p->ucat_t_dev, tokens_dev, (const float*)NULL, p->bu_dev, p->gx_dev, Np, p->I, p->sub_act);
        NBL_LAUNCH_CHECK(ctx, "token_gather_kernel");
    } else if((rc = launch_fc(ctx, x_dev, p->ucat_dev, p->gx_dev, (int)(T * B), (int)Np, (int)p->I, NULL, p->bu_dev,
                              p->sub_act, 0, NULL, NULL)) != NBL_OK) return rc;
    const size_t step = (size_t)B * p->H;
    if(p->G == 8) {
        // Recurrent half, one launch per step (lstm_step_kernel).  h_{t-1} is read straight from y[t-1].
        LstmStepArgs sa;
        sa.w_op = p->wcat_op_dev; sa.bw = p->bw_dev; sa.c = p->c_dev; sa.B = (int)B; sa.H = (int)p->H; sa.Np = (int)Np;
        sa.sub_act = p->sub_act;
        const dim3 grid(Np / 32, nbl_div_up(B, 32));
        for(unsigned t = 0; t < T; t++) {
            sa.hprev_op = p->hop_dev[t & 1];
            sa.hnext_op = p->hop_dev[(t + 1) & 1];
            sa.gx = p->gx_dev + (size_t)t * B * Np;
            sa.hout = y_dev + (size_t)t * step;
            hipLaunchKernelGGL(lstm_step_kernel, grid, dim3(256), 0, ctx->stream, sa);
            NBL_LAUNCH_CHECK(ctx, "lstm_step_kernel");
        }
    } else {
    // Recurrent half for the 32-wide gate interleave.  One step is only [B x H].[H x 4H]: to put work on
    // every CU the k range is split over blockIdx.z into partial sums (deterministic order) and a small
    // cell kernel finishes the step.  Narrow problems keep the single fused kernel.
    GemmArgs a;
    memset(&a, 0, sizeof(a));
    a.Bw = p->wcat_dev; a.M = (int)B; a.N = (int)Np; a.K = (int)p->H; a.lda = (int)p->H; a.ldb = (int)p->H;
    a.ldc = (int)Np;
    a.b = p->bw_dev; a.act = p->sub_act; a.c = p->c_dev; a.H = (int)p->H;
    const int ktiles = nbl_div_up(p->H, GEMM_BK);
    const unsigned gm = nbl_div_up(B, 64), gn = Np / 128;
    int S = 1;
    while(S < 16 && (size_t)gm * gn * S < (size_t)ctx->num_cu && ktiles / (S * 2) >= 2) S *= 2;
    a.k_chunk = nbl_div_up(ktiles, S) * GEMM_BK;
    S = nbl_div_up(p->H, a.k_chunk);
    if(S > 1) {
        const size_t need = (size_t)S * B * Np * sizeof(float);
        if(p->part_bytes < need) {
            if((rc = nbl_free(ctx, p->part_dev)) != NBL_OK) return rc;
            p->part_dev = NULL; p->part_bytes = 0;
            if((rc = nbl_malloc(ctx, (void**)&p->part_dev, need)) != NBL_OK) return rc;
            p->part_bytes = need;
        }
    }
    for(unsigned t = 0; t < T; t++) {
        a.A = t == 0 ? p->h0_dev : y_dev + (size_t)(t - 1) * step;
        a.gx = p->gx_dev + (size_t)t * B * Np;
        a.vec_ok = (p->H % 4 == 0) && aligned16(a.A) && aligned16(a.Bw);
        if(S > 1) {
            a.C = p->part_dev;
            hipLaunchKernelGGL((gemm_nt_kernel<1, 2, 2, 2, EPI_PARTIAL>), dim3(gn, gm, S), dim3(256), 0, ctx->stream, a);
            NBL_LAUNCH_CHECK(ctx, "gemm_nt_kernel(lstm split-k)");
            hipLaunchKernelGGL(lstm_cell_kernel, dim3(nbl_div_up((unsigned)step, 256)), dim3(256), 0, ctx->stream,
                               p->part_dev, a.gx, p->bw_dev, p->c_dev, y_dev + (size_t)t * step,
                               (int)B, (int)p->H, (int)Np, S, p->sub_act);
            NBL_LAUNCH_CHECK(ctx, "lstm_cell_kernel");
        } else {
            a.C = y_dev + (size_t)t * step;
            dim3 grid(p->Hp / 32, nbl_div_up(B, 64), 1);
            hipLaunchKernelGGL((gemm_nt_kernel<1, 4, 2, 1, EPI_LSTM>), grid, dim3(128), 0, ctx->stream, a);
            NBL_LAUNCH_CHECK(ctx, "gemm_nt_kernel(lstm)");
        }
    }
    }
    if(cell_dev)
        NBL_HIP(ctx, hipMemcpyAsync(cell_dev, p->c_dev, st_need, hipMemcpyDeviceToDevice, ctx->stream));
    // The state a carrying plan starts its next pass from: c is in c_dev already; h_T is the buffer the last step
    // wrote (operand-major), or a copy of y[T-1] (the caller may overwrite y before the next pass).
    if(p->G == 8) { if(T & 1) std::swap(p->hop_dev[0], p->hop_dev[1]); }
    else if(p->carry) NBL_HIP(ctx, hipMemcpyAsync(p->h0_dev, y_dev + (size_t)(T - 1) * step, st_need, hipMemcpyDeviceToDevice, ctx->stream));
    p->state_B = B;
    return NBL_OK;
}

int nbl_lstm_plan_carry_state(nbl_ctx *ctx, nbl_lstm_plan *p, int on) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p != NULL, "nbl_lstm_plan_carry_state: NULL plan");
    if(!on || !p->carry) p->state_B = 0;       // a state left by a pass that did not keep h is not a state to start from
    p->carry = on != 0;
    return NBL_OK;
}

int nbl_lstm_plan_reset_state(nbl_ctx *ctx, nbl_lstm_plan *p) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p != NULL, "nbl_lstm_plan_reset_state: NULL plan");
    p->state_B = 0;
    return NBL_OK;
}

int nbl_lstm_plan_set_state(nbl_ctx *ctx, nbl_lstm_plan *p, const float *h_dev, const float *c_dev, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && h_dev && c_dev && B > 0, "nbl_lstm_plan_set_state: NULL argument or empty batch");
    NBL_REQUIRE(ctx, p->carry, "nbl_lstm_plan_set_state: the plan does not carry state (nbl_lstm_plan_carry_state)");
    int rc;
    if((rc = lstm_state_buffers(ctx, p, B)) != NBL_OK) return rc;
    const size_t st = (size_t)B * p->H * sizeof(float);
    NBL_HIP(ctx, hipMemcpyAsync(p->c_dev, c_dev, st, hipMemcpyDeviceToDevice, ctx->stream));
    if(p->G == 8) {
        hipLaunchKernelGGL(lstm_state_to_opmajor_kernel, dim3(nbl_div_up((unsigned)((size_t)B * p->H), 256)), dim3(256), 0, ctx->stream,
                           h_dev, p->hop_dev[0], B, p->H);
        NBL_LAUNCH_CHECK(ctx, "lstm_state_to_opmajor_kernel");
    } else NBL_HIP(ctx, hipMemcpyAsync(p->h0_dev, h_dev, st, hipMemcpyDeviceToDevice, ctx->stream));
    p->state_B = B;
    return NBL_OK;
}

int nbl_lstm_fwd(nbl_ctx *ctx, nbl_lstm_plan *p, const float *x_dev, float *y_dev, float *cell_dev,
                 unsigned T, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && x_dev && y_dev, "nbl_lstm_fwd: NULL argument");
    return lstm_forward(ctx, p, x_dev, NULL, y_dev, cell_dev, T, B);
}

int nbl_lstm_fwd_tokens(nbl_ctx *ctx, nbl_lstm_plan *p, const unsigned *tokens_dev, float *y_dev, float *cell_dev,
                        unsigned T, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && tokens_dev && y_dev, "nbl_lstm_fwd_tokens: NULL argument");
    return lstm_forward(ctx, p, NULL, tokens_dev, y_dev, cell_dev, T, B);
}

int nbl_rnn_pack(nbl_ctx *ctx, const float *const *weight_host, const float *const *bias_host,
                 const float *const *scale_host, const float *const *mean_host, const float *const *var_host,
                 unsigned I, unsigned O, int act, nbl_rnn_plan **out) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, out != NULL, "nbl_rnn_pack: out is NULL");
    *out = NULL;
    NBL_REQUIRE(ctx, weight_host && bias_host, "nbl_rnn_pack: weight/bias is NULL");
    NBL_REQUIRE(ctx, (scale_host != NULL) == (mean_host != NULL) && (scale_host != NULL) == (var_host != NULL),
                "nbl_rnn_pack: scale, mean and var must be given together");
    NBL_REQUIRE(ctx, I && O, "nbl_rnn_pack: zero dimension");
    nbl_rnn_plan *p = new nbl_rnn_plan();
    memset(p, 0, sizeof(*p));
    p->I = I; p->O = O;
    for(int s = 0; s < 3; s++) {
        const int rc = nbl_fc_pack(ctx, weight_host[s], bias_host[s], scale_host ? scale_host[s] : NULL,
                                   mean_host ? mean_host[s] : NULL, var_host ? var_host[s] : NULL,
                                   s == 0 ? I : O, O, act, &p->gate[s]);
        if(rc != NBL_OK) { nbl_rnn_plan_destroy(ctx, p); return rc; }
    }
    if(O % 128 == 0) {      // the per-step kernel reads the hidden gate's weights in operand-major order
        std::vector<float> wop((size_t)O * O);
        for(unsigned n = 0; n < O; n++)
            for(unsigned k = 0; k < O; k++) wop[opmajor_offset(n, k, O)] = weight_host[1][(size_t)n * O + k];
        int rc;
        if((rc = nbl_malloc(ctx, (void**)&p->wh_op, wop.size() * sizeof(float))) != NBL_OK ||
           (rc = nbl_h2d(ctx, p->wh_op, wop.data(), wop.size() * sizeof(float))) != NBL_OK) {
            nbl_rnn_plan_destroy(ctx, p);
            return rc;
        }
    }
    *out = p;
    return NBL_OK;
}

int nbl_rnn_plan_destroy(nbl_ctx *ctx, nbl_rnn_plan *p) {
    if(!ctx || !p) return NBL_EINVAL;
    for(int s = 0; s < 3; s++) if(p->gate[s]) nbl_fc_plan_destroy(ctx, p->gate[s]);
    nbl_free(ctx, p->in_all); nbl_free(ctx, p->states); nbl_free(ctx, p->hid0); nbl_free(ctx, p->tmp);
    nbl_free(ctx, p->wh_op); nbl_free(ctx, p->sop[0]); nbl_free(ctx, p->sop[1]); nbl_free(ctx, p->wi_t);
    delete p;
    return NBL_OK;
}

// x_dev: dense input rows, or NULL with tokens_dev: the position of the single 1.0 of each one-hot row
static int rnn_forward(nbl_ctx *ctx, nbl_rnn_plan *p, const float *x_dev, const unsigned *tokens_dev, float *y_dev,
                       unsigned T, unsigned B) {
    if(T == 0 || B == 0) return NBL_OK;
    const size_t rows = (size_t)T * B;
    if(rows * p->O >= (1ull << 31) || (x_dev && rows * p->I >= (1ull << 31)))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_rnn_fwd: tensors of 2^31 elements or more are not supported");
    int rc;
    if(p->rows_alloc < rows || p->seqs_alloc < B) {
        if((rc = nbl_free(ctx, p->in_all)) != NBL_OK || (rc = nbl_free(ctx, p->states)) != NBL_OK ||
           (rc = nbl_free(ctx, p->hid0)) != NBL_OK || (rc = nbl_free(ctx, p->tmp)) != NBL_OK) return rc;
        p->in_all = p->states = p->hid0 = p->tmp = NULL; p->rows_alloc = p->seqs_alloc = 0;
        if((rc = nbl_malloc(ctx, (void**)&p->in_all, rows * p->O * sizeof(float))) != NBL_OK ||
           (rc = nbl_malloc(ctx, (void**)&p->states, rows * p->O * sizeof(float))) != NBL_OK ||
           (rc = nbl_malloc(ctx, (void**)&p->hid0, (size_t)B * p->O * sizeof(float))) != NBL_OK ||
           (rc = nbl_malloc(ctx, (void**)&p->tmp, (size_t)B * p->O * sizeof(float))) != NBL_OK) return rc;
        p->rows_alloc = rows; p->seqs_alloc = B;
    }
    nbl_fc_plan *gi = p->gate[0], *gh = p->gate[1], *go = p->gate[2];
    // input gate for every step at once: it does not depend on the recurrence
    if(tokens_dev) {
        // one-hot rows: the product is column token[row] of the weights, i.e. a row of their transpose
        if(!p->wi_t) {
            if((rc = nbl_malloc(ctx, (void**)&p->wi_t, (size_t)p->O * p->I * sizeof(float))) != NBL_OK) return rc;
            hipLaunchKernelGGL(transpose_kernel, dim3(nbl_div_up(p->I, 32), nbl_div_up(p->O, 32)), dim3(256), 0, ctx->stream,
                               gi->w_dev, p->wi_t, p->O, p->I);
            NBL_LAUNCH_CHECK(ctx, "transpose_kernel");
        }
        hipLaunchKernelGGL(token_gather_kernel, dim3((unsigned)rows), dim3(256), 0, ctx->stream,
                           p->wi_t, tokens_dev, gi->has_scale ? gi->g_dev : (const float*)NULL, gi->b_dev, p->in_all,
                           p->O, p->I, gi->act);
        NBL_LAUNCH_CHECK(ctx, "token_gather_kernel");
    } else if((rc = launch_fc(ctx, x_dev, gi->w_dev, p->in_all, (int)rows, (int)p->O, (int)p->I, gi->g_dev, gi->b_dev,
                              gi->act, gi->has_scale, &gi->ws_dev, &gi->ws_bytes, gi->w_tiled_dev)) != NBL_OK) return rc;
    const size_t step = (size_t)B * p->O;
    const bool one_launch = p->wh_op != NULL && aligned16(p->in_all) && aligned16(p->states) && aligned16(p->hid0);
    if(one_launch) {
        const size_t need = (size_t)nbl_div_up(B, 32) * 32 * p->O * sizeof(float);
        if(p->sop_bytes < need) {
            if((rc = nbl_free(ctx, p->sop[0])) != NBL_OK || (rc = nbl_free(ctx, p->sop[1])) != NBL_OK) return rc;
            p->sop[0] = p->sop[1] = NULL; p->sop_bytes = 0;
            if((rc = nbl_malloc(ctx, (void**)&p->sop[0], need)) != NBL_OK ||
               (rc = nbl_malloc(ctx, (void**)&p->sop[1], need)) != NBL_OK) return rc;
            p->sop_bytes = need;
            // rows past the batch are read (their sums are dropped) and must hold numbers: zero once, the kernel
            // writes real rows only
            if((rc = nbl_fill_zero(ctx, p->sop[0], need)) != NBL_OK || (rc = nbl_fill_zero(ctx, p->sop[1], need)) != NBL_OK)
                return rc;
        }
    }
    for(unsigned t = 0; t < T; t++) {
        // rnn_layer.cc:103-104: step 0's hidden gate reads the input gate's output, later steps the previous state
        const float *prev = t == 0 ? p->in_all : p->states + (size_t)(t - 1) * step;
        const float *in_t = p->in_all + (size_t)t * step;
        float *state = p->states + (size_t)t * step;
        if(one_launch) {
            RnnStepArgs a;
            a.prev = t == 0 ? prev : p->sop[(t - 1) & 1]; a.prev_opmajor = t == 0 ? 0 : 1;
            a.w_op = p->wh_op; a.state_op = p->sop[t & 1];
            a.g = gh->g_dev; a.b = gh->b_dev; a.in_t = in_t; a.state = state;
            a.hid = t == 0 ? p->hid0 : NULL; a.B = (int)B; a.H = (int)p->O; a.act = gh->act;
            hipLaunchKernelGGL(rnn_step_kernel, dim3(p->O / 32, nbl_div_up(B, 32)), dim3(256), 0, ctx->stream, a);
            NBL_LAUNCH_CHECK(ctx, "rnn_step_kernel");
        } else {
            float *hid = t == 0 ? p->hid0 : p->tmp;
            if((rc = launch_fc(ctx, prev, gh->w_dev, hid, (int)B, (int)p->O, (int)p->O, gh->g_dev, gh->b_dev,
                               gh->act, gh->has_scale, &gh->ws_dev, &gh->ws_bytes, gh->w_tiled_dev)) != NBL_OK) return rc;
            hipLaunchKernelGGL(add_kernel, dim3((unsigned)nbl_div_up_sz(step, 256)), dim3(256), 0, ctx->stream,
                               in_t, (const float*)hid, state, step);
            NBL_LAUNCH_CHECK(ctx, "add_kernel");
        }
    }
    // output gate: step 0 reads the hidden gate's output (rnn_layer.cc:116-117), every later step its state;
    // nothing feeds back, so all later steps are one product
    if((rc = launch_fc(ctx, p->hid0, go->w_dev, y_dev, (int)B, (int)p->O, (int)p->O, go->g_dev, go->b_dev,
                       go->act, go->has_scale, &go->ws_dev, &go->ws_bytes, go->w_tiled_dev)) != NBL_OK) return rc;
    if(T > 1 && (rc = launch_fc(ctx, p->states + step, go->w_dev, y_dev + step, (int)(rows - B), (int)p->O, (int)p->O,
                                go->g_dev, go->b_dev, go->act, go->has_scale, &go->ws_dev, &go->ws_bytes, go->w_tiled_dev)) != NBL_OK) return rc;
    return NBL_OK;
}

int nbl_rnn_fwd(nbl_ctx *ctx, nbl_rnn_plan *p, const float *x_dev, float *y_dev, unsigned T, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && x_dev && y_dev, "nbl_rnn_fwd: NULL argument");
    return rnn_forward(ctx, p, x_dev, NULL, y_dev, T, B);
}

int nbl_rnn_fwd_tokens(nbl_ctx *ctx, nbl_rnn_plan *p, const unsigned *tokens_dev, float *y_dev, unsigned T, unsigned B) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, p && tokens_dev && y_dev, "nbl_rnn_fwd_tokens: NULL argument");
    return rnn_forward(ctx, p, NULL, tokens_dev, y_dev, T, B);
}

}  // extern "C"
