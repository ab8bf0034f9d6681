// The bandwidth-bound layers: pooling, shortcut, softmax, stand-alone activations, bias and
// inference batchnorm.  Each kernel reads its input once and writes its output once; wherever the
// layout allows, a lane moves 16 bytes per access.
#include "nbl_internal.h"
#include <cmath>
#include <vector>
#include <algorithm>

#include <cfloat>

namespace {

// ---- pooling -------------------------------------------------------------------------------------
// One thread per output element, lanes along the output row (coalesced stores, overlapping window
// reads served by L1/L2).  Tap order, sentinel and tie rule follow pooling_layer.cc:126-140:
// rows then columns, taps outside the image read -1e8, strict '>' keeps the first maximum.
// KS > 0 fixes the window size at compile time: all KS*KS loads are issued before the first compare
// (addresses of taps outside the image are clamped and their values replaced), which is what lets
// the kernel run at memory speed instead of one load latency per tap.  KS = 0 is the general loop.
template<bool IS_MAX, bool WRITE_INDEX, int KS>
__global__ __launch_bounds__(256)
void pool_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned *__restrict__ index,
                 unsigned total, int H, int W, int OH, int OW, int ksize, int stride, int pad) {
    const unsigned o = blockIdx.x * blockDim.x + threadIdx.x;
    if(o >= total) return;
    const unsigned ow = o % OW, t = o / OW, oh = t % OH, plane = t / OH;   // plane = b*C + c
    const int h0 = (int)oh * stride - pad, w0 = (int)ow * stride - pad;
    const unsigned base = plane * (unsigned)(H * W);
    float best = -1e8f, acc = 0.0f;
    unsigned best_at = 0xffffffffu;
    if(KS > 0) {
        float v[KS > 0 ? KS * KS : 1];
        #pragma unroll
        for(int i = 0; i < KS; i++)
            #pragma unroll
            for(int j = 0; j < KS; j++) {
                const int ih = h0 + i, iw = w0 + j;
                const bool ok = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
                const float val = x[base + (ok ? (unsigned)(ih * W + iw) : 0u)];
                v[i * KS + j] = ok ? val : (IS_MAX ? -1e8f : 0.0f);
            }
        #pragma unroll
        for(int i = 0; i < KS; i++)
            #pragma unroll
            for(int j = 0; j < KS; j++) {
                if(IS_MAX) {
                    if(v[i * KS + j] > best) { best = v[i * KS + j]; best_at = base + (unsigned)((h0 + i) * W + (w0 + j)); }
                } else {
                    acc += v[i * KS + j];
                }
            }
    } else {
        for(int i = 0; i < ksize; i++) {
            const int ih = h0 + i;
            const bool row_ok = (unsigned)ih < (unsigned)H;
            for(int j = 0; j < ksize; j++) {
                const int iw = w0 + j;
                const bool ok = row_ok && (unsigned)iw < (unsigned)W;
                const unsigned at = base + (unsigned)(ih * W + iw);
                if(IS_MAX) {
                    const float val = ok ? x[at] : -1e8f;
                    if(val > best) { best = val; best_at = at; }
                } else {
                    acc += ok ? x[at] : 0.0f;
                }
            }
        }
    }
    if(IS_MAX) {
        y[o] = best;
        if(WRITE_INDEX) index[o] = best_at;
    } else {
        y[o] = acc / (float)(ksize * ksize);
    }
}

// A KS x KS window whose taps all lie inside the image (no padding, and the last window ends at or before the last row
// and column: AlexNet's 3x3/2 pools on 55, 27 and 13 wide maps), any row length: a window row is KS adjacent floats,
// fetched with ONE load of KS dwords at 4-byte alignment instead of KS loads (the address unit works per instruction,
// and the general kernel's nine 4-byte loads per output held it to 40 % of the memory rate on these maps).
template<int KS> struct __attribute__((packed, aligned(4))) WindowRow { float v[KS]; };
template<bool IS_MAX, bool WRITE_INDEX, int KS, bool STREAM>
__global__ __launch_bounds__(256)
void pool_inside_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned *__restrict__ index,
                        unsigned total, int H, int W, int OH, int OW, int stride) {
    const unsigned o = blockIdx.x * blockDim.x + threadIdx.x;
    if(o >= total) return;
    const unsigned ow = o % OW, t = o / OW, oh = t % OH, plane = t / OH;
    const unsigned at0 = plane * (unsigned)(H * W) + oh * (unsigned)(stride * W) + ow * (unsigned)stride;
    WindowRow<KS> rows[KS];
    #pragma unroll
    for(int i = 0; i < KS; i++) rows[i] = *reinterpret_cast<const WindowRow<KS>*>(x + at0 + i * W);
    float best = -1e8f, acc = 0.0f;
    unsigned best_at = 0xffffffffu;
    #pragma unroll
    for(int i = 0; i < KS; i++)
        #pragma unroll
        for(int j = 0; j < KS; j++) {
            if(IS_MAX) {
                if(rows[i].v[j] > best) { best = rows[i].v[j]; best_at = at0 + (unsigned)(i * W + j); }
            } else {
                acc += rows[i].v[j];
            }
        }
    if(IS_MAX) {
        nbl_put<STREAM>(y + o, best);
        if(WRITE_INDEX) nbl_put<STREAM>(index + o, best_at);
    } else {
        nbl_put<STREAM>(y + o, acc / (float)(KS * KS));
    }
}

// Stride 2, no padding, image width a multiple of 4: a lane produces two adjacent outputs from one
// 16-byte load per window row (plus one scalar for the fifth column of a 3-wide window), so the
// lanes of a wave read whole rows contiguously.  Same scan order, sentinel and tie rule as above.
// STREAM_IN (2-wide windows only: rows are read once) fetches the rows with streaming loads.
template<bool IS_MAX, bool WRITE_INDEX, int KS, bool STREAM, bool STREAM_IN>
__global__ __launch_bounds__(256)
void pool_pair_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned *__restrict__ index,
                      unsigned total_pairs, int H, int W, int OH, int OW2) {
    const unsigned o2 = blockIdx.x * blockDim.x + threadIdx.x;
    if(o2 >= total_pairs) return;
    const unsigned t2 = o2 % OW2, t = o2 / OW2, oh = t % OH, plane = t / OH;
    const unsigned base = plane * (unsigned)(H * W);
    const int h0 = (int)oh * 2, w0 = (int)t2 * 4;
    float v[KS][5];
    #pragma unroll
    for(int i = 0; i < KS; i++) {
        const int ih = h0 + i;
        const bool row_ok = ih < H;
        const unsigned roff = base + (unsigned)((row_ok ? ih : 0) * W + w0);
        const float4 q = nbl_get<STREAM_IN>(reinterpret_cast<const float4*>(x + roff));
        const float pad_v = IS_MAX ? -1e8f : 0.0f;
        v[i][0] = row_ok ? q.x : pad_v; v[i][1] = row_ok ? q.y : pad_v;
        v[i][2] = row_ok ? q.z : pad_v; v[i][3] = row_ok ? q.w : pad_v;
        if(KS == 3) {
            const bool ok = row_ok && w0 + 4 < W;
            const float e = x[ok ? roff + 4 : base];
            v[i][4] = ok ? e : pad_v;
        }
    }
    float out[2]; unsigned at[2];
    #pragma unroll
    for(int p = 0; p < 2; p++) {
        float best = -1e8f, acc = 0.0f;
        unsigned best_at = 0xffffffffu;
        #pragma unroll
        for(int i = 0; i < KS; i++)
            #pragma unroll
            for(int j = 0; j < KS; j++) {
                const float val = v[i][2 * p + j];
                if(IS_MAX) {
                    if(val > best) { best = val; best_at = base + (unsigned)((h0 + i) * W + w0 + 2 * p + j); }
                } else {
                    acc += val;
                }
            }
        out[p] = IS_MAX ? best : acc / (float)(KS * KS);
        at[p] = best_at;
    }
    const size_t o = (size_t)o2 * 2;
    nbl_put<STREAM>(reinterpret_cast<float2*>(y + o), out[0], out[1]);
    if(IS_MAX && WRITE_INDEX) nbl_put<STREAM>(reinterpret_cast<uint2*>(index + o), at[0], at[1]);
}

// Average over whole planes (window = plane, stride = window, no padding: the pool that ends ResNet).  The
// planes are contiguous, so a block stages AVG_PLANES consecutive planes through LDS with 16-byte loads and
// then one thread per plane adds its plane's floats in scan order (the order of pooling_layer.cc:161-170).
// LDS rows have an odd stride so that the threads of a wave read different banks.
constexpr int AVG_PLANES = 128;
__global__ __launch_bounds__(256)
void avgpool_plane_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned planes, unsigned hw, float divisor) {
    extern __shared__ float staged[];
    const unsigned row = hw | 1u;
    const unsigned first = blockIdx.x * AVG_PLANES;
    const unsigned here = min((unsigned)AVG_PLANES, planes - first);
    const unsigned count = here * hw;
    const float *__restrict__ src = x + (size_t)first * hw;
    for(unsigned v = threadIdx.x; v < count / 4; v += 256) {
        const float4 q = *reinterpret_cast<const float4*>(src + 4 * v);
        const float e[4] = { q.x, q.y, q.z, q.w };
        #pragma unroll
        for(unsigned c = 0; c < 4; c++) {
            const unsigned i = 4 * v + c, p = i / hw;
            staged[p * row + (i - p * hw)] = e[c];
        }
    }
    for(unsigned i = (count & ~3u) + threadIdx.x; i < count; i += 256) {
        const unsigned p = i / hw;
        staged[p * row + (i - p * hw)] = src[i];
    }
    __syncthreads();
    if(threadIdx.x < here) {
        const float *mine = staged + threadIdx.x * row;
        float acc = 0.0f;
        for(unsigned e = 0; e < hw; e++) acc += mine[e];
        y[first + threadIdx.x] = acc / divisor;
    }
}

// ---- shortcut ------------------------------------------------------------------------------------
// y = act(prev + conn') where conn' is conn cropped to the common channel/height/width box and
// sampled with stride = max(1, in_w/out_w), sample = max(1, out_w/in_w) (common/utils.cc:28-60).
// Fast path: identical spatial size (stride = sample = 1, same H and W), 4 elements per lane.
template<bool STREAM, bool STREAM_IN>
__global__ void shortcut_same_hw_kernel(const float4 *__restrict__ prev, const float4 *__restrict__ conn,
                                        float4 *__restrict__ y, size_t total4, unsigned hw4,
                                        unsigned in_c, unsigned out_c, int act) {
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(e >= total4) return;
    const size_t plane = e / hw4;                  // b*out_c + c
    const unsigned c = (unsigned)(plane % out_c);
    float4 v = nbl_get<STREAM_IN>(prev + e);
    if(c < in_c) {
        const size_t b = plane / out_c;
        const float4 r = nbl_get<STREAM_IN>(conn + (b * in_c + c) * hw4 + (e - plane * hw4));
        v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
    }
    v.x = nbl_act_apply(act, v.x); v.y = nbl_act_apply(act, v.y);
    v.z = nbl_act_apply(act, v.z); v.w = nbl_act_apply(act, v.w);
    nbl_put<STREAM>(y + e, v);
}

// Spatial sizes differ by an integer stride and the output is not up-sampled (sample = 1): four
// adjacent outputs per lane; with stride 2 their residuals are the even elements of 32 contiguous bytes.
template<bool STRIDE2, bool STREAM>
__global__ void shortcut_strided_kernel(const float4 *__restrict__ prev, const float *__restrict__ conn,
                                        float4 *__restrict__ y, size_t total4,
                                        unsigned in_c, unsigned in_h, unsigned in_w,
                                        unsigned out_c, unsigned out_h, unsigned out_w4,
                                        unsigned stride, unsigned box_c, unsigned box_h, int act) {
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(e >= total4) return;
    const unsigned w4 = (unsigned)(e % out_w4);
    size_t t = e / out_w4;
    const unsigned h = (unsigned)(t % out_h); t /= out_h;
    const unsigned c = (unsigned)(t % out_c);
    const size_t b = t / out_c;
    float4 v = prev[e];
    if(c < box_c && h < box_h) {
        const float *row = conn + ((b * in_c + c) * in_h + (size_t)h * stride) * in_w + (size_t)w4 * 4 * stride;
        if(STRIDE2) {
            const float4 r0 = *reinterpret_cast<const float4*>(row), r1 = *reinterpret_cast<const float4*>(row + 4);
            v.x += r0.x; v.y += r0.z; v.z += r1.x; v.w += r1.z;
        } else {
            v.x += row[0]; v.y += row[stride]; v.z += row[2 * stride]; v.w += row[3 * stride];
        }
    }
    v.x = nbl_act_apply(act, v.x); v.y = nbl_act_apply(act, v.y);
    v.z = nbl_act_apply(act, v.z); v.w = nbl_act_apply(act, v.w);
    nbl_put<STREAM>(y + e, v);
}

__global__ void shortcut_general_kernel(const float *__restrict__ prev, const float *__restrict__ conn,
                                        float *__restrict__ y, size_t total,
                                        unsigned in_c, unsigned in_h, unsigned in_w,
                                        unsigned out_c, unsigned out_h, unsigned out_w,
                                        unsigned stride, unsigned sample, unsigned box_c, unsigned box_h,
                                        unsigned box_w, int act) {
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(e >= total) return;
    const unsigned w = (unsigned)(e % out_w);
    size_t t = e / out_w;
    const unsigned h = (unsigned)(t % out_h); t /= out_h;
    const unsigned c = (unsigned)(t % out_c);
    const size_t b = t / out_c;
    float v = prev[e];
    // element (h, w) receives a residual when it sits on the sample grid inside the common box
    if(c < box_c && h % sample == 0 && w % sample == 0 && h / sample < box_h && w / sample < box_w) {
        const unsigned sh = h / sample * stride, sw = w / sample * stride;
        v += conn[((b * in_c + c) * in_h + sh) * in_w + sw];
    }
    y[e] = nbl_act_apply(act, v);
}

// ---- softmax -------------------------------------------------------------------------------------
// One block per row (softmax_layer.cc:85-106): row maximum, e = exp(x - max), sum, divide.  The CPU code evaluates
// exp in double and rounds to float; here it is the single-precision expf (within an ulp or two of that, against a
// layer tolerance of 1e-4): the double-precision exp held the 4096 x 10000 step of the recurrent driver to 45 % of
// the memory rate.  The sum is a tree over floats where the CPU code adds left to right.
__device__ __forceinline__ float wave_max(float v) {
    for(int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for(int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float softmax_exp(float d) { return expf(d); }

// Rows whose length is a multiple of 4 and whose start is 16-byte aligned, up to 1024 * PER4 entries: a thread keeps
// PER4 pieces of four adjacent entries in registers (pieces tid, tid + 256, ...), so the row moves as 16-byte loads
// and stores, once each way.
template<int PER4, bool STREAM>
__global__ __launch_bounds__(256) void softmax_row_vec4_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned n) {
    typedef float vec4 __attribute__((ext_vector_type(4)));
    __shared__ float red[4];
    const vec4 *in = reinterpret_cast<const vec4*>(x + (size_t)blockIdx.x * n);
    vec4 *out = reinterpret_cast<vec4*>(y + (size_t)blockIdx.x * n);
    const unsigned n4 = n / 4;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    vec4 v[PER4];
    float m = -FLT_MAX;
    #pragma unroll
    for(int i = 0; i < PER4; i++) {
        const unsigned j = tid + i * 256;
        v[i] = j < n4 ? in[j] : vec4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
        m = fmaxf(fmaxf(m, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
    }
    m = wave_max(m);
    if(lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float s = 0.0f;
    #pragma unroll
    for(int i = 0; i < PER4; i++) {
        if(tid + i * 256 < n4) {
            #pragma unroll
            for(int c = 0; c < 4; c++) { v[i][c] = softmax_exp(v[i][c] - m); s += v[i][c]; }
        }
    }
    s = wave_sum(s);
    if(lane == 0) red[wave] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    #pragma unroll
    for(int i = 0; i < PER4; i++) {
        const unsigned j = tid + i * 256;
        if(j < n4) {
            const vec4 q = vec4{v[i][0] / s, v[i][1] / s, v[i][2] / s, v[i][3] / s};
            if constexpr(STREAM) __builtin_nontemporal_store(q, out + j); else out[j] = q;
        }
    }
}

// Rows of up to THREADS * PER entries: a thread keeps its PER entries (columns tid, tid + THREADS, ...) in
// registers, so the row is read once and written once; maximum, partial sums and their trees are those of the
// general kernel below, and so is every result bit.
template<int THREADS, int PER>
__global__ __launch_bounds__(THREADS) void softmax_row_in_registers_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned n) {
    constexpr int WAVES = THREADS / 64;
    __shared__ float red[WAVES];
    const float *in = x + (size_t)blockIdx.x * n;
    float *out = y + (size_t)blockIdx.x * n;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    float v[PER];
    float m = -FLT_MAX;
    #pragma unroll
    for(int i = 0; i < PER; i++) {
        const unsigned j = tid + i * THREADS;
        v[i] = j < n ? in[j] : -FLT_MAX;
        m = fmaxf(m, v[i]);
    }
    m = wave_max(m);
    if(lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
    #pragma unroll
    for(int w = 1; w < WAVES; w++) m = fmaxf(m, red[w]);
    __syncthreads();
    float s = 0.0f;
    #pragma unroll
    for(int i = 0; i < PER; i++) {
        const unsigned j = tid + i * THREADS;
        if(j < n) {
            v[i] = softmax_exp(v[i] - m);
            s += v[i];
        }
    }
    s = wave_sum(s);
    if(lane == 0) red[wave] = s;
    __syncthreads();
    float part[WAVES];
    #pragma unroll
    for(int w = 0; w < WAVES; w++) part[w] = red[w];
    #pragma unroll
    for(int width = WAVES / 2; width >= 1; width /= 2)
        #pragma unroll
        for(int w = 0; w < width; w++) part[w] = part[2 * w] + part[2 * w + 1];
    s = part[0];
    #pragma unroll
    for(int i = 0; i < PER; i++) {
        const unsigned j = tid + i * THREADS;
        if(j < n) out[j] = v[i] / s;
    }
}

// One block of THREADS threads per row of any length; the row is read three times and written twice.
template<int THREADS>
__global__ __launch_bounds__(THREADS) void softmax_kernel(const float *__restrict__ x, float *__restrict__ y, unsigned n) {
    constexpr int WAVES = THREADS / 64;
    __shared__ float red[WAVES];
    const float *in = x + (size_t)blockIdx.x * n;
    float *out = y + (size_t)blockIdx.x * n;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    float m = -FLT_MAX;
    for(unsigned j = tid; j < n; j += THREADS) m = fmaxf(m, in[j]);
    m = wave_max(m);
    if(lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
    #pragma unroll
    for(int w = 1; w < WAVES; w++) m = fmaxf(m, red[w]);
    __syncthreads();
    float s = 0.0f;
    for(unsigned j = tid; j < n; j += THREADS) {
        const float e = softmax_exp(in[j] - m);
        out[j] = e;
        s += e;
    }
    s = wave_sum(s);
    if(lane == 0) red[wave] = s;
    __syncthreads();
    // pairwise over the waves, the same tree for every thread
    float part[WAVES];
    #pragma unroll
    for(int w = 0; w < WAVES; w++) part[w] = red[w];
    #pragma unroll
    for(int width = WAVES / 2; width >= 1; width /= 2)
        #pragma unroll
        for(int w = 0; w < width; w++) part[w] = part[2 * w] + part[2 * w + 1];
    s = part[0];
    for(unsigned j = tid; j < n; j += THREADS) out[j] = out[j] / s;
}

// ---- elementwise ---------------------------------------------------------------------------------
__global__ void activation_kernel(float *__restrict__ x, size_t n, int act) {
    const size_t i4 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if(i4 + 3 < n) {
        float4 v = *reinterpret_cast<float4*>(x + i4);
        v.x = nbl_act_apply(act, v.x); v.y = nbl_act_apply(act, v.y);
        v.z = nbl_act_apply(act, v.z); v.w = nbl_act_apply(act, v.w);
        *reinterpret_cast<float4*>(x + i4) = v;
    } else {
        for(size_t i = i4; i < n; i++) x[i] = nbl_act_apply(act, x[i]);
    }
}

// y[b][c][s] = y * g[c] + b[c]   (bias only: g == NULL).  VEC = 4 needs size % 4 == 0 and a 16-byte aligned tensor:
// the four elements of a piece then share their channel.
template<int VEC>
__global__ void channel_affine_kernel(float *__restrict__ y, const float *__restrict__ g, const float *__restrict__ b,
                                      size_t total, unsigned channel, unsigned size) {
    typedef float __attribute__((ext_vector_type(VEC))) vec;
    const size_t e = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if(e >= total) return;
    const unsigned c = (unsigned)((e / size) % channel);
    const float bc = b[c], gc = g ? g[c] : 1.0f;
    vec v = *reinterpret_cast<vec*>(y + e);
    #pragma unroll
    for(int i = 0; i < VEC; i++) v[i] = g ? v[i] * gc + bc : v[i] + bc;
    *reinterpret_cast<vec*>(y + e) = v;
}

// y = (float)((double)(y - mean[c]) / (sqrt(var[c]) + 1e-5)) * scale[c], the two CPU passes of
// common/batchnorm.cc:58-97 in one.  The quotient is formed as a product with the channel's reciprocal in double,
// one double rounding away from the CPU's division before the rounding to float (the same float in all but about
// one case in 2^29).
template<int VEC>
__global__ void batchnorm_inference_kernel(float *__restrict__ y, const float *__restrict__ mean,
                                           const float *__restrict__ var, const float *__restrict__ scale,
                                           size_t total, unsigned channel, unsigned size) {
    typedef float __attribute__((ext_vector_type(VEC))) vec;
    const size_t e = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if(e >= total) return;
    const unsigned c = (unsigned)((e / size) % channel);
    const float mc = mean[c], sc = scale[c];
    const double r = 1.0 / (sqrt((double)var[c]) + 0.00001);
    vec v = *reinterpret_cast<vec*>(y + e);
    #pragma unroll
    for(int i = 0; i < VEC; i++) v[i] = __fmul_rn((float)((double)__fsub_rn(v[i], mc) * r), sc);
    *reinterpret_cast<vec*>(y + e) = v;
}


// ---- image input contract ---------------------------------------------------------------------------
// 8-bit interleaved images -> network input planes: optional bilinear resize in OpenCV's 8-bit
// fixed-point arithmetic (weights are shorts scaled by 2048, horizontal pass in int, vertical pass
// ((b0 * (S0 >> 4)) >> 16) + ((b1 * (S1 >> 4)) >> 16) + 2) >> 2), then byte / 255.0 and planes 0 and 2
// swapped (models/networks/convolutional.cc:384-412).  One thread per output pixel; the tap tables are
// built on the host.  tab = [xofs | x weights (a0 | a1 << 16) | row0 | row1 | y weights] as ints.
__global__ void image_to_input_kernel(const unsigned char *__restrict__ src, float *__restrict__ dst,
                                      const int *__restrict__ tab, unsigned images, int src_h, int src_w, int ch,
                                      int dst_h, int dst_w, int resize) {
    const int dx = blockIdx.x * blockDim.x + threadIdx.x, dy = blockIdx.y, img = blockIdx.z;
    if(dx >= dst_w) return;
    const unsigned char *__restrict__ in = src + (size_t)img * src_h * src_w * ch;
    float *__restrict__ out = dst + (size_t)img * ch * dst_h * dst_w;
    const size_t plane = (size_t)dst_h * dst_w;
    int sx = dx, sx1 = dx, a0 = 2048, a1 = 0, r0 = dy, r1 = dy, b0 = 2048, b1 = 0;
    if(resize) {
        sx = tab[dx];
        sx1 = sx + 1 < src_w ? sx + 1 : sx;
        const int aw = tab[dst_w + dx];
        a0 = (short)(aw & 0xffff); a1 = (short)(aw >> 16);
        r0 = tab[2 * dst_w + dy]; r1 = tab[2 * dst_w + dst_h + dy];
        const int bw = tab[2 * dst_w + 2 * dst_h + dy];
        b0 = (short)(bw & 0xffff); b1 = (short)(bw >> 16);
    }
    for(int c = 0; c < ch; c++) {
        int v;
        if(resize) {
            const int S0 = in[((size_t)r0 * src_w + sx) * ch + c] * a0 + in[((size_t)r0 * src_w + sx1) * ch + c] * a1;
            const int S1 = in[((size_t)r1 * src_w + sx) * ch + c] * a0 + in[((size_t)r1 * src_w + sx1) * ch + c] * a1;
            v = (((b0 * (S0 >> 4)) >> 16) + ((b1 * (S1 >> 4)) >> 16) + 2) >> 2;
            v = v < 0 ? 0 : v > 255 ? 255 : v;
        } else {
            v = in[((size_t)dy * src_w + dx) * ch + c];
        }
        const int cp = ch >= 3 && c == 0 ? 2 : ch >= 3 && c == 2 ? 0 : c;      // planes 0 and 2 change places
        out[cp * plane + (size_t)dy * dst_w + dx] = (float)((double)v / 255.0);
    }
}

// Source index and the two weights of every destination coordinate along one axis.
// At exactly half size every coordinate falls midway between two source pixels: both weights are 1024 of 2048, the
// fixed-point passes then lose nothing and the result is (a + b + c + d + 2) >> 2 over each 2x2 block -- the same
// bytes as the 2x2 area average that cv::resize substitutes for INTER_LINEAR at that ratio, so the case needs no
// branch of its own.
static void linear_taps(unsigned dst_n, unsigned src_n, bool clamp_weight, std::vector<int> &ofs, std::vector<int> &weights) {
    ofs.resize(dst_n); weights.resize(dst_n);
    const double scale = (double)src_n / (double)dst_n;
    for(unsigned d = 0; d < dst_n; d++) {
        float f = (float)((d + 0.5) * scale - 0.5);
        int s = (int)std::floor((double)f);
        f -= (float)s;
        if(clamp_weight) {
            if(s < 0) { f = 0.0f; s = 0; }
            if(s >= (int)src_n - 1) { f = 0.0f; s = (int)src_n - 1; }
        }
        const int w0 = (int)std::nearbyint((double)((1.0f - f) * 2048.0f)), w1 = (int)std::nearbyint((double)(f * 2048.0f));
        ofs[d] = s;
        weights[d] = (w0 & 0xffff) | (w1 << 16);
    }
}


// sum over rows of probs[row][target[row]] (rows whose target is outside [0, n) add nothing): what the
// recurrent driver accumulates as  sum_i label[i] * output[i]  with one-hot labels
// (models/networks/recurrent.cc:239-241).  One block; per-thread partial sums in row order, then a
// fixed tree, so the result does not depend on scheduling.
__global__ __launch_bounds__(1024) void target_prob_sum_kernel(const float *__restrict__ probs, const unsigned *__restrict__ targets,
                                                               unsigned rows, unsigned n, float *__restrict__ out) {
    __shared__ float red[1024];
    float s = 0.0f;
    for(unsigned r = threadIdx.x; r < rows; r += 1024) {
        const unsigned t = targets[r];
        if(t < n) s += probs[(size_t)r * n + t];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for(unsigned width = 512; width >= 1; width >>= 1) {
        if(threadIdx.x < width) red[threadIdx.x] += red[threadIdx.x + width];
        __syncthreads();
    }
    if(threadIdx.x == 0) *out = red[0];
}


__global__ void clear_u32_kernel(unsigned *p) { *p = 0u; }

// Rows whose label ranks among the k largest entries: one wave per row counts the entries that come
// before the label in descending order (larger value, or equal value and smaller index); one block per
// 4 rows; the per-block counts are added with an integer atomic (order-independent).
__global__ __launch_bounds__(256) void topk_matches_kernel(const float *__restrict__ probs, const unsigned *__restrict__ labels,
                                                           unsigned rows, unsigned n, unsigned k, unsigned *__restrict__ count) {
    const unsigned row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if(row >= rows) return;
    const unsigned l = labels[row];
    if(l >= n) return;
    const float *__restrict__ p = probs + (size_t)row * n;
    const float pl = p[l];
    unsigned before = 0;
    for(unsigned j = lane; j < n; j += 64) {
        const float v = p[j];
        before += (v > pl || (v == pl && j < l)) ? 1u : 0u;
    }
    for(int off = 32; off >= 1; off >>= 1) before += __shfl_down(before, off, 64);
    if(lane == 0 && before < k) atomicAdd(count, 1u);
}

}  // namespace

extern "C" {

int nbl_pool_fwd(nbl_ctx *ctx, const float *x_dev, float *y_dev, unsigned *index_dev,
                 unsigned B, unsigned C, unsigned H, unsigned W,
                 unsigned ksize, unsigned stride, unsigned pad, int mode) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, x_dev && y_dev, "nbl_pool_fwd: NULL pointer");
    NBL_REQUIRE(ctx, mode == NBL_POOL_MAX || mode == NBL_POOL_AVG, "nbl_pool_fwd: undefined pooling layer type %d", mode);
    NBL_REQUIRE(ctx, C && H && W && ksize && stride, "nbl_pool_fwd: zero dimension");
    if(B == 0) return NBL_OK;
    const unsigned OH = nbl_pool_out_dim(H, stride, pad), OW = nbl_pool_out_dim(W, stride, pad);
    const size_t total = (size_t)B * C * OH * OW, in_total = (size_t)B * C * H * W;
    if(total == 0) return NBL_OK;
    if(total >= (1ull << 31) || in_total >= (1ull << 31))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_pool_fwd: tensors of 2^31 elements or more are not supported");
    const bool stream_out = nbl_stream_stores(total * sizeof(float), y_dev, x_dev);
    // two outputs per lane from 16-byte loads
    if(stride == 2 && pad == 0 && (ksize == 2 || ksize == 3) && W % 4 == 0 && OW == W / 2 && OW % 2 == 0 &&
       (((size_t)x_dev | (size_t)y_dev | (size_t)index_dev) & 15) == 0) {
        const unsigned pairs = (unsigned)(total / 2);
        dim3 pgrid(nbl_div_up(pairs, 256)), pblock(256);
#define NBL_PAIR_LAUNCH_AS(IS_MAX, WI, KS, ST, SI) \
        hipLaunchKernelGGL((pool_pair_kernel<IS_MAX, WI, KS, ST, SI>), pgrid, pblock, 0, ctx->stream, x_dev, y_dev, \
                           index_dev, pairs, (int)H, (int)W, (int)OH, (int)(OW / 2))
#define NBL_PAIR_LAUNCH(IS_MAX, WI, KS) \
        do { if(stream_out && KS == 2 && nbl_stream_loads(in_total * sizeof(float))) NBL_PAIR_LAUNCH_AS(IS_MAX, WI, KS, true, KS == 2); \
             else if(stream_out) NBL_PAIR_LAUNCH_AS(IS_MAX, WI, KS, true, false); \
             else NBL_PAIR_LAUNCH_AS(IS_MAX, WI, KS, false, false); } while(0)
        if(mode == NBL_POOL_MAX) {
            if(index_dev) { if(ksize == 2) NBL_PAIR_LAUNCH(true, true, 2); else NBL_PAIR_LAUNCH(true, true, 3); }
            else          { if(ksize == 2) NBL_PAIR_LAUNCH(true, false, 2); else NBL_PAIR_LAUNCH(true, false, 3); }
        } else {
            if(ksize == 2) NBL_PAIR_LAUNCH(false, false, 2); else NBL_PAIR_LAUNCH(false, false, 3);
        }
#undef NBL_PAIR_LAUNCH_AS
#undef NBL_PAIR_LAUNCH
        NBL_LAUNCH_CHECK(ctx, "pool_pair_kernel");
        return NBL_OK;
    }
    // the window is the whole plane: contiguous planes staged through LDS
    if(mode == NBL_POOL_AVG && pad == 0 && ksize == H && ksize == W && OH == 1 && OW == 1 &&
       (size_t)AVG_PLANES * ((H * W) | 1u) * sizeof(float) <= 64 * 1024 && ((size_t)x_dev & 15) == 0) {
        const unsigned planes = B * C, hw = H * W;
        hipLaunchKernelGGL(avgpool_plane_kernel, dim3(nbl_div_up(planes, (unsigned)AVG_PLANES)), dim3(256),
                           AVG_PLANES * (hw | 1u) * sizeof(float), ctx->stream, x_dev, y_dev, planes, hw, (float)(ksize * ksize));
        NBL_LAUNCH_CHECK(ctx, "avgpool_plane_kernel");
        return NBL_OK;
    }
    dim3 grid((unsigned)nbl_div_up_sz(total, 256)), block(256);
    // every tap of every window inside the image: one load per window row
    if(pad == 0 && (ksize == 2 || ksize == 3) && (OH - 1) * stride + ksize <= H && (OW - 1) * stride + ksize <= W) {
#define NBL_INSIDE_LAUNCH(IS_MAX, WI, KS) \
        do { if(stream_out) hipLaunchKernelGGL((pool_inside_kernel<IS_MAX, WI, KS, true>), grid, block, 0, ctx->stream, x_dev, y_dev, \
                                               index_dev, (unsigned)total, (int)H, (int)W, (int)OH, (int)OW, (int)stride); \
             else hipLaunchKernelGGL((pool_inside_kernel<IS_MAX, WI, KS, false>), grid, block, 0, ctx->stream, x_dev, y_dev, \
                                     index_dev, (unsigned)total, (int)H, (int)W, (int)OH, (int)OW, (int)stride); } while(0)
        if(mode == NBL_POOL_MAX) {
            if(index_dev) { if(ksize == 2) NBL_INSIDE_LAUNCH(true, true, 2); else NBL_INSIDE_LAUNCH(true, true, 3); }
            else          { if(ksize == 2) NBL_INSIDE_LAUNCH(true, false, 2); else NBL_INSIDE_LAUNCH(true, false, 3); }
        } else {
            if(ksize == 2) NBL_INSIDE_LAUNCH(false, false, 2); else NBL_INSIDE_LAUNCH(false, false, 3);
        }
#undef NBL_INSIDE_LAUNCH
        NBL_LAUNCH_CHECK(ctx, "pool_inside_kernel");
        return NBL_OK;
    }
#define NBL_POOL_LAUNCH(IS_MAX, WI, KS) \
    hipLaunchKernelGGL((pool_kernel<IS_MAX, WI, KS>), grid, block, 0, ctx->stream, x_dev, y_dev, index_dev, \
                       (unsigned)total, (int)H, (int)W, (int)OH, (int)OW, (int)ksize, (int)stride, (int)pad)
#define NBL_POOL_BY_K(IS_MAX, WI) \
    do { switch(ksize) { case 2: NBL_POOL_LAUNCH(IS_MAX, WI, 2); break; case 3: NBL_POOL_LAUNCH(IS_MAX, WI, 3); break; \
                         case 7: NBL_POOL_LAUNCH(IS_MAX, WI, 7); break; default: NBL_POOL_LAUNCH(IS_MAX, WI, 0); } } while(0)
    if(mode == NBL_POOL_MAX) {
        if(index_dev) NBL_POOL_BY_K(true, true); else NBL_POOL_BY_K(true, false);
    } else {
        NBL_POOL_BY_K(false, false);
    }
#undef NBL_POOL_BY_K
#undef NBL_POOL_LAUNCH
    NBL_LAUNCH_CHECK(ctx, "pool_kernel");
    return NBL_OK;
}

int nbl_shortcut_fwd(nbl_ctx *ctx, const float *prev_dev, const float *conn_dev, float *y_dev, unsigned B,
                     unsigned in_c, unsigned in_h, unsigned in_w,
                     unsigned out_c, unsigned out_h, unsigned out_w, int act) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, prev_dev && conn_dev && y_dev, "nbl_shortcut_fwd: NULL pointer");
    NBL_REQUIRE(ctx, in_c && in_h && in_w && out_c && out_h && out_w, "nbl_shortcut_fwd: zero dimension");
    NBL_REQUIRE(ctx, nbl_act_valid(act), "nbl_shortcut_fwd: undefined activation type %d", act);
    if(B == 0) return NBL_OK;
    const size_t total = (size_t)B * out_c * out_h * out_w;
    if(total >= (1ull << 40)) return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_shortcut_fwd: tensor too large");
    const unsigned hw = out_h * out_w;
    const bool stream_out = nbl_stream_stores(total * sizeof(float), y_dev, prev_dev, conn_dev);
    const bool same_hw = in_h == out_h && in_w == out_w;
    bool vec = same_hw && hw % 4 == 0 && (((size_t)prev_dev | (size_t)conn_dev | (size_t)y_dev) & 15) == 0;
    unsigned hw4 = hw / 4, vin_c = in_c, vout_c = out_c;
    if(!vec && same_hw && in_c == out_c && ((size_t)out_c * hw) % 4 == 0 &&
       (((size_t)prev_dev | (size_t)conn_dev | (size_t)y_dev) & 15) == 0) {
        // identical shapes: element e of conn adds to element e of prev; treat each image as one plane
        vec = true; hw4 = (unsigned)((size_t)out_c * hw / 4); vin_c = vout_c = 1;
    }
    const unsigned stride = in_w / out_w > 1 ? in_w / out_w : 1;
    const unsigned sample = out_w / in_w > 1 ? out_w / in_w : 1;
    const bool aligned = (((size_t)prev_dev | (size_t)conn_dev | (size_t)y_dev) & 15) == 0;
    // four outputs per lane need the whole output row inside the common box and 16-byte aligned rows
    const bool strided_vec = !same_hw && sample == 1 && out_w <= in_w && out_w % 4 == 0 && aligned &&
                             (stride != 2 || in_w % 4 == 0);
    if(vec) {
        const size_t total4 = total / 4;
        const size_t read_bytes = (total + (size_t)B * (in_c < out_c ? in_c : out_c) * hw) * sizeof(float);
#define NBL_SAME_HW_LAUNCH(ST, SI) \
        hipLaunchKernelGGL((shortcut_same_hw_kernel<ST, SI>), dim3((unsigned)nbl_div_up_sz(total4, 256)), dim3(256), 0, ctx->stream, \
                           (const float4*)prev_dev, (const float4*)conn_dev, (float4*)y_dev, total4, hw4, vin_c, vout_c, act)
        if(stream_out && nbl_stream_loads(read_bytes)) NBL_SAME_HW_LAUNCH(true, true);
        else if(stream_out) NBL_SAME_HW_LAUNCH(true, false);
        else NBL_SAME_HW_LAUNCH(false, false);
#undef NBL_SAME_HW_LAUNCH
    } else if(strided_vec) {
        const size_t total4 = total / 4;
        const unsigned box_c = in_c < out_c ? in_c : out_c, box_h = in_h < out_h ? in_h : out_h;
#define NBL_STRIDED_LAUNCH(S2, ST) \
        hipLaunchKernelGGL((shortcut_strided_kernel<S2, ST>), dim3((unsigned)nbl_div_up_sz(total4, 256)), dim3(256), 0, \
                           ctx->stream, (const float4*)prev_dev, conn_dev, (float4*)y_dev, total4, in_c, in_h, in_w, \
                           out_c, out_h, out_w / 4, stride, box_c, box_h, act)
        if(stride == 2) { if(stream_out) NBL_STRIDED_LAUNCH(true, true); else NBL_STRIDED_LAUNCH(true, false); }
        else            { if(stream_out) NBL_STRIDED_LAUNCH(false, true); else NBL_STRIDED_LAUNCH(false, false); }
#undef NBL_STRIDED_LAUNCH
    } else {
        hipLaunchKernelGGL(shortcut_general_kernel, dim3((unsigned)nbl_div_up_sz(total, 256)), dim3(256), 0, ctx->stream,
                           prev_dev, conn_dev, y_dev, total, in_c, in_h, in_w, out_c, out_h, out_w, stride, sample,
                           in_c < out_c ? in_c : out_c, in_h < out_h ? in_h : out_h, in_w < out_w ? in_w : out_w, act);
    }
    NBL_LAUNCH_CHECK(ctx, "shortcut kernel");
    return NBL_OK;
}

int nbl_softmax_fwd(nbl_ctx *ctx, const float *x_dev, float *y_dev, unsigned rows, unsigned n) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, x_dev && y_dev, "nbl_softmax_fwd: NULL pointer");
    if(rows == 0 || n == 0) return NBL_OK;
    if(n % 4 == 0 && n <= 16384 && (((size_t)x_dev | (size_t)y_dev) & 15) == 0) {
        const unsigned per4 = nbl_div_up(n / 4, 256);
        const bool stream_out = nbl_stream_stores((size_t)rows * n * sizeof(float), y_dev, x_dev);
#define NBL_SOFTMAX_VEC(P) \
        do { if(stream_out) hipLaunchKernelGGL((softmax_row_vec4_kernel<P, true>), dim3(rows), dim3(256), 0, ctx->stream, x_dev, y_dev, n); \
             else hipLaunchKernelGGL((softmax_row_vec4_kernel<P, false>), dim3(rows), dim3(256), 0, ctx->stream, x_dev, y_dev, n); } while(0)
        if(per4 <= 1) NBL_SOFTMAX_VEC(1); else if(per4 <= 2) NBL_SOFTMAX_VEC(2); else if(per4 <= 4) NBL_SOFTMAX_VEC(4);
        else if(per4 <= 6) NBL_SOFTMAX_VEC(6); else if(per4 <= 8) NBL_SOFTMAX_VEC(8); else if(per4 <= 10) NBL_SOFTMAX_VEC(10);
        else if(per4 <= 12) NBL_SOFTMAX_VEC(12); else NBL_SOFTMAX_VEC(16);
#undef NBL_SOFTMAX_VEC
    }
    else if(n <= 1024)  hipLaunchKernelGGL((softmax_row_in_registers_kernel<256, 4>), dim3(rows), dim3(256), 0, ctx->stream, x_dev, y_dev, n);
    else if(n <= 2048)  hipLaunchKernelGGL((softmax_row_in_registers_kernel<256, 8>), dim3(rows), dim3(256), 0, ctx->stream, x_dev, y_dev, n);
    else if(n <= 16384) hipLaunchKernelGGL((softmax_row_in_registers_kernel<1024, 16>), dim3(rows), dim3(1024), 0, ctx->stream, x_dev, y_dev, n);
    else                hipLaunchKernelGGL(softmax_kernel<1024>, dim3(rows), dim3(1024), 0, ctx->stream, x_dev, y_dev, n);
    NBL_LAUNCH_CHECK(ctx, "softmax_kernel");
    return NBL_OK;
}

int nbl_activation_fwd(nbl_ctx *ctx, float *x_dev, size_t n, int act) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, nbl_act_valid(act), "nbl_activation_fwd: undefined activation type %d", act);
    if(n == 0 || act == NBL_ACT_LINEAR) return NBL_OK;
    NBL_REQUIRE(ctx, x_dev != NULL, "nbl_activation_fwd: NULL pointer");
    NBL_REQUIRE(ctx, ((size_t)x_dev & 15) == 0, "nbl_activation_fwd: pointer must be 16-byte aligned");
    const size_t threads = nbl_div_up_sz(n, 4);
    hipLaunchKernelGGL(activation_kernel, dim3((unsigned)nbl_div_up_sz(threads, 256)), dim3(256), 0, ctx->stream,
                       x_dev, n, act);
    NBL_LAUNCH_CHECK(ctx, "activation_kernel");
    return NBL_OK;
}

int nbl_forward_bias(nbl_ctx *ctx, float *y_dev, const float *bias_dev,
                     unsigned channel, unsigned size, unsigned batch) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, y_dev && bias_dev, "nbl_forward_bias: NULL pointer");
    const size_t total = (size_t)batch * channel * size;
    if(total == 0) return NBL_OK;
    if(size % 4 == 0 && ((size_t)y_dev & 15) == 0)
        hipLaunchKernelGGL(channel_affine_kernel<4>, dim3((unsigned)nbl_div_up_sz(total / 4, 256)), dim3(256), 0, ctx->stream,
                           y_dev, (const float*)NULL, bias_dev, total, channel, size);
    else
        hipLaunchKernelGGL(channel_affine_kernel<1>, dim3((unsigned)nbl_div_up_sz(total, 256)), dim3(256), 0, ctx->stream,
                           y_dev, (const float*)NULL, bias_dev, total, channel, size);
    NBL_LAUNCH_CHECK(ctx, "channel_affine_kernel");
    return NBL_OK;
}

int nbl_batchnorm_inference(nbl_ctx *ctx, float *y_dev, const float *mean_dev, const float *var_dev,
                            const float *scale_dev, unsigned channel, unsigned size, unsigned batch) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, y_dev && mean_dev && var_dev && scale_dev, "nbl_batchnorm_inference: NULL pointer");
    const size_t total = (size_t)batch * channel * size;
    if(total == 0) return NBL_OK;
    if(size % 4 == 0 && ((size_t)y_dev & 15) == 0)
        hipLaunchKernelGGL(batchnorm_inference_kernel<4>, dim3((unsigned)nbl_div_up_sz(total / 4, 256)), dim3(256), 0, ctx->stream,
                           y_dev, mean_dev, var_dev, scale_dev, total, channel, size);
    else
        hipLaunchKernelGGL(batchnorm_inference_kernel<1>, dim3((unsigned)nbl_div_up_sz(total, 256)), dim3(256), 0, ctx->stream,
                           y_dev, mean_dev, var_dev, scale_dev, total, channel, size);
    NBL_LAUNCH_CHECK(ctx, "batchnorm_inference_kernel");
    return NBL_OK;
}

int nbl_image_to_input(nbl_ctx *ctx, const unsigned char *src_dev, unsigned images, unsigned src_h, unsigned src_w,
                       unsigned channels, float *dst_dev, unsigned dst_h, unsigned dst_w) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, src_dev && dst_dev, "nbl_image_to_input: NULL pointer");
    NBL_REQUIRE(ctx, src_h && src_w && channels && dst_h && dst_w, "nbl_image_to_input: zero dimension");
    if(images == 0) return NBL_OK;
    if(images > 65535 || dst_h > 65535 || src_h >= (1u << 15) || src_w >= (1u << 15))
        return nbl_fail(ctx, NBL_EUNSUPPORTED, "nbl_image_to_input: more than 65535 images or rows, or a source side of 32768 or more");
    const int resize = src_h != dst_h || src_w != dst_w;
    if(resize && !(ctx->rz_tab_dev && ctx->rz_src_h == src_h && ctx->rz_src_w == src_w && ctx->rz_dst_h == dst_h && ctx->rz_dst_w == dst_w)) {
        std::vector<int> xofs, xw, yofs, yw, tab;
        linear_taps(dst_w, src_w, true, xofs, xw);
        linear_taps(dst_h, src_h, false, yofs, yw);
        tab.insert(tab.end(), xofs.begin(), xofs.end());
        tab.insert(tab.end(), xw.begin(), xw.end());
        for(unsigned k = 0; k < 2; k++)       // the two source rows of a destination row, clipped into the image
            for(unsigned d = 0; d < dst_h; d++) tab.push_back(std::min(std::max(yofs[d] + (int)k, 0), (int)src_h - 1));
        tab.insert(tab.end(), yw.begin(), yw.end());
        int rc = nbl_free(ctx, ctx->rz_tab_dev);
        ctx->rz_tab_dev = NULL;
        if(rc != NBL_OK || (rc = nbl_malloc(ctx, (void**)&ctx->rz_tab_dev, tab.size() * sizeof(int))) != NBL_OK ||
           (rc = nbl_h2d(ctx, ctx->rz_tab_dev, tab.data(), tab.size() * sizeof(int))) != NBL_OK) return rc;
        ctx->rz_src_h = src_h; ctx->rz_src_w = src_w; ctx->rz_dst_h = dst_h; ctx->rz_dst_w = dst_w;
    }
    hipLaunchKernelGGL(image_to_input_kernel, dim3(nbl_div_up(dst_w, 256), dst_h, images), dim3(256), 0, ctx->stream,
                       src_dev, dst_dev, ctx->rz_tab_dev, images, (int)src_h, (int)src_w, (int)channels, (int)dst_h, (int)dst_w, resize);
    NBL_LAUNCH_CHECK(ctx, "image_to_input_kernel");
    return NBL_OK;
}

int nbl_target_prob_sum(nbl_ctx *ctx, const float *probs_dev, const unsigned *targets_dev, unsigned rows, unsigned n,
                        float *sum_dev) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, probs_dev && targets_dev && sum_dev, "nbl_target_prob_sum: NULL pointer");
    hipLaunchKernelGGL(target_prob_sum_kernel, dim3(1), dim3(1024), 0, ctx->stream, probs_dev, targets_dev, rows, n, sum_dev);
    NBL_LAUNCH_CHECK(ctx, "target_prob_sum_kernel");
    return NBL_OK;
}

int nbl_topk_matches(nbl_ctx *ctx, const float *probs_dev, const unsigned *labels_dev, unsigned rows, unsigned n,
                     unsigned k, unsigned *count_dev) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, probs_dev && labels_dev && count_dev, "nbl_topk_matches: NULL pointer");
    hipLaunchKernelGGL(clear_u32_kernel, dim3(1), dim3(1), 0, ctx->stream, count_dev);     // a kernel, so the call stays capturable
    NBL_LAUNCH_CHECK(ctx, "clear_u32_kernel");
    if(rows == 0 || n == 0) return NBL_OK;
    hipLaunchKernelGGL(topk_matches_kernel, dim3(nbl_div_up(rows, 4)), dim3(256), 0, ctx->stream,
                       probs_dev, labels_dev, rows, n, k, count_dev);
    NBL_LAUNCH_CHECK(ctx, "topk_matches_kernel");
    return NBL_OK;
}

}  // extern "C"
