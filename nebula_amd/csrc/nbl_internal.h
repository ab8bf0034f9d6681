// Internal declarations shared by the HIP translation units of libnebula_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>

#include "nebula_hip.h"

struct nbl_ctx {
    int device;
    hipStream_t stream;
    bool owns_stream;
    hipEvent_t ev_start, ev_stop;
    int num_cu;
    char err[512];
    // tap tables of the last image resize geometry (nbl_image_to_input), kept on the device
    unsigned rz_src_h, rz_src_w, rz_dst_h, rz_dst_w;
    int *rz_tab_dev;
    float *fc_scratch;      // this device's copy of the static split-K scratch of nbl_fc_fwd_noalloc (NULL: none)
};

// Looks up the device address of the static scratch array for ctx->device (once per device) and stores it in the context.
int nbl_fc_scratch_resolve(nbl_ctx *ctx);

// Records a formatted message on the context and returns `code`.
int nbl_fail(nbl_ctx *ctx, int code, const char *fmt, ...);

#define NBL_REQUIRE(ctx, cond, ...) \
    do { if(!(cond)) return nbl_fail((ctx), NBL_EINVAL, __VA_ARGS__); } while(0)

#define NBL_HIP(ctx, call) \
    do { hipError_t e_ = (call); \
         if(e_ != hipSuccess) return nbl_fail((ctx), e_ == hipErrorOutOfMemory ? NBL_ENOMEM : NBL_EHIP, \
                                              "%s failed: %s", #call, hipGetErrorString(e_)); } while(0)

// After a kernel launch: launch-configuration errors surface here.
#define NBL_LAUNCH_CHECK(ctx, what) \
    do { hipError_t e_ = hipGetLastError(); \
         if(e_ != hipSuccess) return nbl_fail((ctx), NBL_EHIP, "launch of %s failed: %s", what, \
                                              hipGetErrorString(e_)); } while(0)

// A kernel that asks for more than 64 KB of dynamic LDS must have that limit raised first, on every device it runs
// on (hipFuncSetAttribute acts on the current device).  One of these per kernel remembers which devices are done:
// one bit per device ordinal, ordinals from 64 on are asked for every time.
struct nbl_lds_limit_raised {
    std::atomic<unsigned long long> devices{0};
    template<typename Kernel>
    hipError_t ensure(Kernel kernel, int device, int bytes) {
        if(device >= 0 && device < 64 && (devices.load(std::memory_order_acquire) >> device & 1)) return hipSuccess;
        int current = -1;
        hipError_t e = hipGetDevice(&current);
        if(e == hipSuccess && current != device) e = hipSetDevice(device);
        if(e == hipSuccess) e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if(current >= 0 && current != device) (void)hipSetDevice(current);
        if(e == hipSuccess && device >= 0 && device < 64) devices.fetch_or(1ull << device, std::memory_order_release);
        return e;
    }
};

static inline unsigned nbl_div_up(unsigned a, unsigned b) { return (a + b - 1) / b; }
static inline size_t nbl_div_up_sz(size_t a, size_t b) { return (a + b - 1) / b; }

// -------------------------------------------------------------------------------------------------
// Streaming stores.  A kernel that writes a tensor it does not read (out of place) keeps 69 % of the memory rate with
// ordinary stores and 88 % with non-temporal ones on this part (256 MiB copy: 98 us against 76 us); a kernel that
// writes the lines it has just read loses with them (76 us against 89 us), and so does a producer whose consumer
// would have found the tensor in the caches.  Kernels take STREAM as a template argument and the launch site decides
// with nbl_stream_stores(): the output must not alias an input and must be at least NBL_STREAM_MIN_BYTES long, the
// capacity of the eight L2 caches together (a shorter tensor may still be there when the next kernel reads it; whole
// networks time the same either way, so the line is drawn where the isolated kernel starts to gain).
// -------------------------------------------------------------------------------------------------
#ifndef NBL_STREAM_MIN_BYTES
#define NBL_STREAM_MIN_BYTES ((size_t)32 << 20)
#endif
static inline bool nbl_stream_stores(size_t bytes_written, const void *out, const void *in0, const void *in1 = NULL) {
    return bytes_written >= NBL_STREAM_MIN_BYTES && out != in0 && out != in1;
}
// Streaming loads pay only where nothing is read twice and the data cannot already sit in the 256 MiB memory-side cache:
// the 2x2 pool of a 411 MB tensor gains 8 % and the same-shape shortcut of two 205 MB tensors 6 %, while a 3x3/2 pool
// (adjacent windows share rows) loses 60 % and a 164 MB softmax 13 %.
#ifndef NBL_STREAM_IN_MIN_BYTES
#define NBL_STREAM_IN_MIN_BYTES ((size_t)256 << 20)
#endif
static inline bool nbl_stream_loads(size_t bytes_read) { return bytes_read >= NBL_STREAM_IN_MIN_BYTES; }
typedef float    nbl_f32x4 __attribute__((ext_vector_type(4)));
typedef float    nbl_f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned nbl_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned nbl_u32x2 __attribute__((ext_vector_type(2)));
template<bool STREAM> __device__ __forceinline__ void nbl_put(float *p, float v) {
    if constexpr(STREAM) __builtin_nontemporal_store(v, p); else *p = v;
}
template<bool STREAM> __device__ __forceinline__ void nbl_put(unsigned *p, unsigned v) {
    if constexpr(STREAM) __builtin_nontemporal_store(v, p); else *p = v;
}
template<bool STREAM> __device__ __forceinline__ void nbl_put(float2 *p, float a, float b) {
    if constexpr(STREAM) __builtin_nontemporal_store(nbl_f32x2{a, b}, reinterpret_cast<nbl_f32x2*>(p)); else *p = make_float2(a, b);
}
template<bool STREAM> __device__ __forceinline__ void nbl_put(uint2 *p, unsigned a, unsigned b) {
    if constexpr(STREAM) __builtin_nontemporal_store(nbl_u32x2{a, b}, reinterpret_cast<nbl_u32x2*>(p)); else *p = make_uint2(a, b);
}
template<bool STREAM> __device__ __forceinline__ void nbl_put(float4 *p, float4 v) {
    if constexpr(STREAM) __builtin_nontemporal_store(nbl_f32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<nbl_f32x4*>(p)); else *p = v;
}
template<bool STREAM> __device__ __forceinline__ float4 nbl_get(const float4 *p) {
    if constexpr(STREAM) {
        const nbl_f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nbl_f32x4*>(p));
        return make_float4(t.x, t.y, t.z, t.w);
    } else {
        return *p;
    }
}
template<bool STREAM> __device__ __forceinline__ void nbl_put(uint4 *p, uint4 v) {
    if constexpr(STREAM) __builtin_nontemporal_store(nbl_u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<nbl_u32x4*>(p)); else *p = v;
}

// -------------------------------------------------------------------------------------------------
// The thirteen activations of common/activations.cc:6-89, evaluated as the CPU file does: the
// literals there are doubles, so anything that touches one is computed in double and rounded once
// on the store.  relu / leaky / relie keep the `x > 0` predicate on the float value, which is what
// makes their masks agree bit for bit.  elu, hardtan and lhtan are not the textbook functions
// (elu squares positive inputs, the other two return 0/1 indicators); they are reproduced as written.
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ float nbl_act_apply(int act, float x) {
    switch(act) {
        case NBL_ACT_RELU:   return x > 0.0f ? x : 0.0f;
        case NBL_ACT_LINEAR: return x;
        case NBL_ACT_LEAKY:  return x > 0.0f ? x : (float)(0.1 * (double)x);
        case NBL_ACT_RELIE:  return x > 0.0f ? x : (float)(0.01 * (double)x);
        default: break;
    }
    const double d = (double)x;
    switch(act) {
        case NBL_ACT_ELU:      return x > 0.0f ? x * x : (float)(d * (exp(d) - 1.0));
        case NBL_ACT_HARDTAN:  return (x < 1.0f && x > -1.0f) ? 1.0f : 0.0f;
        case NBL_ACT_LHTAN:    return (x > 0.0f && x < 1.0f) ? 1.0f : 0.0f;
        case NBL_ACT_LOGGY:    return (float)(2.0 / (1.0 + exp(0.0 - d)) - 1.0);
        case NBL_ACT_LOGISTIC: return (float)(1.0 / (1.0 + exp(0.0 - d)));
        case NBL_ACT_PLSE:
            if(d < -4.0) return (float)(0.01 * (d + 4.0));
            if(d > 4.0)  return (float)(0.01 * (d - 4.0) + 1.0);
            return (float)(0.125 * d + 0.5);
        case NBL_ACT_RAMP:     return x > 0.0f ? (float)(d * (d + 0.01)) : (float)(0.01 * d);
        case NBL_ACT_STAIR: {
            const int n = (int)x, half = (int)(d / 2.0);
            return (n % 2) ? (x - (float)n) + (float)half : (float)half;
        }
        case NBL_ACT_TANH: {
            const double e = exp(2.0 * d);
            return (float)((e - 1.0) / (e + 1.0));
        }
        default: return x;
    }
}

static inline bool nbl_act_valid(int act) { return act > NBL_ACT_UNDEFINED && act < NBL_ACT_COUNT; }

// Inference batchnorm + bias as one multiply-add per channel, computed on the host in double:
//   g = scale / (sqrt(var) + 1e-5)   (common/batchnorm.cc:70, eps outside the root)
//   b = bias - mean * g
// Without batchnorm g is 1 and b is the bias.
void nbl_fold_batchnorm(const float *bias, const float *scale, const float *mean, const float *var,
                        unsigned n, float *g_out, float *b_out);

// Division by a number known on the host: q = umulhi(n, mul) >> shr for n < 2^31 (mul = ceil(2^(31 + ceil(log2 d)) / d)).
// A runtime integer division costs some 25 ordinary vector instructions, and the block's set-up has half a dozen of
// them; ordinary vector instructions are paid for in matrix-pipe time, which matters for layers with few patch rows.
struct FastDiv {
    unsigned mul, shr, d;
    __host__ __device__ __forceinline__ unsigned div(unsigned n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        return d == 1u ? n : __umulhi(n, mul) >> shr;
#else
        return n / d;
#endif
    }
};
inline FastDiv make_fastdiv(unsigned d) {
    FastDiv f; f.d = d; f.mul = 0; f.shr = 0;
    if(d > 1) {
        unsigned lg = 0;
        while((1ull << lg) < d) lg++;
        const unsigned p = 31 + lg;
        f.mul = (unsigned)(((1ull << p) + d - 1) / d);
        f.shr = p - 32;
    }
    return f;
}

// Convolutions with very few input channels (the first layer of an image network: 3 channels, a large filter):
// their patch rows come from a handful of input rows, so a block stages that strip of the image in LDS once and
// feeds the matrix cores from it (csrc/conv_strip.hip).  Filled by nbl_conv2d_pack when the layer qualifies.
struct nbl_strip_plan {
    bool eligible;
    int C, H, W, F, k, stride, pad, OH, OW, K, Kp, Mp, act;
    int mt;                 // 32-filter MFMA tiles per wave (block tile = 32*mt filters x 128 pixels)
    int rows, pitch;        // strip: input rows a block may need, floats per row (W + 2*pad)
    int *otab_dev;          // [Kp] strip offset of every patch row; padding rows hold 0 (the pixel's own first tap, against a zero weight)
    const float *wq_dev, *g_dev, *b_dev;     // packed weights [Kp / 4][Mp][4], per-filter multiply-add
    size_t lds_bytes;
};
// Builds the offset table (host side of the plan); returns NBL_OK and leaves eligible = false when the layer does not qualify.
int nbl_conv_strip_pack(nbl_ctx *ctx, nbl_strip_plan *sp);
int nbl_conv_strip_forward(nbl_ctx *ctx, const nbl_strip_plan *sp, const float *x_dev, float *y_dev, unsigned B);
void nbl_conv_strip_destroy(nbl_ctx *ctx, nbl_strip_plan *sp);
