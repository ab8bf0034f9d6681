// Context, device memory, stream and timing entry points of the C ABI.
#include "nbl_internal.h"

#include <cmath>

static char g_create_err[512] = "";

int nbl_fail(nbl_ctx *ctx, int code, const char *fmt, ...) {
    char *dst = ctx ? ctx->err : g_create_err;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(dst, 512, fmt, ap);
    va_end(ap);
    return code;
}

void nbl_fold_batchnorm(const float *bias, const float *scale, const float *mean, const float *var,
                        unsigned n, float *g_out, float *b_out) {
    for(unsigned i = 0; i < n; i++) {
        if(scale) {
            const double g = (double)scale[i] / (std::sqrt((double)var[i]) + 0.00001);
            g_out[i] = (float)g;
            b_out[i] = (float)((double)bias[i] - (double)mean[i] * g);
        } else {
            g_out[i] = 1.0f;
            b_out[i] = bias[i];
        }
    }
}

extern "C" {

const char *nbl_version(void) { return "nebula-hip 0.1 (gfx950)"; }

int nbl_ctx_create_on_stream(int device, void *hip_stream, nbl_ctx **out) {
    if(!out) return nbl_fail(NULL, NBL_EINVAL, "nbl_ctx_create: out is NULL");
    *out = NULL;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if(e != hipSuccess || count <= 0)
        return nbl_fail(NULL, NBL_ENODEVICE, "no HIP device visible (%s)", hipGetErrorString(e));
    if(device < 0 || device >= count)
        return nbl_fail(NULL, NBL_EINVAL, "device %d out of range (%d visible)", device, count);
    e = hipSetDevice(device);
    if(e != hipSuccess) return nbl_fail(NULL, NBL_EHIP, "hipSetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if(e != hipSuccess) return nbl_fail(NULL, NBL_EHIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if(strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return nbl_fail(NULL, NBL_ENODEVICE, "device %d is %s; this library holds gfx950 code only",
                        device, prop.gcnArchName);
    nbl_ctx *ctx = new nbl_ctx();
    ctx->device = device;
    ctx->num_cu = prop.multiProcessorCount;
    ctx->err[0] = 0;
    ctx->owns_stream = false;
    ctx->stream = (hipStream_t)hip_stream;
    ctx->ev_start = ctx->ev_stop = nullptr;
    if((e = hipEventCreate(&ctx->ev_start)) != hipSuccess || (e = hipEventCreate(&ctx->ev_stop)) != hipSuccess) {
        delete ctx;
        return nbl_fail(NULL, NBL_EHIP, "hipEventCreate: %s", hipGetErrorString(e));
    }
    const int rc = nbl_fc_scratch_resolve(ctx);
    if(rc != NBL_OK) {
        nbl_fail(NULL, rc, "%s", ctx->err);
        (void)hipEventDestroy(ctx->ev_start); (void)hipEventDestroy(ctx->ev_stop);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return NBL_OK;
}

int nbl_ctx_create(int device, nbl_ctx **out) {
    int rc = nbl_ctx_create_on_stream(device, NULL, out);
    if(rc != NBL_OK) return rc;
    hipStream_t s;
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);   // default priority
    if(e != hipSuccess) {
        nbl_ctx_destroy(*out);
        *out = NULL;
        return nbl_fail(NULL, NBL_EHIP, "hipStreamCreate: %s", hipGetErrorString(e));
    }
    (*out)->stream = s;
    (*out)->owns_stream = true;
    return NBL_OK;
}

int nbl_ctx_destroy(nbl_ctx *ctx) {
    if(!ctx) return NBL_EINVAL;
    // tear-down goes on whatever the individual calls return: there is nobody left to report to
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if(ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if(ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if(ctx->rz_tab_dev) (void)hipFree(ctx->rz_tab_dev);
    if(ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return NBL_OK;
}

const char *nbl_last_error(nbl_ctx *ctx) { return ctx ? ctx->err : g_create_err; }

void *nbl_ctx_stream(nbl_ctx *ctx) { return ctx ? (void*)ctx->stream : NULL; }

int nbl_malloc(nbl_ctx *ctx, void **dev_ptr, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, dev_ptr != NULL, "nbl_malloc: dev_ptr is NULL");
    *dev_ptr = NULL;
    if(bytes == 0) return NBL_OK;
    NBL_HIP(ctx, hipSetDevice(ctx->device));
    NBL_HIP(ctx, hipMalloc(dev_ptr, bytes));
    return NBL_OK;
}

int nbl_free(nbl_ctx *ctx, void *dev_ptr) {
    if(!ctx) return NBL_EINVAL;
    if(!dev_ptr) return NBL_OK;
    NBL_HIP(ctx, hipStreamSynchronize(ctx->stream));
    NBL_HIP(ctx, hipFree(dev_ptr));
    return NBL_OK;
}

int nbl_malloc_host(nbl_ctx *ctx, void **host_ptr, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, host_ptr != NULL, "nbl_malloc_host: host_ptr is NULL");
    *host_ptr = NULL;
    if(bytes == 0) return NBL_OK;
    NBL_HIP(ctx, hipSetDevice(ctx->device));
    NBL_HIP(ctx, hipHostMalloc(host_ptr, bytes, hipHostMallocDefault));
    return NBL_OK;
}

int nbl_free_host(nbl_ctx *ctx, void *host_ptr) {
    if(!ctx) return NBL_EINVAL;
    if(!host_ptr) return NBL_OK;
    NBL_HIP(ctx, hipStreamSynchronize(ctx->stream));
    NBL_HIP(ctx, hipHostFree(host_ptr));
    return NBL_OK;
}

int nbl_h2d(nbl_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    if(bytes == 0) return NBL_OK;
    NBL_REQUIRE(ctx, dst_dev && src_host, "nbl_h2d: NULL pointer");
    NBL_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    NBL_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return NBL_OK;
}

int nbl_d2h(nbl_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    if(bytes == 0) return NBL_OK;
    NBL_REQUIRE(ctx, dst_host && src_dev, "nbl_d2h: NULL pointer");
    NBL_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    NBL_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return NBL_OK;
}

int nbl_d2h_async(nbl_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    if(bytes == 0) return NBL_OK;
    NBL_REQUIRE(ctx, dst_host && src_dev, "nbl_d2h_async: NULL pointer");
    NBL_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    return NBL_OK;
}

__global__ void nbl_fill_zero_kernel(uint4 *dst4, size_t n4, unsigned char *tail, unsigned ntail) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for(size_t j = i; j < n4; j += step) dst4[j] = make_uint4(0, 0, 0, 0);
    if(i < ntail) tail[i] = 0;
}

int nbl_fill_zero(nbl_ctx *ctx, void *dst_dev, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    if(bytes == 0) return NBL_OK;
    NBL_REQUIRE(ctx, dst_dev != NULL, "nbl_fill_zero: NULL pointer");
    NBL_REQUIRE(ctx, ((size_t)dst_dev & 15) == 0, "nbl_fill_zero: pointer must be 16-byte aligned");
    const size_t n4 = bytes / 16;
    const unsigned ntail = (unsigned)(bytes % 16);
    size_t blocks = nbl_div_up_sz(n4 ? n4 : 1, 256);
    if(blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(nbl_fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (uint4*)dst_dev, n4, (unsigned char*)dst_dev + n4 * 16, ntail);
    NBL_LAUNCH_CHECK(ctx, "fill_zero");
    return NBL_OK;
}

__global__ void nbl_copy_kernel(uint4 *__restrict__ dst4, const uint4 *__restrict__ src4, size_t n4,
                                unsigned char *__restrict__ dtail, const unsigned char *__restrict__ stail, unsigned ntail) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for(size_t j = i; j < n4; j += step) dst4[j] = src4[j];
    if(i < ntail) dtail[i] = stail[i];
}

// The same copy with streaming stores (see nbl_stream_stores).
__global__ void nbl_copy_stream_kernel(uint4 *__restrict__ dst4, const uint4 *__restrict__ src4, size_t n4,
                                       unsigned char *__restrict__ dtail, const unsigned char *__restrict__ stail, unsigned ntail) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for(size_t j = i; j < n4; j += step) nbl_put<true>(dst4 + j, src4[j]);
    if(i < ntail) dtail[i] = stail[i];
}

int nbl_copy_d2d(nbl_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    if(!ctx) return NBL_EINVAL;
    if(bytes == 0) return NBL_OK;
    NBL_REQUIRE(ctx, dst_dev && src_dev, "nbl_copy_d2d: NULL pointer");
    NBL_REQUIRE(ctx, (((size_t)dst_dev | (size_t)src_dev) & 15) == 0, "nbl_copy_d2d: pointers must be 16-byte aligned");
    const char *s = (const char*)src_dev, *d = (const char*)dst_dev;
    NBL_REQUIRE(ctx, s + bytes <= d || d + bytes <= s, "nbl_copy_d2d: ranges overlap");
    const size_t n4 = bytes / 16;
    const unsigned ntail = (unsigned)(bytes % 16);
    size_t blocks = nbl_div_up_sz(n4 ? n4 : 1, 256);
    if(blocks > 8192) blocks = 8192;
    if(nbl_stream_stores(bytes, dst_dev, src_dev))
        hipLaunchKernelGGL(nbl_copy_stream_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                           (uint4*)dst_dev, (const uint4*)src_dev, n4,
                           (unsigned char*)dst_dev + n4 * 16, (const unsigned char*)src_dev + n4 * 16, ntail);
    else
        hipLaunchKernelGGL(nbl_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                           (uint4*)dst_dev, (const uint4*)src_dev, n4,
                           (unsigned char*)dst_dev + n4 * 16, (const unsigned char*)src_dev + n4 * 16, ntail);
    NBL_LAUNCH_CHECK(ctx, "copy_d2d");
    return NBL_OK;
}

// Every block writes `words` 32-bit words of its LDS allocation with the pattern and reports one of them, so the
// stores cannot be dropped.
__global__ void nbl_lds_fill_kernel(unsigned pattern, unsigned words, unsigned *sink) {
    extern __shared__ unsigned lds_words[];
    for(unsigned i = threadIdx.x; i < words; i += blockDim.x) lds_words[i] = pattern;
    __syncthreads();
    if(threadIdx.x == 0 && lds_words[words - 1] != pattern) *sink = 1u;
}

int nbl_lds_fill(nbl_ctx *ctx, unsigned pattern) {
    if(!ctx) return NBL_EINVAL;
    int max_bytes = 0;
    NBL_HIP(ctx, hipDeviceGetAttribute(&max_bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, ctx->device));
    if(max_bytes <= 0) return nbl_fail(ctx, NBL_EHIP, "nbl_lds_fill: the device reports no LDS");
    if(max_bytes > 64 * 1024)
        NBL_HIP(ctx, hipFuncSetAttribute((const void*)nbl_lds_fill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, max_bytes));
    unsigned *sink = NULL;
    int rc = nbl_malloc(ctx, (void**)&sink, sizeof(unsigned));
    if(rc != NBL_OK) return rc;
    // a block takes a CU's whole LDS, so at most one is resident per CU; a few rounds reach every CU
    hipLaunchKernelGGL(nbl_lds_fill_kernel, dim3(8u * (unsigned)ctx->num_cu), dim3(256), (size_t)max_bytes, ctx->stream,
                       pattern, (unsigned)max_bytes / 4u, sink);
    hipError_t e = hipGetLastError();
    rc = nbl_free(ctx, sink);       // waits for the kernel
    if(e != hipSuccess) return nbl_fail(ctx, NBL_EHIP, "launch of nbl_lds_fill_kernel failed: %s", hipGetErrorString(e));
    return rc;
}

int nbl_sync(nbl_ctx *ctx) {
    if(!ctx) return NBL_EINVAL;
    NBL_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return NBL_OK;
}

int nbl_timer_start(nbl_ctx *ctx) {
    if(!ctx) return NBL_EINVAL;
    NBL_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    return NBL_OK;
}

int nbl_timer_stop(nbl_ctx *ctx, float *elapsed_ms) {
    if(!ctx) return NBL_EINVAL;
    NBL_REQUIRE(ctx, elapsed_ms != NULL, "nbl_timer_stop: elapsed_ms is NULL");
    NBL_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    NBL_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
    NBL_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
    return NBL_OK;
}

unsigned nbl_pool_out_dim(unsigned in, unsigned stride, unsigned pad) { return stride ? (in + 2 * pad) / stride : 0; }

unsigned nbl_conv_out_dim(unsigned in, unsigned ksize, unsigned stride, unsigned pad) {
    if(!stride || in + 2 * pad < ksize) return 0;
    return (in + 2 * pad - ksize) / stride + 1;
}

}  // extern "C"
