// Context, buffer pool, uploads and downloads: the WgpuContext / UnifiedTensor
// storage / BufferPool side of the boundary (ferrotensor-backend/src/context.rs,
// tensor.rs, pool.rs), on one HIP stream.
#include "ft_common.h"

#include <cstring>

static thread_local std::string g_last_error;

int ft_set_error(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

extern "C" {

const char* ft_last_error(void) { return g_last_error.c_str(); }

static int context_create(int device, void* stream, bool own, ft_context** out) {
    FT_CHECK_ARG(out != nullptr, "ft_context_create: out is NULL");
    int count = 0;
    FT_HIP(hipGetDeviceCount(&count));
    FT_CHECK_ARG(device >= 0 && device < count, "ft_context_create: device %d of %d", device, count);
    FT_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    FT_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return ft_set_error(FT_ERR_INVALID, "ft_context_create: kernels are built for gfx950, device is %s",
                            prop.gcnArchName);
    ft_context* ctx = new ft_context();
    ctx->device = device;
    ctx->num_cus = prop.multiProcessorCount;
    if (own) {
        hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return ft_set_error(FT_ERR_HIP, "hipStreamCreate failed: %s", hipGetErrorString(e));
        }
        ctx->owns_stream = true;
    } else {
        ctx->stream = (hipStream_t)stream;
    }
    *out = ctx;
    return FT_OK;
}

int ft_context_create(int device, ft_context** out) { return context_create(device, nullptr, true, out); }

int ft_context_create_on_stream(int device, void* hip_stream, ft_context** out) {
    return context_create(device, hip_stream, false, out);
}

int ft_pool_trim(ft_context* ctx) {
    FT_CHECK_ARG(ctx, "ft_pool_trim: ctx is NULL");
    FT_HIP(hipSetDevice(ctx->device));
    FT_HIP(hipStreamSynchronize(ctx->stream));
    for (auto& kv : ctx->idle)
        for (void* p : kv.second) FT_HIP(hipFree(p));
    ctx->idle.clear();
    ctx->idle_bytes = 0;
    return FT_OK;
}

int ft_context_destroy(ft_context* ctx) {
    if (!ctx) return FT_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto& kv : ctx->idle)
        for (void* p : kv.second) (void)hipFree(p);
    for (auto& kv : ctx->live) (void)hipFree(kv.first);
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return FT_OK;
}

int ft_synchronize(ft_context* ctx) {
    FT_CHECK_ARG(ctx, "ft_synchronize: ctx is NULL");
    FT_HIP(hipStreamSynchronize(ctx->stream));
    return FT_OK;
}

int ft_flush(ft_context* ctx) {
    FT_CHECK_ARG(ctx, "ft_flush: ctx is NULL");
    return FT_OK;
}

void* ft_context_stream(ft_context* ctx) { return ctx ? (void*)ctx->stream : nullptr; }

int ft_alloc(ft_context* ctx, size_t bytes, void** out_dev) {
    FT_CHECK_ARG(ctx && out_dev, "ft_alloc: NULL argument");
    if (bytes == 0) bytes = 4;                      // storage bindings are whole words
    bytes = (bytes + 255) & ~(size_t)255;           // exact-size classes at 256 B granularity
    auto it = ctx->idle.find(bytes);
    void* p = nullptr;
    if (it != ctx->idle.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        ctx->idle_bytes -= bytes;
    } else {
        FT_HIP(hipSetDevice(ctx->device));
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) {
            // Give the pooled buffers back to the driver and try once more.
            (void)hipGetLastError();
            FT_TRY(ft_pool_trim(ctx));
            e = hipMalloc(&p, bytes);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return ft_set_error(FT_ERR_OOM, "ft_alloc: hipMalloc(%zu) failed: %s", bytes,
                                    hipGetErrorString(e));
            }
        }
    }
    ctx->live[p] = bytes;
    ctx->live_bytes += bytes;
    *out_dev = p;
    return FT_OK;
}

int ft_free(ft_context* ctx, void* dev) {
    FT_CHECK_ARG(ctx, "ft_free: ctx is NULL");
    if (!dev) return FT_OK;
    auto it = ctx->live.find(dev);
    FT_CHECK_ARG(it != ctx->live.end(), "ft_free: %p was not allocated by this context", dev);
    const size_t bytes = it->second;
    ctx->live.erase(it);
    ctx->live_bytes -= bytes;
    // Reuse is safe without a wait: every kernel runs on the one in-order stream.
    ctx->idle[bytes].push_back(dev);
    ctx->idle_bytes += bytes;
    return FT_OK;
}

int ft_pool_stats(ft_context* ctx, size_t* live_bytes, size_t* idle_bytes) {
    FT_CHECK_ARG(ctx, "ft_pool_stats: ctx is NULL");
    if (live_bytes) *live_bytes = ctx->live_bytes;
    if (idle_bytes) *idle_bytes = ctx->idle_bytes;
    return FT_OK;
}

int ft_upload(ft_context* ctx, void* dst_dev, const void* src_host, size_t bytes) {
    FT_CHECK_ARG(ctx && (bytes == 0 || (dst_dev && src_host)), "ft_upload: NULL argument");
    if (bytes == 0) return FT_OK;
    // Pageable source: hipMemcpyAsync stages it before returning, so the
    // caller may reuse src immediately (as with wgpu's write_buffer).
    FT_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    FT_HIP(hipStreamSynchronize(ctx->stream));
    return FT_OK;
}

int ft_download(ft_context* ctx, void* dst_host, const void* src_dev, size_t bytes) {
    FT_CHECK_ARG(ctx && (bytes == 0 || (dst_host && src_dev)), "ft_download: NULL argument");
    if (bytes == 0) return FT_OK;
    FT_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    FT_HIP(hipStreamSynchronize(ctx->stream));
    return FT_OK;
}

int ft_upload_f32_as_f16(ft_context* ctx, void* dst_dev, const float* src_host, size_t n) {
    FT_CHECK_ARG(ctx && (n == 0 || (dst_dev && src_host)), "ft_upload_f32_as_f16: NULL argument");
    size_t bytes = ((n * 2 + 3) / 4) * 4;
    if (bytes < 4) bytes = 4;
    std::vector<uint16_t> packed(bytes / 2, 0);
    for (size_t i = 0; i < n; i++) {
        const _Float16 h = (_Float16)src_host[i];   // IEEE round-to-nearest-even
        std::memcpy(&packed[i], &h, 2);
    }
    return ft_upload(ctx, dst_dev, packed.data(), bytes);
}

int ft_upload_f32_transposed(ft_context* ctx, void* dst_dev, const float* src_host, size_t rows,
                             size_t cols, int dtype) {
    FT_CHECK_ARG(ctx && dst_dev && src_host, "ft_upload_f32_transposed: NULL argument");
    FT_CHECK_ARG(dtype == FT_DTYPE_F32 || dtype == FT_DTYPE_F16,
                 "ft_upload_f32_transposed: dtype %d is not supported", dtype);
    const size_t n = rows * cols;
    if (dtype == FT_DTYPE_F32) {
        std::vector<float> t(n);
        for (size_t c = 0; c < cols; c++)
            for (size_t r = 0; r < rows; r++) t[c * rows + r] = src_host[r * cols + c];
        return ft_upload(ctx, dst_dev, t.data(), n * 4);
    }
    size_t bytes = ((n * 2 + 3) / 4) * 4;
    if (bytes < 4) bytes = 4;
    std::vector<uint16_t> t(bytes / 2, 0);
    for (size_t c = 0; c < cols; c++)
        for (size_t r = 0; r < rows; r++) {
            const _Float16 h = (_Float16)src_host[r * cols + c];
            std::memcpy(&t[c * rows + r], &h, 2);
        }
    return ft_upload(ctx, dst_dev, t.data(), bytes);
}

int ft_copy_tensor(ft_context* ctx, const void* src_dev, size_t bytes, void* dst_dev,
                   size_t dst_byte_offset) {
    FT_CHECK_ARG(ctx && (bytes == 0 || (src_dev && dst_dev)), "ft_copy_tensor: NULL argument");
    if (bytes == 0) return FT_OK;
    FT_HIP(hipMemcpyAsync((char*)dst_dev + dst_byte_offset, src_dev, bytes, hipMemcpyDeviceToDevice,
                          ctx->stream));
    return FT_OK;
}

}  // extern "C"
