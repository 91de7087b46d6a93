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

ft_prof_scope::ft_prof_scope(ft_context* c, const char* name, double flops, double bytes) : ctx(c), index(-1) {
    if (!c || !c->prof_on) return;
    auto it = c->prof_keys.find(name);
    int key;
    if (it == c->prof_keys.end()) {
        key = (int)c->prof_names.size();
        c->prof_names.push_back(name);
        c->prof_keys[name] = key;
        c->prof_totals.emplace_back();
    } else {
        key = it->second;
    }
    ft_context::ProfRecord r{key, nullptr, nullptr, flops, bytes};
    for (hipEvent_t* e : {&r.e0, &r.e1}) {
        if (!c->prof_event_pool.empty()) {
            *e = c->prof_event_pool.back();
            c->prof_event_pool.pop_back();
        } else if (hipEventCreate(e) != hipSuccess) {
            return;
        }
    }
    if (hipEventRecord(r.e0, c->stream) != hipSuccess) return;
    index = (int)c->prof_records.size();
    c->prof_records.push_back(r);
}

ft_prof_scope::~ft_prof_scope() {
    if (index >= 0) (void)hipEventRecord(ctx->prof_records[index].e1, ctx->stream);
}

// Waits for the stream and folds the finished records into the totals.
static int prof_collect(ft_context* ctx) {
    FT_HIP(hipStreamSynchronize(ctx->stream));
    for (auto& r : ctx->prof_records) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, r.e0, r.e1) == hipSuccess) {
            auto& t = ctx->prof_totals[r.key];
            t.launches += 1;
            t.ms += ms;
            t.flops += r.flops;
            t.bytes += r.bytes;
        }
        ctx->prof_event_pool.push_back(r.e0);
        ctx->prof_event_pool.push_back(r.e1);
    }
    ctx->prof_records.clear();
    return FT_OK;
}

extern "C" {

const char* ft_last_error(void) { return g_last_error.c_str(); }

int ft_profile_begin(ft_context* ctx) {
    FT_CHECK_ARG(ctx, "ft_profile_begin: ctx is NULL");
    FT_TRY(prof_collect(ctx));
    for (auto& t : ctx->prof_totals) t = ft_context::ProfTotal();
    ctx->prof_on = true;
    return FT_OK;
}

int ft_profile_end(ft_context* ctx, size_t* kernels) {
    FT_CHECK_ARG(ctx, "ft_profile_end: ctx is NULL");
    ctx->prof_on = false;
    FT_TRY(prof_collect(ctx));
    if (kernels) *kernels = ctx->prof_names.size();
    return FT_OK;
}

int ft_profile_kernel(ft_context* ctx, size_t index, const char** name, uint64_t* launches, double* total_ms,
                      double* flops, double* bytes) {
    FT_CHECK_ARG(ctx && index < ctx->prof_names.size(), "ft_profile_kernel: bad index");
    FT_TRY(prof_collect(ctx));
    const auto& t = ctx->prof_totals[index];
    if (name) *name = ctx->prof_names[index].c_str();
    if (launches) *launches = t.launches;
    if (total_ms) *total_ms = t.ms;
    if (flops) *flops = t.flops;
    if (bytes) *bytes = t.bytes;
    return FT_OK;
}

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
    // Set-up that must not happen later, when a caller may be unable to allocate or load code:
    // the device address of the fixed scratch array of ft_rms_norm_backward_noalloc.
    FT_TRY(ft_internal_noalloc_init(device));
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
    for (auto& r : ctx->prof_records) {
        (void)hipEventDestroy(r.e0);
        (void)hipEventDestroy(r.e1);
    }
    for (hipEvent_t e : ctx->prof_event_pool) (void)hipEventDestroy(e);
    if (ctx->thin_scratch) (void)hipFree(ctx->thin_scratch);
    if (ctx->gemm_scratch) (void)hipFree(ctx->gemm_scratch);
    if (ctx->attn_scratch) (void)hipFree(ctx->attn_scratch);
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
    // Blocks until the copy is done, so the caller may reuse src at once (as with wgpu's
    // write_buffer). The step driver does not come through here: it stages a chunk's arrays in
    // pinned memory and sends them in one asynchronous copy.
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
    // Transposed in 32 x 32 blocks so that both the strided side and the contiguous side stay in cache.
    constexpr size_t kBlock = 32;
    auto for_each_block = [&](auto&& put) {
        for (size_t r0 = 0; r0 < rows; r0 += kBlock)
            for (size_t c0 = 0; c0 < cols; c0 += kBlock) {
                const size_t r1 = r0 + kBlock < rows ? r0 + kBlock : rows;
                const size_t c1 = c0 + kBlock < cols ? c0 + kBlock : cols;
                for (size_t c = c0; c < c1; c++)
                    for (size_t r = r0; r < r1; r++) put(c * rows + r, src_host[r * cols + c]);
            }
    };
    if (dtype == FT_DTYPE_F32) {
        std::vector<float> t(n);
        for_each_block([&](size_t at, float v) { t[at] = v; });
        return ft_upload(ctx, dst_dev, t.data(), n * 4);
    }
    size_t bytes = ((n * 2 + 3) / 4) * 4;
    if (bytes < 4) bytes = 4;
    std::vector<uint16_t> t(bytes / 2, 0);
    for_each_block([&](size_t at, float v) {
        const _Float16 h = (_Float16)v;   // round to nearest even, as half::f16::from_f32
        std::memcpy(&t[at], &h, 2);
    });
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
