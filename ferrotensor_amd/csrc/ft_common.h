// Internal helpers shared by the sources of libferrotensor_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "ferrotensor_hip.h"

// The device-buffer pool: exact-size free lists, like the reference's
// BufferPool (ferrotensor-backend/src/pool.rs), without its 512 MiB cap:
// 288 GB of HBM leaves room to keep every step buffer resident.
// The K shares of a split GEMM left unadded for the kernel that consumes the product (a norm kernel
// that reads the row anyway). Two forms:
//  * every tile split (`splits > 1`): out = (add +) partial[0] + partial[1] + ... in that order, share s of
//    element i at partial[s * stride + i]; `out` holds nothing yet.
//  * tail split (`tail_shift > 0`): `out` is complete except for the 64 x 64 tiles at positions >= tail_first
//    of the tile order (panels of `panel` n tiles, inside a panel row block after row block); tile
//    tail_first + u is (add +) its 1 << tail_shift shares, share s at partial[((u << tail_shift) + s) * 4096],
//    row-major inside the tile.
// Neither: nothing was deferred, `out` is complete.
struct ft_deferred_sum {
    const float* partial = nullptr;
    const float* add = nullptr;
    long stride = 0;
    int splits = 1;
    const float* out = nullptr;
    int tail_first = 0, tail_shift = 0, tiles_m = 0, tiles_n = 0, panel = 1;
    bool pending() const { return splits > 1 || tail_shift > 0; }
};

struct ft_context {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    std::unordered_map<void*, size_t> live;                 // ptr -> bytes handed out
    std::unordered_map<size_t, std::vector<void*>> idle;    // bytes -> free buffers
    size_t live_bytes = 0, idle_bytes = 0;
    int num_cus = 256;

    // Partial sums of the sliced thin products (LoRA dA, dB); allocated on first use.
    float* thin_scratch = nullptr;
    // Partial tiles of split-K GEMMs (few output tiles, long K); allocated on first use.
    float* gemm_scratch = nullptr;
    // Set by the step driver right before one GEMM call whose output's only reader can add the K
    // shares itself; the launch fills it in (and leaves out splitk_reduce_kernel) when it splits K,
    // and clears the pointer either way.
    ft_deferred_sum* defer = nullptr;
    // Per-query-head partial dK/dV of the attention backward at small batch; allocated on first use.
    float* attn_scratch = nullptr;

    // Per-kernel timing with HIP events on the context's stream (off by default).
    struct ProfRecord {
        int key;
        hipEvent_t e0, e1;
        double flops, bytes;
    };
    bool prof_on = false;
    std::vector<std::string> prof_names;
    std::map<std::string, int> prof_keys;
    std::vector<ProfRecord> prof_records;
    std::vector<hipEvent_t> prof_event_pool;
    struct ProfTotal {
        uint64_t launches = 0;
        double ms = 0, flops = 0, bytes = 0;
    };
    std::vector<ProfTotal> prof_totals;
};

// Brackets the launches made during its lifetime with two events when the
// context is profiling; otherwise does nothing.
struct ft_prof_scope {
    ft_context* ctx;
    int index;
    ft_prof_scope(ft_context* c, const char* name, double flops, double bytes);
    ~ft_prof_scope();
};

int ft_set_error(int code, const char* fmt, ...);

// Looks up, once per device, the device address of the fixed scratch array behind
// ft_rms_norm_backward_noalloc (ft_rowops.hip). `device` must be the current device.
int ft_internal_noalloc_init(int device);


#define FT_CHECK_ARG(cond, ...)                                  \
    do {                                                         \
        if (!(cond)) return ft_set_error(FT_ERR_INVALID, __VA_ARGS__); \
    } while (0)

#define FT_HIP(expr)                                                                      \
    do {                                                                                  \
        hipError_t _e = (expr);                                                           \
        if (_e != hipSuccess)                                                             \
            return ft_set_error(FT_ERR_HIP, "%s failed: %s (%s:%d)", #expr,               \
                                hipGetErrorString(_e), __FILE__, __LINE__);               \
    } while (0)

#define FT_TRY(expr)                   \
    do {                               \
        int _rc = (expr);              \
        if (_rc != FT_OK) return _rc;  \
    } while (0)

// Reports a launch-configuration error of the kernel just enqueued.
#define FT_LAUNCH_CHECK() FT_HIP(hipGetLastError())

// A wave-uniform kernel argument fetched once and kept in a register: the empty asm makes the value opaque,
// so the compiler can neither fetch it again from the argument block in front of every use (a scalar load
// and a full wait each time, inside unrolled loops) nor move the fetch into the branches that use it.
// Pointers lose their address space on the way: cast them to ft_global_f (device memory) afterwards so
// that their accesses stay `global_*` instructions.
typedef __attribute__((address_space(1))) float ft_global_f;
template <typename T>
__device__ __forceinline__ T ft_pinned(T v) {
    asm("" : "+s"(v));
    return v;
}

static inline unsigned ft_div_up(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }
