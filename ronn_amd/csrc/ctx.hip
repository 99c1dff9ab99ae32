// Context, device buffers, timers and size rules of the C ABI.
#include <cmath>
#include <cstring>
#include <new>
#include <string>

#include "common.hpp"

namespace {
thread_local std::string g_last_error;

__global__ void fill_u8_kernel(uint8_t *dst, uint8_t value, size_t bytes) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < bytes; i += stride) dst[i] = value;
}
}  // namespace

int rbn_fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

void rbn_clear_error() { g_last_error.clear(); }

int rbn_workspace(rbn_ctx *ctx, size_t bytes, void **out) {
    if (bytes > ctx->ws_bytes) {
        if (ctx->ws) {
            RBN_HIP(hipStreamSynchronize(ctx->stream));
            RBN_HIP(hipFree(ctx->ws));
            ctx->ws = nullptr;
            ctx->ws_bytes = 0;
        }
        size_t want = (size_t)round_up_u64(bytes, 1 << 20);
        hipError_t e = hipMalloc(&ctx->ws, want);
        if (e != hipSuccess) {
            ctx->ws = nullptr;
            return rbn_fail(RBN_ERR_OOM, "workspace allocation of %zu bytes failed: %s", want,
                            hipGetErrorString(e));
        }
        ctx->ws_bytes = want;
    }
    *out = ctx->ws;
    return RBN_OK;
}

int rbn_workspace2(rbn_ctx *ctx, size_t bytes, void **out) {
    if (bytes > ctx->ws2_bytes) {
        if (ctx->ws2) {
            RBN_HIP(hipStreamSynchronize(ctx->stream));
            RBN_HIP(hipFree(ctx->ws2));
            ctx->ws2 = nullptr;
            ctx->ws2_bytes = 0;
        }
        size_t want = (size_t)round_up_u64(bytes, 1 << 20);
        hipError_t e = hipMalloc(&ctx->ws2, want);
        if (e != hipSuccess) {
            ctx->ws2 = nullptr;
            return rbn_fail(RBN_ERR_OOM, "workspace allocation of %zu bytes failed: %s", want,
                            hipGetErrorString(e));
        }
        ctx->ws2_bytes = want;
    }
    *out = ctx->ws2;
    return RBN_OK;
}

int rbn_refuse_while_capturing(rbn_ctx *ctx, const char *what) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
        return rbn_fail(RBN_ERR_INVALID, "%s synchronises the stream and cannot be captured in a graph", what);
    return RBN_OK;
}

extern "C" {

const char *rbn_version(void) { return "ronn-bitnet-hip 0.1 (gfx950)"; }

const char *rbn_last_error(void) { return g_last_error.c_str(); }

int rbn_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int rbn_ctx_create(int device, rbn_ctx **out) {
    rbn_clear_error();
    RBN_REQUIRE(out != nullptr, "out is NULL");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0)
        return rbn_fail(RBN_ERR_NO_DEVICE, "no HIP device visible (%s)",
                        e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    RBN_REQUIRE(device >= 0 && device < n, "device %d out of range [0,%d)", device, n);
    RBN_HIP(hipSetDevice(device));
    rbn_ctx *ctx = new (std::nothrow) rbn_ctx();
    if (!ctx) return rbn_fail(RBN_ERR_OOM, "host allocation failed");
    ctx->device = device;
    e = hipGetDeviceProperties(&ctx->props, device);
    if (e != hipSuccess) {
        delete ctx;
        return rbn_fail(RBN_ERR_HIP, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    }
    if (strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        std::string arch = ctx->props.gcnArchName;
        delete ctx;
        return rbn_fail(RBN_ERR_NO_DEVICE,
                        "device %d is %s; this library carries gfx950 code only", device,
                        arch.c_str());
    }
    // Default priority on purpose: one plain non-blocking stream per context.
    if ((e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev_start)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev_stop)) != hipSuccess ||
        (e = hipHostMalloc(&ctx->mailbox, 4096, hipHostMallocDefault)) != hipSuccess ||
        (e = hipMalloc(&ctx->splitk_partials, (size_t)RBN_SPLITK_TILES * 4096)) != hipSuccess ||
        (e = hipMalloc((void **)&ctx->splitk_tickets, RBN_SPLITK_GROUPS * sizeof(unsigned))) != hipSuccess ||
        (e = hipMemset(ctx->splitk_tickets, 0, RBN_SPLITK_GROUPS * sizeof(unsigned))) != hipSuccess ||
        (e = hipMalloc((void **)&ctx->dev_flags, 256)) != hipSuccess ||
        (e = hipMemset(ctx->dev_flags, 0, 256)) != hipSuccess) {
        int rc = rbn_fail(RBN_ERR_HIP, "context set-up failed: %s", hipGetErrorString(e));
        rbn_ctx_destroy(ctx);
        return rc;
    }
    const int prep = rbn_skinny_prepare(device);
    if (prep != RBN_OK) {
        rbn_ctx_destroy(ctx);
        return prep;
    }
    *out = ctx;
    return RBN_OK;
}

int rbn_ctx_destroy(rbn_ctx *ctx) {
    if (!ctx) return RBN_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    rbn_skinny_release(ctx);
    if (ctx->ws) (void)hipFree(ctx->ws);
    if (ctx->ws2) (void)hipFree(ctx->ws2);
    if (ctx->mailbox) (void)hipHostFree(ctx->mailbox);
    if (ctx->splitk_partials) (void)hipFree(ctx->splitk_partials);
    if (ctx->splitk_tickets) (void)hipFree(ctx->splitk_tickets);
    if (ctx->dev_flags) (void)hipFree(ctx->dev_flags);
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return RBN_OK;
}

int rbn_get_device_info(rbn_ctx *ctx, rbn_device_info *out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(out != nullptr, "out is NULL");
    memset(out, 0, sizeof(*out));
    strncpy(out->name, ctx->props.name, sizeof(out->name) - 1);
    strncpy(out->arch, ctx->props.gcnArchName, sizeof(out->arch) - 1);
    out->compute_units = ctx->props.multiProcessorCount;
    out->clock_khz = ctx->props.clockRate;
    out->mem_clock_khz = ctx->props.memoryClockRate;
    out->mem_bus_bits = ctx->props.memoryBusWidth;
    out->hbm_bytes = ctx->props.totalGlobalMem;
    out->l2_bytes = (uint64_t)ctx->props.l2CacheSize;
    return RBN_OK;
}

int rbn_malloc(rbn_ctx *ctx, size_t bytes, void **d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_out != nullptr, "d_out is NULL");
    *d_out = nullptr;
    size_t want = bytes == 0 ? 256 : (size_t)round_up_u64(bytes, 256);
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess)
        return rbn_fail(RBN_ERR_OOM, "hipMalloc(%zu) failed: %s", want, hipGetErrorString(e));
    ctx->allocated += want;
    if (ctx->allocated > ctx->peak) ctx->peak = ctx->allocated;
    *d_out = p;
    return RBN_OK;
}

int rbn_free(rbn_ctx *ctx, void *d_ptr) {
    RBN_ENTER(ctx);
    if (!d_ptr) return RBN_OK;
    size_t size = 0;
    hipDeviceptr_t base = nullptr;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)d_ptr) == hipSuccess &&
        ctx->allocated >= size)
        ctx->allocated -= size;
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    RBN_HIP(hipFree(d_ptr));
    return RBN_OK;
}

int rbn_h2d(rbn_ctx *ctx, void *d_dst, const void *h_src, size_t bytes) {
    RBN_ENTER(ctx);
    if (bytes == 0) return RBN_OK;
    RBN_REQUIRE(d_dst && h_src, "null pointer in rbn_h2d");
    RBN_HIP(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    return RBN_OK;
}

int rbn_d2h(rbn_ctx *ctx, void *h_dst, const void *d_src, size_t bytes) {
    RBN_ENTER(ctx);
    if (bytes == 0) return RBN_OK;
    RBN_REQUIRE(h_dst && d_src, "null pointer in rbn_d2h");
    RBN_HIP(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    return RBN_OK;
}

int rbn_d2d(rbn_ctx *ctx, void *d_dst, const void *d_src, size_t bytes) {
    RBN_ENTER(ctx);
    if (bytes == 0) return RBN_OK;
    RBN_REQUIRE(d_dst && d_src, "null pointer in rbn_d2d");
    RBN_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return RBN_OK;
}

int rbn_fill_u8(rbn_ctx *ctx, void *d_dst, int value, size_t bytes) {
    RBN_ENTER(ctx);
    if (bytes == 0) return RBN_OK;
    RBN_REQUIRE(d_dst != nullptr, "d_dst is NULL");
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_u8_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((uint8_t *)d_dst,
                                                                         (uint8_t)value, bytes);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_sync(rbn_ctx *ctx) {
    RBN_ENTER(ctx);
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    return RBN_OK;
}

int rbn_device_flags(rbn_ctx *ctx, uint32_t *h_flags) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_flags != nullptr, "h_flags is NULL");
    RBN_CHECK(rbn_refuse_while_capturing(ctx, "rbn_device_flags"));
    unsigned *box = static_cast<unsigned *>(ctx->mailbox) + 512;  // the mailbox's second half
    RBN_HIP(hipMemcpyAsync(box, ctx->dev_flags, sizeof(unsigned), hipMemcpyDeviceToHost, ctx->stream));
    fill_u8_kernel<<<dim3(1), dim3(64), 0, ctx->stream>>>((uint8_t *)ctx->dev_flags, 0, sizeof(unsigned));
    RBN_HIP(hipGetLastError());
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    *h_flags = *box;
    return RBN_OK;
}

int rbn_memory_info(rbn_ctx *ctx, uint64_t *allocated, uint64_t *peak) {
    RBN_ENTER(ctx);
    if (allocated) *allocated = ctx->allocated;
    if (peak) *peak = ctx->peak;
    return RBN_OK;
}

int64_t rbn_tensor_bytes(uint64_t element_count, int dtype) {
    switch (dtype) {
        case 8: return (int64_t)((element_count + 7) / 8);
        case 6: return (int64_t)((element_count + 3) / 4);
        case 0: return (int64_t)(element_count * 4);
        case 1:
        case 2: return (int64_t)(element_count * 2);
        default: return -1;
    }
}

size_t rbn_tensor_alignment(int dtype) {
    switch (dtype) {
        case 8:
        case 6:
        case 0: return 32;
        case 1:
        case 2: return 16;
        default: return 8;
    }
}

size_t rbn_packed_capacity(uint64_t n) { return (size_t)round_up_u64((n + 3) / 4, 16) + 16; }

size_t rbn_tiled_bytes(uint64_t K, uint64_t N) {
    return (size_t)(rbn_kpad(K) / 16 * rbn_npad(N) * 4);
}

size_t rbn_act_pitch(uint64_t K) { return (size_t)rbn_kpad(K); }

int rbn_timer_start(rbn_ctx *ctx) {
    RBN_ENTER(ctx);
    RBN_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
    return RBN_OK;
}

int rbn_timer_stop(rbn_ctx *ctx, float *h_ms) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_ms != nullptr, "h_ms is NULL");
    RBN_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
    RBN_HIP(hipEventSynchronize(ctx->ev_stop));
    RBN_HIP(hipEventElapsedTime(h_ms, ctx->ev_start, ctx->ev_stop));
    return RBN_OK;
}

// ---- HIP graphs -----------------------------------------------------------------
struct rbn_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

int rbn_graph_begin_capture(rbn_ctx *ctx) {
    RBN_ENTER(ctx);
    RBN_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    return RBN_OK;
}

int rbn_graph_end_capture(rbn_ctx *ctx, rbn_graph **out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(out != nullptr, "out is NULL");
    *out = nullptr;
    hipGraph_t g = nullptr;
    RBN_HIP(hipStreamEndCapture(ctx->stream, &g));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return rbn_fail(RBN_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    // Resources of the executable graph go to the device now, not inside its first launch
    // (a launch-bound sequence would otherwise see one slow first replay).  Best effort.
    (void)hipGraphUpload(exec, ctx->stream);
    (void)hipGetLastError();
    rbn_graph *r = new (std::nothrow) rbn_graph();
    if (!r) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(g);
        return rbn_fail(RBN_ERR_OOM, "host allocation failed");
    }
    r->graph = g;
    r->exec = exec;
    *out = r;
    return RBN_OK;
}

int rbn_graph_launch(rbn_ctx *ctx, rbn_graph *graph) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(graph && graph->exec, "graph is NULL");
    RBN_HIP(hipGraphLaunch(graph->exec, ctx->stream));
    return RBN_OK;
}

int rbn_graph_destroy(rbn_ctx *ctx, rbn_graph *graph) {
    RBN_ENTER(ctx);
    if (!graph) return RBN_OK;
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
    return RBN_OK;
}

// ---- synthetic inputs ---------------------------------------------------------
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t index) {
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void rbn_synth_normal_f32(uint64_t seed, double sigma, uint64_t first, uint64_t count,
                          float *h_out) {
    // Pair p yields elements 2p and 2p+1 (the cosine and sine branches of Box-Muller).
    const double two_pi = 6.283185307179586476925286766559;
    uint64_t i = first, end = first + count;
    while (i < end) {
        uint64_t pair = i >> 1;
        uint64_t bits = splitmix64_at(seed, pair);
        double u1 = ((double)((bits >> 40) & 0xffffffull) + 1.0) * (1.0 / 16777216.0);  // (0,1]
        double u2 = (double)((bits >> 8) & 0xffffffull) * (1.0 / 16777216.0);           // [0,1)
        double r = sqrt(-2.0 * log(u1));
        double a = two_pi * u2;
        if ((i & 1) == 0) {
            h_out[i - first] = (float)(sigma * (r * cos(a)));
            ++i;
            if (i < end) {
                h_out[i - first] = (float)(sigma * (r * sin(a)));
                ++i;
            }
        } else {
            h_out[i - first] = (float)(sigma * (r * sin(a)));
            ++i;
        }
    }
}

}  // extern "C"
