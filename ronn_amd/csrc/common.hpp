// Internal declarations shared by the translation units of libronn_bitnet_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "../../include/ronn_bitnet_hip.h"

struct rbn_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr;
    hipEvent_t ev_stop = nullptr;
    hipDeviceProp_t props{};
    std::recursive_mutex lock;
    uint64_t allocated = 0;
    uint64_t peak = 0;
    // Small device workspace owned by the context (reductions, sequential-sum
    // state); grown on demand by rbn_workspace().
    void *ws = nullptr;
    size_t ws_bytes = 0;
    // Second grow-only buffer: the packed image of the activations in rbn_act_quant_ternary
    // (ws is in use by the sums at the same time).
    void *ws2 = nullptr;
    size_t ws2_bytes = 0;
    // Pinned host mailbox for the few scalars that come back from the device.
    void *mailbox = nullptr;
    // Split-k workspace of the matmuls: RBN_SPLITK_TILES partial tiles of 16 x 64 int32
    // (the prefill kernel takes sixteen of them per 64 x 256 partial) and one ticket counter
    // per output tile.  Allocated once with the
    // context and never moved, so launches captured in a HIP graph stay valid.
    void *splitk_partials = nullptr;
    unsigned *splitk_tickets = nullptr;
    // One word of RBN_FLAG_* bits that kernels set when they refuse to do something a host
    // check could not see coming (rbn_device_flags reads and clears it).
    unsigned *dev_flags = nullptr;
    // the window-end kernel of the exact sums has been given its dynamic-LDS limit on this device
    bool seq_scan_prepared = false;
    // the size (in blocks of the exact sums) of the last tensor summed and the windows its sums took
    uint64_t seq_seen_blocks = 0;
    int seq_seen_windows = 0;
};

constexpr int RBN_SPLITK_TILES = 16384;  // 64 MiB
constexpr int RBN_SPLITK_GROUPS = 1024;

// Records `fmt...` as the calling thread's last error and returns `code`.
int rbn_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void rbn_clear_error();

// Per-device set-up of the small-batch kernels (dynamic-LDS limit, address of their static
// scratch array); called with `device` current.
int rbn_skinny_prepare(int device);
// gives up the context's claim on its GPU's static scratch array (rbn_ctx_destroy)
void rbn_skinny_release(const rbn_ctx *ctx);

// Ensures ctx->ws has at least `bytes` bytes; returns it through *out.
int rbn_workspace(rbn_ctx *ctx, size_t bytes, void **out);
// The same for ctx->ws2.
int rbn_workspace2(rbn_ctx *ctx, size_t bytes, void **out);
// RBN_ERR_INVALID with a message naming `what` when the context's stream is being captured
// (for entry points that synchronise, allocate or return scalars to the host).
int rbn_refuse_while_capturing(rbn_ctx *ctx, const char *what);

#define RBN_HIP(expr)                                                                      \
    do {                                                                                   \
        hipError_t _e = (expr);                                                            \
        if (_e != hipSuccess)                                                              \
            return rbn_fail(RBN_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                   \
                            hipGetErrorString(_e), __FILE__, __LINE__);                    \
    } while (0)

#define RBN_REQUIRE(cond, ...)                                                             \
    do {                                                                                   \
        if (!(cond)) return rbn_fail(RBN_ERR_INVALID, __VA_ARGS__);                        \
    } while (0)

#define RBN_CHECK(expr)                                                                    \
    do {                                                                                   \
        int _rc = (expr);                                                                  \
        if (_rc != RBN_OK) return _rc;                                                     \
    } while (0)

// Locks the context and makes its device current for the calling thread.
struct CtxGuard {
    std::unique_lock<std::recursive_mutex> lk;
    int rc;
    explicit CtxGuard(rbn_ctx *ctx) : lk(), rc(RBN_OK) {
        if (!ctx) {
            rc = rbn_fail(RBN_ERR_INVALID, "context is NULL");
            return;
        }
        lk = std::unique_lock<std::recursive_mutex>(ctx->lock);
        hipError_t e = hipSetDevice(ctx->device);
        if (e != hipSuccess)
            rc = rbn_fail(RBN_ERR_HIP, "hipSetDevice(%d) failed: %s", ctx->device,
                          hipGetErrorString(e));
    }
};

#define RBN_ENTER(ctx)      \
    rbn_clear_error();      \
    CtxGuard _guard(ctx);   \
    if (_guard.rc != RBN_OK) return _guard.rc

static inline uint64_t round_up_u64(uint64_t v, uint64_t m) { return (v + m - 1) / m * m; }

// Layout helpers (see the header for the formats).
static inline uint64_t rbn_kpad(uint64_t K) { return round_up_u64(K, 128); }
static inline uint64_t rbn_npad(uint64_t N) { return round_up_u64(N, 64); }
