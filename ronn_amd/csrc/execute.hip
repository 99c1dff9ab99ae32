// CompiledKernel::execute, TernaryMatMul arm
// (crates/ronn-providers/src/bitnet/kernels.rs:271-283): host tensors in, both
// operands ternarised per tensor on every call, ternary matmul, host tensor out.
#include <vector>

#include "common.hpp"

namespace {
// Frees every device pointer it was given when it goes out of scope.
struct DeviceScope {
    rbn_ctx *ctx;
    std::vector<void *> ptrs;
    explicit DeviceScope(rbn_ctx *c) : ctx(c) {}
    ~DeviceScope() {
        (void)hipStreamSynchronize(ctx->stream);
        for (void *p : ptrs) (void)hipFree(p);
    }
    int alloc(size_t bytes, void **out) {
        hipError_t e = hipMalloc(out, bytes == 0 ? 256 : bytes);
        if (e != hipSuccess) {
            *out = nullptr;
            return rbn_fail(RBN_ERR_OOM, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        }
        ptrs.push_back(*out);
        return RBN_OK;
    }
};
}  // namespace

extern "C" int rbn_execute_ternary_matmul(rbn_ctx *ctx, const float *h_a, const float *h_b,
                                          uint64_t M, uint64_t N, uint64_t K, int mode,
                                          float *h_out, int32_t *h_acc) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_a && h_b && h_out, "null pointer in rbn_execute_ternary_matmul");
    RBN_REQUIRE(M > 0 && N > 0 && K > 0, "M, N and K must be positive");
    RBN_CHECK(rbn_refuse_while_capturing(ctx, "rbn_execute_ternary_matmul"));
    DeviceScope scope(ctx);
    float *d_a = nullptr, *d_b = nullptr, *d_out = nullptr, *d_as = nullptr;
    int8_t *d_q = nullptr;
    int32_t *d_rs = nullptr, *d_acc = nullptr;
    uint8_t *d_bp = nullptr;
    uint32_t *d_bt = nullptr;
    RBN_CHECK(scope.alloc(M * K * 4, (void **)&d_a));
    RBN_CHECK(scope.alloc(K * N * 4, (void **)&d_b));
    RBN_CHECK(scope.alloc(M * rbn_act_pitch(K), (void **)&d_q));
    RBN_CHECK(scope.alloc(M * 4, (void **)&d_as));
    RBN_CHECK(scope.alloc(M * 4, (void **)&d_rs));
    RBN_CHECK(scope.alloc(rbn_packed_capacity(K * N), (void **)&d_bp));
    RBN_CHECK(scope.alloc(rbn_tiled_bytes(K, N), (void **)&d_bt));
    RBN_CHECK(scope.alloc(M * N * 4, (void **)&d_out));
    if (h_acc) RBN_CHECK(scope.alloc(M * N * 4, (void **)&d_acc));
    RBN_CHECK(rbn_h2d(ctx, d_a, h_a, M * K * 4));
    RBN_CHECK(rbn_h2d(ctx, d_b, h_b, K * N * 4));
    // kernels.rs:277-278
    float a_scale, a_thr, b_scale, b_thr;
    RBN_CHECK(rbn_act_quant_ternary(ctx, d_a, M, K, mode, d_q, d_as, d_rs, &a_scale, &a_thr));
    RBN_CHECK(rbn_quantize_ternary(ctx, d_b, K * N, mode, d_bp, &b_scale, &b_thr, nullptr));
    RBN_CHECK(rbn_tile_weights(ctx, d_bp, K, N, d_bt));
    // kernels.rs:280-281
    RBN_CHECK(rbn_matmul_t2_i8(ctx, d_q, d_as, d_rs, d_bt, b_scale, M, K, N, d_acc, d_out));
    RBN_CHECK(rbn_d2h(ctx, h_out, d_out, M * N * 4));
    if (h_acc) RBN_CHECK(rbn_d2h(ctx, h_acc, d_acc, M * N * 4));
    return RBN_OK;
}
