/*
 * CPU oracle for the BitNet ternary path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, statement by statement, the scalar CPU algorithm of the
 * reference's BitNet provider so that the HIP kernels can be checked against it.
 * Nothing in the shipped library links, loads or calls it; only the test-suite,
 * the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Reference functions restated (paths relative to the reference checkout,
 * crates/ronn-providers/src/bitnet/):
 *   orc_quantize_ternary      quantization.rs:67-109   BitNetQuantizer::quantize_ternary
 *   orc_pack_ternary_bits     quantization.rs:131-153  pack_ternary_bits
 *   orc_get_value             quantization.rs:275-291  TernaryTensor::get_value
 *   orc_dequantize_ternary    quantization.rs:182-207  dequantize_ternary
 *   orc_ternary_matmul        kernels.rs:134-178       execute_ternary_matmul
 *   orc_execute_ternary       kernels.rs:271-283       CompiledKernel::execute, TernaryMatMul arm
 *   orc_packed_size / orc_alignment  allocator.rs:39-75
 *
 * Rust semantics that matter and how they are kept:
 *   - `iter().sum::<f32>()` is a strict left fold in f32.  The loops below are
 *     plain sequential `s = s + x` in `float`; build with -O2 -ffp-contract=off
 *     and without -ffast-math so the compiler may not reassociate or vectorise.
 *   - `usize as f32` rounds to nearest even: C's (float)(uint64_t) does the same.
 *   - `0.7` in an f32 expression is the f32 literal 0.7f.
 *   - `f32::abs` clears the sign bit (NaN stays NaN): fabsf.
 *   - comparisons with NaN are false, so a NaN weight packs as 0b00 (-1).
 *
 * Parity status.  The ternary functions above are pinned by the reference's own
 * known-answer test (quantization.rs:348-361), by hand-derived vectors for the
 * inputs its other tests use (quantization.rs:316, kernels.rs:388-389), by
 * closed forms and by brute force on tiny inputs (tests/test_oracle.py).
 * The int8 functions at the end (orc_act_quant_i8, orc_matmul_i8_ternary) have
 * NO counterpart in the reference: PARITY UNPINNED against the reference; they
 * are pinned only by closed forms and an exact integer library cross-check.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- quantization.rs:131-153 -------------------------------------------- */
/* `scale` is accepted and ignored, as in the reference signature. */
void orc_pack_ternary_bits(const float *data, size_t element_count, float threshold,
                           float scale, uint8_t *packed /* ceil(n/4) bytes */)
{
    (void)scale;
    const size_t bit_pairs_per_byte = 4;
    size_t byte_count = (element_count + bit_pairs_per_byte - 1) / bit_pairs_per_byte;
    memset(packed, 0, byte_count);
    for (size_t i = 0; i < element_count; i++) {
        float value = data[i];
        uint8_t quantized;
        if (fabsf(value) <= threshold) {
            quantized = 0x1; /* zero -> 01 */
        } else if (value > 0.0f) {
            quantized = 0x2; /* +1 -> 10 */
        } else {
            quantized = 0x0; /* -1 -> 00 */
        }
        size_t byte_idx = i / bit_pairs_per_byte;
        unsigned bit_offset = (unsigned)(i % bit_pairs_per_byte) * 2u;
        packed[byte_idx] |= (uint8_t)(quantized << bit_offset);
    }
}

/* ---- quantization.rs:67-109 --------------------------------------------- */
/* Returns the number of survivors (|x| > threshold) for the caller's interest. */
uint64_t orc_quantize_ternary(const float *data, size_t total_elements, uint8_t *packed,
                              float *out_scale, float *out_threshold)
{
    /* :79  data.iter().map(|x| x.abs()).sum::<f32>() / total_elements as f32 * 0.7 */
    float sum = -0.0f; /* Rust's float Sum starts from -0.0; immaterial unless n == 0 */
    for (size_t i = 0; i < total_elements; i++) {
        sum = sum + fabsf(data[i]);
    }
    float threshold = sum / (float)(uint64_t)total_elements * 0.7f;

    /* :82-97  survivors in index order, then their sequential f32 mean */
    float nz_sum = -0.0f;
    uint64_t nz_count = 0;
    for (size_t i = 0; i < total_elements; i++) {
        float a = fabsf(data[i]);
        if (a > threshold) {
            nz_sum = nz_sum + a;
            nz_count++;
        }
    }
    float scale = (nz_count == 0) ? 1.0f : nz_sum / (float)nz_count;

    orc_pack_ternary_bits(data, total_elements, threshold, scale, packed);
    *out_scale = scale;
    *out_threshold = threshold;
    return nz_count;
}

/* ---- quantization.rs:275-291 -------------------------------------------- */
int8_t orc_get_value(const uint8_t *packed, size_t element_count, size_t index)
{
    if (index >= element_count) {
        return 0;
    }
    const size_t bit_pairs_per_byte = 4;
    size_t byte_idx = index / bit_pairs_per_byte;
    unsigned bit_offset = (unsigned)(index % bit_pairs_per_byte) * 2u;
    unsigned bit_pair = (packed[byte_idx] >> bit_offset) & 0x3u;
    switch (bit_pair) {
    case 0x0: return -1;
    case 0x1: return 0;
    case 0x2: return 1;
    default:  return 0; /* invalid, default to zero */
    }
}

/* ---- quantization.rs:182-207 -------------------------------------------- */
void orc_dequantize_ternary(const uint8_t *packed, size_t element_count, float scale, float *out)
{
    const size_t bit_pairs_per_byte = 4;
    for (size_t i = 0; i < element_count; i++) {
        size_t byte_idx = i / bit_pairs_per_byte;
        unsigned bit_offset = (unsigned)(i % bit_pairs_per_byte) * 2u;
        unsigned bit_pair = (packed[byte_idx] >> bit_offset) & 0x3u;
        float v;
        switch (bit_pair) {
        case 0x0: v = -scale; break;
        case 0x1: v = 0.0f; break;
        case 0x2: v = scale; break;
        default:  v = 0.0f; break;
        }
        out[i] = v;
    }
}

/* ---- kernels.rs:134-178 -------------------------------------------------- */
/* a: [m,k] ternary, b: [k,n] ternary, both flat row-major 2-bit packed.
 * The shape check of :142-152 is done by the caller on the host mirror; here the
 * element counts are m*k and k*n by construction.  `acc` (optional) receives the
 * int32 dot products before scaling. */
void orc_ternary_matmul(const uint8_t *a_packed, float a_scale, const uint8_t *b_packed,
                        float b_scale, size_t m, size_t n, size_t k, float *result,
                        int32_t *acc /* may be NULL */)
{
    size_t a_count = m * k, b_count = k * n;
    for (size_t i = 0; i < m; i++) {
        for (size_t j = 0; j < n; j++) {
            int32_t dot_product = 0;
            for (size_t l = 0; l < k; l++) {
                int32_t a_val = (int32_t)orc_get_value(a_packed, a_count, i * k + l);
                int32_t b_val = (int32_t)orc_get_value(b_packed, b_count, l * n + j);
                dot_product += a_val * b_val;
            }
            /* :168  dot_product as f32 * a.scale * b.scale, left to right */
            float r = (float)dot_product * a_scale;
            r = r * b_scale;
            result[i * n + j] = r;
            if (acc) acc[i * n + j] = dot_product;
        }
    }
}

/* ---- kernels.rs:271-283 -------------------------------------------------- */
/* Full execute() of the TernaryMatMul arm: both operands are ternarised, per
 * tensor, on every call, then multiplied.  Returns 0, or -1 on allocation failure. */
int orc_execute_ternary(const float *a, const float *b, size_t m, size_t n, size_t k,
                        float *result, int32_t *acc /* may be NULL */)
{
    size_t a_count = m * k, b_count = k * n;
    uint8_t *ap = (uint8_t *)malloc((a_count + 3) / 4 + 1);
    uint8_t *bp = (uint8_t *)malloc((b_count + 3) / 4 + 1);
    if (!ap || !bp) { free(ap); free(bp); return -1; }
    float a_scale, a_thr, b_scale, b_thr;
    orc_quantize_ternary(a, a_count, ap, &a_scale, &a_thr);
    orc_quantize_ternary(b, b_count, bp, &b_scale, &b_thr);
    orc_ternary_matmul(ap, a_scale, bp, b_scale, m, n, k, result, acc);
    free(ap);
    free(bp);
    return 0;
}

/* ---- allocator.rs:39-75 --------------------------------------------------- */
/* dtype codes: 0=F32 1=F16 2=BF16 6=U8 (2-bit ternary) 8=Bool (1-bit binary);
 * the numbering follows the declaration order of DataType, ronn-core types.rs:39-60.
 * Returns -1 for a dtype the allocator rejects (:60-63). */
int64_t orc_packed_size(const size_t *shape, size_t ndim, int dtype)
{
    size_t element_count = 1;
    for (size_t i = 0; i < ndim; i++) element_count *= shape[i];
    switch (dtype) {
    case 8: return (int64_t)((element_count + 7) / 8);
    case 6: return (int64_t)((element_count + 3) / 4);
    case 0: return (int64_t)(element_count * 4);
    case 1: case 2: return (int64_t)(element_count * 2);
    default: return -1;
    }
}

size_t orc_alignment(int dtype)
{
    switch (dtype) {
    case 8: case 6: return 32;
    case 0: return 32;
    case 1: case 2: return 16;
    default: return 8;
    }
}

/* =========================================================================
 * Build-defined int8 activation path.  NO REFERENCE COUNTERPART: the reference
 * ternarises activations with quantize_ternary (kernels.rs:277).  PARITY
 * UNPINNED against the reference.  Definition (one row = one token):
 *   amax  = max_k |x[k]|            (NaN-free input assumed; fmaxf ignores NaN)
 *   g     = max(amax, 1e-5f)
 *   inv   = 127.0f / g
 *   q[k]  = clamp(round_half_even(x[k] * inv), -128, 127)
 *   scale = g / 127.0f
 *   rowsum = sum_k q[k]             (int32)
 * ========================================================================= */
void orc_act_quant_i8(const float *x, size_t m, size_t k, int8_t *q, float *scale,
                      int32_t *rowsum)
{
    for (size_t i = 0; i < m; i++) {
        const float *row = x + i * k;
        float amax = 0.0f;
        for (size_t l = 0; l < k; l++) amax = fmaxf(amax, fabsf(row[l]));
        float g = fmaxf(amax, 1e-5f);
        float inv = 127.0f / g;
        int32_t s = 0;
        for (size_t l = 0; l < k; l++) {
            float v = nearbyintf(row[l] * inv); /* default rounding mode: half to even */
            v = fminf(fmaxf(v, -128.0f), 127.0f);
            int8_t qi = (int8_t)v;
            q[i * k + l] = qi;
            s += qi;
        }
        scale[i] = g / 127.0f;
        if (rowsum) rowsum[i] = s;
    }
}

/* int8 activations x ternary weights with the reference's inner loop
 * (get_value on the weight side, kernels.rs:161-165) and the reference's
 * epilogue order (kernels.rs:168), with act_scale per row in place of a.scale. */
void orc_matmul_i8_ternary(const int8_t *q, const float *act_scale, const uint8_t *b_packed,
                           float b_scale, size_t m, size_t n, size_t k, float *result,
                           int32_t *acc /* may be NULL */)
{
    size_t b_count = k * n;
    for (size_t i = 0; i < m; i++) {
        for (size_t j = 0; j < n; j++) {
            int32_t dot_product = 0;
            for (size_t l = 0; l < k; l++) {
                int32_t a_val = (int32_t)q[i * k + l];
                int32_t b_val = (int32_t)orc_get_value(b_packed, b_count, l * n + j);
                dot_product += a_val * b_val;
            }
            float r = (float)dot_product * act_scale[i];
            r = r * b_scale;
            result[i * n + j] = r;
            if (acc) acc[i * n + j] = dot_product;
        }
    }
}

/* Ternary activations as int8 {-1,0,+1}: what quantize_ternary + get_value give
 * for the activation operand (kernels.rs:162, 277), unpacked for the device path. */
void orc_unpack_values(const uint8_t *packed, size_t element_count, int8_t *out)
{
    for (size_t i = 0; i < element_count; i++) out[i] = orc_get_value(packed, element_count, i);
}
