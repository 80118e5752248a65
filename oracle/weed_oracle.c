/*
 * weed_oracle.c -- CPU restatement of vm6502q/weed's quantized-KV attention path.
 *
 * TEST INFRASTRUCTURE ONLY (see weed_oracle.h).  Plain C, scalar, one thread: at every decode
 * configuration the reference's own work splitter runs on one core too, because it starts
 * min(cores, items / 2^18) workers (src/common/parallel_for.cpp:93-106).
 *
 * What pins each function (tests/test_oracle_*.py):
 *   wo_uniform_write_row / read_row / codes : known answers recorded from the reference's own build
 *       (words 0x00ffea40, 0x3ff24600 0x0000003f, 0xe8887000 0x0000ffff, 0x00007f39 and the four
 *       dequantised floats), plus brute-force interval checks.
 *   wo_matmul, wo_softmax, wo_reduce        : the reference's unit tests (test/tests.cpp:177-228,
 *       1020-1041, 1110-1171, 1206-1221) and float64 numpy closed forms.
 *   wo_triu_fill                            : brute force against the rule i + diag <= j.
 *   wo_rope_tables / wo_rope_forward        : the reference has no test of RoPE -- PARITY UNPINNED against
 *       the reference; pinned by float64 closed forms of the tables, the identity at position 0 and the
 *       per-coordinate formula evaluated independently in numpy.
 *   wo_unary, wo_silu_mul                   : the reference's unit tests (test/tests.cpp:230-244, 284-291,
 *       314-321: relu(2) = 2, relu(-2) = 0, sigmoid(0) = 0.5, tanh(0) = 0) and float64 closed forms of every
 *       function; gelu additionally against erf-free float64 evaluation of the same tanh formula.
 *   wo_rms_norm, wo_layer_norm              : the reference has no test of either module -- PARITY UNPINNED
 *       against the reference; pinned by float64 closed forms, by what the mathematics fixes (unit mean square /
 *       zero mean and unit variance of the result before the affine step, scale invariance, a constant row) and by
 *       the reference's test of the axis mean they are built from (test/tests.cpp:111-120: mean(1, 2, 3) = 2).
 *   wo_block_scale                          : float64 closed form (order-dependent in the last ulps).
 *   wo_orthonormalize_columns, wo_apply_rotation : invariants only (R^T R = I, y = x R, R R^T = I);
 *       the reference draws its Gaussian matrix from std::random_device, so no vector exists.
 *   wo_encode_row / wo_decode_row (mode 1), wo_decode_attn : the reference has no such code and no
 *       test of attention at all -- PARITY UNPINNED against the reference; pinned by brute-force
 *       nearest-centroid search, textbook Lloyd-Max tables, and a float64 dense attention.
 */
#include "weed_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* Weed's uniform coder                                                                        */
/* ------------------------------------------------------------------------------------------ */

/* include/modules/multihead_attention.hpp:31 -- values_per_word = 32 / bits */
int wo_values_per_word(int bits) { return (int)(sizeof(int32_t) * 8) / bits; }

/* src/modules/multihead_attention.cpp:38-39 */
int wo_words_per_row(int d, int bits)
{
    const int vpw = wo_values_per_word(bits);
    return (d + vpw - 1) / vpw;
}

/* src/modules/multihead_attention.cpp:49-58: the bucket arithmetic of write_row */
static int uniform_bucket(float v, float lo, float hi, float step, int levels)
{
    int bucket = 0;
    if (step > 1e-8f) {
        const float hs = hi - step;
        const float m = (v < hs) ? v : hs;       /* std::min(hi - step, v) */
        const float clamped = (lo < m) ? m : lo; /* std::max(lo, .) */
        bucket = (int)((clamped - lo) / step);
        if (bucket > levels - 1) {
            bucket = levels - 1;
        }
        if (bucket < 0) {
            bucket = 0;
        }
    }
    return bucket;
}

/* src/modules/multihead_attention.cpp:43-62.  ORs into the word, as the reference does. */
void wo_uniform_write_row(int32_t *packed, uint32_t row, const float *vals, int d, int bits, float block_scale)
{
    const int vpw = wo_values_per_word(bits);
    const int levels = 1 << bits;
    const uint32_t wpr = (uint32_t)wo_words_per_row(d, bits);
    const uint32_t base = row * wpr;
    const float lo = -3.0f * block_scale;
    const float hi = 3.0f * block_scale;
    const float step = (hi - lo) / (float)levels;
    for (int j = 0; j < d; ++j) {
        const int bucket = uniform_bucket(vals[j], lo, hi, step, levels);
        const uint32_t word_idx = base + (uint32_t)(j / vpw);
        const int bit_offset = (j % vpw) * bits;
        packed[word_idx] = (int32_t)((uint32_t)packed[word_idx] | ((uint32_t)bucket << bit_offset));
    }
}

void wo_uniform_codes(const float *vals, int d, int bits, float block_scale, uint8_t *codes)
{
    const int levels = 1 << bits;
    const float lo = -3.0f * block_scale;
    const float hi = 3.0f * block_scale;
    const float step = (hi - lo) / (float)levels;
    for (int j = 0; j < d; ++j) {
        codes[j] = (uint8_t)uniform_bucket(vals[j], lo, hi, step, levels);
    }
}

/* src/modules/multihead_attention.cpp:64-79 */
void wo_uniform_read_row(const int32_t *packed, uint32_t row, float *vals, int d, int bits, float block_scale)
{
    const int vpw = wo_values_per_word(bits);
    const int levels = 1 << bits;
    const int mask = levels - 1;
    const uint32_t wpr = (uint32_t)wo_words_per_row(d, bits);
    const uint32_t base = row * wpr;
    const float lo = -3.0f * block_scale;
    const float hi = 3.0f * block_scale;
    const float step = (hi - lo) / (float)levels;
    for (int j = 0; j < d; ++j) {
        const uint32_t word_idx = base + (uint32_t)(j / vpw);
        const int bit_offset = (j % vpw) * bits;
        const int bucket = (int)((packed[word_idx] >> bit_offset) & mask);
        vals[j] = lo + ((float)bucket + 0.5f) * step;
    }
}

/* src/modules/multihead_attention.cpp:226-241 */
float wo_block_scale(const float *x, size_t n)
{
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        sum += x[i] * x[i];
    }
    return sqrtf(sum / (float)n + 1e-8f);
}

/* ------------------------------------------------------------------------------------------ */
/* rotation                                                                                    */
/* ------------------------------------------------------------------------------------------ */

/* src/modules/multihead_attention.cpp:94-118: normalise column j, then remove its projection from every
 * later column; column j starts at R[j*d]. */
void wo_orthonormalize_columns(float *R, int d)
{
    for (int j = 0; j < d; ++j) {
        float norm = 0.0f;
        for (int i = 0; i < d; ++i) {
            norm += R[j * d + i] * R[j * d + i];
        }
        norm = sqrtf(norm);
        if (norm < 1e-8f) {
            norm = 1e-8f;
        }
        for (int i = 0; i < d; ++i) {
            R[j * d + i] /= norm;
        }
        for (int k = j + 1; k < d; ++k) {
            float dot = 0.0f;
            for (int i = 0; i < d; ++i) {
                dot += R[j * d + i] * R[k * d + i];
            }
            for (int i = 0; i < d; ++i) {
                R[k * d + i] -= dot * R[j * d + i];
            }
        }
    }
}

/* src/modules/multihead_attention.cpp:125-140 -> Tensor::matmul -> src/ops/matmul.cpp:34-47 */
void wo_apply_rotation(const float *x, size_t rows, int d, const float *R, float *y)
{
    for (size_t r = 0; r < rows; ++r) {
        for (int j = 0; j < d; ++j) {
            float sum = 0.0f;
            for (int i = 0; i < d; ++i) {
                sum += x[r * (size_t)d + i] * R[i + d * j];
            }
            y[r * (size_t)d + j] = sum;
        }
    }
}

/* src/modules/multihead_attention.cpp:181-186 */
void wo_transpose_square(const float *R, int d, float *Rt)
{
    for (int i = 0; i < d; ++i) {
        for (int j = 0; j < d; ++j) {
            Rt[i * d + j] = R[j * d + i];
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* table-driven coder                                                                          */
/* ------------------------------------------------------------------------------------------ */

/* Mode 0 follows write_row (cpp:43-62).  Mode 1 has no counterpart in the reference:
 *   n2 = fma-accumulated sum of squares, j ascending;  norm = sqrt(n2);
 *   inv = sqrt(d) / norm, alpha = norm / sqrt(d) (both 0 when norm <= 1e-30);
 *   u_j = y_j * inv;  code_j = #{k : u_j >= bounds[k]};  sign_j = (u_j >= levels[code_j]). */
void wo_encode_row(const wo_coder *c, const float *y, uint8_t *fields, float *alpha)
{
    if (c->mode == 0) {
        wo_uniform_codes(y, c->d, c->bits, c->block_scale, fields);
        return;
    }
    float n2 = 0.0f;
    for (int j = 0; j < c->d; ++j) {
        n2 = fmaf(y[j], y[j], n2);
    }
    const float norm = sqrtf(n2);
    const float sqrt_d = sqrtf((float)c->d);
    float inv = 0.0f, a = 0.0f;
    if (norm > 1e-30f) {
        inv = sqrt_d / norm;
        a = norm / sqrt_d;
    }
    *alpha = a;
    const int nb = (1 << c->bits) - 1;
    for (int j = 0; j < c->d; ++j) {
        const float u = y[j] * inv;
        int code = 0;
        for (int k = 0; k < nb; ++k) {
            code += (u >= c->bounds[k]) ? 1 : 0;
        }
        if (c->sign) {
            const int s = (u >= c->levels[code]) ? 1 : 0;
            fields[j] = (uint8_t)((code << 1) | s);
        } else {
            fields[j] = (uint8_t)code;
        }
    }
}

/* Mode 0 follows read_row (cpp:64-79); mode 1: yhat_j = alpha * recon[field_j]. */
void wo_decode_row(const wo_coder *c, const uint8_t *fields, float alpha, float *yhat)
{
    if (c->mode == 0) {
        const int levels = 1 << c->bits;
        const float lo = -3.0f * c->block_scale;
        const float hi = 3.0f * c->block_scale;
        const float step = (hi - lo) / (float)levels;
        for (int j = 0; j < c->d; ++j) {
            yhat[j] = lo + ((float)fields[j] + 0.5f) * step;
        }
        return;
    }
    for (int j = 0; j < c->d; ++j) {
        yhat[j] = alpha * c->recon[fields[j]];
    }
}

/* Batched forms (plain loops over the row functions). */
void wo_encode_rows(const wo_coder *c, const float *y, size_t rows, uint8_t *fields, float *alpha)
{
    for (size_t r = 0; r < rows; ++r) {
        wo_encode_row(c, y + r * (size_t)c->d, fields + r * (size_t)c->d, alpha + r);
    }
}

void wo_decode_rows(const wo_coder *c, const uint8_t *fields, const float *alpha, size_t rows, float *yhat)
{
    for (size_t r = 0; r < rows; ++r) {
        wo_decode_row(c, fields + r * (size_t)c->d, alpha ? alpha[r] : 0.0f, yhat + r * (size_t)c->d);
    }
}

void wo_uniform_write_rows(int32_t *packed, const float *vals, size_t rows, int d, int bits, float block_scale)
{
    for (size_t r = 0; r < rows; ++r) {
        wo_uniform_write_row(packed, (uint32_t)r, vals + r * (size_t)d, d, bits, block_scale);
    }
}

void wo_uniform_read_rows(const int32_t *packed, float *vals, size_t rows, int d, int bits, float block_scale)
{
    for (size_t r = 0; r < rows; ++r) {
        wo_uniform_read_row(packed, (uint32_t)r, vals + r * (size_t)d, d, bits, block_scale);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* dense ops                                                                                   */
/* ------------------------------------------------------------------------------------------ */

/* src/ops/matmul.cpp:34-47: one output per (i, j), k-ascending accumulation in fp32. */
void wo_matmul(uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t a_o, uint32_t a_s0, uint32_t a_s1,
               const float *B, uint32_t b_o, uint32_t b_s0, uint32_t b_s1, float *C, uint32_t c_o, uint32_t c_s0,
               uint32_t c_s1)
{
    for (uint32_t i = 0; i < M; ++i) {
        for (uint32_t j = 0; j < N; ++j) {
            float sum = 0.0f;
            for (uint32_t k = 0; k < K; ++k) {
                sum += A[a_o + i * a_s0 + k * a_s1] * B[b_o + k * b_s0 + j * b_s1];
            }
            C[c_o + i * c_s0 + j * c_s1] = sum;
        }
    }
}

/* Offset of outer index o into a strided tensor, skipping `axis`; the last dimension is the fastest
 * digit of o (src/ops/softmax.cpp:23-45, src/ops/reduce.cpp:17-31). */
static uint32_t outer_base(int rank, const uint32_t *shape, const uint32_t *stride, int axis, uint32_t o)
{
    uint32_t base = 0;
    uint32_t tmp = o;
    for (int dd = rank - 1; dd >= 0; --dd) {
        if (dd == axis) {
            continue;
        }
        const uint32_t dim = shape[dd];
        const uint32_t i_d = tmp % dim;
        tmp /= dim;
        base += i_d * stride[dd];
    }
    return base;
}

/* src/ops/softmax.cpp:82-103: max, then sum of exp(x - max), then exp(x - max) / sum; exp is evaluated
 * twice per element and the sum runs in index order. */
void wo_softmax(int rank, const uint32_t *shape, int axis, const float *a, uint32_t a_off, const uint32_t *a_stride,
                float *out, uint32_t o_off, const uint32_t *o_stride)
{
    uint32_t n = 1;
    for (int dd = 0; dd < rank; ++dd) {
        if (dd != axis) {
            n *= shape[dd];
        }
    }
    const uint32_t axis_size = shape[axis];
    const uint32_t as = a_stride[axis];
    const uint32_t os = o_stride[axis];
    for (uint32_t o = 0; o < n; ++o) {
        const uint32_t base = a_off + outer_base(rank, shape, a_stride, axis, o);
        const uint32_t out_base = o_off + outer_base(rank, shape, o_stride, axis, o);
        float mx = a[base];
        for (uint32_t j = 1; j < axis_size; ++j) {
            const float v = a[base + j * as];
            if (v > mx) {
                mx = v;
            }
        }
        float s = 0.0f;
        for (uint32_t j = 0; j < axis_size; ++j) {
            s += expf(a[base + j * as] - mx);
        }
        for (uint32_t j = 0; j < axis_size; ++j) {
            out[out_base + j * os] = expf(a[base + j * as] - mx) / s;
        }
    }
}

/* src/ops/reduce.cpp:33-58 */
void wo_reduce(int op, int rank, const uint32_t *shape, int axis, const float *a, uint32_t a_off,
               const uint32_t *a_stride, float *out, uint32_t o_off, const uint32_t *o_stride)
{
    uint32_t n = 1;
    for (int dd = 0; dd < rank; ++dd) {
        if (dd != axis) {
            n *= shape[dd];
        }
    }
    const uint32_t axis_size = shape[axis];
    const uint32_t as = a_stride[axis];
    for (uint32_t o = 0; o < n; ++o) {
        const uint32_t base = a_off + outer_base(rank, shape, a_stride, axis, o);
        const uint32_t out_idx = o_off + outer_base(rank, shape, o_stride, axis, o);
        float r;
        if (op == 0) {
            r = 0.0f;
            for (uint32_t j = 0; j < axis_size; ++j) {
                r += a[base + j * as];
            }
        } else {
            r = a[base];
            for (uint32_t j = 1; j < axis_size; ++j) {
                const float v = a[base + j * as];
                if ((op == 1) ? (v > r) : (v < r)) {
                    r = v;
                }
            }
        }
        out[out_idx] = r;
    }
}

/* src/ops/triu_fill.cpp:42-59 */
void wo_triu_fill(float *a, uint32_t off, uint32_t rows, uint32_t cols, uint32_t s0, uint32_t s1, float val,
                  uint32_t diagonal)
{
    for (uint32_t idx = 0; idx < rows * cols; ++idx) {
        const uint32_t i = idx % rows;
        const uint32_t j = idx / rows;
        if ((i + diagonal) <= j) {
            a[off + i * s0 + j * s1] = val;
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* rotary position embedding                                                                   */
/* ------------------------------------------------------------------------------------------ */

/* src/modules/rope.cpp:18-51 (RoPE::_build_tables): theta_i = base^(-2i/head_dim) in fp32 (std::pow on floats),
 * angle = pos * theta_i, the cosine / sine stored for BOTH coordinates 2i and 2i+1; tables are column-major
 * [max_seq_len, head_dim]: entry (pos, j) at pos + j * max_seq_len. */
void wo_rope_tables(uint32_t head_dim, uint32_t max_seq_len, float base, float *cos_t, float *sin_t)
{
    const uint32_t half = head_dim >> 1;
    for (uint32_t pos = 0; pos < max_seq_len; ++pos) {
        for (uint32_t i = 0; i < half; ++i) {
            const float theta = powf(base, -2.0f * (float)i / (float)head_dim);
            const float angle = (float)pos * theta;
            const float c = cosf(angle), sn = sinf(angle);
            cos_t[pos + (size_t)(2 * i) * max_seq_len] = c;
            cos_t[pos + (size_t)(2 * i + 1) * max_seq_len] = c;
            sin_t[pos + (size_t)(2 * i) * max_seq_len] = sn;
            sin_t[pos + (size_t)(2 * i + 1) * max_seq_len] = sn;
        }
    }
}

/* src/modules/rope.cpp:53-98 (RoPE::_rotate_half + RoPE::forward): out = x * cos + rotate_half(x) * sin with
 * rotate_half(x) = [-x[half:], x[:half]] along the last dimension, each product rounded before the add.  x, out:
 * dense [B, H, T, head_dim] in C order here (the strides are the caller's business on the device).  The reference
 * always uses positions 0..T-1; `pos0` shifts them (0 = reference behaviour). */
void wo_rope_forward(const float *x, uint32_t B, uint32_t H, uint32_t T, uint32_t head_dim, const float *cos_t,
                     const float *sin_t, uint32_t max_seq_len, uint32_t pos0, float *out)
{
    const uint32_t half = head_dim >> 1;
    for (size_t bh = 0; bh < (size_t)B * H; ++bh) {
        for (uint32_t t = 0; t < T; ++t) {
            const float *row = x + (bh * T + t) * head_dim;
            float *dst = out + (bh * T + t) * head_dim;
            for (uint32_t j = 0; j < head_dim; ++j) {
                const float rot = (j < half) ? -row[j + half] : row[j - half];
                const float c = cos_t[(pos0 + t) + (size_t)j * max_seq_len];
                const float sn = sin_t[(pos0 + t) + (size_t)j * max_seq_len];
                const float a = row[j] * c;
                const float b = rot * sn;
                dst[j] = a + b;
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* activations and norms                                                                       */
/* ------------------------------------------------------------------------------------------ */

/* include/common/weed_types.hpp:213-214: FP_NORM_EPSILON = epsilon / 4 of the real type */
float wo_norm_epsilon(void) { return 1.1920928955078125e-07f / 4.0f; }

/* src/ops/real_unary.cpp:80 (relu: std::max(x, 0)), :135 (sigmoid: 1 / (1 + exp(-x)), float exp), :191 (tanh);
 * src/tensors/tensor.cpp:841-851 (gelu): x3 = x * x * x; inner = k2 * (x + k1 * x3); t = tanh(inner);
 * k0 * x * (ones + t) -- every operator is a separate elementwise op, so every intermediate is rounded to float. */
void wo_unary(int op, const float *x, size_t n, float *out)
{
    const float k0 = 0.5f, k1 = 0.044715f, k2 = 0.7978845608028654f;
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        float r;
        if (op == 0) {
            r = (v > 0.0f) ? v : 0.0f;
        } else if (op == 1) {
            r = 1.0f / (1.0f + expf(-v));
        } else if (op == 2) {
            r = tanhf(v);
        } else {
            const float xx = v * v;
            const float x3 = xx * v;
            const float s = k1 * x3;
            const float u = v + s;
            const float inner = k2 * u;
            const float t = tanhf(inner);
            const float half_x = k0 * v;
            const float one_t = 1.0f + t;
            r = half_x * one_t;
        }
        out[i] = r;
    }
}

/* include/modules/swiglu.hpp:75: gate * Tensor::sigmoid(gate) * up, left to right */
void wo_silu_mul(const float *gate, const float *up, size_t n, float *out)
{
    for (size_t i = 0; i < n; ++i) {
        const float sg = 1.0f / (1.0f + expf(-gate[i]));
        const float a = gate[i] * sg;
        out[i] = a * up[i];
    }
}

/* Tensor::mean(a, axis) (src/tensors/tensor.cpp:682-693): Weed::reduce adds along the axis in index order
 * (src/ops/reduce.cpp:33-38), then one division by the length */
static float axis_mean(const float *v, size_t n)
{
    float sum = 0.0f;
    for (size_t j = 0; j < n; ++j) {
        sum += v[j];
    }
    return sum / (float)n;
}

/* include/modules/rms_norm.hpp:34-38: (x / ((mean(x * x, axis) + eps) ^ 0.5)) * weight; `^` is std::pow on floats
 * (src/ops/pow.cpp:52-56) */
void wo_rms_norm(const float *x, size_t rows, size_t n, const float *w, float eps, float *out)
{
    float *sq = (float *)malloc(sizeof(float) * n);
    for (size_t r = 0; r < rows; ++r) {
        const float *row = x + r * n;
        for (size_t j = 0; j < n; ++j) {
            sq[j] = row[j] * row[j];
        }
        const float t = axis_mean(sq, n) + eps;
        const float root = powf(t, 0.5f);
        for (size_t j = 0; j < n; ++j) {
            const float q = row[j] / root;
            out[r * n + j] = q * w[j];
        }
    }
    free(sq);
}

/* src/modules/layernorm.cpp:29-42: xc = x - mean(x, -1); y = xc / ((mean(xc * xc, -1) + eps) ^ 0.5);
 * y = y * gamma + beta */
void wo_layer_norm(const float *x, size_t rows, size_t n, const float *gamma, const float *beta, float eps, float *out)
{
    float *xc = (float *)malloc(sizeof(float) * n);
    float *sq = (float *)malloc(sizeof(float) * n);
    for (size_t r = 0; r < rows; ++r) {
        const float *row = x + r * n;
        const float mu = axis_mean(row, n);
        for (size_t j = 0; j < n; ++j) {
            xc[j] = row[j] - mu;
            sq[j] = xc[j] * xc[j];
        }
        const float t = axis_mean(sq, n) + eps;
        const float root = powf(t, 0.5f);
        for (size_t j = 0; j < n; ++j) {
            const float q = xc[j] / root;
            const float g = q * gamma[j];
            out[r * n + j] = g + beta[j];
        }
    }
    free(xc);
    free(sq);
}

/* ------------------------------------------------------------------------------------------ */
/* single-query decode attention in the reference's cost structure                             */
/* ------------------------------------------------------------------------------------------ */

void wo_decode_attn(const wo_attn_geom *g, const wo_coder *kc, const wo_coder *vc, const uint8_t *kf, const float *ka,
                    const uint8_t *vf, const float *va, const float *q, const float *Rk, const float *Rv, float *out,
                    float *scores_out)
{
    const int d = g->d;
    const int Hq = g->n_q_heads;
    const int Hkv = g->n_kv_heads;
    const int groups = Hq / Hkv;
    const size_t pitch = (size_t)g->max_tokens;
    float *Rvt = NULL;
    if (g->unrotate_out) {
        Rvt = (float *)malloc(sizeof(float) * (size_t)d * d);
        wo_transpose_square(Rv, d, Rvt); /* cpp:181-186 */
    }
    for (int b = 0; b < g->n_seq; ++b) {
        const size_t L = (size_t)g->seq_lens[b];
        if (!L) {
            memset(out + (size_t)b * Hq * d, 0, sizeof(float) * (size_t)Hq * d);
            continue;
        }
        /* cpp:259-273: dequantise the whole cache into dense [Hkv][L][d] tensors */
        float *Kd = (float *)malloc(sizeof(float) * Hkv * L * d);
        float *Vd = (float *)malloc(sizeof(float) * Hkv * L * d);
        for (int h = 0; h < Hkv; ++h) {
            for (size_t n = 0; n < L; ++n) {
                const size_t row = ((size_t)b * Hkv + h) * pitch + n;
                wo_decode_row(kc, kf + row * d, ka ? ka[row] : 0.0f, Kd + ((size_t)h * L + n) * d);
                wo_decode_row(vc, vf + row * d, va ? va[row] : 0.0f, Vd + ((size_t)h * L + n) * d);
            }
        }
        /* cpp:276: rotate Q into K's basis */
        float *Q = (float *)malloc(sizeof(float) * Hq * d);
        if (g->rotate_q) {
            wo_apply_rotation(q + (size_t)b * Hq * d, (size_t)Hq, d, Rk, Q);
        } else {
            memcpy(Q, q + (size_t)b * Hq * d, sizeof(float) * Hq * d);
        }
        /* cpp:291-311: replicate KV heads up to the query heads (dense copy) */
        float *Krep = (float *)malloc(sizeof(float) * Hq * L * d);
        float *Vrep = (float *)malloc(sizeof(float) * Hq * L * d);
        for (int h = 0; h < Hq; ++h) {
            const int kvh = g->gqa_weed_mapping ? (h % Hkv) : (h / groups);
            memcpy(Krep + (size_t)h * L * d, Kd + (size_t)kvh * L * d, sizeof(float) * L * d);
            memcpy(Vrep + (size_t)h * L * d, Vd + (size_t)kvh * L * d, sizeof(float) * L * d);
        }
        float *Kt = (float *)malloc(sizeof(float) * L * d);
        float *scores = (float *)malloc(sizeof(float) * L);
        float *weights = (float *)malloc(sizeof(float) * L);
        float *o_rot = (float *)malloc(sizeof(float) * d);
        const float sqrt_d = sqrtf((float)d); /* cpp:319 */
        for (int h = 0; h < Hq; ++h) {
            const float *Kh = Krep + (size_t)h * L * d;
            const float *Vh = Vrep + (size_t)h * L * d;
            /* cpp:314 + tensor.cpp:1245: the transposed K is materialised */
            for (size_t n = 0; n < L; ++n) {
                for (int j = 0; j < d; ++j) {
                    Kt[(size_t)j * L + n] = Kh[n * d + j];
                }
            }
            /* cpp:315: scores = Q Kt, k ascending (matmul.cpp:40-44) */
            wo_matmul(1, (uint32_t)L, (uint32_t)d, Q + (size_t)h * d, 0, 0, 1, Kt, 0, (uint32_t)L, 1, scores, 0, 0, 1);
            /* cpp:319 -> div.cpp:17-20: a true division pass */
            for (size_t n = 0; n < L; ++n) {
                scores[n] = scores[n] / sqrt_d;
            }
            if (scores_out) {
                memcpy(scores_out + ((size_t)b * Hq + h) * pitch, scores, sizeof(float) * L);
            }
            /* cpp:334 */
            {
                const uint32_t shape[1] = { (uint32_t)L };
                const uint32_t stride[1] = { 1 };
                wo_softmax(1, shape, 0, scores, 0, stride, weights, 0, stride);
            }
            /* cpp:337: out = weights V, n ascending */
            wo_matmul(1, (uint32_t)d, (uint32_t)L, weights, 0, 0, 1, Vh, 0, (uint32_t)d, 1, o_rot, 0, 0, 1);
            /* cpp:343-348 */
            float *dst = out + ((size_t)b * Hq + h) * d;
            if (g->unrotate_out) {
                wo_apply_rotation(o_rot, 1, d, Rvt, dst);
            } else {
                memcpy(dst, o_rot, sizeof(float) * d);
            }
        }
        free(Kd);
        free(Vd);
        free(Q);
        free(Krep);
        free(Vrep);
        free(Kt);
        free(scores);
        free(weights);
        free(o_rot);
    }
    free(Rvt);
}
