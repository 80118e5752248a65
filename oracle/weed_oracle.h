/*
 * weed_oracle.h -- CPU restatement of vm6502q/weed's quantized-KV attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing under weed_amd/ may include, link or call
 * this; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.
 *
 * Every function cites the reference file:line it follows (paths relative to the
 * reference checkout).  Build: `make -C oracle` (plain gcc, -O3, no -march,
 * -ffp-contract=off, as the reference is built: CMakeLists.txt:161-167).
 *
 * Pinning status of each function is in weed_oracle.c's header comment.
 */
#ifndef WEED_ORACLE_H
#define WEED_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- Weed's uniform coder (src/modules/multihead_attention.cpp:31-79) ---- */
int wo_values_per_word(int bits);
int wo_words_per_row(int d, int bits);
void wo_uniform_write_row(int32_t *packed, uint32_t row, const float *vals, int d, int bits, float block_scale);
void wo_uniform_read_row(const int32_t *packed, uint32_t row, float *vals, int d, int bits, float block_scale);
/* one code per byte, same arithmetic as write_row */
void wo_uniform_codes(const float *vals, int d, int bits, float block_scale, uint8_t *codes);
/* block_scale = sqrt(sum(x^2)/n + 1e-8), sequential fp32 (multihead_attention.cpp:226-241) */
float wo_block_scale(const float *x, size_t n);

/* ---- rotation (multihead_attention.cpp:84-140) ---- */
/* In-place Gram-Schmidt over the columns of a column-major d x d matrix. */
void wo_orthonormalize_columns(float *R, int d);
/* y[r,j] = sum_i x[r,i] * R[i + d*j], i ascending; x,y row-contiguous [rows][d]. */
void wo_apply_rotation(const float *x, size_t rows, int d, const float *R, float *y);
void wo_transpose_square(const float *R, int d, float *Rt);

/* ---- table-driven coder: Lloyd-Max codes + optional sign residual + row scale ---- */
typedef struct {
    int mode;          /* 0 = Weed uniform (block_scale), 1 = Lloyd-Max with per-row scale */
    int d;             /* head_dim */
    int bits;          /* code bits */
    int sign;          /* 1 = a residual sign bit is kept (mode 1 only) */
    float block_scale; /* mode 0 */
    const float *bounds; /* mode 1: 2^bits - 1 ascending decision thresholds */
    const float *levels; /* mode 1: 2^bits centroids */
    const float *recon;  /* mode 1: 2^(bits+sign) reconstruction levels, index (code<<sign)|signbit */
} wo_coder;

/* fields[j] = code (mode 0 / sign==0) or (code<<1)|sign; *alpha = row scale (mode 1), untouched in mode 0 */
void wo_encode_row(const wo_coder *c, const float *y, uint8_t *fields, float *alpha);
void wo_decode_row(const wo_coder *c, const uint8_t *fields, float alpha, float *yhat);
/* loops over the row functions; alpha may be NULL in mode 0 for wo_decode_rows */
void wo_encode_rows(const wo_coder *c, const float *y, size_t rows, uint8_t *fields, float *alpha);
void wo_decode_rows(const wo_coder *c, const uint8_t *fields, const float *alpha, size_t rows, float *yhat);
void wo_uniform_write_rows(int32_t *packed, const float *vals, size_t rows, int d, int bits, float block_scale);
void wo_uniform_read_rows(const int32_t *packed, float *vals, size_t rows, int d, int bits, float block_scale);

/* ---- dense ops ---- */
/* strided 2-D GEMM, k-ascending fp32 sums (src/ops/matmul.cpp:34-47,95-122) */
void wo_matmul(uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t a_o, uint32_t a_s0, uint32_t a_s1,
               const float *B, uint32_t b_o, uint32_t b_s0, uint32_t b_s1, float *C, uint32_t c_o, uint32_t c_s0,
               uint32_t c_s1);
/* three-pass softmax along `axis` of a strided tensor (src/ops/softmax.cpp:23-45,82-103) */
void wo_softmax(int rank, const uint32_t *shape, int axis, const float *a, uint32_t a_off, const uint32_t *a_stride,
                float *out, uint32_t o_off, const uint32_t *o_stride);
/* axis sum/max/min; op 0 sum, 1 max, 2 min (src/ops/reduce.cpp:17-58).  Output element o (index over the
 * non-reduced dims, dim 0 fastest) is written to out[o_off + sum_d i_d*o_stride[d]]. */
void wo_reduce(int op, int rank, const uint32_t *shape, int axis, const float *a, uint32_t a_off,
               const uint32_t *a_stride, float *out, uint32_t o_off, const uint32_t *o_stride);
/* fill where i + diagonal <= j on a col-major-indexed 2-D tensor (src/ops/triu_fill.cpp:42-59) */
void wo_triu_fill(float *a, uint32_t off, uint32_t rows, uint32_t cols, uint32_t s0, uint32_t s1, float val,
                  uint32_t diagonal);

/* ---- activations and norms of the attention module's two callers ---- */
/* op 0 relu, 1 sigmoid, 2 tanh (src/ops/real_unary.cpp:80,135,191), 3 gelu as Tensor::gelu composes it from
 * elementwise ops (src/tensors/tensor.cpp:841-851) */
void wo_unary(int op, const float *x, size_t n, float *out);
/* SwiGLU::forward's gate (include/modules/swiglu.hpp:71-77): (gate * sigmoid(gate)) * up */
void wo_silu_mul(const float *gate, const float *up, size_t n, float *out);
/* RMSNorm::forward (include/modules/rms_norm.hpp:34-38) over dense rows [rows][n]; w: [n] */
void wo_rms_norm(const float *x, size_t rows, size_t n, const float *w, float eps, float *out);
/* LayerNorm::forward (src/modules/layernorm.cpp:29-42) over dense rows [rows][n]; gamma, beta: [n] */
void wo_layer_norm(const float *x, size_t rows, size_t n, const float *gamma, const float *beta, float eps, float *out);
/* FP_NORM_EPSILON at fp32 (include/common/weed_types.hpp:213-214): the eps both norms default to */
float wo_norm_epsilon(void);

/* ---- single-query decode attention over a quantized cache, in the reference's cost structure
 * (multihead_attention.cpp:259-348): dequantise the whole cache to dense fp32, replicate KV heads,
 * materialise K^T, naive dots, divide by sqrt(d), three-pass softmax, naive P.V, un-rotate. ---- */
/* RoPE::_build_tables and RoPE::forward (src/modules/rope.cpp:18-98); tables column-major [max_seq_len, head_dim];
 * x, out dense [B, H, T, head_dim] in C order; pos0 = position of token 0 (the reference always uses 0). */
void wo_rope_tables(uint32_t head_dim, uint32_t max_seq_len, float base, float *cos_t, float *sin_t);
void wo_rope_forward(const float *x, uint32_t B, uint32_t H, uint32_t T, uint32_t head_dim, const float *cos_t,
                     const float *sin_t, uint32_t max_seq_len, uint32_t pos0, float *out);

typedef struct {
    int n_seq, n_q_heads, n_kv_heads, d;
    int max_tokens;          /* row pitch of the field/alpha arrays */
    const int32_t *seq_lens; /* [n_seq] */
    int gqa_weed_mapping;    /* 1: kv = q_head % n_kv_heads (reference, cpp:301-306); 0: kv = q_head / groups */
    int rotate_q;            /* q is multiplied by Rk first (cpp:276) */
    int unrotate_out;        /* out is multiplied by Rv^T last (cpp:343-348) */
} wo_attn_geom;

/* kf/vf: [n_seq][n_kv_heads][max_tokens][d] uint8 fields; ka/va: [n_seq][n_kv_heads][max_tokens] row scales
 * (ignored in mode 0); q,out: [n_seq][n_q_heads][d]; Rk,Rv: column-major d x d (may be NULL when the flags are 0).
 * scores_out (optional, may be NULL): [n_seq][n_q_heads][max_tokens] scaled scores before softmax. */
void wo_decode_attn(const wo_attn_geom *g, const wo_coder *kc, const wo_coder *vc, const uint8_t *kf, const float *ka,
                    const uint8_t *vf, const float *va, const float *q, const float *Rk, const float *Rv, float *out,
                    float *scores_out);

#ifdef __cplusplus
}
#endif
#endif
