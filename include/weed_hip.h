/*
 * weed_hip.h -- C ABI of the MI355X (gfx950) device layer for Weed's quantized-KV attention path.
 *
 * This is the seam a Weed build binds instead of its OpenCL device (include/devices/gpu_device.hpp,
 * include/common/oclengine.hpp): plain C types only -- uint32_t for Weed's tcapint, int32_t for symint,
 * float for real1 -- raw device pointers, explicit geometry in ELEMENTS exactly as Weed's ops pass it
 * (offset + per-dimension stride, column-major by convention, see include/tensors/base_tensor.hpp:123-142).
 *
 * Conventions
 *   - Every function returns an int status: WEED_HIP_OK (0) or a WEED_HIP_E* code, and never throws.
 *     weed_hip_last_error() returns the message of the calling thread's last failure.  Weed's device layer
 *     throws std::runtime_error / Weed::bad_alloc / std::invalid_argument instead
 *     (include/devices/pool_item.hpp:32-40, src/devices/gpu_device.cpp:60-73,177, src/ops/matmul.cpp:96-109);
 *     a host wrapper maps WEED_HIP_EINVAL -> std::invalid_argument, WEED_HIP_ENOMEM -> bad_alloc,
 *     WEED_HIP_EDEVICE -> std::runtime_error.
 *   - All launches are ordered on one HIP stream per process (weed_hip_set_stream / weed_hip_stream); an
 *     asynchronous kernel fault surfaces at the next weed_hip_sync(), like Weed's callbackError latch
 *     (include/devices/gpu_device.hpp:101-111).
 *   - Entry points are not re-entrant per cache object; serialise callers per device as Weed serialises
 *     enqueues under GpuDevice::queue_mutex (include/devices/gpu_device.hpp:41).
 *   - Pointers named *_dev are device pointers; everything else is host memory.
 */
#ifndef WEED_HIP_H
#define WEED_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    WEED_HIP_OK = 0,
    WEED_HIP_EINVAL = 1,   /* bad argument / shape mismatch (Weed: std::invalid_argument)      */
    WEED_HIP_ENOMEM = 2,   /* device allocation failed (Weed: Weed::bad_alloc)                 */
    WEED_HIP_EDEVICE = 3,  /* HIP runtime / kernel failure (Weed: std::runtime_error)          */
    WEED_HIP_ECAPACITY = 4 /* append beyond max_tokens (Weed: unchecked std::vector overrun)   */
};

/* ------------------------------------------------------------------------------------------------ */
/* device, stream, memory.  Replaces OCLEngine::GetWeedDevice (src/common/oclengine.cpp:186-194),      */
/* GpuDevice::MakeBuffer (src/devices/gpu_device.cpp:34-76) and the blocking read/write helpers         */
/* (src/devices/gpu_device.cpp:396-402, src/storage/gpu_real_storage.cpp:18-23).                        */
/* ------------------------------------------------------------------------------------------------ */
int weed_hip_init(int device_id);
/* The other end of weed_hip_init (the reference's device object goes away with its queue and buffers,
 * include/devices/gpu_device.hpp:60-82): waits for everything queued, then frees what the library itself holds on the
 * device -- the cached blocks of weed_hip_malloc, the scratch of split products, its timing events, its own stream.
 * Caches (weed_hip_kv_cache_destroy) and blocks from weed_hip_malloc that are still in use belong to the caller and
 * are not touched; free them before or after.  A later weed_hip_init (or any call) starts the library again. */
int weed_hip_shutdown(void);
int weed_hip_device_count(int *count);
int weed_hip_device_name(char *buf, size_t buf_len);
/* Use an existing hipStream_t for all later launches (NULL restores the library's own stream). */
int weed_hip_set_stream(void *hip_stream);
void *weed_hip_stream(void);
int weed_hip_sync(void);
const char *weed_hip_last_error(void);
const char *weed_hip_version(void);

/* Device memory for tensors.  Freed blocks are kept and handed out again in stream order (no wait, no driver call)
 * while the working set repeats, as the intermediates of a module's forward do; weed_hip_release_cached drains the
 * stream and returns them to the driver.  WEED_HIP_POOL_MAX_MB caps the cached bytes (default 64 GiB, 0 = no cache). */
int weed_hip_malloc(void **ptr_dev, size_t bytes);
int weed_hip_free(void *ptr_dev);
int weed_hip_release_cached(void);
int weed_hip_memset(void *ptr_dev, int byte_value, size_t bytes);
int weed_hip_memcpy_h2d(void *dst_dev, const void *src, size_t bytes);
int weed_hip_memcpy_d2h(void *dst, const void *src_dev, size_t bytes);
int weed_hip_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes);

/* Per-kernel device timing (HIP events on the launch stream), off by default.  When enabled, each entry
 * point brackets its dominant kernel with events; weed_hip_profile_read returns the accumulated time. */
int weed_hip_profile_enable(int on);
int weed_hip_profile_reset(void);
/* name: "kv_decode_attn", "kv_decode_combine", "kv_encode", "kv_pack", "matmul", "softmax", "reduce", "elementwise",
 * "copy", "rope", "rms_norm", "layer_norm", "read_sweep" */
int weed_hip_profile_read(const char *name, double *total_ms, uint64_t *launches);

/* ------------------------------------------------------------------------------------------------ */
/* dense ops on strided fp32 tensors                                                                  */
/* ------------------------------------------------------------------------------------------------ */

/* out[M,N] = a[M,K] . b[K,N].  Replaces Weed::matmul's real branch (src/ops/matmul.cpp:242-279; geometry as
 * get_dim, matmul.cpp:95-122; OpenCL kernel matmul_real, src/common/qengine.cl:598-640).  Element (i,k) of a is
 * a_dev[a_off + i*a_s0 + k*a_s1], and likewise for b and out. */
int weed_hip_matmul_f32(uint32_t M, uint32_t N, uint32_t K, const float *a_dev, uint32_t a_off, uint32_t a_s0,
                        uint32_t a_s1, const float *b_dev, uint32_t b_off, uint32_t b_s0, uint32_t b_s1, float *out_dev,
                        uint32_t o_off, uint32_t o_s0, uint32_t o_s1);

/* Which matrix instruction the large products run on (no counterpart in the reference; process-wide, takes effect
 * with the next call).  0, the default: products whose operands are contiguous along one dimension and 16-byte aligned,
 * with more than 64 rows, run on the bfloat16 instruction with both operands split exactly into three bfloat16 parts and
 * six of the nine products of parts accumulated in fp32 -- 1.5 times the fp32 instruction's speed and more.  The error
 * against the exact product is the fp32 instruction's own: relative to sum_k |a_ik| |b_kj| per element, at k = 1028 over
 * operands spanning 2^-20 .. 2^20, largest 7.1e-7 against 5.9e-7 and mean 5.8e-8 against 5.1e-8; for operands of one
 * magnitude 8.0e-8 against 1.0e-7 and 9.1e-9 against 1.1e-8 (a sequential fp32 sum: 3.4e-7 and 2.0e-8).  Two things are
 * not kept: an operand that is not finite gives NaN where the fp32 instruction would give an infinity, and operand
 * values below 2^-112 in magnitude lose accuracy, because their second and third parts fall below bfloat16's normal
 * range and the instruction takes them as zeros (largest error 1.3e-6 for values around 2^-115, 3e-5 around 2^-120,
 * 9e-4 around 2^-125; fp32 denormals count as zero), where the fp32 instruction keeps 2e-7 down to the denormals.  1: the fp32 instruction everywhere (v_mfma_f32_32x32x2_f32: every product
 * exact, sums rounded to fp32 in ascending k per 16-k slice), also for the products of 17 to 64 rows against a
 * k-contiguous weight, which otherwise split their operands the same way.  Products with at most 16 rows, and unaligned
 * or doubly strided operands, do not depend on it.  The process-wide default is read once from the environment
 * variable WEED_HIP_MATMUL_FP32 (1 = the fp32 instruction). */
int weed_hip_matmul_tuning(int32_t fp32_instruction);

/* batch[0] * batch[1] independent products in one launch: product (c0, c1) uses the offsets
 * off + c0 * bs[0] + c1 * bs[1] of each operand.  The reference has no device entry for this: Tensor::matmul loops
 * over the leading dimensions on the host and calls the 2-D product once per index (src/tensors/tensor.cpp:1213-1272);
 * the attention scores and weights of a prefill are (batch x heads) such products.  At most 65535 products. */
int weed_hip_matmul_batched_f32(const uint32_t batch[2], uint32_t M, uint32_t N, uint32_t K, const float *a_dev,
                                uint32_t a_off, uint32_t a_s0, uint32_t a_s1, const uint32_t a_bs[2],
                                const float *b_dev, uint32_t b_off, uint32_t b_s0, uint32_t b_s1,
                                const uint32_t b_bs[2], float *out_dev, uint32_t o_off, uint32_t o_s0, uint32_t o_s1,
                                const uint32_t o_bs[2]);

/* out[M,N] = a[M,K] . w[K,N] + bias[N]: Linear::forward (src/modules/linear.cpp:86-100: `x >> weight`, then
 * `+ bias` broadcast over the rows) as one launch.  The bias (element n at bias_dev[bias_off + n*bias_stride]) is added
 * to the rounded sum, so the result is bit-identical to weed_hip_matmul_f32 followed by the broadcast add of
 * weed_hip_elementwise_f32; bias_dev may be null (no bias). */
int weed_hip_linear_f32(uint32_t M, uint32_t N, uint32_t K, const float *a_dev, uint32_t a_off, uint32_t a_s0,
                        uint32_t a_s1, const float *w_dev, uint32_t w_off, uint32_t w_s0, uint32_t w_s1,
                        const float *bias_dev, uint32_t bias_off, uint32_t bias_stride, float *out_dev, uint32_t o_off,
                        uint32_t o_s0, uint32_t o_s1);

/* out[o_off + i*o_stride] = a[a_off + i*a_stride] for i < n.  Replaces the OpenCL kernel copy_real
 * (src/common/qengine.cl:979, launched from src/ops/copy_broadcast.cpp:66); also the plain copy used to calibrate the
 * HBM traffic counters. */
int weed_hip_copy_f32(uint64_t n, const float *a_dev, uint32_t a_off, uint32_t a_stride, float *out_dev, uint32_t o_off,
                      uint32_t o_stride);

/* Calibration, no counterpart in the reference: read `bytes` of device memory once with 16-byte loads and write
 * nothing, by 256 workgroups of 8 wavefronts in units of 8 KB with the next unit in flight (a tail below 8 KB is not
 * read).  per_wavefront_runs = 1: every wavefront walks one contiguous run, the decode kernel's launch shape; 0: the
 * device's wavefronts take the units in turns, so that the device reads one contiguous stretch at any moment.  The
 * time of such a launch is what merely reading the bytes of a decode step costs on this part.  sink_dev: one word that
 * is (practically) never written. */
int weed_hip_read_sweep(const void *src_dev, uint64_t bytes, int per_wavefront_runs, uint32_t *sink_dev);

/* Broadcasting elementwise ops on tensors of one logical shape (rank <= 8, strides in elements, stride 0 repeats a
 * dimension): out = a (COPY; b may be NULL), a + b, a - b, a * b, a / b, and the activations below.  Replace Weed's add / mul
 * (src/ops/commuting.cpp:17-25), sub (src/ops/sub.cpp), div with IEEE division (src/ops/div.cpp:17-20), add_in_place
 * (src/ops/in_place.cpp:17-25, out aliasing a) and the strided gather behind Tensor::contiguous
 * (include/tensors/tensor.hpp:319-331). */
enum {
    WEED_HIP_EW_COPY = 0,
    WEED_HIP_EW_ADD = 1,
    WEED_HIP_EW_SUB = 2,
    WEED_HIP_EW_MUL = 3,
    WEED_HIP_EW_DIV = 4,
    /* a * sigmoid(a) * b: the gate of SwiGLU::forward (include/modules/swiglu.hpp:71-77: `gate * Tensor::sigmoid(gate)
     * * up`, three elementwise ops in the reference) as one pass */
    WEED_HIP_EW_SILU_MUL = 5,
    /* unary (b may be NULL): Weed::relu / sigmoid / tanh (src/ops/real_unary.cpp:80,135,191) and Tensor::gelu
     * (src/tensors/tensor.cpp:841-851: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), eight elementwise ops in the
     * reference) */
    WEED_HIP_EW_RELU = 6,
    WEED_HIP_EW_SIGMOID = 7,
    WEED_HIP_EW_TANH = 8,
    WEED_HIP_EW_GELU = 9
};
int weed_hip_elementwise_f32(int op, uint32_t rank, const uint32_t *shape, const float *a_dev, uint32_t a_off,
                             const uint32_t *a_stride, const float *b_dev, uint32_t b_off, const uint32_t *b_stride,
                             float *out_dev, uint32_t o_off, const uint32_t *o_stride);

/* a[i,j] = val wherever i + diagonal <= j, on a rows x cols matrix.  Replaces Weed::triu_fill
 * (src/ops/triu_fill.cpp:42-59), the causal mask builder of MultiHeadAttention::forward. */
int weed_hip_triu_fill_f32(uint32_t rows, uint32_t cols, float val, uint32_t diagonal, float *a_dev, uint32_t a_off,
                           uint32_t a_s0, uint32_t a_s1);

/* Rotary position embedding: out = x * cos + rotate_half(x) * sin over the last dimension of a strided
 * [B, H, T, head_dim] tensor, rotate_half(x) = [-x[half:], x[:half]].  Replaces RoPE::forward
 * (src/modules/rope.cpp:77-98) and its helper _rotate_half (53-75).  cos_dev / sin_dev are the module's tables,
 * column-major [table_rows, head_dim] as RoPE::_build_tables lays them out (rope.cpp:18-51).  Token t of the call
 * uses table row pos0 + t; the reference always uses pos0 = 0, a decode step with a cache passes the cache length. */
int weed_hip_rope_f32(const uint32_t shape[4], const float *x_dev, uint32_t x_off, const uint32_t x_stride[4],
                      const float *cos_dev, const float *sin_dev, uint32_t table_rows, uint32_t pos0, float *out_dev,
                      uint32_t o_off, const uint32_t o_stride[4]);

/* RMSNorm::forward (include/modules/rms_norm.hpp:34-38: `x / ((mean(x * x, axis) + eps) ^ 0.5) * weight`, seven ops
 * and an axis reduction in the reference) as one kernel: out = x / sqrt(mean(x^2 over axis) + eps) * w, with
 * w[w_off + j * w_stride] for index j along the axis.  rank <= 8; x and out may be the same tensor. */
int weed_hip_rms_norm_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *x_dev, uint32_t x_off,
                          const uint32_t *x_stride, const float *w_dev, uint32_t w_off, uint32_t w_stride, float eps,
                          float *out_dev, uint32_t o_off, const uint32_t *o_stride);

/* LayerNorm::forward (src/modules/layernorm.cpp:29-42) as one kernel: xc = x - mean(x over axis),
 * out = xc / sqrt(mean(xc^2) + eps) * gamma + beta, gamma and beta indexed along the axis like w above. */
int weed_hip_layer_norm_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *x_dev, uint32_t x_off,
                            const uint32_t *x_stride, const float *gamma_dev, uint32_t gamma_off, uint32_t gamma_stride,
                            const float *beta_dev, uint32_t beta_off, uint32_t beta_stride, float eps, float *out_dev,
                            uint32_t o_off, const uint32_t *o_stride);

/* Numerically stable softmax along `axis`.  Replaces Weed::softmax (src/ops/softmax.cpp:276-287; OpenCL kernel
 * softmax_forward, qengine.cl:1001-1033).  rank <= 8. */
int weed_hip_softmax_f32(uint32_t rank, const uint32_t *shape, uint32_t axis, const float *a_dev, uint32_t a_off,
                         const uint32_t *a_stride, float *out_dev, uint32_t o_off, const uint32_t *o_stride);

/* Axis reductions.  Replace Weed::reduce / Weed::max / Weed::min (src/ops/reduce.cpp:342-386; OpenCL kernels
 * reduce_real / axis_max / axis_min, qengine.cl:136-159,244-297).  out has the shape of a with `axis` removed;
 * o_stride has `rank` entries and the one at `axis` is ignored. */
enum { WEED_HIP_REDUCE_SUM = 0, WEED_HIP_REDUCE_MAX = 1, WEED_HIP_REDUCE_MIN = 2 };
int weed_hip_reduce_f32(int op, uint32_t rank, const uint32_t *shape, uint32_t axis, const float *a_dev,
                        uint32_t a_off, const uint32_t *a_stride, float *out_dev, uint32_t o_off,
                        const uint32_t *o_stride);

/* ------------------------------------------------------------------------------------------------ */
/* rotation                                                                                            */
/* ------------------------------------------------------------------------------------------------ */

/* Seeded replacement of make_random_rotation (src/modules/multihead_attention.cpp:84-121): draws d*d N(0,1)
 * values with std::mt19937(seed) + std::normal_distribution<float> on the host (column-major), uploads them and
 * orthonormalises the columns on the device in the reference's order (normalise column j, remove its projection
 * from every later column).  r_dev receives d*d floats, column-major. */
int weed_hip_make_rotation(uint32_t seed, uint32_t d, float *r_dev);
/* Device Gram-Schmidt only (input already in r_dev). */
int weed_hip_orthonormalize_columns(uint32_t d, float *r_dev);

/* apply_rotation (src/modules/multihead_attention.cpp:125-140): y = x . R over the last dimension (length d) of a
 * strided tensor of rank <= 8; R is d x d column-major.  Products are added in ascending index order with separate
 * multiplies and adds, the order of the reference's naive matmul (src/ops/matmul.cpp:40-44), so the rotated values
 * match a BLAS-less reference build bit for bit.  x_dev and out_dev must not overlap. */
int weed_hip_apply_rotation_f32(uint32_t d, const float *r_dev, uint32_t rank, const uint32_t *shape,
                                const float *x_dev, uint32_t x_off, const uint32_t *x_stride, float *out_dev,
                                uint32_t o_off, const uint32_t *o_stride);

/* ------------------------------------------------------------------------------------------------ */
/* quantized KV cache: device twin of Weed::QuantizedKVCache (include/modules/multihead_attention.hpp:22-36)  */
/* ------------------------------------------------------------------------------------------------ */

enum {
    WEED_HIP_KV_UNIFORM = 0, /* Weed's coder: 2^bits uniform cells on [-3s, 3s), one block_scale per tensor     */
    WEED_HIP_KV_LLOYDMAX = 1 /* per-row scale, Lloyd-Max codes for N(0,1), optional residual sign bit           */
};
enum {
    WEED_HIP_GQA_WEED = 0,    /* kv_head = q_head % n_kv_heads  (multihead_attention.cpp:301-306)               */
    WEED_HIP_GQA_BLOCKED = 1  /* kv_head = q_head / (n_q_heads / n_kv_heads)                                    */
};

typedef struct {
    int32_t mode;          /* WEED_HIP_KV_UNIFORM or WEED_HIP_KV_LLOYDMAX                                      */
    int32_t n_seq;         /* B: sequences held side by side                                                  */
    int32_t n_kv_heads;    /* Hkv                                                                             */
    int32_t head_dim;      /* d, any value in 1..256 as QuantizedKVCache::allocate takes (cpp:31-41); rows are
                            * stored with d rounded up to a multiple of 32, zeros in the extra coordinates      */
    int32_t max_tokens;    /* capacity per sequence (Weed: max_seq_len)                                        */
    int32_t k_bits;        /* code bits for keys: 1..8 (UNIFORM, any kv_quant_bits of the reference), 1..4 (LLOYDMAX) */
    int32_t v_bits;        /* code bits for values, likewise                                                   */
    int32_t k_sign;        /* 1: keep a residual sign bit per key coordinate (LLOYDMAX only)                   */
    int32_t v_sign;        /* 1: same for values                                                              */
} weed_hip_kv_config;

typedef struct weed_hip_kv_cache weed_hip_kv_cache;

/* QuantizedKVCache::allocate for both K and V (multihead_attention.cpp:31-41,190-193). */
int weed_hip_kv_cache_create(weed_hip_kv_cache **cache, const weed_hip_kv_config *cfg);
int weed_hip_kv_cache_destroy(weed_hip_kv_cache *cache);
/* MultiHeadAttention::reset_cache (include/modules/multihead_attention.hpp:140-149): lengths to 0; rotations,
 * scales and tables are kept unless `drop_rotations` is non-zero. */
int weed_hip_kv_cache_reset(weed_hip_kv_cache *cache, int drop_rotations);
/* Bytes of device memory a decode step reads for the packed K and V fields and row scales of `n_tokens` tokens of
 * one (sequence, kv head): the algorithmic bytes used for roofline accounting. */
int weed_hip_kv_cache_row_bytes(const weed_hip_kv_cache *cache, uint32_t *k_row_bytes, uint32_t *v_row_bytes);
int weed_hip_kv_cache_seq_lens(const weed_hip_kv_cache *cache, int32_t *lens /* [n_seq] host */);

/* k_rotation / v_rotation (multihead_attention.cpp:177-178): column-major d x d, copied from device memory. */
int weed_hip_kv_cache_set_rotations(weed_hip_kv_cache *cache, const float *rk_dev, const float *rv_dev);
/* block_scale of the two caches (multihead_attention.cpp:240-241); UNIFORM mode only. */
int weed_hip_kv_cache_set_scales(weed_hip_kv_cache *cache, float k_scale, float v_scale);
int weed_hip_kv_cache_get_scales(const weed_hip_kv_cache *cache, float *k_scale, float *v_scale);
/* Replace the built-in Lloyd-Max tables (host arrays): bounds[2^bits-1], levels[2^bits], recon[2^(bits+sign)].
 * `which` 0 = keys, 1 = values.  Reconstruction levels are rounded to IEEE binary16 (the fused decode kernel keeps
 * them in fp16 so that products with the split query are exact); recon_rounded receives the values in use. */
int weed_hip_kv_cache_set_tables(weed_hip_kv_cache *cache, int which, const float *bounds, const float *levels,
                                 const float *recon, float *recon_rounded);
int weed_hip_kv_cache_get_tables(const weed_hip_kv_cache *cache, int which, float *bounds, float *levels, float *recon);

/* sqrt(sum(x^2)/n + 1e-8) over a strided [n_seq, n_kv_heads, T, d] tensor (multihead_attention.cpp:226-241).
 * `sequential` != 0 reproduces the reference's one-thread fp32 summation order bit for bit: the flat column-major
 * index of the logical tensor (first dimension fastest, d slowest), whatever the strides of the view are; 0 uses a
 * tree reduction. */
int weed_hip_block_scale_f32(const float *x_dev, uint32_t off, const uint32_t shape[4], const uint32_t stride[4],
                             int sequential, float *scale_out /* host */);

/* Encode-and-append: apply_rotation + write_row for T_new tokens of every sequence in
 * [seq_begin, seq_begin + seq_count) (multihead_attention.cpp:206-257).  k_dev / v_dev are logical
 * [seq_count, n_kv_heads, T_new, d] tensors with strides in elements.  `rotate` = 0: the inputs are already in the
 * rotated basis; 1: rotate on the matrix cores (fp32, fastest; sums in a different order than the reference's loop);
 * 2: rotate with the reference's order and rounding (src/ops/matmul.cpp:40-44), so that codes match a BLAS-less
 * reference build bit for bit.  Tokens are appended in logical order (token t of the call becomes token len+t).
 * An append of one token per sequence (a decode step's) and an append of whole 32-token half blocks behind whole half
 * blocks (a prefill, in chunks or not) are one kernel launch (a large one is followed by a small kernel that moves
 * the lengths); other appends take two.  However the tokens arrive, the
 * cache ends up with the same bits. */
int weed_hip_kv_encode_append(weed_hip_kv_cache *cache, int32_t seq_begin, int32_t seq_count, int32_t T_new,
                              const float *k_dev, uint32_t k_off, const uint32_t k_stride[4], const float *v_dev,
                              uint32_t v_off, const uint32_t v_stride[4], int rotate);

/* read_row for a token range (multihead_attention.cpp:64-79,259-273): dense fp32 [seq_count, n_kv_heads, T, d]
 * with caller strides, still in the rotated basis.  `which` 0 = keys, 1 = values. */
int weed_hip_kv_dequant(const weed_hip_kv_cache *cache, int which, int32_t seq_begin, int32_t seq_count,
                        int32_t tok_begin, int32_t T, float *out_dev, uint32_t o_off, const uint32_t o_stride[4]);

/* Unpack for inspection: one field per byte, fields_dev[seq_count][n_kv_heads][T][d] (field = code, or
 * (code<<1)|sign when a sign bit is kept), scales_dev[seq_count][n_kv_heads][T] (row scale alpha = |y|/sqrt(d);
 * LLOYDMAX only, may be NULL). */
int weed_hip_kv_export_fields(const weed_hip_kv_cache *cache, int which, int32_t seq_begin, int32_t seq_count,
                              int32_t tok_begin, int32_t T, uint8_t *fields_dev, float *scales_dev);
/* UNIFORM mode: the rows in Weed's own word packing, floor(32/bits) codes per int32
 * (QuantizedKVCache::packed, multihead_attention.cpp:43-62); words_dev[seq_count][n_kv_heads][T][wpr]. */
int weed_hip_kv_export_weed_words(const weed_hip_kv_cache *cache, int which, int32_t seq_begin, int32_t seq_count,
                                  int32_t tok_begin, int32_t T, int32_t *words_dev);

/* The reverse of weed_hip_kv_export_weed_words: append T_new tokens per sequence whose rows arrive already coded in
 * Weed's word packing (QuantizedKVCache::packed as write_row leaves it, multihead_attention.cpp:43-62; both arrays
 * [seq_count][n_kv_heads][T_new][words per row], on the device).  A cache built by the reference on another device is
 * moved over this way without a round trip through floats; set the two block scales with
 * weed_hip_kv_cache_set_scales first.  UNIFORM mode only. */
int weed_hip_kv_append_weed_words(weed_hip_kv_cache *cache, int32_t seq_begin, int32_t seq_count, int32_t T_new,
                                  const int32_t *k_words_dev, const int32_t *v_words_dev);

/* Fused single-query decode attention over the packed cache: everything MultiHeadAttention::forward does between
 * the cache rebuild and the output projection for T = 1 (multihead_attention.cpp:259-348): un-pack, Q.K^T,
 * /sqrt(d), softmax over each sequence's own length (split over the context and merged), P.V, un-rotate.
 * q_dev / out_dev: logical [n_seq, n_q_heads, d] with strides in elements.
 * flags: bit 0 rotate q by k_rotation first (cpp:276); bit 1 multiply the result by v_rotation^T (cpp:343-348). */
enum { WEED_HIP_ATTN_ROTATE_Q = 1, WEED_HIP_ATTN_UNROTATE_OUT = 2 };
int weed_hip_kv_decode_attn(weed_hip_kv_cache *cache, int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev,
                            uint32_t q_off, const uint32_t q_stride[3], float *out_dev, uint32_t o_off,
                            const uint32_t o_stride[3], uint32_t flags);

/* How the decode kernels cut a launch's list of 64-token blocks into per-wavefront runs (no counterpart in the
 * reference; results do not depend on it, only speed).  wavefronts: number of runs, 0 = as many wavefronts as the
 * device holds at once; skew_percent: how much longer than the mean the runs of a workgroup's oldest wavefronts are
 * (and the youngest shorter), negative = the built-in 16 (28 for kernel instances with three wavefronts per SIMD);
 * always_search: bit 0: find every run's first region by search even when all sequences have equal lengths;
 * bit 1: never let the matrix-core kernel merge its partials itself; bit 2: never let it rotate the queries itself;
 * bit 3: every wavefront takes one contiguous piece of the cache (otherwise, in batches of equal sequences,
 * neighbouring wavefronts take the blocks of their common piece in turns)
 * (when every workgroup's share of the launch is a whole number of (sequence, kv head) regions, or every region a
 * whole number of such shares, one kernel does the whole call: that is so for batches of 1 to 256 sequences whose
 * lengths are equal or not too different -- sequences are counted as having as many blocks as the longest while that
 * adds at most 3/4 to the blocks of the batch; other batches of up to 63
 * sequences are one kernel too, with partial results in memory -- all of this at head_dims up to 128 (65 to 96 with at
 * most eight query heads per kv head and fields of at most 5 bits); at 129 to 256 (with at most eight query heads per
 * kv head) only the first two cases; otherwise, or with these bits, a kernel ahead rotates
 * the queries and one behind merges the partials; the ways differ in the rounding of the last bits).  A number of
 * wavefronts other than 0 switches the choice of run lengths for whole regions off.  The process-wide defaults are read once from the environment variables WEED_HIP_DECODE_WAVES,
 * WEED_HIP_DECODE_SKEW and WEED_HIP_DECODE_SEARCH; with WEED_HIP_DECODE_PLAN=1 every decode call writes the partition
 * it chose (run length, wavefronts, which of the cases above) to stderr. */
int weed_hip_kv_decode_tuning(int32_t wavefronts, int32_t skew_percent, int32_t always_search);

/* weed_hip_kv_decode_attn for callers that cannot allocate device memory (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results; the workspace (rotated queries, split partials) is a 32 MiB array that is part of the
 * library's device image and that every device the library was initialised on holds until the process ends.  Calls
 * no hipMalloc / hipFree and creates no events (the library's timing scopes skip it).  Shapes whose workspace
 * 64 KiB + n_seq * n_q_heads * (d * 8 + 8 + slots * (d + 2) * 4) bytes (slots: context splits, at most a few dozen)
 * exceeds the array return WEED_HIP_EINVAL.  The first 64 KiB are arrival counters of the kernel's own merge: they start
 * as zeros with the array and every launch that completes leaves them at zero; weed_hip_kv_cache_reset (of any cache)
 * and weed_hip_shutdown clear them too, which is how a process recovers them after a launch the device aborted.  All calls on one device share the
 * array: calls that overlap on one device (two host threads, two streams) race; weed_hip_init must have run on the
 * device. */
int weed_hip_kv_decode_attn_noalloc(weed_hip_kv_cache *cache, int32_t n_q_heads, int32_t gqa_mapping,
                                    const float *q_dev, uint32_t q_off, const uint32_t q_stride[3], float *out_dev,
                                    uint32_t o_off, const uint32_t o_stride[3], uint32_t flags);

/* The same, attending only over the first lens_dev[s] tokens of sequence s (device array of n_seq lengths, each at
 * most the cached length).  This is how a causal mask with a cache offset is expressed for one query position at a
 * time: the reference adds a triangular mask to a dense score matrix instead (multihead_attention.cpp:322-328,
 * src/ops/triu_fill.cpp:42-59). */
int weed_hip_kv_decode_attn_prefix(weed_hip_kv_cache *cache, const int32_t *lens_dev, int32_t n_q_heads,
                                   int32_t gqa_mapping, const float *q_dev, uint32_t q_off, const uint32_t q_stride[3],
                                   float *out_dev, uint32_t o_off, const uint32_t o_stride[3], uint32_t flags);

/* A chunk of n_tokens (1..64) query positions per sequence with the causal mask inside the kernel (speculative or
 * chunked decoding; MultiHeadAttention::forward with 1 < T, multihead_attention.cpp:259-348 with the triangular mask of
 * 322-328).  The last n_tokens of the attended tokens (lens_dev[s], or the cached length when lens_dev is NULL) are
 * the chunk's own: position t attends to all but the last n_tokens - 1 - t of them.  q_dev / out_dev: logical
 * [n_seq, n_tokens, n_q_heads, d] with strides in elements.  The (position, head) pairs of a KV head are the rows of
 * matrix tiles of 16 (8 above head_dim 128): up to that many pairs cost ONE pass over the packed cache, more pairs
 * one pass per tile.  Needs a shape the matrix-core kernel serves: fields of 2..5 bits, or of equal width 1, 6, 7
 * or 8 (up to 4 bits above head_dim 128). */
int weed_hip_kv_decode_attn_chunk(weed_hip_kv_cache *cache, const int32_t *lens_dev, int32_t n_tokens,
                                  int32_t n_q_heads, int32_t gqa_mapping, const float *q_dev, uint32_t q_off,
                                  const uint32_t q_stride[4], float *out_dev, uint32_t o_off,
                                  const uint32_t o_stride[4], uint32_t flags);

#ifdef __cplusplus
}
#endif
#endif
