// Device twin of Weed::QuantizedKVCache (include/modules/multihead_attention.hpp:22-36) plus the state
// MultiHeadAttention keeps beside it (k_rotation, v_rotation, v_rotation_trans, cache_len; hpp:56-68).
#pragma once

#include <vector>

#include "common.h"
#include "kv_layout.h"

namespace weedhip {

// What a kernel needs to turn one tensor's fields back into numbers: value = alpha * table[field] + beta,
// with alpha the row scale (LLOYDMAX) or the cell width (UNIFORM, where table[c] = c + 0.5 and beta = -3s).
struct SideParams {
    const uint8_t *fields;  // packed items, one region per (sequence, kv head)
    const float *alpha;     // [n_seq][n_kv_heads][padded_tokens] row scales, LLOYDMAX only
    const uint32_t *alpha_max; // [n_seq][n_kv_heads][kScaleMaxSlots]: the largest of them is the bit pattern of the largest row scale seen, LLOYDMAX only
    uint64_t region_bytes;
    uint32_t w;             // field width
    float alpha_const;      // UNIFORM: step
    float beta;             // UNIFORM: lo
    float table[32];        // reconstruction levels, 2^w entries
};

struct Side {
    int bits = 0;
    int sign = 0;
    uint32_t w = 0;
    uint8_t *fields = nullptr;
    float *alpha = nullptr;
    uint32_t *alpha_max = nullptr;
    uint64_t region_bytes = 0;
    float block_scale = 1.0f; // UNIFORM (Weed: QuantizedKVCache::block_scale)
    float bounds[15] = {};
    float levels[16] = {};
    float recon[32] = {};
    float *rot = nullptr;   // column-major d x d (k_rotation / v_rotation)
    float *rot_t = nullptr; // its transpose (v_rotation_trans and the coalesced form of k_rotation)
};

} // namespace weedhip

struct weed_hip_kv_cache {
    weed_hip_kv_config cfg;
    // head_dim as stored: cfg.head_dim rounded up to a multiple of 32.  Rows are coded with zeros in the coordinates
    // beyond cfg.head_dim (the query has zeros there too, so their key fields are inert; their value coordinates
    // are never written out) and the rotations are kept as dp x dp matrices with an identity block for them.  Every
    // layout, kernel instance and scratch size below goes by dp; cfg.head_dim bounds what is read from and written
    // to the caller's tensors and enters the two scale factors sqrt(head_dim).
    uint32_t dp = 0;
    uint32_t padded_tokens = 0;
    weedhip::Side k, v;
    bool has_rotations = false;
    std::vector<int32_t> lens; // host mirror of lens_dev
    std::vector<uint64_t> plan_region_end; // host scratch of the decode planner, kept between calls
    int32_t *lens_dev = nullptr;
    uint32_t *append_done = nullptr; // behind lens_dev: workgroups of the append under way that are through
    // scratch for encode: one field per byte + row scales for the tokens being appended
    uint8_t *enc_fields = nullptr;
    float *enc_alpha = nullptr;
    size_t enc_rows_cap = 0;
    // scratch for decode: rotated queries and split partials
    float *dec_ws = nullptr;
    size_t dec_ws_bytes = 0;
    // LDS image of both sides' lookup tables for the matrix-core decode kernel (kMfmaTableImageBytes), rebuilt
    // whenever the tables change
    uint32_t *table_image = nullptr;
};

namespace weedhip {
// Builds the kernel-side view of one tensor of the cache.
SideParams side_params(const weed_hip_kv_cache *c, int which);
// (Re)builds c->table_image from the current tables; a blocking copy, done when a cache is created or its tables set.
int upload_table_image(weed_hip_kv_cache *c);
} // namespace weedhip
