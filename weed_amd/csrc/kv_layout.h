// Packed-cache layout of libweed_hip, shared by host code, every kernel and the CPU layout test.
//
// A *field* is what one coordinate of one cached row stores: the scalar code, or (code << 1) | sign when a
// residual sign bit is kept.  Field width w = bits + sign: 1..5 with Lloyd-Max codes, 1..8 with Weed's uniform coder.
//
// Fields are stored in *items*: 8 fields in exactly w bytes, field e at bits [e*w, (e+1)*w) of the item
// (little-endian bit string).  Consecutive fields (2p, 2p+1) form *pair* p of the item: the decode kernel turns one
// pair into one 32-bit matrix-operand register (two fp16 values) with a single table lookup.
//
// Tokens are stored in blocks of 64 = 4 tiles of 16.  With d = head_dim, a block of either cache is 8*d*w bytes and
// is laid out so that each lane of the decode kernel's 64-lane wavefront reads ONE contiguous run of bytes.  A lane
// is (r, g): r = lane % 16, g = lane / 16.
//
//   K block: lane (r, g) owns token rows 16*t + r (t = 0..3) and the coordinates [g*d/4, (g+1)*d/4), as d/32 items
//            per tile:  item (g, r, t, ks) holds coordinates g*d/4 + 8*ks + e (e = 0..7) of token 16*t + r, at byte
//            (((g*16 + r)*4 + t)*(d/32) + ks)*w.   Token rows feed the A operand of the Q.K^T matrix instruction.
//
//   V block: lane (c, g) owns the coordinates 16*jb + c (jb = 0..d/16-1) and, in each 32-token half u of the block,
//            the eight tokens 16*(2u + e/4) + 4*g + e%4 (e = 0..7) -- the order in which the score tile leaves the
//            Q.K^T instruction, so probabilities feed the P.V instruction without any cross-lane movement:
//            item (g, c, u, jb) sits at byte (((g*16 + c)*2 + u)*(d/16) + jb)*w.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define WK_HD __host__ __device__ __forceinline__
#else
#define WK_HD inline
#endif

namespace weedkv {

constexpr uint32_t kBlockTokens = 64;
// The largest row scale of a region is kept as the maximum over this many words (64 bytes per region): the encoder's
// workgroups raise different words, because raising ONE word from the 128 workgroups of a 4096-token prefill is served
// one after the other (4 us of a 45 us encode); a reader takes the largest of them.
constexpr uint32_t kScaleMaxSlots = 16;

WK_HD uint32_t block_bytes(uint32_t d, uint32_t w) { return 8u * d * w; }

WK_HD uint32_t padded_tokens(uint32_t max_tokens) { return (max_tokens + kBlockTokens - 1) / kBlockTokens * kBlockTokens; }

// bytes per (sequence, kv head) region; always a multiple of 16
WK_HD uint64_t region_bytes(uint32_t max_tokens, uint32_t d, uint32_t w)
{
    return (uint64_t)(padded_tokens(max_tokens) / kBlockTokens) * block_bytes(d, w);
}

// Position of one field inside a region.
struct FieldPos {
    uint64_t byte; // first byte of the item
    uint32_t bit;  // bit offset of the field inside the item
};

WK_HD FieldPos k_field_pos(uint32_t n, uint32_t j, uint32_t d, uint32_t w)
{
    const uint32_t block = n >> 6, t = (n >> 4) & 3, r = n & 15;
    const uint32_t per_lane = d / 4; // coordinates per lane group
    const uint32_t g = j / per_lane, ks = (j % per_lane) >> 3, e = j & 7;
    FieldPos p;
    p.byte = (uint64_t)block * block_bytes(d, w) + (uint64_t)((((g * 16 + r) * 4 + t) * (d / 32) + ks) * w);
    p.bit = e * w;
    return p;
}

WK_HD FieldPos v_field_pos(uint32_t n, uint32_t j, uint32_t d, uint32_t w)
{
    const uint32_t block = n >> 6, nb = n & 63;
    const uint32_t t = nb >> 4, u = t >> 1, rr = nb & 15;
    const uint32_t g = rr >> 2, e = (rr & 3) + 4 * (t & 1);
    const uint32_t c = j & 15, jb = j >> 4;
    FieldPos p;
    p.byte = (uint64_t)block * block_bytes(d, w) + (uint64_t)((((g * 16 + c) * 2 + u) * (d / 16) + jb) * w);
    p.bit = e * w;
    return p;
}

// Token (inside its 64-block) stored in field e of a V item of lane group g, half u.
WK_HD uint32_t v_item_token(uint32_t u, uint32_t g, uint32_t e) { return 16 * (2 * u + (e >> 2)) + 4 * g + (e & 3); }

// Read / write one field of an item through byte accesses (w <= 8, so a field spans at most two bytes).
WK_HD uint32_t item_get(const uint8_t *item, uint32_t bit, uint32_t w)
{
    const uint32_t b = bit >> 3, s = bit & 7;
    uint32_t v = item[b];
    if (s + w > 8) {
        v |= (uint32_t)item[b + 1] << 8;
    }
    return (v >> s) & ((1u << w) - 1u);
}

// Assemble the w bytes of an item from 8 fields.
WK_HD void item_build(const uint8_t *fields8, uint32_t w, uint8_t *out)
{
    uint64_t bits = 0;
    for (uint32_t e = 0; e < 8; ++e) {
        bits |= (uint64_t)fields8[e] << (e * w);
    }
    for (uint32_t b = 0; b < w; ++b) {
        out[b] = (uint8_t)(bits >> (8 * b));
    }
}

} // namespace weedkv
