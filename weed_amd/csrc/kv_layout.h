// Packed-cache layout of libweed_hip, shared by host code, every kernel and the CPU layout test.
//
// A *field* is what one coordinate of one cached row stores: the scalar code, or (code << 1) | sign when a
// residual sign bit is kept.  Field width w = bits + sign, 1..5.
//
// Fields are stored in *groups of 32*: 32 fields in exactly w dwords.
//   K cache: a group is 32 consecutive coordinates of one token.
//   V cache: a group is one coordinate of 32 tokens (half of a 64-token block).
// Inside a group the 32 fields form 16 pairs (fields 2P, 2P+1); pair P = 4*g + p is "slot (g, p)": the decode kernel's
// lane-group g consumes the four pairs of slot row g, one MFMA operand register per pair.
//
//   w = 1, 2, 4 : fields in index order, field f at bit f*w of the group's bit string.
//   w = 3       : dword g (g < 3) holds slot row g in bits 0..23 (pair p at bit 6p) and pair (3, g) in bits 24..29;
//                 pair (3, 3) is assembled from bits 30..31 of the three dwords (dword m supplies bits 2m, 2m+1).
//   w = 5       : pair P < 15 sits in dword P/3 at bit 10*(P%3); pair 15 is assembled from bits 30..31 of the five
//                 dwords (dword m supplies bits 2m, 2m+1).
//
// Tokens are stored in blocks of 64.  With groups = d/32, a block of either cache is 2*d*w dwords.
//   K block: dword ((G*16 + r)*4 + t)*w + m   holds dword m of coordinate group G of token 16*t + r.
//            A lane (r, G) of the decode kernel therefore reads 4*w consecutive dwords: its rows of all four
//            16-token tiles.
//   V block: dword ((m*16 + c)*2 + u)*(d/16) + jb   holds dword m of the group of coordinate 16*jb + c, half u.
//            Field 8*g + i of that group belongs to token 16*(2u + i/4) + 4*g + i%4, which is the order in which
//            the score tile leaves the Q.K^T matrix instruction.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define WK_HD __host__ __device__ __forceinline__
#else
#define WK_HD inline
#endif

namespace weedkv {

constexpr uint32_t kBlockTokens = 64;

struct FieldPos {
    uint32_t dword; // dword within the group, or 0xffffffff when the field lives in the spare bits
    uint32_t bit;   // bit offset inside that dword, or bit offset inside the assembled spare value
};

WK_HD FieldPos field_pos(uint32_t f, uint32_t w)
{
    FieldPos r;
    if (w == 3) {
        const uint32_t P = f >> 1, half = f & 1;
        if (P < 12) {
            r.dword = P >> 2;
            r.bit = 6 * (P & 3) + 3 * half;
        } else if (P < 15) {
            r.dword = P - 12;
            r.bit = 24 + 3 * half;
        } else {
            r.dword = 0xffffffffu;
            r.bit = 3 * half;
        }
    } else if (w == 5) {
        const uint32_t P = f >> 1, half = f & 1;
        if (P < 15) {
            r.dword = P / 3;
            r.bit = 10 * (P % 3) + 5 * half;
        } else {
            r.dword = 0xffffffffu;
            r.bit = 5 * half;
        }
    } else {
        const uint32_t b = f * w;
        r.dword = b >> 5;
        r.bit = b & 31;
    }
    return r;
}

// Value assembled from bits 30..31 of each dword (odd widths only).
WK_HD uint32_t group_spare(const uint32_t *g, uint32_t w)
{
    uint32_t s = 0;
    for (uint32_t m = 0; m < w; ++m) {
        s |= (g[m] >> 30) << (2 * m);
    }
    return s;
}

WK_HD uint32_t group_get(const uint32_t *g, uint32_t f, uint32_t w)
{
    const FieldPos p = field_pos(f, w);
    const uint32_t mask = (1u << w) - 1u;
    if (p.dword == 0xffffffffu) {
        return (group_spare(g, w) >> p.bit) & mask;
    }
    return (g[p.dword] >> p.bit) & mask;
}

// ORs field f into a group whose bits for f are zero.
WK_HD void group_or(uint32_t *g, uint32_t f, uint32_t w, uint32_t val)
{
    const FieldPos p = field_pos(f, w);
    if (p.dword == 0xffffffffu) {
        const uint32_t s = val << p.bit; // bits of the assembled spare value
        for (uint32_t m = 0; m < w; ++m) {
            g[m] |= ((s >> (2 * m)) & 3u) << 30;
        }
        return;
    }
    g[p.dword] |= val << p.bit;
}

// Mask, per dword, of the bits field f occupies.
WK_HD void group_field_mask(uint32_t *mask, uint32_t f, uint32_t w)
{
    group_or(mask, f, w, (1u << w) - 1u);
}

WK_HD uint32_t block_dwords(uint32_t d, uint32_t w) { return 2u * d * w; }

WK_HD uint32_t padded_tokens(uint32_t max_tokens) { return (max_tokens + kBlockTokens - 1) / kBlockTokens * kBlockTokens; }

// dwords per (sequence, kv head) region
WK_HD uint64_t region_dwords(uint32_t max_tokens, uint32_t d, uint32_t w)
{
    return (uint64_t)(padded_tokens(max_tokens) / kBlockTokens) * block_dwords(d, w);
}

// K cache: index (within the region) of dword 0 of coordinate group G of token n.
WK_HD uint64_t k_group_index(uint32_t n, uint32_t G, uint32_t d, uint32_t w)
{
    const uint32_t block = n >> 6, t = (n >> 4) & 3, r = n & 15;
    return (uint64_t)block * block_dwords(d, w) + (uint64_t)(((G * 16 + r) * 4 + t) * w);
}

// V cache: where the field of (token n, coordinate j) lives.
struct VPos {
    uint64_t base;   // index (within the region) of dword 0 of the group; dword m is at base + m*stride
    uint32_t stride; // distance between the dwords of one group
    uint32_t field;  // field index inside the group
};

WK_HD VPos v_pos(uint32_t n, uint32_t j, uint32_t d, uint32_t w)
{
    const uint32_t block = n >> 6, nb = n & 63;
    const uint32_t t = nb >> 4, u = t >> 1, rr = nb & 15;
    const uint32_t g = rr >> 2, i = (rr & 3) + 4 * (t & 1);
    const uint32_t c = j & 15, jb = j >> 4;
    VPos p;
    p.stride = 16 * 2 * (d / 16);
    p.base = (uint64_t)block * block_dwords(d, w) + (uint64_t)((c * 2 + u) * (d / 16) + jb);
    p.field = 8 * g + i;
    return p;
}

// Inverse of the token part of v_pos: token (inside its 64-block) of field f of half u.
WK_HD uint32_t v_field_token(uint32_t u, uint32_t f)
{
    const uint32_t g = f >> 3, i = f & 7;
    return 16 * (2 * u + (i >> 2)) + 4 * g + (i & 3);
}

} // namespace weedkv
