// CPU check of the packed-cache layout arithmetic in weed_amd/csrc/kv_layout.h (built and run by
// tests/test_layout_cpu.py with g++; no GPU involved).
#include <cstdio>
#include <cstdlib>
#include <set>
#include <utility>
#include <vector>

#include "../weed_amd/csrc/kv_layout.h"

using namespace weedkv;

#define CHECK(cond)                                                                                                    \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                              \
            return 1;                                                                                                  \
        }                                                                                                              \
    } while (0)

int main()
{
    // items: 8 fields of w bits in w bytes
    for (uint32_t w = 1; w <= 8; ++w) {
        std::srand(w);
        for (int trial = 0; trial < 200; ++trial) {
            uint8_t f8[8], bytes[9] = { 0 };
            for (uint32_t e = 0; e < 8; ++e) {
                f8[e] = (uint8_t)(std::rand() & ((1 << w) - 1));
            }
            item_build(f8, w, bytes);
            uint64_t bits = 0;
            for (uint32_t b = 0; b < w; ++b) {
                bits |= (uint64_t)bytes[b] << (8 * b);
            }
            for (uint32_t e = 0; e < 8; ++e) {
                CHECK(item_get(bytes, e * w, w) == f8[e]);
                CHECK(((bits >> (e * w)) & ((1u << w) - 1)) == f8[e]); // little-endian bit string
            }
            CHECK(bytes[w] == 0); // exactly w bytes are written
        }
    }
    // token / coordinate addressing: every (token, coordinate) gets its own field, blocks hold exactly their 64
    // tokens, no byte of a region is wasted
    const uint32_t dims[] = { 32, 64, 96, 128, 256 };
    for (uint32_t d : dims) {
        for (uint32_t w = 1; w <= 8; ++w) {
            const uint32_t max_tokens = 200; // 4 blocks after padding
            const uint64_t region = region_bytes(max_tokens, d, w);
            CHECK(padded_tokens(max_tokens) == 256);
            CHECK(region == 4ull * 8 * d * w && region % 16 == 0);
            for (int which = 0; which < 2; ++which) {
                std::set<std::pair<uint64_t, uint32_t>> seen;
                std::set<uint64_t> items;
                for (uint32_t n = 0; n < 256; ++n) {
                    for (uint32_t j = 0; j < d; ++j) {
                        const FieldPos p = which ? v_field_pos(n, j, d, w) : k_field_pos(n, j, d, w);
                        CHECK(p.byte % w == 0 && p.byte + w <= region);
                        CHECK(p.bit % w == 0 && p.bit < 8 * w);
                        CHECK(p.byte / block_bytes(d, w) == n / 64);
                        CHECK(seen.insert(std::make_pair(p.byte, p.bit)).second);
                        items.insert(p.byte);
                    }
                }
                CHECK(seen.size() == 256ull * d);
                CHECK(items.size() * w == region);
            }
            // K: the 8 fields of an item are 8 consecutive coordinates of one token; a lane's items are contiguous
            for (uint32_t n = 0; n < 64; ++n) {
                for (uint32_t j = 0; j < d; j += 8) {
                    const FieldPos p0 = k_field_pos(n, j, d, w);
                    for (uint32_t e = 0; e < 8; ++e) {
                        const FieldPos p = k_field_pos(n, j + e, d, w);
                        CHECK(p.byte == p0.byte && p.bit == e * w);
                    }
                }
                const uint32_t r = n & 15, t = n >> 4;
                for (uint32_t g = 0; g < 4; ++g) {
                    const uint64_t lane_base = (uint64_t)(g * 16 + r) * 4 * (d / 32) * w;
                    for (uint32_t ks = 0; ks < d / 32; ++ks) {
                        CHECK(k_field_pos(n, g * (d / 4) + 8 * ks, d, w).byte == lane_base + (t * (d / 32) + ks) * w);
                    }
                }
            }
            // V: the 8 fields of an item are the tokens v_item_token(u, g, e) of one coordinate
            for (uint32_t u = 0; u < 2; ++u) {
                for (uint32_t g = 0; g < 4; ++g) {
                    for (uint32_t j = 0; j < d; ++j) {
                        const FieldPos p0 = v_field_pos(v_item_token(u, g, 0), j, d, w);
                        CHECK(p0.byte == (uint64_t)(((g * 16 + (j & 15)) * 2 + u) * (d / 16) + (j >> 4)) * w);
                        for (uint32_t e = 0; e < 8; ++e) {
                            const FieldPos p = v_field_pos(v_item_token(u, g, e), j, d, w);
                            CHECK(p.byte == p0.byte && p.bit == e * w);
                        }
                    }
                }
            }
            // every token of a block appears exactly once among the item slots
            std::set<uint32_t> toks;
            for (uint32_t u = 0; u < 2; ++u) {
                for (uint32_t g = 0; g < 4; ++g) {
                    for (uint32_t e = 0; e < 8; ++e) {
                        toks.insert(v_item_token(u, g, e));
                    }
                }
            }
            CHECK(toks.size() == 64 && *toks.rbegin() == 63);
        }
    }
    std::printf("OK\n");
    return 0;
}
