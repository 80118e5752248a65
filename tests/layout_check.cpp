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
    // groups of 32 fields
    for (uint32_t w = 1; w <= 5; ++w) {
        uint32_t all[5] = { 0, 0, 0, 0, 0 };
        for (uint32_t f = 0; f < 32; ++f) {
            uint32_t m[5] = { 0, 0, 0, 0, 0 };
            group_field_mask(m, f, w);
            uint32_t bits = 0;
            for (uint32_t k = 0; k < 5; ++k) {
                CHECK(k < w || m[k] == 0);
                CHECK((all[k] & m[k]) == 0); // fields never overlap
                all[k] |= m[k];
                bits += (uint32_t)__builtin_popcount(m[k]);
            }
            CHECK(bits == w);
        }
        for (uint32_t k = 0; k < w; ++k) {
            CHECK(all[k] == 0xffffffffu); // no bit is wasted
        }
        std::srand(w);
        for (int trial = 0; trial < 50; ++trial) {
            uint32_t g[5] = { 0, 0, 0, 0, 0 }, vals[32];
            for (uint32_t f = 0; f < 32; ++f) {
                vals[f] = (uint32_t)std::rand() & ((1u << w) - 1u);
                group_or(g, f, w, vals[f]);
            }
            for (uint32_t f = 0; f < 32; ++f) {
                CHECK(group_get(g, f, w) == vals[f]);
            }
        }
        // pair structure the decode kernel relies on: both fields of a pair sit in the same dword (or both in
        // the spare value), the second one w bits above the first
        for (uint32_t P = 0; P < 16; ++P) {
            const FieldPos a = field_pos(2 * P, w), b = field_pos(2 * P + 1, w);
            CHECK(a.dword == b.dword && b.bit == a.bit + w);
        }
    }
    // token / coordinate addressing
    const uint32_t dims[] = { 32, 64, 96, 128, 256 };
    for (uint32_t d : dims) {
        for (uint32_t w = 1; w <= 5; ++w) {
            const uint32_t max_tokens = 200; // 4 blocks after padding
            const uint64_t region = region_dwords(max_tokens, d, w);
            CHECK(padded_tokens(max_tokens) == 256);
            CHECK(region == 4ull * 2 * d * w);
            std::set<uint64_t> seen;
            for (uint32_t n = 0; n < 256; ++n) {
                for (uint32_t G = 0; G < d / 32; ++G) {
                    const uint64_t idx = k_group_index(n, G, d, w);
                    CHECK(idx % w == 0 && idx + w <= region);
                    CHECK(idx / block_dwords(d, w) == n / 64); // a block holds exactly its 64 tokens
                    CHECK(seen.insert(idx).second);
                }
            }
            CHECK(seen.size() * w == region);
            std::set<std::pair<uint64_t, uint32_t>> vseen;
            std::set<uint64_t> vdwords;
            for (uint32_t n = 0; n < 256; ++n) {
                for (uint32_t j = 0; j < d; ++j) {
                    const VPos p = v_pos(n, j, d, w);
                    CHECK(p.field < 32);
                    CHECK(p.base + (uint64_t)(w - 1) * p.stride < region);
                    CHECK(p.base / block_dwords(d, w) == n / 64);
                    CHECK(vseen.insert(std::make_pair(p.base, p.field)).second);
                    for (uint32_t m = 0; m < w; ++m) {
                        vdwords.insert(p.base + (uint64_t)m * p.stride);
                    }
                    const uint32_t u = ((n & 63) >> 4) >> 1;
                    CHECK(v_field_token(u, p.field) == (n & 63));
                }
            }
            CHECK(vseen.size() == 256ull * d);
            CHECK(vdwords.size() == region);
        }
    }
    std::printf("OK\n");
    return 0;
}
