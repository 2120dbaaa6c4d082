/*
 * CPU oracle, test infrastructure only: random streams.
 *
 * SplitMix64 / xoshiro256++ follow sampling.rs:1621-1670 and are pinned by the
 * golden vectors of sampling.rs:1817-1864.  Philox4x32-10 is the published
 * Random123 generator (Salmon et al., SC'11), pinned by its known-answer vectors;
 * the reference has no Philox, it exists here for the counter-based stream the
 * stochastic-acceptance workload asks for.
 */
#include "dflash_oracle.h"

uint64_t orc_splitmix64_next(uint64_t *state) {
    *state += 0x9e3779b97f4a7c15ull;
    uint64_t v = *state;
    v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
    v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
    return v ^ (v >> 31);
}

void orc_xoshiro_seed(uint64_t seed, uint64_t s[4]) {
    uint64_t sm = seed;
    for (int i = 0; i < 4; i++) s[i] = orc_splitmix64_next(&sm);
}

static uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

uint64_t orc_xoshiro_next(uint64_t s[4]) {
    uint64_t result = rotl64(s[0] + s[3], 23) + s[0];
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}

/* sampling.rs:1654-1657 */
double orc_unit_f64(uint64_t raw) { return (double)(raw >> 11) / 9007199254740992.0; }

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; round++) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}
