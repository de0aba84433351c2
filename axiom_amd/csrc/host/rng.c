/* xoshiro256** with splitmix64 seeding, per thread (Axiom's src/core/rng.c): identical
 * output sequence for a given seed, including the cached second value of the polar normal. */
#include <math.h>
#include <time.h>
#include <unistd.h>

#include "axiom/rng.h"

static _Thread_local uint64_t tl_s[4];
static _Thread_local bool tl_seeded = false;
static _Thread_local bool tl_have_spare = false;
static _Thread_local float tl_spare = 0.0f;

static uint64_t splitmix(uint64_t *ctr) {
    uint64_t z = (*ctr += 0x9e3779b97f4a7c15ULL);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

static inline uint64_t rol(uint64_t v, int r) { return (v << r) | (v >> (64 - r)); }

void ax_rng_seed(uint64_t seed) {
    uint64_t ctr = seed;
    for (int i = 0; i < 4; i++) tl_s[i] = splitmix(&ctr);
    tl_seeded = true;
}

bool ax_rng_is_seeded(void) { return tl_seeded; }

uint64_t ax_rng_uint64(void) {
    if (!tl_seeded) {   /* first use without a seed: time and pid, as the reference does */
        uint64_t t = (uint64_t)time(NULL), p = (uint64_t)getpid();
        ax_rng_seed(t ^ (p << 32) ^ (p * 0x517cc1b727220a95ULL));
    }
    const uint64_t out = rol(tl_s[1] * 5, 7) * 9;
    const uint64_t sh = tl_s[1] << 17;
    tl_s[2] ^= tl_s[0];
    tl_s[3] ^= tl_s[1];
    tl_s[1] ^= tl_s[2];
    tl_s[0] ^= tl_s[3];
    tl_s[2] ^= sh;
    tl_s[3] = rol(tl_s[3], 45);
    return out;
}

float ax_rng_float(void) { return (float)(ax_rng_uint64() >> 40) * 0x1.0p-24f; }
float ax_rng_uniform(float low, float high) { return low + ax_rng_float() * (high - low); }

float ax_rng_normal(void) {
    if (tl_have_spare) {
        tl_have_spare = false;
        return tl_spare;
    }
    float u, v, r2;
    do {
        u = ax_rng_float() * 2.0f - 1.0f;
        v = ax_rng_float() * 2.0f - 1.0f;
        r2 = u * u + v * v;
    } while (r2 >= 1.0f || r2 == 0.0f);
    const float f = sqrtf(-2.0f * logf(r2) / r2);
    tl_spare = v * f;
    tl_have_spare = true;
    return u * f;
}

float ax_rng_normal_params(float mean, float std) { return mean + std * ax_rng_normal(); }

uint64_t ax_rng_bounded(uint64_t n) {
    if (n <= 1) return 0;
    const uint64_t reject_below = (0 - n) % n;
    for (;;) {
        uint64_t r = ax_rng_uint64();
        if (r >= reject_below) return r % n;
    }
}
