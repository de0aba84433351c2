/* Per-thread pseudo-random numbers with the output sequence of Axiom's generator (src/core/rng.c):
 * the xoshiro256** recurrence, its state filled from the seed by four splitmix64 steps; floats
 * from the top 24 bits; normals by the polar method, which yields two values per accepted point
 * (the second is kept for the next call).  Seeded weights therefore match the reference bit for
 * bit (known answers in the tests). */
#include <math.h>
#include <time.h>
#include <unistd.h>

#include "axiom/rng.h"

typedef struct {
    uint64_t word[4];      /* xoshiro256** state */
    float kept;            /* second value of the last accepted polar point */
    bool ready, has_kept;
} generator_t;

static _Thread_local generator_t tl_gen;

/* one step of the splitmix64 sequence that starts at *counter */
static uint64_t splitmix64_next(uint64_t *counter) {
    *counter += UINT64_C(0x9e3779b97f4a7c15);
    uint64_t mixed = *counter;
    mixed ^= mixed >> 30;
    mixed *= UINT64_C(0xbf58476d1ce4e5b9);
    mixed ^= mixed >> 27;
    mixed *= UINT64_C(0x94d049bb133111eb);
    mixed ^= mixed >> 31;
    return mixed;
}

#define ROTATE_LEFT(value, bits) (((value) << (bits)) | ((value) >> (64 - (bits))))

void ax_rng_seed(uint64_t seed) {
    generator_t *g = &tl_gen;
    uint64_t counter = seed;
    g->word[0] = splitmix64_next(&counter);
    g->word[1] = splitmix64_next(&counter);
    g->word[2] = splitmix64_next(&counter);
    g->word[3] = splitmix64_next(&counter);
    g->ready = true;
}

bool ax_rng_is_seeded(void) { return tl_gen.ready; }

/* a first draw without a seed takes one from the clock and the process id, as the reference does */
static void seed_from_environment(void) {
    const uint64_t now = (uint64_t)time(NULL), pid = (uint64_t)getpid();
    ax_rng_seed(now ^ (pid << 32) ^ (pid * UINT64_C(0x517cc1b727220a95)));
}

uint64_t ax_rng_uint64(void) {
    generator_t *g = &tl_gen;
    if (!g->ready) seed_from_environment();
    uint64_t a = g->word[0], b = g->word[1], c = g->word[2], d = g->word[3];
    const uint64_t result = ROTATE_LEFT(b * 5, 7) * 9;
    const uint64_t shifted = b << 17;
    c ^= a;
    d ^= b;
    b ^= c;
    a ^= d;
    c ^= shifted;
    d = ROTATE_LEFT(d, 45);
    g->word[0] = a;
    g->word[1] = b;
    g->word[2] = c;
    g->word[3] = d;
    return result;
}

/* [0, 1): the top 24 bits of a draw, scaled by 2^-24 */
float ax_rng_float(void) { return ldexpf((float)(ax_rng_uint64() >> 40), -24); }

float ax_rng_uniform(float low, float high) {
    const float unit = ax_rng_float();
    return low + unit * (high - low);
}

float ax_rng_normal(void) {
    generator_t *g = &tl_gen;
    if (g->has_kept) {
        g->has_kept = false;
        return g->kept;
    }
    for (;;) {
        const float x = ax_rng_float() * 2.0f - 1.0f;
        const float y = ax_rng_float() * 2.0f - 1.0f;
        const float radius2 = x * x + y * y;
        if (radius2 >= 1.0f || radius2 == 0.0f) continue;     /* outside the unit disc, or its centre */
        const float factor = sqrtf(-2.0f * logf(radius2) / radius2);
        g->kept = y * factor;
        g->has_kept = true;
        return x * factor;
    }
}

float ax_rng_normal_params(float mean, float std) { return mean + std * ax_rng_normal(); }

/* uniform on [0, n) by rejection: draws below 2^64 mod n would make some residues more likely */
uint64_t ax_rng_bounded(uint64_t n) {
    if (n < 2) return 0;
    const uint64_t threshold = (UINT64_C(0) - n) % n;
    uint64_t draw = ax_rng_uint64();
    while (draw < threshold) draw = ax_rng_uint64();
    return draw % n;
}
