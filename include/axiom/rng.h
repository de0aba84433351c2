/* axiom/rng.h — xoshiro256** generator of the Axiom C API (include/axiom/rng.h,
 * src/core/rng.c): same seeding, same float mapping, same polar normal, so seeded
 * weights match the reference bit for bit. */
#ifndef AX_RNG_H
#define AX_RNG_H
#include <stdbool.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
void     ax_rng_seed(uint64_t seed);
bool     ax_rng_is_seeded(void);
uint64_t ax_rng_uint64(void);
float    ax_rng_float(void);                    /* [0,1), 24 bits */
float    ax_rng_uniform(float low, float high);
float    ax_rng_normal(void);
float    ax_rng_normal_params(float mean, float std);
uint64_t ax_rng_bounded(uint64_t n);            /* [0,n) without modulo bias */
#ifdef __cplusplus
}
#endif
#endif
