/* TEST INFRASTRUCTURE — the benchmark harness's input generator: one
 * std::mt19937_64 stream per tensor (seed = base seed + tensor id), so that the
 * GPU side and the CPU baseline of bench.py are fed identical bits.
 * Uniform numbers are (x >> 40) * 2^-24, normal ones come from Box-Muller on
 * those.  The generator is the published MT19937-64 recurrence (Matsumoto &
 * Nishimura), pinned by the C++ standard's known answer: the 10000th output of
 * a generator seeded with 5489 is 9981545732273789042 (tests/test_harness_rng.py).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define NN 312
#define MM 156
#define UM 0xFFFFFFFF80000000ULL
#define LM 0x7FFFFFFFULL

typedef struct {
  uint64_t mt[NN];
  int idx;
} mt64;

static void mt64_seed(mt64 *g, uint64_t seed) {
  g->mt[0] = seed;
  for (int i = 1; i < NN; ++i) g->mt[i] = 6364136223846793005ULL * (g->mt[i - 1] ^ (g->mt[i - 1] >> 62)) + (uint64_t)i;
  g->idx = NN;
}

static uint64_t mt64_next(mt64 *g) {
  if (g->idx >= NN) {
    int i;
    for (i = 0; i < NN - MM; ++i) {
      uint64_t const x = (g->mt[i] & UM) | (g->mt[i + 1] & LM);
      g->mt[i] = g->mt[i + MM] ^ (x >> 1) ^ ((x & 1ULL) ? 0xB5026F5AA96619E9ULL : 0ULL);
    }
    for (; i < NN - 1; ++i) {
      uint64_t const x = (g->mt[i] & UM) | (g->mt[i + 1] & LM);
      g->mt[i] = g->mt[i + (MM - NN)] ^ (x >> 1) ^ ((x & 1ULL) ? 0xB5026F5AA96619E9ULL : 0ULL);
    }
    uint64_t const x = (g->mt[NN - 1] & UM) | (g->mt[0] & LM);
    g->mt[NN - 1] = g->mt[MM - 1] ^ (x >> 1) ^ ((x & 1ULL) ? 0xB5026F5AA96619E9ULL : 0ULL);
    g->idx = 0;
  }
  uint64_t x = g->mt[g->idx++];
  x ^= (x >> 29) & 0x5555555555555555ULL;
  x ^= (x << 17) & 0x71D67FFFEDA60000ULL;
  x ^= (x << 37) & 0xFFF7EEE000000000ULL;
  x ^= (x >> 43);
  return x;
}

static float u24(mt64 *g) { return (float)(mt64_next(g) >> 40) * (1.0f / 16777216.0f); }

void dlo_rng_raw(uint64_t seed, size_t n, uint64_t *out) {
  mt64 g;
  mt64_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) out[i] = mt64_next(&g);
}

/* out[i] = lo + (hi - lo) * u, u in [0, 1) */
void dlo_rng_uniform(uint64_t seed, size_t n, float lo, float hi, float *out) {
  mt64 g;
  mt64_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) out[i] = lo + (hi - lo) * u24(&g);
}

/* standard normal by Box-Muller: two uniforms give two normals (u1 shifted into (0, 1]) */
void dlo_rng_normal(uint64_t seed, size_t n, float *out) {
  mt64 g;
  mt64_seed(&g, seed);
  for (size_t i = 0; i < n; i += 2) {
    double const u1 = ((double)(mt64_next(&g) >> 40) + 1.0) * (1.0 / 16777216.0);
    double const u2 = (double)(mt64_next(&g) >> 40) * (1.0 / 16777216.0);
    double const rad = sqrt(-2.0 * log(u1)), ang = 6.283185307179586476925 * u2;
    out[i] = (float)(rad * cos(ang));
    if (i + 1 < n) out[i + 1] = (float)(rad * sin(ang));
  }
}

/* out[i] = 1 with probability keep */
void dlo_rng_bernoulli_u8(uint64_t seed, size_t n, float keep, uint8_t *out) {
  mt64 g;
  mt64_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) out[i] = u24(&g) < keep ? 1 : 0;
}

/* out[i] = u mod k (labels) */
void dlo_rng_index(uint64_t seed, size_t n, uint32_t k, uint32_t *out) {
  mt64 g;
  mt64_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) out[i] = (uint32_t)(mt64_next(&g) % k);
}
