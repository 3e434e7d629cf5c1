/*
 * Sanitizer driver for the scalar C emulator (oracle/scalar_ref.c).
 *
 * TEST INFRASTRUCTURE ONLY.  Runs every entry point of the emulator over exactly-sized heap
 * buffers (so that AddressSanitizer sees any access one element past an end), for every dtype,
 * sizes 0, 1 and odd ones on both sides of the reduction block of StableAdamW, every flag
 * combination the entry point reads, NULL for the buffers a variant must not touch, and
 * gradients that include zeros, sub-eps values, huge values and NaN.  Prints one checksum per
 * entry point; the test builds this file twice - with -fsanitize=address,undefined and
 * without - and demands a clean sanitizer run and equal output.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

enum { F32 = 0, BF16 = 1, F16 = 2 };
enum { KAHAN = 1, UPDATE = 2, DECOUPLE_WD = 4, ADAM_WD = 8, DECOUPLE_LR = 16, DAMPENING = 32, RECTIFY = 64, LOOKAHEAD = 128 };

float optimi_ref_round(float x, int dt);
void optimi_ref_adam(void*, const void*, void*, void*, void*, int64_t, int, double, double, double, double, double, double, int);
void optimi_ref_lion(void*, const void*, void*, void*, int64_t, int, double, double, double, double, int);
double optimi_ref_stableadamw(void*, const void*, void*, void*, void*, int64_t, int, double, double, double, double, double,
                              double, double, int);
void optimi_ref_adan(void*, const void*, void*, void*, void*, void*, void*, int64_t, int, double, double, double, double,
                     double, double, double, double, int);
void optimi_ref_sgd(void*, const void*, void*, void*, int64_t, int, double, double, double, int);
void optimi_ref_ranger(void*, const void*, void*, void*, void*, void*, int64_t, int, double, double, double, double, double,
                       double, double, double, int);

static uint64_t rng_state = 88172645463325252ull;
static uint32_t rng(void) {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (uint32_t)(rng_state >> 16);
}
static float uniform(float scale) { return ((float)(rng() & 0xffffff) / 8388608.0f - 1.0f) * scale; }

static size_t esize(int dt) { return dt == F32 ? 4 : 2; }

/* a float as the 16-bit or 32-bit pattern of dtype dt, through the emulator's own rounding */
static void put(void* buf, int64_t i, float x, int dt) {
  float r = optimi_ref_round(x, dt);
  uint32_t u;
  memcpy(&u, &r, 4);
  if (dt == F32) ((uint32_t*)buf)[i] = u;
  else if (dt == BF16) ((uint16_t*)buf)[i] = (uint16_t)(u >> 16);
  else {  /* the rounded value is exactly representable in fp16: rebuild its pattern */
    uint32_t sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
    uint16_t h;
    if (mag == 0) h = 0;
    else if (mag >= 0x7f800000u) h = (uint16_t)(0x7c00u | (mag > 0x7f800000u ? 0x200u : 0u));
    else {
      int e = (int)(mag >> 23) - 127 + 15;
      uint32_t m = mag & 0x7fffffu;
      if (e <= 0) h = (uint16_t)((m | 0x800000u) >> (14 - e));
      else h = (uint16_t)(((uint32_t)e << 10) | (m >> 13));
    }
    ((uint16_t*)buf)[i] = (uint16_t)(h | sign);
  }
}

static void* fresh(int64_t n, int dt, float scale, int special) {
  void* p = malloc(n > 0 ? (size_t)n * esize(dt) : 1);  /* exactly n elements */
  static const float odd[] = {0.0f, -0.0f, 1e-9f, -1e-9f, 1.0f, -65504.0f, 3e-7f};
  for (int64_t i = 0; i < n; ++i) put(p, i, (special && i < 7) ? odd[i] : uniform(scale), dt);
  return p;
}

static uint64_t fnv(uint64_t h, const void* p, int64_t n, int dt) {
  const unsigned char* b = (const unsigned char*)p;
  for (size_t i = 0; i < (size_t)n * esize(dt); ++i) h = (h ^ b[i]) * 1099511628211ull;
  return h;
}

static const int64_t SIZES[] = {0, 1, 3, 31, 33, 1000, 4095, 4097, 8200};

int main(void) {
  const int n_sizes = (int)(sizeof(SIZES) / sizeof(SIZES[0]));
  uint64_t h_adam = 14695981039346656037ull, h_lion = h_adam, h_stable = h_adam, h_adan = h_adam, h_sgd = h_adam, h_ranger = h_adam;
  for (int dt = 0; dt < 3; ++dt)
    for (int si = 0; si < n_sizes; ++si) {
      const int64_t n = SIZES[si];
      for (int variant = 0; variant < 6; ++variant) {
        const int update = variant != 1, kahan = (variant & 1) == 0, low = dt != F32;
        const int base = (update ? UPDATE : 0) | (kahan ? KAHAN : 0);
        const int need_k = kahan && update && low;
        void *p = fresh(n, dt, 0.02f, 0), *g = fresh(n, dt, 1e-3f, 1), *m = fresh(n, dt, 1e-3f, 0), *v = fresh(n, dt, 1e-6f, 0);
        void *d = fresh(n, dt, 1e-3f, 0), *pg = fresh(n, dt, 1e-3f, 0), *la = fresh(n, dt, 0.02f, 0);
        void* k = need_k ? fresh(n, dt, 1e-5f, 0) : NULL;
        for (int i = 0; i < n; ++i) put(v, i, uniform(1e-6f) * uniform(1.0f) + 1e-6f, dt);  /* second moments are not negative */
        for (int step = 1; step <= 3; ++step) {
          const double wd = variant == 2 ? 0.0 : (variant == 3 ? 1e-2 : 1 - 1e-3 * 1e-2);
          const int decoupled = variant == 3 ? 0 : DECOUPLE_WD;
          optimi_ref_adam(p, g, m, v, k, n, dt, 1e-3, 0.3, 0.9, 0.1, wd, 1e-6, base | decoupled);
          h_adam = fnv(fnv(fnv(h_adam, p, n, dt), m, n, dt), v, n, dt);
          optimi_ref_lion(p, g, m, k, n, dt, 1e-4, 0.1, 0.01, variant == 2 ? 0.0 : 1 - 1e-5, base);
          h_lion = fnv(fnv(h_lion, p, n, dt), m, n, dt);
          double r = optimi_ref_stableadamw(p, g, m, v, k, n, dt, 1e-3, 0.3, 0.9, 0.1, variant == 2 ? 0.0 : 1e-2, 1e-6,
                                            variant == 4 ? 2e-3 : 0.0, base | (variant == 4 ? DECOUPLE_LR : 0));
          h_stable = fnv(fnv(h_stable, p, n, dt), &r, 1, F32);
          optimi_ref_adan(p, g, m, d, v, pg, k, n, dt, 1e-3, 0.2, 0.92, 0.3, 0.9, 0.1, 1e-6, variant == 2 ? 0.0 : 1 + 2e-5,
                          base | (variant == 5 ? ADAM_WD : 0));
          h_adan = fnv(fnv(fnv(h_adan, p, n, dt), d, n, dt), pg, n, dt);
          optimi_ref_sgd(p, g, variant == 2 ? NULL : m, k, n, dt, 1e-2, variant == 2 ? 0.0 : 0.9, wd,
                         base | decoupled | (variant == 4 ? DAMPENING : 0));
          h_sgd = fnv(fnv(h_sgd, p, n, dt), m, n, dt);
          optimi_ref_ranger(p, g, m, v, variant == 2 ? NULL : la, k, n, dt, 1e-3, 0.3, 0.9, 0.1, wd, 1e-6, 0.7, 0.5,
                            base | decoupled | (step > 1 ? RECTIFY : 0) | (step == 3 ? LOOKAHEAD : 0));
          h_ranger = fnv(fnv(h_ranger, p, n, dt), la, n, dt);
          if (k) h_adam = fnv(h_adam, k, n, dt);
        }
        free(p); free(g); free(m); free(v); free(d); free(pg); free(la); free(k);
      }
    }
  printf("adam %016llx\nlion %016llx\nstableadamw %016llx\nadan %016llx\nsgd %016llx\nranger %016llx\n",
         (unsigned long long)h_adam, (unsigned long long)h_lion, (unsigned long long)h_stable, (unsigned long long)h_adan,
         (unsigned long long)h_sgd, (unsigned long long)h_ranger);
  return 0;
}
