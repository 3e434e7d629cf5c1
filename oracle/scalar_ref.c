/*
 * Scalar C emulator of optimi's PyTorch for-loop optimizer step.
 *
 * TEST INFRASTRUCTURE ONLY: the checker the HIP kernels are compared against.
 * Nothing in the shipped library includes or links this file.
 *
 * The reference (optimi/adam.py:354-396, lion.py:301-338, stableadamw.py:421-472,
 * adan.py:405-469) is a chain of in-place torch ops.  On CPU each op reads its
 * operands, computes in fp32 and rounds the result to the tensor dtype once.  This
 * file spells that chain out one element at a time with every rounding point
 * written down:
 *
 *   R(x)    round fp32 x to the tensor dtype (bf16, fp16: round-to-nearest-even; fp32: x)
 *   S(s)    a Python-double scalar narrowed to fp32 (mul_, lerp_, addcmul_, addcdiv_, div_)
 *   Sd(s)   a Python-double scalar narrowed to the tensor dtype (add_ with a scalar
 *           operand or an alpha: ATen's CPU add kernel casts both to the tensor dtype)
 *   lerp    ATen CPU form: d = end-start; |w|<0.5 ? fma(w,d,start) : fma(w-1,d,end)
 *   addcmul fma(S(value)*t1, t2, self)
 *   addcdiv self + (S(value)*t1)/t2
 *   add(alpha) fma(other, Sd(alpha), self)
 *
 * Those forms were measured against torch 2.10 CPU (AVX-512 build) and are pinned by the
 * golden fixtures the reference wrote (tests/golden).  Compile with contraction off so
 * that only the fmaf() calls written here fuse.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { OPTIMI_REF_F32 = 0, OPTIMI_REF_BF16 = 1, OPTIMI_REF_F16 = 2 };
enum {
  OPTIMI_REF_KAHAN = 1,       /* kahan_sum requested (only acts on bf16 tensors)   */
  OPTIMI_REF_UPDATE = 2,      /* update_parameters                                  */
  OPTIMI_REF_DECOUPLE_WD = 4, /* Adam: decoupled decay; unset = L2 into the gradient */
  OPTIMI_REF_ADAM_WD = 8,     /* Adan: Adam-style decay instead of Adan-style       */
  OPTIMI_REF_DECOUPLE_LR = 16,/* StableAdamW: fully decoupled decay                 */
  OPTIMI_REF_DAMPENING = 32,  /* SGD: dampened momentum (lerp)                       */
  OPTIMI_REF_RECTIFY = 64,    /* RAdam/Ranger: rectified step                        */
  OPTIMI_REF_LOOKAHEAD = 128  /* Ranger: Lookahead sync on this step                 */
};

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline uint16_t bf16_from_f32(float f) {
  uint32_t u = f32_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
/* IEEE binary16, round-to-nearest-even, subnormals kept, overflow to infinity */
static inline uint16_t f16_from_f32(float f) {
  const uint32_t inf32 = 255u << 23, max16 = (127u + 16u) << 23, magic = ((127u - 15u) + (23u - 10u) + 1u) << 23;
  uint32_t u = f32_to_bits(f);
  const uint32_t sign = u & 0x80000000u;
  u ^= sign;
  uint16_t o;
  if (u >= max16) {
    o = u > inf32 ? 0x7e00 : 0x7c00;
  } else if (u < (113u << 23)) { /* below 2^-14: lands on the subnormal grid by adding a float whose ulp is 2^-24 */
    float t = bits_to_f32(u) + bits_to_f32(magic);
    o = (uint16_t)(f32_to_bits(t) - magic);
  } else {
    const uint32_t odd = (u >> 13) & 1u;
    u += ((uint32_t)(15 - 127) << 23) + 0xfffu + odd;
    o = (uint16_t)(u >> 13);
  }
  return (uint16_t)(o | (sign >> 16));
}
static inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, ex = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (ex == 0) {
    float v = (float)man * 5.9604644775390625e-8f; /* man * 2^-24 */
    return sign ? -v : v;
  }
  if (ex == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
  return bits_to_f32(sign | ((ex + 112u) << 23) | (man << 13));
}
static inline int low_precision(int dt) { return dt != OPTIMI_REF_F32; }
static inline float R(float x, int dt) {
  if (dt == OPTIMI_REF_BF16) return bits_to_f32((uint32_t)bf16_from_f32(x) << 16);
  if (dt == OPTIMI_REF_F16) return f16_to_f32(f16_from_f32(x));
  return x;
}
static inline float LD(const void* a, int64_t i, int dt) {
  if (dt == OPTIMI_REF_BF16) return bits_to_f32((uint32_t)((const uint16_t*)a)[i] << 16);
  if (dt == OPTIMI_REF_F16) return f16_to_f32(((const uint16_t*)a)[i]);
  return ((const float*)a)[i];
}
static inline void ST(void* a, int64_t i, int dt, float x) {
  if (dt == OPTIMI_REF_BF16) ((uint16_t*)a)[i] = bf16_from_f32(x);
  else if (dt == OPTIMI_REF_F16) ((uint16_t*)a)[i] = f16_from_f32(x);
  else ((float*)a)[i] = x;
}
/* test hook: R() as the emulator applies it */
float optimi_ref_round(float x, int dt) { return R(x, dt); }

static inline float S(double s) { return (float)s; }
static inline float Sd(double s, int dt) { return R((float)s, dt); }

static inline float lerp_f(float start, float end, float w) {
  float d = end - start;
  return fabsf(w) < 0.5f ? fmaf(w, d, start) : fmaf(w - 1.0f, d, end);
}

/* param += kahan; kahan += (old param - new param)      optimi/adam.py:388-393 */
static inline void kahan_commit(float* p, float* k, int dt) {
  float old = *p;
  *p = R(old + *k, dt);
  float err = R(old - *p, dt);
  *k = R(*k + err, dt);
}

/* ---------------------------------------------------------------------------
 * Adam / AdamW                                          optimi/adam.py:354-396
 * weight_decay: the formed factor when decoupled, the raw coefficient for L2.
 * kahan may be NULL when the Kahan branch is not taken.
 * ------------------------------------------------------------------------- */
void optimi_ref_adam(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan, int64_t n, int dt,
                     double lr, double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay,
                     double eps, int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const int do_wd = weight_decay != 0 && update;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), g = LD(grad, i, dt), m = LD(exp_avg, i, dt), v = LD(exp_avg_sq, i, dt);
    if (do_wd) {
      if (flags & OPTIMI_REF_DECOUPLE_WD) p = R(p * S(weight_decay), dt);   /* adam.py:375 */
      else g = R(fmaf(p, Sd(weight_decay, dt), g), dt);                     /* adam.py:377 */
    }
    m = R(lerp_f(m, g, S(beta1_comp)), dt);                                  /* adam.py:380 */
    v = R(v * S(beta2_hat), dt);                                             /* adam.py:381 */
    v = R(fmaf(S(beta2_comp) * g, g, v), dt);
    ST(exp_avg, i, dt, m);
    ST(exp_avg_sq, i, dt, v);
    if (!update) continue;
    float d = R(sqrtf(v), dt);
    d = R(d + Sd(eps, dt), dt);
    if (do_kahan) {
      float k = LD(kahan, i, dt);
      k = R(k + (S(-lr) * m) / d, dt);                                       /* adam.py:386 */
      kahan_commit(&p, &k, dt);
      ST(kahan, i, dt, k);
    } else {
      p = R(p + (S(-lr) * m) / d, dt);                                       /* adam.py:396 */
    }
    ST(param, i, dt, p);
  }
}

/* ---------------------------------------------------------------------------
 * Lion                                                  optimi/lion.py:301-338
 * weight_decay: the formed factor (or 0).
 * ------------------------------------------------------------------------- */
void optimi_ref_lion(void* param, const void* grad, void* exp_avg, void* kahan, int64_t n, int dt, double lr,
                     double beta1_comp, double beta2_comp, double weight_decay, int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const int do_wd = weight_decay != 0 && update;
  const float neg_lr = Sd(-lr, dt); /* add_(update, alpha=-lr): alpha takes the tensor dtype */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), g = LD(grad, i, dt), m = LD(exp_avg, i, dt);
    if (do_wd) p = R(p * S(weight_decay), dt);                               /* lion.py:315 */
    float u = 0.0f;
    if (update) {
      float c = R(lerp_f(m, g, S(beta1_comp)), dt);                          /* lion.py:319 */
      u = (float)((c > 0.0f) - (c < 0.0f));
    }
    m = R(lerp_f(m, g, S(beta2_comp)), dt);                                  /* lion.py:322 */
    ST(exp_avg, i, dt, m);
    if (!update) continue;
    if (do_kahan) {
      float k = LD(kahan, i, dt);
      k = R(fmaf(u, neg_lr, k), dt);                                         /* lion.py:327 */
      kahan_commit(&p, &k, dt);
      ST(kahan, i, dt, k);
    } else {
      p = R(fmaf(u, neg_lr, p), dt);                                         /* lion.py:338 */
    }
    ST(param, i, dt, p);
  }
}

/* ---------------------------------------------------------------------------
 * StableAdamW                                    optimi/stableadamw.py:421-472
 * weight_decay: the raw coefficient.  Returns the clipped learning rate.
 * The mean is accumulated in double over fixed blocks, then narrowed to fp32,
 * divided by fp32(n) and rounded to the tensor dtype, as torch's CPU mean does
 * (fp32 sum -> fp32 divide -> cast).
 * ------------------------------------------------------------------------- */
double optimi_ref_stableadamw(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan, int64_t n,
                              int dt, double lr, double beta1_comp, double beta2_hat, double beta2_comp,
                              double weight_decay, double eps, double max_lr, int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const float eps_sq = R((float)(eps * eps), dt);                 /* stableadamw.py:119 */
  enum { BLK = 4096 };
  const int64_t nblk = (n + BLK - 1) / BLK;
  double* part = (double*)calloc((size_t)(nblk > 0 ? nblk : 1), sizeof(double));
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nblk; ++b) {
    const int64_t hi = (b + 1) * BLK < n ? (b + 1) * BLK : n;
    double acc = 0.0;
    for (int64_t i = b * BLK; i < hi; ++i) {
      float g = LD(grad, i, dt), m = LD(exp_avg, i, dt), v = LD(exp_avg_sq, i, dt);
      m = R(lerp_f(m, g, S(beta1_comp)), dt);                                /* stableadamw.py:442 */
      v = R(v * S(beta2_hat), dt);                                           /* stableadamw.py:443 */
      v = R(fmaf(S(beta2_comp) * g, g, v), dt);
      ST(exp_avg, i, dt, m);
      ST(exp_avg_sq, i, dt, v);
      if (update) {
        float q = R(g * g, dt);                                              /* stableadamw.py:447 */
        float mx = v > eps_sq ? v : eps_sq;
        q = R(q / mx, dt);
        acc += (double)q;
      }
    }
    part[b] = acc;
  }
  double total = 0.0;
  for (int64_t b = 0; b < nblk; ++b) total += part[b];
  free(part);
  if (!update) return lr;

  float ms = R((float)total / (float)n, dt);
  float rms = R(sqrtf(ms), dt);
  double rmsd = (double)rms;
  lr = lr / (rmsd > 1.0 ? rmsd : 1.0);                                       /* stableadamw.py:450 */
  double factor = 0.0;
  if (weight_decay != 0)                                                     /* stableadamw.py:453-458 */
    factor = (flags & OPTIMI_REF_DECOUPLE_LR) ? 1 - (lr / max_lr) * weight_decay : 1 - lr * weight_decay;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), m = LD(exp_avg, i, dt), v = LD(exp_avg_sq, i, dt);
    if (weight_decay != 0) p = R(p * S(factor), dt);
    float d = R(sqrtf(v), dt);
    d = R(d + Sd(eps, dt), dt);
    if (do_kahan) {
      float k = LD(kahan, i, dt);
      k = R(k + (S(-lr) * m) / d, dt);                                       /* stableadamw.py:462 */
      kahan_commit(&p, &k, dt);
      ST(kahan, i, dt, k);
    } else {
      p = R(p + (S(-lr) * m) / d, dt);                                       /* stableadamw.py:472 */
    }
    ST(param, i, dt, p);
  }
  return lr;
}

/* ---------------------------------------------------------------------------
 * Adan                                                  optimi/adan.py:405-469
 * weight_decay: the formed factor 1+lr*wd (Adan style) or 1-lr*wd (ADAM_WD), or 0.
 * prev_grad holds the negated previous gradient.
 * ------------------------------------------------------------------------- */
void optimi_ref_adan(void* param, const void* grad, void* exp_avg, void* exp_avg_diff, void* exp_avg_sq,
                     void* prev_grad, void* kahan, int64_t n, int dt, double lr, double beta1_comp, double beta2,
                     double beta2_comp, double beta3_hat, double beta3_comp, double eps, double weight_decay,
                     int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const int adam_wd = (flags & OPTIMI_REF_ADAM_WD) != 0;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), g = LD(grad, i, dt), m = LD(exp_avg, i, dt), df = LD(exp_avg_diff, i, dt);
    float nn = LD(exp_avg_sq, i, dt), pg = LD(prev_grad, i, dt);
    pg = R(pg + g, dt);                                                      /* adan.py:427 */
    m = R(lerp_f(m, g, S(beta1_comp)), dt);                                  /* adan.py:430 */
    df = R(lerp_f(df, pg, S(beta2_comp)), dt);                               /* adan.py:433 */
    pg = R(pg * S(beta2), dt);                                               /* adan.py:436 */
    pg = R(pg + g, dt);
    nn = R(nn * S(beta3_hat), dt);                                           /* adan.py:437 */
    nn = R(fmaf(S(beta3_comp) * pg, pg, nn), dt);
    pg = R(g * -1.0f, dt);                                                   /* adan.py:440 */
    ST(exp_avg, i, dt, m);
    ST(exp_avg_diff, i, dt, df);
    ST(exp_avg_sq, i, dt, nn);
    ST(prev_grad, i, dt, pg);
    if (!update) continue;
    float d = R(sqrtf(nn), dt);                                              /* adan.py:444 */
    d = R(d + Sd(eps, dt), dt);
    if (adam_wd && weight_decay != 0) p = R(p * S(weight_decay), dt);        /* adan.py:447-448 */
    if (do_kahan) {
      float k = LD(kahan, i, dt);
      k = R(k + (S(-lr) * m) / d, dt);                                       /* adan.py:451 */
      k = R(k + (S(-lr * beta2) * df) / d, dt);                              /* adan.py:452 */
      kahan_commit(&p, &k, dt);
      ST(kahan, i, dt, k);
    } else {
      p = R(p + (S(-lr) * m) / d, dt);                                       /* adan.py:461 */
      p = R(p + (S(-lr * beta2) * df) / d, dt);                              /* adan.py:462 */
    }
    if (!adam_wd && weight_decay != 0) p = R(p / S(weight_decay), dt);       /* adan.py:465-466 */
    ST(param, i, dt, p);
  }
}

/* ---------------------------------------------------------------------------
 * SGD                                                    optimi/sgd.py:329-372
 * weight_decay as for Adam.  exp_avg may be NULL when momentum == 0.
 * ------------------------------------------------------------------------- */
void optimi_ref_sgd(void* param, const void* grad, void* exp_avg, void* kahan, int64_t n, int dt, double lr,
                    double momentum, double weight_decay, int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const int do_wd = weight_decay != 0 && update;
  const float neg_lr = Sd(-lr, dt); /* add_(exp_avg, alpha=-lr) */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), g = LD(grad, i, dt), m;
    if (do_wd) {
      if (flags & OPTIMI_REF_DECOUPLE_WD) p = R(p * S(weight_decay), dt);    /* sgd.py:345 */
      else g = R(fmaf(p, Sd(weight_decay, dt), g), dt);                      /* sgd.py:347 */
    }
    if (momentum != 0) {
      m = LD(exp_avg, i, dt);
      if (flags & OPTIMI_REF_DAMPENING) {
        m = R(lerp_f(m, g, S(1 - momentum)), dt);                            /* sgd.py:353 */
      } else {
        m = R(m * S(momentum), dt);                                          /* sgd.py:355 */
        m = R(m + g, dt);
      }
      ST(exp_avg, i, dt, m);
    } else {
      m = g;                                                                 /* sgd.py:357 */
    }
    if (!update) continue;
    if (do_kahan) {
      float k = LD(kahan, i, dt);
      k = R(fmaf(m, neg_lr, k), dt);                                         /* sgd.py:362 */
      kahan_commit(&p, &k, dt);
      ST(kahan, i, dt, k);
    } else {
      p = R(fmaf(m, neg_lr, p), dt);                                         /* sgd.py:372 */
    }
    ST(param, i, dt, p);
  }
}

/* ---------------------------------------------------------------------------
 * RAdam and Ranger                     optimi/radam.py:368-417, ranger.py:402-473
 * rect is read only with OPTIMI_REF_RECTIFY.  la_param (Ranger) may be NULL for
 * RAdam; with OPTIMI_REF_LOOKAHEAD the Lookahead interpolation follows the step.
 * ------------------------------------------------------------------------- */
void optimi_ref_ranger(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* la_param, void* kahan,
                       int64_t n, int dt, double lr, double beta1_comp, double beta2_hat, double beta2_comp,
                       double weight_decay, double eps, double rect, double alpha, int flags) {
  const int update = (flags & OPTIMI_REF_UPDATE) != 0;
  const int do_kahan = (flags & OPTIMI_REF_KAHAN) && low_precision(dt);
  const int do_wd = weight_decay != 0 && update;
  const int rectify = (flags & OPTIMI_REF_RECTIFY) != 0;
  const int lookahead = update && (flags & OPTIMI_REF_LOOKAHEAD) && la_param;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float p = LD(param, i, dt), g = LD(grad, i, dt), m = LD(exp_avg, i, dt), v = LD(exp_avg_sq, i, dt);
    if (do_wd) {
      if (flags & OPTIMI_REF_DECOUPLE_WD) p = R(p * S(weight_decay), dt);    /* radam.py:389 */
      else g = R(fmaf(p, Sd(weight_decay, dt), g), dt);                      /* radam.py:391 */
    }
    m = R(lerp_f(m, g, S(beta1_comp)), dt);                                  /* radam.py:394 */
    v = R(v * S(beta2_hat), dt);                                             /* radam.py:395 */
    v = R(fmaf(S(beta2_comp) * g, g, v), dt);
    ST(exp_avg, i, dt, m);
    ST(exp_avg_sq, i, dt, v);
    if (!update) continue;
    float k = do_kahan ? LD(kahan, i, dt) : p;   /* the accumulator the step lands in */
    if (rectify) {
      float d = R(sqrtf(v), dt);
      d = R(d + Sd(eps, dt), dt);
      k = R(k + (S(-lr * rect) * m) / d, dt);                                /* radam.py:401, 415 */
    } else {
      k = R(fmaf(m, Sd(-lr, dt), k), dt);                                    /* radam.py:403, 417 */
    }
    if (do_kahan) kahan_commit(&p, &k, dt); else p = k;
    if (lookahead) {
      float la = LD(la_param, i, dt);
      float t = R(p - la, dt);                                               /* ranger.py:453, 472 */
      if (do_kahan) {
        k = R(fmaf(t, Sd(alpha, dt), k), dt);                                /* ranger.py:453 */
        float old = la;
        la = R(old + k, dt);                                                 /* ranger.py:457 */
        float err = R(old - la, dt);
        k = R(fmaf(err, Sd(alpha, dt), k), dt);                              /* ranger.py:460 */
      } else {
        la = R(fmaf(t, Sd(alpha, dt), la), dt);                              /* ranger.py:472 */
      }
      p = la;                                                                /* ranger.py:462, 473 */
      ST(la_param, i, dt, la);
    }
    if (do_kahan) ST(kahan, i, dt, k);
    ST(param, i, dt, p);
  }
}
