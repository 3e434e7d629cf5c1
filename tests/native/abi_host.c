/*
 * The C ABI from a host that has no PyTorch and no Python: plain C, the HIP runtime for device
 * memory, include/optimi_hip.h for the optimizer steps.
 *
 * TEST PROGRAM.  For AdamW, Lion, Adan and SGD, in bf16 with Kahan summation and in fp32, it steps
 * a list of 20 tensors (sizes 0, 1, around the 512-element tile and the 8192-element chunk, up to
 * 70,001 elements; more than 16 tensors, so the tables live in device memory) three times through
 * the whole-list entry point, a copy of the same list through the per-tensor entry points, and a
 * third copy on the host through the scalar C emulator (oracle/scalar_ref.c, the checker of the
 * test suite).  All three must agree bit for bit in every buffer.  Prints one line per case and
 * "abi_host ok" at the end; exit status 1 on any mismatch or error.
 *
 * `abi_host paths` instead walks the host side of the library (see run_paths below).
 *
 * Build:  gcc -O1 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -Iinclude tests/native/abi_host.c \
 *             -Loptimi_amd -loptimi_hip -Loracle -loptimi_ref -L/opt/rocm/lib -lamdhip64 -lm
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "optimi_hip.h"

/* the emulator's entry points (oracle/scalar_ref.c); its dtype and flag values are the ABI's */
float optimi_ref_round(float x, int dt);
void optimi_ref_adam(void*, const void*, void*, void*, void*, int64_t, int, double, double, double, double, double, double, int);
void optimi_ref_lion(void*, const void*, void*, void*, int64_t, int, double, double, double, double, int);
void optimi_ref_adan(void*, const void*, void*, void*, void*, void*, void*, int64_t, int, double, double, double, double,
                     double, double, double, double, int);
void optimi_ref_sgd(void*, const void*, void*, void*, int64_t, int, double, double, double, int);

#define N_TENSORS 20
#define MAX_ARRAYS 7 /* param, grad, up to four states, Kahan buffer */
#define STEPS 3

static const int64_t kSizes[N_TENSORS] = {70001, 0, 1, 511, 512, 513, 8191, 8192, 8193, 7, 0, 16384,
                                          4097, 30000, 3, 1000, 24577, 64, 65, 12345};

#define HIP_OK(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__); \
      exit(1);                                                                         \
    }                                                                                  \
  } while (0)
#define ABI_OK(call)                                                                          \
  do {                                                                                        \
    int rc_ = (call);                                                                         \
    if (rc_ != 0) {                                                                           \
      fprintf(stderr, "%s: %s (line %d)\n", #call, optimi_hip_error_string(rc_), __LINE__); \
      exit(1);                                                                                \
    }                                                                                         \
  } while (0)

static uint64_t rng_state;
static uint32_t rng(void) {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (uint32_t)(rng_state >> 16);
}
static float uniform(float scale) { return ((float)(rng() & 0xffffff) / 8388608.0f - 1.0f) * scale; }

static size_t esize(int dt) { return dt == OPTIMI_F32 ? 4 : 2; }

/* stores x rounded to bf16 or as fp32 (the two dtypes this program runs) */
static void put(void* buf, int64_t i, float x, int dt) {
  float r = optimi_ref_round(x, dt);
  uint32_t u;
  memcpy(&u, &r, 4);
  if (dt == OPTIMI_F32) ((uint32_t*)buf)[i] = u;
  else ((uint16_t*)buf)[i] = (uint16_t)(u >> 16);
}

/* One copy of the list: array a of tensor t is host[a][t] on the host and dev[a][t] on the device. */
typedef struct {
  void* host[MAX_ARRAYS][N_TENSORS];
  void* dev[MAX_ARRAYS][N_TENSORS];
} List;

static void list_alloc(List* l, int n_arrays, int dt, int on_device) {
  memset(l, 0, sizeof(*l));
  for (int a = 0; a < n_arrays; ++a)
    for (int t = 0; t < N_TENSORS; ++t) {
      size_t bytes = (size_t)kSizes[t] * esize(dt);
      l->host[a][t] = malloc(bytes ? bytes : 1);
      if (on_device && bytes) HIP_OK(hipMalloc(&l->dev[a][t], bytes));
    }
}
static void list_free(List* l, int n_arrays) {
  for (int a = 0; a < n_arrays; ++a)
    for (int t = 0; t < N_TENSORS; ++t) {
      free(l->host[a][t]);
      if (l->dev[a][t]) HIP_OK(hipFree(l->dev[a][t]));
    }
}
static void upload(List* l, int a, int dt) {
  for (int t = 0; t < N_TENSORS; ++t)
    if (kSizes[t]) HIP_OK(hipMemcpy(l->dev[a][t], l->host[a][t], (size_t)kSizes[t] * esize(dt), hipMemcpyHostToDevice));
}
static void download(List* l, int a, int dt) {
  for (int t = 0; t < N_TENSORS; ++t)
    if (kSizes[t]) HIP_OK(hipMemcpy(l->host[a][t], l->dev[a][t], (size_t)kSizes[t] * esize(dt), hipMemcpyDeviceToHost));
}

enum { ADAMW, LION, ADAN, SGD, N_OPT };
static const char* kName[N_OPT] = {"adamw", "lion", "adan", "sgd"};
/* arrays in the ABI's order: param, grad, states..., Kahan buffer last */
static const int kArrays[N_OPT] = {5, 4, 7, 4};

/* the debiased beta of optimi/utils.py:31-36 */
static double debias(double beta, int step) {
  double bt = pow(beta, step);
  return (bt - beta) / (bt - 1.0);
}

typedef struct {
  double s[8];
  uint32_t flags;
} Scalars;

static Scalars scalars_of(int opt, int step, int kahan) {
  Scalars c;
  memset(&c, 0, sizeof(c));
  c.flags = OPTIMI_UPDATE | (kahan ? OPTIMI_KAHAN : 0);
  const double lr = 1e-3;
  switch (opt) {
    case ADAMW: { /* lr, 1-b1^, b2^, 1-b2^, decay factor, eps */
      double b1 = debias(0.9, step), b2 = debias(0.99, step);
      double v[6] = {lr, 1 - b1, b2, 1 - b2, 1 - lr * 1e-2, 1e-6};
      memcpy(c.s, v, sizeof(v));
      c.flags |= OPTIMI_DECOUPLE_WD;
      break;
    }
    case LION: { /* lr, 1-b1, 1-b2, decay factor */
      double v[4] = {1e-4, 1 - 0.9, 1 - 0.99, 1 - 1e-4 * 0.1};
      memcpy(c.s, v, sizeof(v));
      break;
    }
    case ADAN: { /* lr, 1-b1^, b2, 1-b2^, b3^, 1-b3^, eps, decay factor */
      double b1 = debias(0.98, step), b2 = debias(0.92, step), b3 = debias(0.99, step);
      double v[8] = {lr, 1 - b1, 0.92, 1 - b2, b3, 1 - b3, 1e-8, 1 + lr * 2e-2};
      memcpy(c.s, v, sizeof(v));
      break;
    }
    case SGD: { /* lr, momentum, decay factor */
      double v[3] = {1e-2, 0.9, 1 - 1e-2 * 1e-2};
      memcpy(c.s, v, sizeof(v));
      c.flags |= OPTIMI_DECOUPLE_WD;
      break;
    }
  }
  return c;
}

static void ref_step(int opt, void* const* a, int64_t n, int dt, const Scalars* c) {
  const double* s = c->s;
  const int f = (int)c->flags;
  switch (opt) {
    case ADAMW: optimi_ref_adam(a[0], a[1], a[2], a[3], a[4], n, dt, s[0], s[1], s[2], s[3], s[4], s[5], f); break;
    case LION: optimi_ref_lion(a[0], a[1], a[2], a[3], n, dt, s[0], s[1], s[2], s[3], f); break;
    case ADAN: optimi_ref_adan(a[0], a[1], a[2], a[3], a[4], a[5], a[6], n, dt, s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], f); break;
    case SGD: optimi_ref_sgd(a[0], a[1], a[2], a[3], n, dt, s[0], s[1], s[2], f); break;
  }
}

static void hip_single(int opt, void* const* a, int64_t n, int dt, const Scalars* c) {
  const double* s = c->s;
  switch (opt) {
    case ADAMW: ABI_OK(optimi_hip_adam_single(a[0], a[1], a[2], a[3], a[4], n, dt, s[0], s[1], s[2], s[3], s[4], s[5], c->flags, NULL)); break;
    case LION: ABI_OK(optimi_hip_lion_single(a[0], a[1], a[2], a[3], n, dt, s[0], s[1], s[2], s[3], c->flags, NULL)); break;
    case ADAN:
      ABI_OK(optimi_hip_adan_single(a[0], a[1], a[2], a[3], a[4], a[5], a[6], n, dt, s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7],
                                    c->flags, NULL));
      break;
    case SGD: ABI_OK(optimi_hip_sgd_single(a[0], a[1], a[2], a[3], n, dt, s[0], s[1], s[2], c->flags, NULL)); break;
  }
}

static void hip_multi(int opt, optimi_group* g, List* l, int dt, const Scalars* c) {
  const double* s = c->s;
  void* const* p = l->dev[0];
  const void* const* gr = (const void* const*)l->dev[1];
  switch (opt) {
    case ADAMW:
      ABI_OK(optimi_hip_adam_multi(g, N_TENSORS, p, gr, l->dev[2], l->dev[3], l->dev[4], kSizes, dt, s[0], s[1], s[2], s[3], s[4], s[5],
                                   c->flags, NULL));
      break;
    case LION:
      ABI_OK(optimi_hip_lion_multi(g, N_TENSORS, p, gr, l->dev[2], l->dev[3], kSizes, dt, s[0], s[1], s[2], s[3], c->flags, NULL));
      break;
    case ADAN:
      ABI_OK(optimi_hip_adan_multi(g, N_TENSORS, p, gr, l->dev[2], l->dev[3], l->dev[4], l->dev[5], l->dev[6], kSizes, dt, s[0], s[1],
                                   s[2], s[3], s[4], s[5], s[6], s[7], c->flags, NULL));
      break;
    case SGD:
      ABI_OK(optimi_hip_sgd_multi(g, N_TENSORS, p, gr, l->dev[2], l->dev[3], kSizes, dt, s[0], s[1], s[2], c->flags, NULL));
      break;
  }
}

static int run_case(int opt, int dt) {
  const int A = kArrays[opt], kahan = dt != OPTIMI_F32;
  List multi, single, ref;
  list_alloc(&multi, A, dt, 1);
  list_alloc(&single, A, dt, 1);
  list_alloc(&ref, A, dt, 0);
  rng_state = 88172645463325252ull + (uint64_t)(opt * 7 + dt);
  /* parameters, zeroed states (Adan's prev_grad starts as the negated first gradient, below) */
  for (int t = 0; t < N_TENSORS; ++t) {
    for (int64_t i = 0; i < kSizes[t]; ++i) put(ref.host[0][t], i, uniform(0.05f), dt);
    for (int a = 2; a < A; ++a) memset(ref.host[a][t], 0, (size_t)kSizes[t] * esize(dt));
  }
  optimi_group* group = NULL;
  ABI_OK(optimi_hip_group_create(&group));
  for (int step = 1; step <= STEPS; ++step) {
    for (int t = 0; t < N_TENSORS; ++t)
      for (int64_t i = 0; i < kSizes[t]; ++i) {
        float g = uniform(step == 2 ? 4e-3f : 1e-3f);
        put(ref.host[1][t], i, g, dt);
        if (opt == ADAN && step == 1) put(ref.host[5][t], i, -g, dt); /* optimi/adan.py:109 */
      }
    if (step == 1) {
      for (int a = 0; a < A; ++a)
        for (int t = 0; t < N_TENSORS; ++t) {
          memcpy(multi.host[a][t], ref.host[a][t], (size_t)kSizes[t] * esize(dt));
          memcpy(single.host[a][t], ref.host[a][t], (size_t)kSizes[t] * esize(dt));
        }
      for (int a = 0; a < A; ++a) {
        upload(&multi, a, dt);
        upload(&single, a, dt);
      }
    } else {
      for (int t = 0; t < N_TENSORS; ++t) {
        memcpy(multi.host[1][t], ref.host[1][t], (size_t)kSizes[t] * esize(dt));
        memcpy(single.host[1][t], ref.host[1][t], (size_t)kSizes[t] * esize(dt));
      }
      upload(&multi, 1, dt);
      upload(&single, 1, dt);
    }
    const Scalars c = scalars_of(opt, step, kahan);
    hip_multi(opt, group, &multi, dt, &c);
    for (int t = 0; t < N_TENSORS; ++t) {
      void* dev[MAX_ARRAYS];
      void* host[MAX_ARRAYS];
      for (int a = 0; a < MAX_ARRAYS; ++a) {
        dev[a] = a < A ? single.dev[a][t] : NULL;
        host[a] = a < A ? ref.host[a][t] : NULL;
      }
      if (!kahan) dev[A - 1] = NULL; /* an fp32 tensor has no Kahan buffer: NULL is fine */
      hip_single(opt, dev, kSizes[t], dt, &c);
      ref_step(opt, host, kSizes[t], dt, &c);
    }
  }
  HIP_OK(hipDeviceSynchronize());
  int bad = 0;
  for (int a = 0; a < A; ++a) {
    if (a == 1) continue; /* the gradient is read-only */
    if (a == A - 1 && !kahan) continue;
    download(&multi, a, dt);
    download(&single, a, dt);
    for (int t = 0; t < N_TENSORS; ++t) {
      size_t bytes = (size_t)kSizes[t] * esize(dt);
      if (memcmp(multi.host[a][t], ref.host[a][t], bytes)) {
        fprintf(stderr, "%s: array %d of tensor %d: whole-list step differs from the emulator\n", kName[opt], a, t);
        bad = 1;
      }
      if (memcmp(single.host[a][t], ref.host[a][t], bytes)) {
        fprintf(stderr, "%s: array %d of tensor %d: per-tensor step differs from the emulator\n", kName[opt], a, t);
        bad = 1;
      }
    }
  }
  /* the parameters did move */
  int moved = 0;
  rng_state = 88172645463325252ull + (uint64_t)(opt * 7 + dt);
  for (int64_t i = 0; i < kSizes[0] && !moved; ++i) {
    char first[4];
    put(first, 0, uniform(0.05f), dt);
    moved = memcmp(first, (char*)ref.host[0][0] + (size_t)i * esize(dt), esize(dt)) != 0;
  }
  if (!moved) {
    fprintf(stderr, "%s: the parameters did not move\n", kName[opt]);
    bad = 1;
  }
  optimi_hip_group_destroy(group);
  list_free(&multi, A);
  list_free(&single, A);
  list_free(&ref, A);
  printf("%s %s: %s\n", kName[opt], dt == OPTIMI_F32 ? "fp32" : "bf16+kahan", bad ? "MISMATCH" : "ok");
  fflush(stdout);
  return bad;
}

/* ---- "paths" mode: the library's host side walked over its own ground ----
 * Lists that grow and shrink between 0 and 1000 tensors on one group (kernel-argument table, device
 * tables that are rebuilt, re-uploaded or left alone, workspaces that grow), every whole-list entry
 * point with one dtype and with a dtype per tensor, pointers that change between calls, tensors two
 * bytes off the 16-byte grid, StableAdamW's per-tensor entry points on growing tensors, the traffic
 * probe, the copy probe and launches split into pieces.  Results are not inspected here (the other
 * mode and the Python tests do that): every call must succeed, and the program is meant to be run
 * with the library's host code under AddressSanitizer as well. */
static int64_t launches_before;

static void paths_list(optimi_group* g, char* arena, size_t arena_bytes, int n, int variant) {
  static void* ptr[MAX_ARRAYS][1000];
  static int64_t numel[1000];
  static int dtypes[1000];
  size_t pos = 0;
  for (int t = 0; t < n; ++t) {
    numel[t] = (int64_t)(rng() % 3 == 0 ? rng() % 40 : rng() % 20000);
    if (rng() % 11 == 0) numel[t] = 0;
    dtypes[t] = (t % 3 == 1) ? OPTIMI_F32 : OPTIMI_BF16;
    for (int a = 0; a < MAX_ARRAYS; ++a) {
      size_t bytes = ((size_t)numel[t] * 4 + 15) & ~(size_t)15;
      size_t off = (variant & 2) && a == 1 && t % 5 == 0 ? 4 : 0; /* a gradient that is a view into a bucket */
      if (pos + bytes + 16 > arena_bytes) pos = 0;                 /* wrap: buffers may alias, values do not matter */
      ptr[a][t] = arena + pos + off;
      pos += bytes + 16;
    }
  }
  const uint32_t f = OPTIMI_UPDATE | OPTIMI_KAHAN;
  const void* const* gr = (const void* const*)ptr[1];
  for (int rep = 0; rep < 2; ++rep) { /* the second time nothing has changed: no upload */
    ABI_OK(optimi_hip_adam_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, OPTIMI_BF16, 1e-3, 0.1, 0.98, 0.02, 0.99999, 1e-6,
                                 f | OPTIMI_DECOUPLE_WD | ((variant & 1) ? OPTIMI_RESIDENT : 0), NULL));
  }
  if (n > 2) { /* one gradient moves: table only */
    void* keep = ptr[1][n / 2];
    ptr[1][n / 2] = ptr[1][0];
    ABI_OK(optimi_hip_adam_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, OPTIMI_BF16, 1e-3, 0.1, 0.98, 0.02, 0.0, 1e-6, f, NULL));
    ptr[1][n / 2] = keep;
  }
  ABI_OK(optimi_hip_adam_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, dtypes, 1e-3, 0.1, 0.98, 0.02, 1e-2, 1e-6, f, NULL));
  ABI_OK(optimi_hip_lion_multi(g, n, ptr[0], gr, ptr[2], ptr[3], numel, OPTIMI_F16, 1e-4, 0.1, 0.01, 0.9999, f, NULL));
  ABI_OK(optimi_hip_lion_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], numel, dtypes, 1e-4, 0.1, 0.01, 0.0, OPTIMI_KAHAN, NULL));
  ABI_OK(optimi_hip_stableadamw_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, OPTIMI_BF16, 1e-3, 0.1, 0.98, 0.02, 1e-2, 1e-6,
                                      0.0, f, NULL));
  ABI_OK(optimi_hip_stableadamw_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, dtypes, 1e-3, 0.1, 0.98, 0.02, 1e-2,
                                            1e-6, 2e-3, f | OPTIMI_DECOUPLE_LR, NULL));
  ABI_OK(optimi_hip_stableadamw_multi(g, n, ptr[0], gr, ptr[2], ptr[3], NULL, numel, OPTIMI_F32, 1e-3, 0.1, 0.98, 0.02, 1e-2, 1e-6, 0.0,
                                      0 /* accumulate only */, NULL));
  ABI_OK(optimi_hip_adan_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], ptr[5], ptr[6], numel, OPTIMI_BF16, 1e-3, 0.02, 0.92, 0.08, 0.98,
                               0.02, 1e-8, 1.00002, f, NULL));
  ABI_OK(optimi_hip_adan_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], ptr[5], ptr[6], numel, dtypes, 1e-3, 0.02, 0.92, 0.08,
                                     0.98, 0.02, 1e-8, 0.99998, f | OPTIMI_ADAM_WD, NULL));
  ABI_OK(optimi_hip_sgd_multi(g, n, ptr[0], gr, ptr[2], ptr[3], numel, OPTIMI_BF16, 1e-2, 0.9, 0.9999, f | OPTIMI_DECOUPLE_WD, NULL));
  ABI_OK(optimi_hip_sgd_multi_mixed(g, n, ptr[0], gr, NULL, ptr[3], numel, dtypes, 1e-2, 0.0, 1e-2, f, NULL));
  ABI_OK(optimi_hip_radam_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, OPTIMI_BF16, 1e-3, 0.1, 0.98, 0.02, 0.99999, 1e-6, 0.7,
                                f | OPTIMI_DECOUPLE_WD | OPTIMI_RECTIFY, NULL));
  ABI_OK(optimi_hip_radam_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[4], numel, dtypes, 1e-3, 0.1, 0.98, 0.02, 0.99999, 1e-6,
                                      0.0, f | OPTIMI_DECOUPLE_WD, NULL));
  ABI_OK(optimi_hip_ranger_multi(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[5], ptr[4], numel, OPTIMI_BF16, 1e-3, 0.1, 0.98, 0.02, 0.99999,
                                 1e-6, 0.7, 0.5, f | OPTIMI_DECOUPLE_WD | OPTIMI_RECTIFY | OPTIMI_LOOKAHEAD, NULL));
  ABI_OK(optimi_hip_ranger_multi_mixed(g, n, ptr[0], gr, ptr[2], ptr[3], ptr[5], ptr[4], numel, dtypes, 1e-3, 0.1, 0.98, 0.02, 0.99999,
                                       1e-6, 0.7, 0.5, f | OPTIMI_DECOUPLE_WD, NULL));
  /* the traffic probe on the same tensors (sizes in bytes, multiples of 16: the aligned ones only) */
  if (!(variant & 2) && n > 0) {
    static int64_t bytes[1000];
    void* const* cols[MAX_ARRAYS];
    for (int t = 0; t < n; ++t) bytes[t] = (numel[t] * 2) & ~(int64_t)15;
    for (int a = 0; a < MAX_ARRAYS; ++a) cols[a] = ptr[a];
    ABI_OK(optimi_hip_stream_probe(g, n, cols, bytes, 7, 6, 0, 0, NULL));
    ABI_OK(optimi_hip_stream_probe(g, n, cols, bytes, 3, 1, 9, OPTIMI_PROBE_SCRAMBLE, NULL));
  }
}

static int run_paths(void) {
  const size_t arena_bytes = (size_t)192 << 20;
  char* arena = NULL;
  HIP_OK(hipMalloc((void**)&arena, arena_bytes));
  HIP_OK(hipMemset(arena, 0, arena_bytes));
  rng_state = 1234567891234567ull;
  optimi_group* g = NULL;
  ABI_OK(optimi_hip_group_create(&g));
  static const int lengths[] = {1, 16, 17, 40, 17, 300, 5, 1000, 0, 33, 2, 999, 16, 64};
  for (size_t i = 0; i < sizeof(lengths) / sizeof(lengths[0]); ++i) {
    if (i == 6) optimi_hip_launch_limit(48);   /* three chunks per launch from here on ... */
    if (i == 10) optimi_hip_launch_limit(-1);  /* ... to here */
    paths_list(g, arena, arena_bytes, lengths[i], (int)i);
    HIP_OK(hipDeviceSynchronize());
  }
  /* per-tensor StableAdamW on tensors that grow and shrink (the group's partials grow), with and without a group */
  static const int64_t sizes[] = {1, 8192, 100000, 513, 3000000, 0, 70000, 10000000, 9};
  for (size_t i = 0; i < sizeof(sizes) / sizeof(sizes[0]); ++i) {
    char* p = arena;
    size_t stride = ((size_t)sizes[i] * 2 + 255) & ~(size_t)255;
    if (6 * stride > arena_bytes) {
      fprintf(stderr, "paths: the arena is too small for six arrays of %lld elements\n", (long long)sizes[i]);
      return 1;
    }
    const uint32_t f = OPTIMI_UPDATE | OPTIMI_KAHAN;
    ABI_OK(optimi_hip_stableadamw_single(g, p, p + stride, p + 2 * stride, p + 3 * stride, p + 4 * stride, sizes[i], OPTIMI_BF16, 1e-3,
                                         0.1, 0.98, 0.02, 1e-2, 1e-6, 0.0, f, NULL));
    ABI_OK(optimi_hip_stableadamw_single_noalloc(p, p + stride, p + 2 * stride, p + 3 * stride, p + 4 * stride, sizes[i], OPTIMI_F16,
                                                 1e-3, 0.1, 0.98, 0.02, 1e-2, 1e-6, 0.0, f, NULL));
    ABI_OK(optimi_hip_ranger_single(p, p + stride, p + 2 * stride, p + 3 * stride, p + 5 * stride, p + 4 * stride, sizes[i], OPTIMI_BF16,
                                    1e-3, 0.1, 0.98, 0.02, 0.99999, 1e-6, 0.7, 0.5, f | OPTIMI_DECOUPLE_WD | OPTIMI_LOOKAHEAD, NULL));
    ABI_OK(optimi_hip_radam_single(p, p + stride, p + 2 * stride, p + 3 * stride, NULL, sizes[i] / 2, OPTIMI_F32, 1e-3, 0.1, 0.98, 0.02,
                                   0.0, 1e-6, 0.0, OPTIMI_UPDATE, NULL));
  }
  ABI_OK(optimi_hip_copy_probe(arena, arena + (arena_bytes >> 1), (int64_t)(arena_bytes >> 1), NULL));
  HIP_OK(hipDeviceSynchronize());
  /* a second group on the same lists, destroyed while the first lives on */
  optimi_group* g2 = NULL;
  ABI_OK(optimi_hip_group_create(&g2));
  paths_list(g2, arena, arena_bytes, 50, 0);
  ABI_OK(optimi_hip_group_destroy(g2));
  paths_list(g, arena, arena_bytes, 50, 1);
  HIP_OK(hipDeviceSynchronize());
  ABI_OK(optimi_hip_group_destroy(g));
  HIP_OK(hipFree(arena));
  printf("abi_host paths ok (%lld kernels, %lld table uploads)\n", (long long)(optimi_hip_launch_count() - launches_before),
         (long long)optimi_hip_upload_count());
  return 0;
}

int main(int argc, char** argv) {
  int n_dev = 0;
  HIP_OK(hipGetDeviceCount(&n_dev));
  if (n_dev < 1) {
    fprintf(stderr, "no HIP device\n");
    return 1;
  }
  HIP_OK(hipSetDevice(0));
  printf("abi version %d, %lld kernels launched so far\n", optimi_hip_version(), (long long)optimi_hip_launch_count());
  if (argc > 1 && strcmp(argv[1], "paths") == 0) {
    launches_before = optimi_hip_launch_count();
    return run_paths();
  }
  int bad = 0;
  for (int opt = 0; opt < N_OPT; ++opt) {
    bad |= run_case(opt, OPTIMI_BF16);
    bad |= run_case(opt, OPTIMI_F32);
  }
  if (bad) return 1;
  printf("abi_host ok (%lld kernels)\n", (long long)optimi_hip_launch_count());
  return 0;
}
