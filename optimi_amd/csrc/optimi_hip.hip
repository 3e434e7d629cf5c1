// Fused optimizer-step kernels for MI355X (gfx950) and the C ABI around them.
//
// Every kernel here is a bandwidth-bound stream over a handful of equally sized arrays
// (param, grad, moments, Kahan buffer).  One workgroup of 256 lanes covers one chunk of
// 16 KiB per array: each lane issues kUnroll 16-byte loads per array before the first
// use, does the arithmetic in fp32 registers, and writes 16-byte stores back in place.
// A whole parameter list runs as ONE launch: a chunk map (chunk -> tensor) and a tensor
// table (pointers, size, first chunk) tell each workgroup where it works.
//
// Arithmetic contract.  Results follow optimi's PyTorch for-loop path
// (optimi/adam.py:354-396, lion.py:301-338, stableadamw.py:421-472, adan.py:405-469),
// which rounds to the tensor dtype after every in-place op.  The element functions below
// replay those rounding points in registers: R() is "round to the tensor dtype", each
// fmaf() is a fusion ATen's CPU kernels perform, and the file is compiled with
// -ffp-contract=off so nothing else fuses.  Division and sqrt are the correctly rounded
// ones.  Scalars are narrowed on the host: S() to fp32, Sd() to the tensor dtype (ATen's
// CPU add kernel casts a scalar operand / alpha to the tensor dtype).

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "optimi_hip.h"

namespace {

constexpr int kThreads = 256;   // lanes per workgroup (4 wavefronts of 64)
constexpr int kUnroll = 4;      // 16-byte vectors per lane per array
constexpr int kMaxArrays = 7;   // Adan: p g m diff sq prev kahan
constexpr int kAbiVersion = 1000;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------------
// dtype policies
// ------------------------------------------------------------------------------------
struct F32 {
  static constexpr int kVec = 4;  // elements per 16-byte vector
  static constexpr int kElemBytes = 4;
  static constexpr int kDtype = OPTIMI_F32;
  static constexpr bool kLowPrecision = false;
  __device__ static __forceinline__ float R(float x) { return x; }
  __device__ static __forceinline__ void unpack(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r[i]);
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __float_as_uint(f[i]);
    return r;
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) { return ((const float*)p)[i]; }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float x) { ((float*)p)[i] = x; }
};

struct BF16 {
  static constexpr int kVec = 8;
  static constexpr int kElemBytes = 2;
  static constexpr int kDtype = OPTIMI_BF16;
  static constexpr bool kLowPrecision = true;
  // round-to-nearest-even to bf16, returned widened (v_cvt_pk_bf16_f32 + shift on gfx950)
  __device__ static __forceinline__ float R(float x) { return (float)(__bf16)x; }
  __device__ static __forceinline__ void unpack(const u32x4& r, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(r[i] << 16);
      f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {  // f[] hold exact bf16 values
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x2 v = {f[2 * i], f[2 * i + 1]};
      r[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    return r;
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) {
    return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16);
  }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float x) {
    ((uint16_t*)p)[i] = (uint16_t)(__float_as_uint(x) >> 16);
  }
};

// ------------------------------------------------------------------------------------
// tables
// ------------------------------------------------------------------------------------
struct TensorEntry {
  void* ptr[kMaxArrays];
  int64_t numel;
  int64_t first_chunk;  // index of this tensor's first chunk within the launch
  uint32_t vec_ok;      // all buffers 16-byte aligned
  uint32_t pad;
};
static_assert(sizeof(TensorEntry) == 80, "TensorEntry layout");

struct TensorScalars {  // StableAdamW: what pass 2 needs per tensor, written on the device
  float neg_lr;
  float wd_factor;
};

// ATen's lerp with a scalar weight: |w| < 0.5 ? fma(w, e-s, s) : fma(w-1, e-s, e).
// The branch and the coefficient depend on the weight only, so the host picks them.
struct Lerp {
  float coef;
  uint32_t small;
};
__device__ __forceinline__ float lerp_apply(float start, float end, const Lerp& l) {
  float d = end - start;
  return fmaf(l.coef, d, l.small ? start : end);
}

template <class DT>
__device__ __forceinline__ void kahan_commit(float& p, float& k) {
  float old = p;
  p = DT::R(old + k);
  float err = DT::R(old - p);
  k = DT::R(k + err);
}

constexpr uint32_t bit(int i) { return 1u << i; }

// ------------------------------------------------------------------------------------
// element functions.  x[] is indexed by array slot; each Op names its slots.
// ------------------------------------------------------------------------------------
struct AdamScalars {
  Lerp l1;
  float wd, wd_alpha, b2h, b2c, eps_d, neg_lr;
  uint32_t wd_mode;  // 0 none, 1 decoupled (p *= wd), 2 L2 (g += wd_alpha * p)
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 exp_avg_sq, 4 kahan_comp     optimi/adam.py:354-396
template <class DT_, bool KAHAN, bool UPDATE>
struct AdamOp {
  using DT = DT_;
  using Scalars = AdamScalars;
  static constexpr int kArrays = 5;
  static constexpr uint32_t kLoad = UPDATE ? (bit(0) | bit(1) | bit(2) | bit(3) | (KAHAN ? bit(4) : 0)) : (bit(1) | bit(2) | bit(3));
  static constexpr uint32_t kStore = UPDATE ? (bit(0) | bit(2) | bit(3) | (KAHAN ? bit(4) : 0)) : (bit(2) | bit(3));
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(float* x, const Scalars& s, float&) {
    float p = x[0], g = x[1], m = x[2], v = x[3];
    if (UPDATE) {
      if (s.wd_mode == 1) p = DT::R(p * s.wd);
      else if (s.wd_mode == 2) g = DT::R(fmaf(p, s.wd_alpha, g));
    }
    m = DT::R(lerp_apply(m, g, s.l1));
    v = DT::R(v * s.b2h);
    v = DT::R(fmaf(s.b2c * g, g, v));
    x[2] = m;
    x[3] = v;
    if (UPDATE) {
      float d = DT::R(sqrtf(v));
      d = DT::R(d + s.eps_d);
      if (KAHAN) {
        float k = x[4];
        k = DT::R(k + (s.neg_lr * m) / d);
        kahan_commit<DT>(p, k);
        x[4] = k;
      } else {
        p = DT::R(p + (s.neg_lr * m) / d);
      }
      x[0] = p;
    }
  }
};

struct LionScalars {
  Lerp l1, l2;
  float wd, neg_lr_d;
  uint32_t do_wd;
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 kahan_comp                  optimi/lion.py:301-338
template <class DT_, bool KAHAN, bool UPDATE>
struct LionOp {
  using DT = DT_;
  using Scalars = LionScalars;
  static constexpr int kArrays = 4;
  static constexpr uint32_t kLoad = UPDATE ? (bit(0) | bit(1) | bit(2) | (KAHAN ? bit(3) : 0)) : (bit(1) | bit(2));
  static constexpr uint32_t kStore = UPDATE ? (bit(0) | bit(2) | (KAHAN ? bit(3) : 0)) : bit(2);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(float* x, const Scalars& s, float&) {
    float p = x[0], g = x[1], m = x[2];
    float u = 0.0f;
    if (UPDATE) {
      if (s.do_wd) p = DT::R(p * s.wd);
      float c = DT::R(lerp_apply(m, g, s.l1));
      u = (float)((c > 0.0f) - (c < 0.0f));
    }
    m = DT::R(lerp_apply(m, g, s.l2));
    x[2] = m;
    if (UPDATE) {
      if (KAHAN) {
        float k = x[3];
        k = DT::R(fmaf(u, s.neg_lr_d, k));
        kahan_commit<DT>(p, k);
        x[3] = k;
      } else {
        p = DT::R(fmaf(u, s.neg_lr_d, p));
      }
      x[0] = p;
    }
  }
};

struct StableP1Scalars {
  Lerp l1;
  float b2h, b2c, eps_sq_d;
};

// StableAdamW pass 1: moments and sum of g^2/max(v, eps^2).  Slots as Adam.   stableadamw.py:442-447
template <class DT_, bool UPDATE>
struct StablePass1Op {
  using DT = DT_;
  using Scalars = StableP1Scalars;
  static constexpr int kArrays = 5;
  static constexpr uint32_t kLoad = bit(1) | bit(2) | bit(3);
  static constexpr uint32_t kStore = bit(2) | bit(3);
  static constexpr bool kReduce = UPDATE;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(float* x, const Scalars& s, float& acc) {
    float g = x[1], m = x[2], v = x[3];
    m = DT::R(lerp_apply(m, g, s.l1));
    v = DT::R(v * s.b2h);
    v = DT::R(fmaf(s.b2c * g, g, v));
    x[2] = m;
    x[3] = v;
    if (UPDATE) {
      float q = DT::R(g * g);
      float mx = v > s.eps_sq_d ? v : s.eps_sq_d;
      q = DT::R(q / mx);
      acc += q;
    }
  }
};

struct StableP2Scalars {
  const TensorScalars* per_tensor;
  float eps_d, neg_lr, wd;  // neg_lr, wd are filled per tensor by prepare()
  uint32_t do_wd;
};

// StableAdamW pass 2: decay with the clipped lr, then the Adam tail.          stableadamw.py:453-472
template <class DT_, bool KAHAN>
struct StablePass2Op {
  using DT = DT_;
  using Scalars = StableP2Scalars;
  static constexpr int kArrays = 5;
  static constexpr uint32_t kLoad = bit(0) | bit(2) | bit(3) | (KAHAN ? bit(4) : 0);
  static constexpr uint32_t kStore = bit(0) | (KAHAN ? bit(4) : 0);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars& s, int tensor) {
    TensorScalars t = s.per_tensor[tensor];
    s.neg_lr = t.neg_lr;
    s.wd = t.wd_factor;
  }
  __device__ static __forceinline__ void elem(float* x, const Scalars& s, float&) {
    float p = x[0], m = x[2], v = x[3];
    if (s.do_wd) p = DT::R(p * s.wd);
    float d = DT::R(sqrtf(v));
    d = DT::R(d + s.eps_d);
    if (KAHAN) {
      float k = x[4];
      k = DT::R(k + (s.neg_lr * m) / d);
      kahan_commit<DT>(p, k);
      x[4] = k;
    } else {
      p = DT::R(p + (s.neg_lr * m) / d);
    }
    x[0] = p;
  }
};

struct AdanScalars {
  Lerp l1, l2;
  float b2, b3h, b3c, eps_d, neg_lr, neg_lr_b2, wd;
  uint32_t wd_mode;  // 0 none, 1 Adam style (p *= wd before), 2 Adan style (p /= wd after)
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 exp_avg_diff, 4 exp_avg_sq, 5 prev_grad, 6 kahan   adan.py:405-469
template <class DT_, bool KAHAN, bool UPDATE>
struct AdanOp {
  using DT = DT_;
  using Scalars = AdanScalars;
  static constexpr int kArrays = 7;
  static constexpr uint32_t kState = bit(2) | bit(3) | bit(4) | bit(5);
  static constexpr uint32_t kLoad = bit(1) | kState | (UPDATE ? (bit(0) | (KAHAN ? bit(6) : 0)) : 0);
  static constexpr uint32_t kStore = kState | (UPDATE ? (bit(0) | (KAHAN ? bit(6) : 0)) : 0);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(float* x, const Scalars& s, float&) {
    float p = x[0], g = x[1], m = x[2], df = x[3], n = x[4], pg = x[5];
    pg = DT::R(pg + g);
    m = DT::R(lerp_apply(m, g, s.l1));
    df = DT::R(lerp_apply(df, pg, s.l2));
    pg = DT::R(pg * s.b2);
    pg = DT::R(pg + g);
    n = DT::R(n * s.b3h);
    n = DT::R(fmaf(s.b3c * pg, pg, n));
    pg = DT::R(g * -1.0f);
    x[2] = m;
    x[3] = df;
    x[4] = n;
    x[5] = pg;
    if (UPDATE) {
      float d = DT::R(sqrtf(n));
      d = DT::R(d + s.eps_d);
      if (s.wd_mode == 1) p = DT::R(p * s.wd);
      if (KAHAN) {
        float k = x[6];
        k = DT::R(k + (s.neg_lr * m) / d);
        k = DT::R(k + (s.neg_lr_b2 * df) / d);
        kahan_commit<DT>(p, k);
        x[6] = k;
      } else {
        p = DT::R(p + (s.neg_lr * m) / d);
        p = DT::R(p + (s.neg_lr_b2 * df) / d);
      }
      if (s.wd_mode == 2) p = DT::R(p / s.wd);
      x[0] = p;
    }
  }
};

// ------------------------------------------------------------------------------------
// the streaming kernel
// ------------------------------------------------------------------------------------
template <class DT>
constexpr int64_t chunk_elems() { return (int64_t)kThreads * DT::kVec * kUnroll; }

// Block-wide sum of one double per lane; the result is valid in lane 0 of wave 0.
__device__ __forceinline__ double block_sum(double v, double* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    v = lds[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) v += lds[w];
  }
  return v;
}

// Unpacks one 16-byte vector per loaded array, runs the element function on each lane's
// elements and writes the stored arrays back to element offset `off` of the tensor.
template <class Op>
__device__ __forceinline__ void compute_store(const TensorEntry& e, int64_t off, const u32x4* raw,
                                              const typename Op::Scalars& s, float& acc) {
  using DT = typename Op::DT;
  constexpr int V = DT::kVec;
  constexpr int A = Op::kArrays;
  float f[A][V];
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kLoad & bit(a)) DT::unpack(raw[a], f[a]);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float x[A];
#pragma unroll
    for (int a = 0; a < A; ++a) x[a] = (Op::kLoad & bit(a)) ? f[a][i] : 0.0f;
    Op::elem(x, s, acc);
#pragma unroll
    for (int a = 0; a < A; ++a)
      if (Op::kStore & bit(a)) f[a][i] = x[a];
  }
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kStore & bit(a))
      __builtin_nontemporal_store(DT::pack(f[a]), (u32x4*)((char*)e.ptr[a] + off * DT::kElemBytes));
}

template <class Op>
__device__ __forceinline__ void load_vec(const TensorEntry& e, int64_t off, u32x4* raw) {
  using DT = typename Op::DT;
#pragma unroll
  for (int a = 0; a < Op::kArrays; ++a)
    if (Op::kLoad & bit(a))
      raw[a] = __builtin_nontemporal_load((const u32x4*)((const char*)e.ptr[a] + off * DT::kElemBytes));
}

template <class Op>
__device__ __forceinline__ void one_element(const TensorEntry& e, int64_t i, const typename Op::Scalars& s, float& acc) {
  using DT = typename Op::DT;
  constexpr int A = Op::kArrays;
  float x[A];
#pragma unroll
  for (int a = 0; a < A; ++a) x[a] = (Op::kLoad & bit(a)) ? DT::load1(e.ptr[a], i) : 0.0f;
  Op::elem(x, s, acc);
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kStore & bit(a)) DT::store1(e.ptr[a], i, x[a]);
}

template <class Op, bool MULTI>
__global__ void __launch_bounds__(kThreads)
step_kernel(const TensorEntry* __restrict__ table, const int32_t* __restrict__ chunk_map, const TensorEntry single,
            typename Op::Scalars s, double* __restrict__ partials) {
  using DT = typename Op::DT;
  constexpr int V = DT::kVec;
  constexpr int A = Op::kArrays;
  constexpr int64_t kChunk = chunk_elems<DT>();

  int tensor = 0;
  if (MULTI) tensor = chunk_map[blockIdx.x];
  const TensorEntry& e = MULTI ? table[tensor] : single;
  const int64_t chunk = (int64_t)blockIdx.x - (MULTI ? e.first_chunk : 0);
  const int64_t base = chunk * kChunk;
  const int64_t remain = e.numel - base;
  Op::prepare(s, tensor);

  float acc = 0.0f;
  if (e.vec_ok && remain >= kChunk) {
    // full chunk: every load is issued before the first use
    u32x4 raw[kUnroll][A];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) load_vec<Op>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, raw[u]);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      compute_store<Op>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, raw[u], s, acc);
  } else if (e.vec_ok) {
    // last chunk of a tensor: whole vectors while they fit, then the few leftover elements
    const int64_t end = e.numel;
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t off = base + ((int64_t)u * kThreads + threadIdx.x) * V;
      if (off + V <= end) {
        u32x4 raw[A];
        load_vec<Op>(e, off, raw);
        compute_store<Op>(e, off, raw, s, acc);
      } else {
        for (int64_t i = off; i < end; ++i) one_element<Op>(e, i, s, acc);
      }
    }
  } else {
    // buffers that are not 16-byte aligned: one element at a time
    const int64_t n = remain < kChunk ? remain : kChunk;
    for (int64_t i = threadIdx.x; i < n; i += kThreads) one_element<Op>(e, base + i, s, acc);
  }

  if (Op::kReduce) {
    __shared__ double lds[kThreads / 64];
    double total = block_sum((double)acc, lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = total;
  }
}

// StableAdamW: one workgroup per tensor turns that tensor's chunk partials into its clipped
// learning rate and decay factor (optimi/stableadamw.py:447-458), in double like the Python
// scalars of the reference.  The mean and its square root are rounded to the tensor dtype,
// as torch's mean()/sqrt() on a tensor of that dtype are.
struct FinalizeArgs {
  double lr, weight_decay, max_lr;
  uint32_t decouple_lr;
};

template <class DT, bool MULTI>
__global__ void __launch_bounds__(kThreads)
stable_finalize_kernel(const TensorEntry* __restrict__ table, const TensorEntry single, const double* __restrict__ partials,
                       TensorScalars* __restrict__ out, FinalizeArgs a) {
  constexpr int64_t kChunk = chunk_elems<DT>();
  const TensorEntry& e = MULTI ? table[blockIdx.x] : single;
  const int64_t first = MULTI ? e.first_chunk : 0;
  const int64_t count = (e.numel + kChunk - 1) / kChunk;
  double v = 0.0;
  for (int64_t c = threadIdx.x; c < count; c += kThreads) v += partials[first + c];
  __shared__ double lds[kThreads / 64];
  double total = block_sum(v, lds);
  if (threadIdx.x == 0) {
    double lr = a.lr;
    if (e.numel > 0) {
      float ms = DT::R((float)total / (float)e.numel);
      float rms = DT::R(sqrtf(ms));
      double r = (double)rms;
      lr = lr / (r > 1.0 ? r : 1.0);
    }
    double factor = a.decouple_lr ? 1.0 - (lr / a.max_lr) * a.weight_decay : 1.0 - lr * a.weight_decay;
    TensorScalars t;
    t.neg_lr = (float)(-lr);
    t.wd_factor = (float)factor;
    out[blockIdx.x] = t;
  }
}

__global__ void __launch_bounds__(kThreads) copy_probe_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * kThreads * kUnroll;
  u32x4 r[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    int64_t i = base + (int64_t)u * kThreads + threadIdx.x;
    if (i < n_vec) r[u] = __builtin_nontemporal_load(src + i);
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    int64_t i = base + (int64_t)u * kThreads + threadIdx.x;
    if (i < n_vec) __builtin_nontemporal_store(r[u], dst + i);
  }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
inline float S(double x) { return (float)x; }
inline float round_bf16_host(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) u = 0x7fc00000u;
  else { u += 0x7fffu + ((u >> 16) & 1u); u &= 0xffff0000u; }
  std::memcpy(&f, &u, 4);
  return f;
}
inline float Sd(double x, int dtype) { return dtype == OPTIMI_BF16 ? round_bf16_host((float)x) : (float)x; }
inline Lerp make_lerp(double weight) {
  float w = (float)weight;
  Lerp l;
  l.small = std::fabs(w) < 0.5f ? 1u : 0u;
  l.coef = l.small ? w : w - 1.0f;
  return l;
}
inline int64_t chunk_elems_rt(int dtype) { return dtype == OPTIMI_BF16 ? chunk_elems<BF16>() : chunk_elems<F32>(); }
inline int elem_bytes(int dtype) { return dtype == OPTIMI_BF16 ? 2 : 4; }

#define HIP_TRY(expr)                          \
  do {                                         \
    hipError_t err__ = (expr);                 \
    if (err__ != hipSuccess) return (int)err__; \
  } while (0)

struct DeviceBuf {
  void* ptr = nullptr;
  size_t cap = 0;
  int reserve(size_t bytes) {
    if (bytes <= cap) return 0;
    size_t want = bytes + bytes / 2 + 4096;
    void* p = nullptr;
    HIP_TRY(hipMalloc(&p, want));
    if (ptr) (void)hipFree(ptr);
    ptr = p;
    cap = want;
    return 0;
  }
  void release() {
    if (ptr) (void)hipFree(ptr);
    ptr = nullptr;
    cap = 0;
  }
};

struct StagingSlot {
  void* host = nullptr;
  size_t cap = 0;
  hipEvent_t done = nullptr;
  bool in_flight = false;
};

}  // namespace

struct optimi_group {
  int device = 0;
  DeviceBuf table, chunk_map, partials, tensor_scalars;
  std::vector<TensorEntry> host_table;   // what the device table holds
  std::vector<int32_t> host_map;         // scratch for building the chunk map
  std::vector<int64_t> map_numel;        // sizes the device chunk map was built for
  int64_t map_chunk = 0;
  int64_t n_chunks = 0;
  StagingSlot ring[4];
  int ring_pos = 0;
  hipEvent_t last_launch = nullptr;
  hipStream_t last_stream = nullptr;
  bool launched = false;
};

namespace {

// Copies `bytes` host bytes to device memory through a pinned ring slot, on `stream`.
int staged_upload(optimi_group* g, void* dst, const void* src, size_t bytes, hipStream_t stream) {
  StagingSlot& slot = g->ring[g->ring_pos];
  g->ring_pos = (g->ring_pos + 1) % 4;
  if (slot.in_flight) {
    HIP_TRY(hipEventSynchronize(slot.done));
    slot.in_flight = false;
  }
  if (slot.cap < bytes) {
    if (slot.host) (void)hipHostFree(slot.host);
    slot.host = nullptr;
    slot.cap = 0;
    size_t want = bytes + bytes / 2 + 4096;
    HIP_TRY(hipHostMalloc(&slot.host, want, hipHostMallocDefault));
    slot.cap = want;
  }
  if (!slot.done) HIP_TRY(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
  std::memcpy(slot.host, src, bytes);
  HIP_TRY(hipMemcpyAsync(dst, slot.host, bytes, hipMemcpyHostToDevice, stream));
  HIP_TRY(hipEventRecord(slot.done, stream));
  slot.in_flight = true;
  return 0;
}

int check_ptrs(int n_tensors, const void* const* list) { return (n_tensors > 0 && list == nullptr) ? OPTIMI_ERR_NULL : 0; }

// Validates the list, (re)builds the chunk map and tensor table and uploads what changed.
// `lists[a]` may be nullptr for an array the launch does not touch (`need` has its bit clear).
int prepare_tables(optimi_group* g, int n_tensors, const void* const* const* lists, int n_arrays, uint32_t need,
                   const int64_t* numel, int dtype, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  if (n_tensors < 0) return OPTIMI_ERR_SIZE;
  if (dtype != OPTIMI_F32 && dtype != OPTIMI_BF16) return OPTIMI_ERR_DTYPE;
  if (n_tensors > 0 && !numel) return OPTIMI_ERR_NULL;
  for (int a = 0; a < n_arrays; ++a)
    if ((need & bit(a)) && check_ptrs(n_tensors, lists[a])) return OPTIMI_ERR_NULL;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev != g->device) return OPTIMI_ERR_DEVICE;

  const int64_t chunk = chunk_elems_rt(dtype);
  const int eb = elem_bytes(dtype);
  std::vector<TensorEntry> fresh;
  try {
    fresh.resize((size_t)n_tensors);
  } catch (const std::bad_alloc&) {
    return OPTIMI_ERR_NOMEM;
  }
  int64_t n_chunks = 0;
  for (int t = 0; t < n_tensors; ++t) {
    TensorEntry& e = fresh[(size_t)t];
    std::memset(&e, 0, sizeof(e));
    if (numel[t] < 0) return OPTIMI_ERR_SIZE;
    e.numel = numel[t];
    e.first_chunk = n_chunks;
    e.vec_ok = 1;
    for (int a = 0; a < n_arrays; ++a) {
      if (!(need & bit(a))) continue;
      const void* p = lists[a][t];
      if (!p && numel[t] > 0) return OPTIMI_ERR_NULL;
      uintptr_t u = (uintptr_t)p;
      if (u % (uintptr_t)eb) return OPTIMI_ERR_ALIGN;
      if (u % 16) e.vec_ok = 0;
      e.ptr[a] = const_cast<void*>(p);
    }
    n_chunks += (numel[t] + chunk - 1) / chunk;
  }
  if (n_chunks > 0x7fffffff) return OPTIMI_ERR_SIZE;

  // a group moved to another stream must not overwrite tables a previous launch still reads
  if (g->launched && g->last_stream != stream) HIP_TRY(hipStreamWaitEvent(stream, g->last_launch, 0));

  bool same_sizes = g->map_chunk == chunk && g->map_numel.size() == (size_t)n_tensors &&
                    (n_tensors == 0 || std::memcmp(g->map_numel.data(), numel, sizeof(int64_t) * (size_t)n_tensors) == 0);
  if (!same_sizes && n_chunks > 0) {
    g->map_chunk = 0;  // the cached map is void until the new one is on its way
    try {
      g->host_map.resize((size_t)n_chunks);
      g->map_numel.assign(numel, numel + n_tensors);
    } catch (const std::bad_alloc&) {
      return OPTIMI_ERR_NOMEM;
    }
    for (int t = 0; t < n_tensors; ++t) {
      const int64_t c0 = fresh[(size_t)t].first_chunk;
      const int64_t c1 = c0 + (numel[t] + chunk - 1) / chunk;
      for (int64_t c = c0; c < c1; ++c) g->host_map[(size_t)c] = t;
    }
    int rc = g->chunk_map.reserve(sizeof(int32_t) * (size_t)n_chunks);
    if (rc) return rc;
    rc = staged_upload(g, g->chunk_map.ptr, g->host_map.data(), sizeof(int32_t) * (size_t)n_chunks, stream);
    if (rc) return rc;
    g->map_chunk = chunk;
  }
  g->n_chunks = n_chunks;

  bool same_table = g->host_table.size() == fresh.size() &&
                    (fresh.empty() || std::memcmp(g->host_table.data(), fresh.data(), sizeof(TensorEntry) * fresh.size()) == 0);
  if (!same_table && n_tensors > 0) {
    int rc = g->table.reserve(sizeof(TensorEntry) * fresh.size());
    if (rc) {
      g->host_table.clear();
      return rc;
    }
    rc = staged_upload(g, g->table.ptr, fresh.data(), sizeof(TensorEntry) * fresh.size(), stream);
    if (rc) {
      g->host_table.clear();
      return rc;
    }
    g->host_table.swap(fresh);
  }
  return 0;
}

int note_launch(optimi_group* g, hipStream_t stream) {
  HIP_TRY(hipGetLastError());
  if (!g->last_launch) HIP_TRY(hipEventCreateWithFlags(&g->last_launch, hipEventDisableTiming));
  HIP_TRY(hipEventRecord(g->last_launch, stream));
  g->last_stream = stream;
  g->launched = true;
  return 0;
}

template <class Op>
void launch_multi(optimi_group* g, const typename Op::Scalars& s, hipStream_t stream) {
  TensorEntry none;
  std::memset(&none, 0, sizeof(none));
  step_kernel<Op, true><<<dim3((unsigned)g->n_chunks), dim3(kThreads), 0, stream>>>(
      (const TensorEntry*)g->table.ptr, (const int32_t*)g->chunk_map.ptr, none, s, (double*)g->partials.ptr);
}

template <class Op>
void launch_single(const TensorEntry& e, const typename Op::Scalars& s, double* partials, hipStream_t stream) {
  const int64_t chunk = chunk_elems<typename Op::DT>();
  const unsigned blocks = (unsigned)((e.numel + chunk - 1) / chunk);
  step_kernel<Op, false><<<dim3(blocks), dim3(kThreads), 0, stream>>>(nullptr, nullptr, e, s, partials);
}

// Runs F<Op>::go() for the Op selected by dtype x kahan x update.
template <template <class, bool, bool> class OpT, class Fn>
void dispatch3(int dtype, bool kahan, bool update, Fn&& fn) {
  if (dtype == OPTIMI_BF16) {
    if (update) {
      if (kahan) fn(OpT<BF16, true, true>{});
      else fn(OpT<BF16, false, true>{});
    } else {
      fn(OpT<BF16, false, false>{});
    }
  } else {
    if (update) fn(OpT<F32, false, true>{});
    else fn(OpT<F32, false, false>{});
  }
}

int single_entry(TensorEntry& e, const void* const* ptrs, int n_arrays, uint32_t need, int64_t numel, int dtype) {
  if (numel < 0) return OPTIMI_ERR_SIZE;
  if (dtype != OPTIMI_F32 && dtype != OPTIMI_BF16) return OPTIMI_ERR_DTYPE;
  if (numel > chunk_elems_rt(dtype) * (int64_t)0x7fffffff) return OPTIMI_ERR_SIZE;
  std::memset(&e, 0, sizeof(e));
  e.numel = numel;
  e.vec_ok = 1;
  const int eb = elem_bytes(dtype);
  for (int a = 0; a < n_arrays; ++a) {
    if (!(need & bit(a))) continue;
    if (!ptrs[a] && numel > 0) return OPTIMI_ERR_NULL;
    uintptr_t u = (uintptr_t)ptrs[a];
    if (u % (uintptr_t)eb) return OPTIMI_ERR_ALIGN;
    if (u % 16) e.vec_ok = 0;
    e.ptr[a] = const_cast<void*>(ptrs[a]);
  }
  return 0;
}

// ---- scalar packs ------------------------------------------------------------------
AdamScalars adam_scalars(int dtype, double lr, double beta1_comp, double beta2_hat, double beta2_comp,
                         double weight_decay, double eps, uint32_t flags) {
  AdamScalars s;
  s.l1 = make_lerp(beta1_comp);
  s.wd = S(weight_decay);
  s.wd_alpha = Sd(weight_decay, dtype);
  s.b2h = S(beta2_hat);
  s.b2c = S(beta2_comp);
  s.eps_d = Sd(eps, dtype);
  s.neg_lr = S(-lr);
  s.wd_mode = (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? ((flags & OPTIMI_DECOUPLE_WD) ? 1u : 2u) : 0u;
  return s;
}
uint32_t adam_need(bool kahan, bool update) {
  return update ? (bit(0) | bit(1) | bit(2) | bit(3) | (kahan ? bit(4) : 0)) : (bit(1) | bit(2) | bit(3));
}

LionScalars lion_scalars(int dtype, double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags) {
  LionScalars s;
  s.l1 = make_lerp(beta1_comp);
  s.l2 = make_lerp(beta2_comp);
  s.wd = S(weight_decay);
  s.neg_lr_d = Sd(-lr, dtype);
  s.do_wd = (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? 1u : 0u;
  return s;
}
uint32_t lion_need(bool kahan, bool update) {
  return update ? (bit(0) | bit(1) | bit(2) | (kahan ? bit(3) : 0)) : (bit(1) | bit(2));
}

AdanScalars adan_scalars(int dtype, double lr, double beta1_comp, double beta2, double beta2_comp, double beta3_hat,
                         double beta3_comp, double eps, double weight_decay, uint32_t flags) {
  AdanScalars s;
  s.l1 = make_lerp(beta1_comp);
  s.l2 = make_lerp(beta2_comp);
  s.b2 = S(beta2);
  s.b3h = S(beta3_hat);
  s.b3c = S(beta3_comp);
  s.eps_d = Sd(eps, dtype);
  s.neg_lr = S(-lr);
  s.neg_lr_b2 = S(-lr * beta2);
  s.wd = S(weight_decay);
  s.wd_mode = (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? ((flags & OPTIMI_ADAM_WD) ? 1u : 2u) : 0u;
  return s;
}
uint32_t adan_need(bool kahan, bool update) {
  return bit(1) | bit(2) | bit(3) | bit(4) | bit(5) | (update ? (bit(0) | (kahan ? bit(6) : 0)) : 0);
}

StableP1Scalars stable_p1_scalars(int dtype, double beta1_comp, double beta2_hat, double beta2_comp, double eps) {
  StableP1Scalars s;
  s.l1 = make_lerp(beta1_comp);
  s.b2h = S(beta2_hat);
  s.b2c = S(beta2_comp);
  s.eps_sq_d = Sd(eps * eps, dtype);  // the reference keeps eps**2 in a tensor of the param dtype
  return s;
}

inline bool kahan_on(int dtype, uint32_t flags) {
  return dtype == OPTIMI_BF16 && (flags & OPTIMI_KAHAN) && (flags & OPTIMI_UPDATE);
}

template <class DT>
int stable_run(bool multi, optimi_group* g, const TensorEntry& single, int n_tensors, int dtype, double lr,
               double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps, double max_lr,
               uint32_t flags, hipStream_t stream) {
  const bool update = (flags & OPTIMI_UPDATE) != 0;
  const bool kahan = kahan_on(dtype, flags);
  const int64_t chunk = chunk_elems<DT>();
  const int64_t n_chunks = multi ? g->n_chunks : (single.numel + chunk - 1) / chunk;
  if (n_chunks == 0) return 0;
  StableP1Scalars s1 = stable_p1_scalars(dtype, beta1_comp, beta2_hat, beta2_comp, eps);
  if (!update) {
    if (multi) launch_multi<StablePass1Op<DT, false>>(g, s1, stream);
    else launch_single<StablePass1Op<DT, false>>(single, s1, nullptr, stream);
    return 0;
  }
  int rc = g->partials.reserve(sizeof(double) * (size_t)n_chunks);
  if (rc) return rc;
  rc = g->tensor_scalars.reserve(sizeof(TensorScalars) * (size_t)(multi ? n_tensors : 1));
  if (rc) return rc;
  FinalizeArgs fa;
  fa.lr = lr;
  fa.weight_decay = weight_decay;
  fa.max_lr = max_lr;
  fa.decouple_lr = (flags & OPTIMI_DECOUPLE_LR) ? 1u : 0u;
  StableP2Scalars s2;
  s2.per_tensor = (const TensorScalars*)g->tensor_scalars.ptr;
  s2.eps_d = Sd(eps, dtype);
  s2.neg_lr = 0.0f;
  s2.wd = 0.0f;
  s2.do_wd = weight_decay != 0 ? 1u : 0u;
  if (multi) {
    launch_multi<StablePass1Op<DT, true>>(g, s1, stream);
    TensorEntry none;
    std::memset(&none, 0, sizeof(none));
    stable_finalize_kernel<DT, true><<<dim3((unsigned)n_tensors), dim3(kThreads), 0, stream>>>(
        (const TensorEntry*)g->table.ptr, none, (const double*)g->partials.ptr, (TensorScalars*)g->tensor_scalars.ptr, fa);
    if (kahan) launch_multi<StablePass2Op<DT, true>>(g, s2, stream);
    else launch_multi<StablePass2Op<DT, false>>(g, s2, stream);
  } else {
    launch_single<StablePass1Op<DT, true>>(single, s1, (double*)g->partials.ptr, stream);
    stable_finalize_kernel<DT, false><<<dim3(1), dim3(kThreads), 0, stream>>>(
        nullptr, single, (const double*)g->partials.ptr, (TensorScalars*)g->tensor_scalars.ptr, fa);
    if (kahan) launch_single<StablePass2Op<DT, true>>(single, s2, nullptr, stream);
    else launch_single<StablePass2Op<DT, false>>(single, s2, nullptr, stream);
  }
  return 0;
}

}  // namespace

// ------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------
extern "C" {

const char* optimi_hip_error_string(int status) {
  switch (status) {
    case OPTIMI_OK: return "success";
    case OPTIMI_ERR_NULL: return "optimi_hip: a required pointer is NULL";
    case OPTIMI_ERR_SIZE: return "optimi_hip: negative or too large element/tensor count";
    case OPTIMI_ERR_DTYPE: return "optimi_hip: unsupported dtype (expected OPTIMI_F32 or OPTIMI_BF16)";
    case OPTIMI_ERR_ALIGN: return "optimi_hip: buffer not aligned to its element size";
    case OPTIMI_ERR_DEVICE: return "optimi_hip: group used on a different device than it was created on";
    case OPTIMI_ERR_NOMEM: return "optimi_hip: host allocation failed";
    case OPTIMI_ERR_ARG: return "optimi_hip: inconsistent scalar argument";
    default: break;
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "optimi_hip: unknown status";
}

int optimi_hip_version(void) { return kAbiVersion; }

int64_t optimi_hip_chunk_elems(int dtype) {
  if (dtype != OPTIMI_F32 && dtype != OPTIMI_BF16) return OPTIMI_ERR_DTYPE;
  return chunk_elems_rt(dtype);
}

int optimi_hip_group_create(optimi_group** out) {
  if (!out) return OPTIMI_ERR_NULL;
  *out = nullptr;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  optimi_group* g = new (std::nothrow) optimi_group();
  if (!g) return OPTIMI_ERR_NOMEM;
  g->device = dev;
  *out = g;
  return 0;
}

int optimi_hip_group_destroy(optimi_group* g) {
  if (!g) return 0;
  int rc = 0;
  if (g->launched) {
    hipError_t e = hipEventSynchronize(g->last_launch);
    if (e != hipSuccess) rc = (int)e;
  }
  for (StagingSlot& s : g->ring) {
    if (s.in_flight) (void)hipEventSynchronize(s.done);
    if (s.done) (void)hipEventDestroy(s.done);
    if (s.host) (void)hipHostFree(s.host);
  }
  if (g->last_launch) (void)hipEventDestroy(g->last_launch);
  g->table.release();
  g->chunk_map.release();
  g->partials.release();
  g->tensor_scalars.release();
  delete g;
  return rc;
}

int optimi_hip_adam_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                          const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                          double beta2_comp, double weight_decay, double eps, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[5] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp};
  int rc = prepare_tables(g, n_tensors, lists, 5, adam_need(kahan, update), numel, dtype, stream);
  if (rc) return rc;
  if (g->n_chunks == 0) return 0;
  AdamScalars s = adam_scalars(dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, flags);
  dispatch3<AdamOp>(dtype, kahan, update, [&](auto op) { launch_multi<decltype(op)>(g, s, stream); });
  return note_launch(g, stream);
}

int optimi_hip_lion_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                          optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[4] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)kahan_comp};
  int rc = prepare_tables(g, n_tensors, lists, 4, lion_need(kahan, update), numel, dtype, stream);
  if (rc) return rc;
  if (g->n_chunks == 0) return 0;
  LionScalars s = lion_scalars(dtype, lr, beta1_comp, beta2_comp, weight_decay, flags);
  dispatch3<LionOp>(dtype, kahan, update, [&](auto op) { launch_multi<decltype(op)>(g, s, stream); });
  return note_launch(g, stream);
}

int optimi_hip_stableadamw_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                 void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                 const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                                 double beta2_comp, double weight_decay, double eps, double max_lr, uint32_t flags,
                                 optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if ((flags & OPTIMI_DECOUPLE_LR) && weight_decay != 0 && !(max_lr > 0)) return OPTIMI_ERR_ARG;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[5] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp};
  int rc = prepare_tables(g, n_tensors, lists, 5, adam_need(kahan, update), numel, dtype, stream);
  if (rc) return rc;
  if (g->n_chunks == 0) return 0;
  TensorEntry none;
  std::memset(&none, 0, sizeof(none));
  rc = dtype == OPTIMI_BF16
           ? stable_run<BF16>(true, g, none, n_tensors, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
           : stable_run<F32>(true, g, none, n_tensors, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream);
  if (rc) return rc;
  return note_launch(g, stream);
}

int optimi_hip_adan_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_diff, void* const* exp_avg_sq,
                          void* const* prev_grad, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2, double beta2_comp, double beta3_hat, double beta3_comp,
                          double eps, double weight_decay, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[7] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_diff, (const void* const*)exp_avg_sq,
                                 (const void* const*)prev_grad, (const void* const*)kahan_comp};
  int rc = prepare_tables(g, n_tensors, lists, 7, adan_need(kahan, update), numel, dtype, stream);
  if (rc) return rc;
  if (g->n_chunks == 0) return 0;
  AdanScalars s = adan_scalars(dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags);
  dispatch3<AdanOp>(dtype, kahan, update, [&](auto op) { launch_multi<decltype(op)>(g, s, stream); });
  return note_launch(g, stream);
}

int optimi_hip_adam_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan_comp,
                           int64_t numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                           double beta2_comp, double weight_decay, double eps, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* ptrs[5] = {param, grad, exp_avg, exp_avg_sq, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 5, adam_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  AdamScalars s = adam_scalars(dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, flags);
  dispatch3<AdamOp>(dtype, kahan, update, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_lion_single(void* param, const void* grad, void* exp_avg, void* kahan_comp, int64_t numel, int dtype,
                           double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                           optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* ptrs[4] = {param, grad, exp_avg, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 4, lion_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  LionScalars s = lion_scalars(dtype, lr, beta1_comp, beta2_comp, weight_decay, flags);
  dispatch3<LionOp>(dtype, kahan, update, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_stableadamw_single(optimi_group* g, void* param, const void* grad, void* exp_avg, void* exp_avg_sq,
                                  void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                                  double beta2_hat, double beta2_comp, double weight_decay, double eps, double max_lr,
                                  uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!g) return OPTIMI_ERR_NULL;
  if ((flags & OPTIMI_DECOUPLE_LR) && weight_decay != 0 && !(max_lr > 0)) return OPTIMI_ERR_ARG;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* ptrs[5] = {param, grad, exp_avg, exp_avg_sq, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 5, adam_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev != g->device) return OPTIMI_ERR_DEVICE;
  if (g->launched && g->last_stream != stream) HIP_TRY(hipStreamWaitEvent(stream, g->last_launch, 0));
  rc = dtype == OPTIMI_BF16
           ? stable_run<BF16>(false, g, e, 1, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
           : stable_run<F32>(false, g, e, 1, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream);
  if (rc) return rc;
  return note_launch(g, stream);
}

int optimi_hip_adan_single(void* param, const void* grad, void* exp_avg, void* exp_avg_diff, void* exp_avg_sq,
                           void* prev_grad, void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                           double beta2, double beta2_comp, double beta3_hat, double beta3_comp, double eps,
                           double weight_decay, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* ptrs[7] = {param, grad, exp_avg, exp_avg_diff, exp_avg_sq, prev_grad, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 7, adan_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  AdanScalars s = adan_scalars(dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags);
  dispatch3<AdanOp>(dtype, kahan, update, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_copy_probe(void* dst, const void* src, int64_t bytes, optimi_stream_t stream_) {
  if (!dst || !src) return OPTIMI_ERR_NULL;
  if (bytes < 0 || bytes % 16) return OPTIMI_ERR_SIZE;
  if (((uintptr_t)dst % 16) || ((uintptr_t)src % 16)) return OPTIMI_ERR_ALIGN;
  const int64_t n_vec = bytes / 16;
  if (n_vec == 0) return 0;
  const int64_t per_block = (int64_t)kThreads * kUnroll;
  const int64_t blocks = (n_vec + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return OPTIMI_ERR_SIZE;
  copy_probe_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream_>>>((u32x4*)dst, (const u32x4*)src, n_vec);
  HIP_TRY(hipGetLastError());
  return 0;
}

}  // extern "C"
