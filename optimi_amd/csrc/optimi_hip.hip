// Fused optimizer-step kernels for MI355X (gfx950) and the C ABI around them.
//
// Every kernel here is a bandwidth-bound stream over a handful of equally sized arrays
// (param, grad, moments, Kahan buffer).  Tensors are cut into chunks of 16 KiB per array;
// kSub workgroups of kThreads lanes share a chunk, each lane issuing kUnroll 16-byte loads
// per array before the first use, doing the arithmetic in fp32 registers and writing
// 16-byte stores back in place.  A whole parameter list runs as ONE launch: a tensor table
// (pointers, size, first chunk) tells each workgroup where it works - found through a chunk
// map (chunk -> tensor) in device memory, or, for lists of at most 16 tensors, searched in a
// copy that travels as a kernel argument (tables.h).  How many workgroups a CU holds at once
// is throttled with a dummy dynamic-LDS request (see launch_shape): with up to thirteen
// concurrent streams HBM runs best when only a few tens of KiB per CU are in flight.
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
#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <cstring>
#include <initializer_list>
#include <mutex>
#include <new>
#include <type_traits>
#include <utility>
#include <vector>

#include "optimi_hip.h"
#include "tables.h"

namespace {

using optimi_tables::bit;
using optimi_tables::FewTable;
using optimi_tables::kChunkBytes;
using optimi_tables::kFew;
using optimi_tables::kMaxArrays;
using optimi_tables::TensorEntry;
using optimi_tables::valid_dtype;

#ifndef OPTIMI_THREADS
#define OPTIMI_THREADS 64
#endif
#ifndef OPTIMI_UNROLL
#define OPTIMI_UNROLL 1
#endif
constexpr int kThreads = OPTIMI_THREADS;  // lanes per workgroup
constexpr int kUnroll = OPTIMI_UNROLL;    // 16-byte vectors per lane per array
constexpr int kSub = kChunkBytes / (kThreads * kUnroll * 16);  // workgroups per chunk
static_assert(kSub >= 1 && kSub * kThreads * kUnroll * 16 == kChunkBytes, "workgroup tile must divide the chunk");
static_assert(kThreads % 64 == 0 && kThreads <= 1024, "whole wavefronts");
constexpr int kReduceThreads = 1024;      // lanes of the per-tensor finalize workgroup
static_assert((int64_t)optimi_tables::kMaxTensors * kReduceThreads < ((int64_t)1 << 32), "one finalize workgroup per tensor must fit a grid");
constexpr int kAbiVersion = 1004;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Pointers come out of the tensor table as plain addresses; telling the compiler they are
// global memory gets global_load/global_store instead of flat accesses.
#define OPTIMI_GLOBAL __attribute__((address_space(1)))
// Streaming load: the data will not be used again before it has left every cache (`nt` policy).
__device__ __forceinline__ u32x4 load16(const void* base, int64_t byte_off) {
  return __builtin_nontemporal_load((const OPTIMI_GLOBAL u32x4*)((uintptr_t)base + (uintptr_t)byte_off));
}
// Ordinary cached load of a lane's vector of a full tile, for a working set small enough to stay
// in the 256 MB last-level cache between steps.  Written as a buffer load so that the compiler
// cannot merge it with the streaming load of the other branch (merging two loads that differ only
// in the `nt` hint drops the hint from both).  `tile` (wave-uniform) points at the workgroup's
// tile of one array, `lane_off` is the lane's byte offset in it.
__device__ __forceinline__ u32x4 load16_tile_cached(const void* tile, uint32_t lane_off) {
  __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(tile), 0, (uint32_t)(kThreads * kUnroll * 16), 0x00020000);
  return __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, 0, 0);
}
__device__ __forceinline__ void store16(void* base, int64_t byte_off, u32x4 v) {
  __builtin_nontemporal_store(v, (OPTIMI_GLOBAL u32x4*)((uintptr_t)base + (uintptr_t)byte_off));
}
// The same vector at an address that is only aligned to one element (ELEM = 2 or 4 bytes): the
// reduced alignment of the type tells the compiler so, and it emits what the target guarantees
// to work (one 16-byte access on gfx950, whose memory unit handles unaligned global accesses).
typedef u32x4 u32x4_align2 __attribute__((aligned(2)));
typedef u32x4 u32x4_align4 __attribute__((aligned(4)));
template <int ELEM>
__device__ __forceinline__ u32x4 load16_unaligned(const void* base, int64_t byte_off) {
  const uintptr_t at = (uintptr_t)base + (uintptr_t)byte_off;
  if (ELEM == 2) return __builtin_nontemporal_load((const OPTIMI_GLOBAL u32x4_align2*)at);
  return __builtin_nontemporal_load((const OPTIMI_GLOBAL u32x4_align4*)at);
}
template <int ELEM>
__device__ __forceinline__ void store16_unaligned(void* base, int64_t byte_off, u32x4 v) {
  const uintptr_t at = (uintptr_t)base + (uintptr_t)byte_off;
  if (ELEM == 2) __builtin_nontemporal_store(v, (OPTIMI_GLOBAL u32x4_align2*)at);
  else __builtin_nontemporal_store(v, (OPTIMI_GLOBAL u32x4_align4*)at);
}

// The store of a full tile: a buffer store with the sc0 sc1 cache policy, i.e. written through
// to memory instead of left dirty in L2 (or marked for early eviction, as `nt` does).  With nine
// streams per wave this is worth about 3 % of HBM bandwidth on MI355X: dirty lines evicted later
// reach the DRAM out of step with the reads.  The clang builtin for global stores cannot
// express the policy, the buffer builtin can, and unlike inline assembly it is tracked by the
// compiler's wait-count insertion.  `tile` (wave-uniform) points at the workgroup's tile of
// one array, `lane_off` is the lane's byte offset in it.
#ifndef OPTIMI_STORE_POLICY
#define OPTIMI_STORE_POLICY (1 | 16)
#endif
constexpr int kStorePolicy = OPTIMI_STORE_POLICY;  // aux bits of the buffer instructions on gfx94x/gfx950: 1 sc0, 2 nt, 16 sc1
__device__ __forceinline__ void store16_tile(void* tile, uint32_t lane_off, u32x4 v) {
  // dword 3 = 0x00020000: raw buffer, 32-bit data format; stride 0; bounds = the tile
  __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(tile, 0, (uint32_t)(kThreads * kUnroll * 16), 0x00020000);
  __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_off, 0, kStorePolicy);
}

// Element math runs on pairs of neighbouring elements (f32x2): one v_cvt_pk_bf16_f32 then
// rounds two values.  With packed fp32 ops disabled the pair arithmetic is two scalar ops.
__device__ __forceinline__ f32x2 splat(float x) { return f32x2{x, x}; }
__device__ __forceinline__ f32x2 fma2(f32x2 a, f32x2 b, f32x2 c) { return f32x2{fmaf(a.x, b.x, c.x), fmaf(a.y, b.y, c.y)}; }
__device__ __forceinline__ f32x2 sqrt2(f32x2 a) { return f32x2{sqrtf(a.x), sqrtf(a.y)}; }
__device__ __forceinline__ f32x2 div2(f32x2 a, f32x2 b) { return f32x2{a.x / b.x, a.y / b.y}; }

// ------------------------------------------------------------------------------------
// dtype policies
// ------------------------------------------------------------------------------------
struct F32 {
  static constexpr int kVec = 4;    // elements per 16-byte vector
  static constexpr int kPairs = 2;  // element pairs per vector
  static constexpr int kElemBytes = 4;
  __device__ static __forceinline__ f32x2 R2(f32x2 x) { return x; }
  __device__ static __forceinline__ void unpack(const u32x4& r, f32x2* f) {
    f[0] = f32x2{__uint_as_float(r[0]), __uint_as_float(r[1])};
    f[1] = f32x2{__uint_as_float(r[2]), __uint_as_float(r[3])};
  }
  __device__ static __forceinline__ u32x4 pack(const f32x2* f) {
    return u32x4{__float_as_uint(f[0].x), __float_as_uint(f[0].y), __float_as_uint(f[1].x), __float_as_uint(f[1].y)};
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) { return ((const OPTIMI_GLOBAL float*)(uintptr_t)p)[i]; }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float x) { ((OPTIMI_GLOBAL float*)(uintptr_t)p)[i] = x; }
};

struct BF16 {
  static constexpr int kVec = 8;
  static constexpr int kPairs = 4;
  static constexpr int kElemBytes = 2;
  __device__ static __forceinline__ f32x2 widen(uint32_t two) {  // two packed bf16 -> two floats
    return f32x2{__uint_as_float(two << 16), __uint_as_float(two & 0xffff0000u)};
  }
  __device__ static __forceinline__ uint32_t narrow(f32x2 x) {  // round-to-nearest-even, v_cvt_pk_bf16_f32
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
  }
  __device__ static __forceinline__ f32x2 R2(f32x2 x) { return widen(narrow(x)); }
  __device__ static __forceinline__ void unpack(const u32x4& r, f32x2* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = widen(r[i]);
  }
  // Two floats that hold exact bf16 values, packed: their upper halves.  Written with plain bit
  // operations so that the compiler sees through join(widen(u)) == u: a value that R2 has just
  // rounded is stored without a second conversion (4 to 6 % fewer vector instructions per tile).
  __device__ static __forceinline__ uint32_t join(f32x2 x) {
    return (__float_as_uint(x.y) & 0xffff0000u) | (__float_as_uint(x.x) >> 16);
  }
  __device__ static __forceinline__ u32x4 pack(const f32x2* f) {  // f[] hold exact bf16 values
    return u32x4{join(f[0]), join(f[1]), join(f[2]), join(f[3])};
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) {
    return __uint_as_float((uint32_t)((const OPTIMI_GLOBAL uint16_t*)(uintptr_t)p)[i] << 16);
  }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float x) {
    ((OPTIMI_GLOBAL uint16_t*)(uintptr_t)p)[i] = (uint16_t)(__float_as_uint(x) >> 16);
  }
};

struct F16 {
  static constexpr int kVec = 8;
  static constexpr int kPairs = 4;
  static constexpr int kElemBytes = 2;
  __device__ static __forceinline__ f32x2 widen(uint32_t two) {  // two packed halves -> two floats
    return __builtin_convertvector(__builtin_bit_cast(f16x2, two), f32x2);
  }
  // Round to nearest even, subnormals kept.  The conversion is written as an instruction so that
  // the compiler cannot merge it with the fma that feeds it: the merged form (v_fma_mixlo_f16)
  // rounds the exact result once, while the reference rounds to fp32 first and to fp16 second.
  __device__ static __forceinline__ uint32_t narrow(f32x2 x) {
    uint32_t r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(x.x), "v"(x.y));
    return r;
  }
  __device__ static __forceinline__ f32x2 R2(f32x2 x) { return widen(narrow(x)); }
  __device__ static __forceinline__ void unpack(const u32x4& r, f32x2* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = widen(r[i]);
  }
  __device__ static __forceinline__ u32x4 pack(const f32x2* f) {
    return u32x4{narrow(f[0]), narrow(f[1]), narrow(f[2]), narrow(f[3])};
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) {
    return (float)((const OPTIMI_GLOBAL _Float16*)(uintptr_t)p)[i];
  }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float x) {
    ((OPTIMI_GLOBAL uint16_t*)(uintptr_t)p)[i] = (uint16_t)narrow(f32x2{x, x});
  }
};

// ------------------------------------------------------------------------------------
// tables
// ------------------------------------------------------------------------------------
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
__device__ __forceinline__ f32x2 lerp2(f32x2 start, f32x2 end, const Lerp& l) {
  f32x2 d = end - start;
  return fma2(splat(l.coef), d, l.small ? start : end);
}

// param += kahan; kahan += (old param - new param)
template <class DT>
__device__ __forceinline__ void kahan_commit(f32x2& p, f32x2& k) {
  f32x2 old = p;
  p = DT::R2(old + k);
  f32x2 err = DT::R2(old - p);
  k = DT::R2(k + err);
}

// ------------------------------------------------------------------------------------
// element functions on pairs.  x[] is indexed by array slot; each Op names its slots.
// KAHAN / UPDATE / WD are compile-time so the inner code is branch-free; UPDATE=false is the
// accumulate-only step, which touches neither the parameter nor the Kahan buffer.
// ------------------------------------------------------------------------------------
struct AdamScalars {
  Lerp l1;
  float wd, wd_alpha, b2h, b2c, eps_d, neg_lr, neg_lr_d;
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 exp_avg_sq, 4 kahan_comp     optimi/adam.py:354-396
// WD: 0 none, 1 decoupled (p *= wd), 2 L2 (g += wd_alpha * p)
// TAIL: 0 the Adam step -lr*m/(sqrt(v)+eps); 1 RAdam's unrectified step -lr*m (optimi/radam.py:398-417)
template <class DT_, bool KAHAN, bool UPDATE, int WD, int TAIL>
struct AdamTailOp {
  using DT = DT_;
  using F32Partner = AdamTailOp<F32, false, UPDATE, WD, TAIL>;  // the same step on an fp32 tensor of a mixed list
  using Scalars = AdamScalars;
  static constexpr int kArrays = 5;
  static constexpr uint32_t kLoad = UPDATE ? (bit(0) | bit(1) | bit(2) | bit(3) | (KAHAN ? bit(4) : 0)) : (bit(1) | bit(2) | bit(3));
  static constexpr uint32_t kStore = UPDATE ? (bit(0) | bit(2) | bit(3) | (KAHAN ? bit(4) : 0)) : (bit(2) | bit(3));
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    f32x2 p = x[0], g = x[1], m = x[2], v = x[3];
    if (UPDATE && WD == 1) p = DT::R2(p * s.wd);
    if (UPDATE && WD == 2) g = DT::R2(fma2(p, splat(s.wd_alpha), g));
    m = DT::R2(lerp2(m, g, s.l1));
    v = DT::R2(v * s.b2h);
    v = DT::R2(fma2(g * s.b2c, g, v));
    x[2] = m;
    x[3] = v;
    if (UPDATE) {
      f32x2 k = KAHAN ? x[4] : p;  // the accumulator the step lands in
      if (TAIL == 0) {
        f32x2 d = DT::R2(sqrt2(v));
        d = DT::R2(d + s.eps_d);
        k = DT::R2(k + div2(m * s.neg_lr, d));
      } else {
        k = DT::R2(fma2(m, splat(s.neg_lr_d), k));
      }
      if (KAHAN) {
        kahan_commit<DT>(p, k);
        x[4] = k;
      } else {
        p = k;
      }
      x[0] = p;
    }
  }
};
template <class DT, bool KAHAN, bool UPDATE, int WD> using AdamOp = AdamTailOp<DT, KAHAN, UPDATE, WD, 0>;
template <class DT, bool KAHAN, bool UPDATE, int WD> using RAdamEarlyOp = AdamTailOp<DT, KAHAN, UPDATE, WD, 1>;

struct RangerScalars {
  AdamScalars a;
  float alpha_d;
};

// Ranger = the RAdam step, then every k-th step (step % k == 0) a Lookahead sync with the slow
// weights.  This Op is such a synchronising step; every other Ranger step is RAdam's Op.
// slots: 0 param, 1 grad, 2 exp_avg, 3 exp_avg_sq, 4 kahan_comp, 5 la_param   optimi/ranger.py:402-473
template <class DT_, bool KAHAN, int WD, int TAIL>
struct RangerOp {
  using DT = DT_;
  using F32Partner = RangerOp<F32, false, WD, TAIL>;
  using Scalars = RangerScalars;
  using Inner = AdamTailOp<DT_, KAHAN, true, WD, TAIL>;
  static constexpr int kArrays = 6;
  static constexpr uint32_t kLoad = Inner::kLoad | bit(5);
  static constexpr uint32_t kStore = Inner::kStore | bit(5);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2& q) {
    Inner::elem(x, s.a, q);
    f32x2 p = x[0], la = x[5];
    f32x2 t = DT::R2(p - la);
    if (KAHAN) {
      f32x2 k = x[4];
      k = DT::R2(fma2(t, splat(s.alpha_d), k));
      f32x2 old = la;
      la = DT::R2(old + k);
      f32x2 err = DT::R2(old - la);
      k = DT::R2(fma2(err, splat(s.alpha_d), k));
      x[4] = k;
    } else {
      la = DT::R2(fma2(t, splat(s.alpha_d), la));
    }
    x[0] = la;
    x[5] = la;
  }
};

struct SgdScalars {
  Lerp damp;
  float wd, wd_alpha, momentum, neg_lr_d;
};

// slots: 0 param, 1 grad, 2 exp_avg (momentum buffer), 3 kahan_comp          optimi/sgd.py:329-372
// WD as Adam.  MOM: 0 no momentum (the step uses the gradient), 1 m = m*momentum + g, 2 dampening (lerp)
template <class DT_, bool KAHAN, bool UPDATE, int WD, int MOM>
struct SgdOp {
  using DT = DT_;
  using F32Partner = SgdOp<F32, false, UPDATE, WD, MOM>;
  using Scalars = SgdScalars;
  static constexpr int kArrays = 4;
  static constexpr uint32_t kLoad = bit(1) | (MOM ? bit(2) : 0) | (UPDATE ? (bit(0) | (KAHAN ? bit(3) : 0)) : 0);
  static constexpr uint32_t kStore = (MOM ? bit(2) : 0) | (UPDATE ? (bit(0) | (KAHAN ? bit(3) : 0)) : 0);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    f32x2 p = x[0], g = x[1], m = x[2];
    if (UPDATE && WD == 1) p = DT::R2(p * s.wd);
    if (UPDATE && WD == 2) g = DT::R2(fma2(p, splat(s.wd_alpha), g));
    if (MOM == 1) {
      m = DT::R2(m * s.momentum);
      m = DT::R2(m + g);
    } else if (MOM == 2) {
      m = DT::R2(lerp2(m, g, s.damp));
    } else {
      m = g;
    }
    if (MOM) x[2] = m;
    if (UPDATE) {
      if (KAHAN) {
        f32x2 k = x[3];
        k = DT::R2(fma2(m, splat(s.neg_lr_d), k));
        kahan_commit<DT>(p, k);
        x[3] = k;
      } else {
        p = DT::R2(fma2(m, splat(s.neg_lr_d), p));
      }
      x[0] = p;
    }
  }
};

struct LionScalars {
  Lerp l1, l2;
  float wd, neg_lr_d;
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 kahan_comp                  optimi/lion.py:301-338
// WD: 0 none, 1 decoupled
template <class DT_, bool KAHAN, bool UPDATE, int WD>
struct LionOp {
  using DT = DT_;
  using F32Partner = LionOp<F32, false, UPDATE, WD>;
  using Scalars = LionScalars;
  static constexpr int kArrays = 4;
  static constexpr uint32_t kLoad = UPDATE ? (bit(0) | bit(1) | bit(2) | (KAHAN ? bit(3) : 0)) : (bit(1) | bit(2));
  static constexpr uint32_t kStore = UPDATE ? (bit(0) | bit(2) | (KAHAN ? bit(3) : 0)) : bit(2);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ float sign1(float c) { return (float)((c > 0.0f) - (c < 0.0f)); }
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    f32x2 p = x[0], g = x[1], m = x[2];
    f32x2 u = splat(0.0f);
    if (UPDATE) {
      if (WD == 1) p = DT::R2(p * s.wd);
      f32x2 c = DT::R2(lerp2(m, g, s.l1));
      u = f32x2{sign1(c.x), sign1(c.y)};
    }
    m = DT::R2(lerp2(m, g, s.l2));
    x[2] = m;
    if (UPDATE) {
      if (KAHAN) {
        f32x2 k = x[3];
        k = DT::R2(fma2(u, splat(s.neg_lr_d), k));
        kahan_commit<DT>(p, k);
        x[3] = k;
      } else {
        p = DT::R2(fma2(u, splat(s.neg_lr_d), p));
      }
      x[0] = p;
    }
  }
};

struct StableP1Scalars {
  Lerp l1;
  float b2h, b2c, eps_sq_d;
};

// StableAdamW pass 1: moments and g^2/max(v, eps^2) per element (summed by the kernel).
// Slots as Adam.                                                optimi/stableadamw.py:442-447
template <class DT_, bool UPDATE>
struct StablePass1Op {
  using DT = DT_;
  using F32Partner = StablePass1Op<F32, UPDATE>;
  using Scalars = StableP1Scalars;
  static constexpr int kArrays = 5;
  static constexpr uint32_t kLoad = bit(1) | bit(2) | bit(3);
  static constexpr uint32_t kStore = bit(2) | bit(3);
  static constexpr bool kReduce = UPDATE;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2& q) {
    f32x2 g = x[1], m = x[2], v = x[3];
    m = DT::R2(lerp2(m, g, s.l1));
    v = DT::R2(v * s.b2h);
    v = DT::R2(fma2(g * s.b2c, g, v));
    x[2] = m;
    x[3] = v;
    if (UPDATE) {
      q = DT::R2(g * g);
      f32x2 mx = f32x2{v.x > s.eps_sq_d ? v.x : s.eps_sq_d, v.y > s.eps_sq_d ? v.y : s.eps_sq_d};
      q = DT::R2(div2(q, mx));
    }
  }
};

struct StableP2Scalars {
  const TensorScalars* per_tensor;
  float eps_d, neg_lr, wd;  // neg_lr, wd are filled per tensor by prepare()
};

// StableAdamW pass 2: decay with the clipped lr, then the Adam tail.   stableadamw.py:453-472
// WD: 0 none, 1 decoupled with the per-tensor factor
template <class DT_, bool KAHAN, int WD>
struct StablePass2Op {
  using DT = DT_;
  using F32Partner = StablePass2Op<F32, false, WD>;
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
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    f32x2 p = x[0], m = x[2], v = x[3];
    if (WD == 1) p = DT::R2(p * s.wd);
    f32x2 d = DT::R2(sqrt2(v));
    d = DT::R2(d + s.eps_d);
    if (KAHAN) {
      f32x2 k = x[4];
      k = DT::R2(k + div2(m * s.neg_lr, d));
      kahan_commit<DT>(p, k);
      x[4] = k;
    } else {
      p = DT::R2(p + div2(m * s.neg_lr, d));
    }
    x[0] = p;
  }
};

struct AdanScalars {
  Lerp l1, l2;
  float b2, b3h, b3c, eps_d, neg_lr, neg_lr_b2, wd;
};

// slots: 0 param, 1 grad, 2 exp_avg, 3 exp_avg_diff, 4 exp_avg_sq, 5 prev_grad, 6 kahan   adan.py:405-469
// WD: 0 none, 1 Adam style (p *= wd before the step), 2 Adan style (p /= wd after it)
template <class DT_, bool KAHAN, bool UPDATE, int WD>
struct AdanOp {
  using DT = DT_;
  using F32Partner = AdanOp<F32, false, UPDATE, WD>;
  using Scalars = AdanScalars;
  static constexpr int kArrays = 7;
  static constexpr uint32_t kState = bit(2) | bit(3) | bit(4) | bit(5);
  static constexpr uint32_t kLoad = bit(1) | kState | (UPDATE ? (bit(0) | (KAHAN ? bit(6) : 0)) : 0);
  static constexpr uint32_t kStore = kState | (UPDATE ? (bit(0) | (KAHAN ? bit(6) : 0)) : 0);
  static constexpr bool kReduce = false;
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    f32x2 p = x[0], g = x[1], m = x[2], df = x[3], n = x[4], pg = x[5];
    pg = DT::R2(pg + g);
    m = DT::R2(lerp2(m, g, s.l1));
    df = DT::R2(lerp2(df, pg, s.l2));
    pg = DT::R2(pg * s.b2);
    pg = DT::R2(pg + g);
    n = DT::R2(n * s.b3h);
    n = DT::R2(fma2(pg * s.b3c, pg, n));
    pg = -g;  // R(g * -1): the negation of a value of the tensor dtype is exact, so only the sign bit moves
    x[2] = m;
    x[3] = df;
    x[4] = n;
    x[5] = pg;
    if (UPDATE) {
      f32x2 d = DT::R2(sqrt2(n));
      d = DT::R2(d + s.eps_d);
      if (WD == 1) p = DT::R2(p * s.wd);
      if (KAHAN) {
        f32x2 k = x[6];
        k = DT::R2(k + div2(m * s.neg_lr, d));
        k = DT::R2(k + div2(df * s.neg_lr_b2, d));
        kahan_commit<DT>(p, k);
        x[6] = k;
      } else {
        p = DT::R2(p + div2(m * s.neg_lr, d));
        p = DT::R2(p + div2(df * s.neg_lr_b2, d));
      }
      if (WD == 2) p = DT::R2(div2(p, splat(s.wd)));
      x[0] = p;
    }
  }
};

struct ProbeScalars {
  uint32_t salt, mask;
};

// Measurement aid, not an optimizer: the memory traffic of a step with NR arrays read and the
// first NW of them written in place, and no floating-point work.  It runs through the very
// kernel, tiles, loads, stores, tables and occupancy throttle the optimizers use, so what it
// reaches is the ceiling of that access mix on the machine at hand: AdamW with Kahan is 5 read /
// 4 written, Lion 4 / 3, StableAdamW's passes 3 / 2 and 4 / 2, Adan 7 / 6.  The 16-byte vectors
// pass through as raw bits (the F32 policy neither converts nor rounds).  Every stored vector
// depends on every loaded one - as the parameter, the first array an optimizer stores, depends on
// all of its inputs - so no load can be dropped and a lane's stores follow all of its loads.
// What is stored is the array's own content xor (a mix of everything loaded & mask): the mask is 0
// unless the caller asks for scrambling, so the arrays keep their bits (the bandwidth of this
// memory depends a little on the data, and a probe that filled the arrays with noise would be
// measured on other data than the step it stands for); the compiler cannot know that.
template <int NR, int NW>
struct ProbeOp {
  using DT = F32;
  using F32Partner = ProbeOp<NR, NW>;
  using Scalars = ProbeScalars;
  static constexpr bool kProbe = true;
  static constexpr int kArrays = kMaxArrays;
  static constexpr uint32_t kLoad = (1u << NR) - 1u;
  static constexpr uint32_t kStore = (1u << NW) - 1u;
  static constexpr bool kReduce = false;
  static_assert(NW >= 1 && NW <= NR && NR <= kMaxArrays, "written arrays are among the read ones");
  __device__ static __forceinline__ void prepare(Scalars&, int) {}
  __device__ static __forceinline__ void elem(f32x2* x, const Scalars& s, f32x2&) {
    uint32_t d0 = s.salt, d1 = s.salt;
#pragma unroll
    for (int a = 0; a < NR; ++a) {
      d0 ^= __float_as_uint(x[a].x);
      d1 ^= __float_as_uint(x[a].y);
    }
#pragma unroll
    for (int a = 0; a < NW; ++a)
      x[a] = f32x2{__uint_as_float(__float_as_uint(x[a].x) ^ ((d0 + (uint32_t)a) & s.mask)),
                   __uint_as_float(__float_as_uint(x[a].y) ^ ((d1 + (uint32_t)a) & s.mask))};
  }
};

template <class Op, class = void>
struct is_probe : std::false_type {};
template <class Op>
struct is_probe<Op, std::enable_if_t<Op::kProbe>> : std::true_type {};

// ------------------------------------------------------------------------------------
// the streaming kernel
// ------------------------------------------------------------------------------------
template <class DT>
constexpr int64_t chunk_elems() { return kChunkBytes / DT::kElemBytes; }

// Block-wide sum of one double per lane; the result is valid in lane 0 of wave 0.
template <int THREADS>
__device__ __forceinline__ double block_sum(double v, double* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  if (THREADS == 64) return v;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    v = lds[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) v += lds[w];
  }
  return v;
}

// Unpacks one 16-byte vector per loaded array, runs the element function on each pair and
// writes the stored arrays back to element offset `off` of the tensor.
// `TILE`: the workgroup owns a full tile starting at element `tile_base` (wave-uniform) and
// stores through store16_tile; otherwise element `off` onwards is stored with plain stores -
// `UNALIGNED`: at addresses that are only aligned to one element.
template <class Op, bool TILE = false, bool UNALIGNED = false>
__device__ __forceinline__ void compute_store(const TensorEntry& e, int64_t off, const u32x4* raw,
                                              const typename Op::Scalars& s, float& acc, int64_t tile_base = 0) {
  using DT = typename Op::DT;
  constexpr int P = DT::kPairs;
  constexpr int A = Op::kArrays;
  f32x2 f[A][P];
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kLoad & bit(a)) DT::unpack(raw[a], f[a]);
#pragma unroll
  for (int i = 0; i < P; ++i) {
    f32x2 x[A];
#pragma unroll
    for (int a = 0; a < A; ++a) x[a] = (Op::kLoad & bit(a)) ? f[a][i] : splat(0.0f);
    f32x2 q = splat(0.0f);
    Op::elem(x, s, q);
    if (Op::kReduce) {
      acc += q.x;
      acc += q.y;
    }
#pragma unroll
    for (int a = 0; a < A; ++a)
      if (Op::kStore & bit(a)) f[a][i] = x[a];
  }
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kStore & bit(a)) {
      if (TILE)
        store16_tile((void*)((uintptr_t)e.ptr[a] + (uintptr_t)(tile_base * DT::kElemBytes)),
                     (uint32_t)((off - tile_base) * DT::kElemBytes), DT::pack(f[a]));
      else if (UNALIGNED)
        store16_unaligned<DT::kElemBytes>(e.ptr[a], off * DT::kElemBytes, DT::pack(f[a]));
      else
        store16(e.ptr[a], off * DT::kElemBytes, DT::pack(f[a]));
    }
}

template <class Op>
__device__ __forceinline__ void load_vec(const TensorEntry& e, int64_t off, u32x4* raw) {
  using DT = typename Op::DT;
#pragma unroll
  for (int a = 0; a < Op::kArrays; ++a)
    if (Op::kLoad & bit(a)) raw[a] = load16(e.ptr[a], off * DT::kElemBytes);
}

// The same from addresses that are only aligned to one element.
template <class Op>
__device__ __forceinline__ void load_vec_unaligned(const TensorEntry& e, int64_t off, u32x4* raw) {
  using DT = typename Op::DT;
#pragma unroll
  for (int a = 0; a < Op::kArrays; ++a)
    if (Op::kLoad & bit(a)) raw[a] = load16_unaligned<DT::kElemBytes>(e.ptr[a], off * DT::kElemBytes);
}

// The same for a lane of a full tile that starts at element `tile_base`, with cached loads.
template <class Op>
__device__ __forceinline__ void load_vec_cached(const TensorEntry& e, int64_t off, int64_t tile_base, u32x4* raw) {
  using DT = typename Op::DT;
#pragma unroll
  for (int a = 0; a < Op::kArrays; ++a)
    if (Op::kLoad & bit(a))
      raw[a] = load16_tile_cached((const void*)((uintptr_t)e.ptr[a] + (uintptr_t)(tile_base * DT::kElemBytes)),
                                  (uint32_t)((off - tile_base) * DT::kElemBytes));
}

template <class Op>
__device__ __forceinline__ void one_element(const TensorEntry& e, int64_t i, const typename Op::Scalars& s, float& acc) {
  using DT = typename Op::DT;
  constexpr int A = Op::kArrays;
  f32x2 x[A];
#pragma unroll
  for (int a = 0; a < A; ++a) x[a] = splat((Op::kLoad & bit(a)) ? DT::load1(e.ptr[a], i) : 0.0f);
  f32x2 q = splat(0.0f);
  Op::elem(x, s, q);
  if (Op::kReduce) acc += q.x;
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (Op::kStore & bit(a)) DT::store1(e.ptr[a], i, x[a].x);
}

// The work of one workgroup: the tile `sub` of chunk `chunk_id`, which belongs to tensor `tensor`
// (entry `e`).  `s` is the workgroup's own copy of the launch scalars.
template <class Op>
__device__ __forceinline__ void tile_step(const TensorEntry& e, int tensor, int64_t chunk_id, int sub,
                                          typename Op::Scalars s, double* __restrict__ partials) {
  using DT = typename Op::DT;
  constexpr int V = DT::kVec;
  constexpr int A = Op::kArrays;
  constexpr int64_t kChunk = chunk_elems<DT>();
  constexpr int64_t kTile = (int64_t)kThreads * kUnroll * V;  // elements one workgroup covers

  const int64_t base = optimi_tables::tile_base(chunk_id, sub, e.first_chunk, kChunk, kTile);
  const int64_t remain = e.numel - base;  // <= 0 for tiles past the end of the tensor's last chunk
  const bool vec_ok = (e.flags & optimi_tables::kEntryVec) != 0;
  Op::prepare(s, tensor);

  float acc = 0.0f;
  if (vec_ok && remain >= kTile) {
    // full tile: every load is issued before the first use.  The two cache policies are two
    // copies of the whole tile body, so that each keeps its own schedule of waits.
    if (e.flags & optimi_tables::kEntryCached) {
      u32x4 raw[kUnroll][A];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) load_vec_cached<Op>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, base, raw[u]);
      __builtin_amdgcn_sched_barrier(0);  // as below
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        compute_store<Op, true>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, raw[u], s, acc, base);
    } else {
      u32x4 raw[kUnroll][A];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) load_vec<Op>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, raw[u]);
      // nothing moves across this line: the scheduler has been seen to sink the last load below the
      // first use of the first one (a wait for one load before the next is issued, i.e. two memory
      // round trips per tile: 5 % on the 7B AdamW list)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        compute_store<Op, true>(e, base + ((int64_t)u * kThreads + threadIdx.x) * V, raw[u], s, acc, base);
    }
  } else if (vec_ok) {
    // end of a tensor: whole vectors while they fit, then the few leftover elements
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
    // some buffer is not 16-byte aligned (a view into a flat buffer, a gradient inside a
    // communication bucket): the same vectors through element-aligned accesses, then the few
    // leftover elements (one element at a time this path ran at 2.8 TB/s in bf16)
    const int64_t end = e.numel;
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t off = base + ((int64_t)u * kThreads + threadIdx.x) * V;
      if (off + V <= end) {
        u32x4 raw[A];
        load_vec_unaligned<Op>(e, off, raw);
        compute_store<Op, false, true>(e, off, raw, s, acc);
      } else {
        for (int64_t i = off; i < end; ++i) one_element<Op>(e, i, s, acc);
      }
    }
  }

  if (Op::kReduce) {
    __shared__ double lds[kThreads / 64];
    double total = block_sum<kThreads>((double)acc, lds);
    if (threadIdx.x == 0) partials[chunk_id * kSub + sub] = total;
  }
}

// MULTI: the tensor table and the chunk map are in device memory.  Otherwise the table travels
// as the kernel argument `few` (one tensor for the per-tensor entry points, up to kFew for
// short lists) and the workgroup searches it.
template <class Op, bool MULTI>
__global__ void __launch_bounds__(kThreads)
step_kernel(const TensorEntry* __restrict__ table, const int32_t* __restrict__ chunk_map, const FewTable few,
            typename Op::Scalars s, double* __restrict__ partials, int64_t first_workgroup) {
  // a list too long for one grid is stepped by several launches; this one starts at `first_workgroup`
  const int64_t workgroup = first_workgroup + blockIdx.x;
  const int64_t chunk_id = workgroup / kSub;
  const int sub = (int)(workgroup % kSub);
  // a table of one (the per-tensor entry points) needs no search
  const int tensor = MULTI ? chunk_map[chunk_id] : (few.n == 1 ? 0 : optimi_tables::few_lookup(few, chunk_id));
  const TensorEntry& e = MULTI ? table[tensor] : few.e[tensor];
  tile_step<Op>(e, tensor, chunk_id, sub, s, partials);
}

// A list that holds fp32 tensors beside tensors of one 16-bit dtype (a model kept in bf16 whose
// embeddings or norms stay fp32): every workgroup looks its tensor up as above and runs that
// dtype's step on its tile, with that dtype's scalars.  Chunks are kChunkBytes per array for
// both, so the grid does not care which is which.
template <class OpLow, class OpF32, bool MULTI>
__global__ void __launch_bounds__(kThreads)
mixed_kernel(const TensorEntry* __restrict__ table, const int32_t* __restrict__ chunk_map, const FewTable few,
             typename OpLow::Scalars s_low, typename OpF32::Scalars s_f32, double* __restrict__ partials,
             int64_t first_workgroup) {
  const int64_t workgroup = first_workgroup + blockIdx.x;
  const int64_t chunk_id = workgroup / kSub;
  const int sub = (int)(workgroup % kSub);
  const int tensor = MULTI ? chunk_map[chunk_id] : optimi_tables::few_lookup(few, chunk_id);
  const TensorEntry& e = MULTI ? table[tensor] : few.e[tensor];
  if (e.flags & optimi_tables::kEntryF32) tile_step<OpF32>(e, tensor, chunk_id, sub, s_f32, partials);
  else tile_step<OpLow>(e, tensor, chunk_id, sub, s_low, partials);
}

// StableAdamW: one workgroup per tensor turns that tensor's chunk partials into its clipped
// learning rate and decay factor (optimi/stableadamw.py:447-458), in double like the Python
// scalars of the reference.  The mean and its square root are rounded to the tensor dtype,
// as torch's mean()/sqrt() on a tensor of that dtype are.  `DT` is the dtype of the list's
// tensors that are not marked fp32 in their entry.
struct FinalizeArgs {
  double lr, weight_decay, max_lr;
  uint32_t decouple_lr;
};

template <class DT, bool MULTI>
__global__ void __launch_bounds__(kReduceThreads)
stable_finalize_kernel(const TensorEntry* __restrict__ table, const FewTable few, const double* __restrict__ partials,
                       TensorScalars* __restrict__ out, FinalizeArgs a) {
  const TensorEntry& e = MULTI ? table[blockIdx.x] : few.e[blockIdx.x];
  const bool f32 = (e.flags & optimi_tables::kEntryF32) != 0;
  const int64_t chunk = f32 ? chunk_elems<F32>() : chunk_elems<DT>();
  const int64_t first = e.first_chunk * kSub;  // one partial per workgroup of pass 1
  const int64_t count = (e.numel + chunk - 1) / chunk * kSub;
  // sixteen independent accumulators keep that many loads per lane in flight (the largest tensors
  // of a 7B-parameter list bring a quarter of a million partials to their one workgroup; 89 -> 79 us
  // for that list against four accumulators); the order is fixed, so the sum is the same on every run
  constexpr int kAcc = 16;
  double acc[kAcc];
#pragma unroll
  for (int j = 0; j < kAcc; ++j) acc[j] = 0.0;
  int64_t c = threadIdx.x;
  for (; c + (kAcc - 1) * kReduceThreads < count; c += kAcc * kReduceThreads) {
#pragma unroll
    for (int j = 0; j < kAcc; ++j) acc[j] += partials[first + c + j * kReduceThreads];
  }
  for (; c < count; c += kReduceThreads) acc[0] += partials[first + c];
#pragma unroll
  for (int span = kAcc / 2; span > 0; span >>= 1) {
#pragma unroll
    for (int j = 0; j < span; ++j) acc[j] += acc[j + span];
  }
  double v = acc[0];
  __shared__ double lds[kReduceThreads / 64];
  double total = block_sum<kReduceThreads>(v, lds);
  if (threadIdx.x == 0) {
    double lr = a.lr;
    if (e.numel > 0) {
      float ms = (float)total / (float)e.numel;
      if (!f32) ms = DT::R2(splat(ms)).x;
      float rms = sqrtf(ms);
      if (!f32) rms = DT::R2(splat(rms)).x;
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

__global__ void __launch_bounds__(256) copy_probe_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, int64_t n_vec) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n_vec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
constexpr int popcount(uint32_t x) { return x ? (int)(x & 1u) + popcount(x >> 1) : 0; }
inline float S(double x) { return (float)x; }
inline float round_bf16_host(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) u = 0x7fc00000u;
  else { u += 0x7fffu + ((u >> 16) & 1u); u &= 0xffff0000u; }
  std::memcpy(&f, &u, 4);
  return f;
}
inline float round_f16_host(float f) { return (float)(_Float16)f; }  // round-to-nearest-even, subnormals kept
inline float Sd(double x, int dtype) {
  return dtype == OPTIMI_BF16 ? round_bf16_host((float)x) : dtype == OPTIMI_F16 ? round_f16_host((float)x) : (float)x;
}
inline Lerp make_lerp(double weight) {
  float w = (float)weight;
  Lerp l;
  l.small = std::fabs(w) < 0.5f ? 1u : 0u;
  l.coef = l.small ? w : w - 1.0f;
  return l;
}
inline int64_t chunk_elems_rt(int dtype) { return optimi_tables::chunk_elems(dtype); }
using optimi_tables::elem_bytes;

#define HIP_TRY(expr)                          \
  do {                                         \
    hipError_t err__ = (expr);                 \
    if (err__ != hipSuccess) return (int)err__; \
  } while (0)

struct DeviceBuf {
  void* ptr = nullptr;
  size_t cap = 0;
  int reserve(size_t bytes) {
    bytes = (bytes + 15) & ~(size_t)15;  // whole 16-byte vectors: what the upload kernel writes
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

std::atomic<int64_t> table_uploads{0};  // tensor tables and chunk maps copied to the device so far

struct StagingSlot {
  void* host = nullptr;
  size_t cap = 0;
  hipEvent_t done = nullptr;
  bool in_flight = false;
};

}  // namespace

// A tensor table on the device and the host copy of what it holds.
struct TableSlot {
  DeviceBuf dev;
  std::vector<TensorEntry> host;
  bool holds(const std::vector<TensorEntry>& fresh) const {
    return host.size() == fresh.size() && std::memcmp(host.data(), fresh.data(), sizeof(TensorEntry) * fresh.size()) == 0;
  }
};

struct optimi_group {
  int device = 0;
  // Two tables: gradients that alternate between two sets of buffers (a new gradient assigned before
  // the old one is freed, double-buffered buckets) then find their table on the device every time.
  TableSlot tables[2];
  int table_cur = 0;                     // the slot the last launch read
  DeviceBuf chunk_map, partials, tensor_scalars;
  std::vector<int32_t> host_map;         // scratch for building the chunk map
  std::vector<int64_t> map_first;        // what the device chunk map was built for: every tensor's first chunk, then the chunk count
  StagingSlot ring[4];
  int ring_pos = 0;
  hipEvent_t last_launch = nullptr;
  hipStream_t last_stream = nullptr;
  bool launched = false;
};

namespace {

// Copies `bytes` host bytes to device memory (a DeviceBuf, whose capacity is in whole 16-byte
// vectors) through a pinned ring slot, on `stream`.
int staged_upload(optimi_group* g, void* dst, const void* src, size_t bytes, hipStream_t stream) {
  StagingSlot& slot = g->ring[g->ring_pos];
  g->ring_pos = (g->ring_pos + 1) % 4;
  if (slot.in_flight) {
    HIP_TRY(hipEventSynchronize(slot.done));
    slot.in_flight = false;
  }
  const size_t need = (bytes + 15) & ~(size_t)15;  // whole 16-byte vectors: what the upload kernel reads
  if (slot.cap < need) {
    if (slot.host) (void)hipHostFree(slot.host);
    slot.host = nullptr;
    slot.cap = 0;
    size_t want = need + need / 2 + 4096;
    HIP_TRY(hipHostMalloc(&slot.host, want, hipHostMallocDefault));
    slot.cap = want;
  }
  if (!slot.done) HIP_TRY(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
  std::memcpy(slot.host, src, bytes);
  // A small kernel on the launch stream reads the pinned slot and writes the device table.  The
  // runtime's own host-to-device copy takes 5 us for 3 KB and 27 us for 24 KB on the stream here
  // (a 300-tensor list whose gradients move every step: 252 us per step against 226 us with the
  // table unchanged); the kernel takes a few microseconds whatever the size.  Both buffers are
  // sized in whole 16-byte vectors, so the copy may round up to them.
  const int64_t n_vec = (int64_t)((bytes + 15) / 16);
  copy_probe_kernel<<<dim3((unsigned)((n_vec + 255) / 256)), dim3(256), 0, stream>>>((u32x4*)dst, (const u32x4*)slot.host, n_vec);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipEventRecord(slot.done, stream));
  slot.in_flight = true;
  ++table_uploads;
  return 0;
}


// Whether work put on `stream` is being recorded into a HIP graph instead of run.  A capture
// must not see the group's own bookkeeping: an event recorded inside a capture cannot be waited
// for or synchronised on by eager work afterwards, and a copy recorded from the pinned staging
// ring would replay from a slot that later uploads overwrite.
int stream_capturing(hipStream_t stream, bool* capturing) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  HIP_TRY(hipStreamIsCapturing(stream, &status));
  *capturing = status != hipStreamCaptureStatusNone;
  return 0;
}

// A list whose arrays add up to at most this many bytes stays in the 256 MB last-level cache
// from one optimizer step to the next when nothing else runs in between (measured: cached loads
// beat `nt` loads up to 270 MB of arrays and lose from 335 MB on).  A caller that knows this is so
// says OPTIMI_RESIDENT, and such a launch then uses cached loads: 1 % faster than streaming ones
// on a 269 MB fp32 list stepped back to back.  It is a hint to opt in with, not the default: a
// training loop runs a forward and a backward pass between two optimizer steps, after which the
// list has to come from memory, and there streaming loads are the faster ones (the same list with
// 2 GiB moved through the caches before every step: 71.5 us streaming, 77.2 us cached).
// Per-tensor entry points never take this path: they step one tensor of a larger model.
constexpr int64_t kResidentBytes = (int64_t)288 << 20;

// What one list launch works on, as the entry points hand it to the launchers.
struct ListPlan {
  bool few = false;           // the table travels as a kernel argument; the group's tables are untouched
  FewTable table;             // valid when `few`
  int n_tensors = 0;
  int64_t n_chunks = 0;
  bool resident = false;      // the list's arrays fit the last-level cache and were touched recently
  bool mixed = false;         // fp32 tensors beside 16-bit ones
  bool misaligned = false;    // most of the list's elements are in tensors with a buffer off the 16-byte grid
};

constexpr int64_t kMaxChunks = (int64_t)0x7fffffff / kSub;  // chunk and workgroup numbers fit 31 bits (2 TiB per array)

// The dtypes a mixed list may hold: fp32 and at most one 16-bit dtype.  `*low` becomes the
// dtype of the tensors that are not fp32 (fp32 if there are none), `*mixed` whether both kinds
// are present.
int list_dtypes(int n_tensors, const int* dtypes, int* low, bool* mixed) {
  if (n_tensors > 0 && !dtypes) return OPTIMI_ERR_NULL;
  int low_dtype = OPTIMI_F32;
  bool any_f32 = false;
  for (int t = 0; t < n_tensors; ++t) {
    if (!valid_dtype(dtypes[t])) return OPTIMI_ERR_DTYPE;
    if (dtypes[t] == OPTIMI_F32) any_f32 = true;
    else if (low_dtype == OPTIMI_F32) low_dtype = dtypes[t];
    else if (low_dtype != dtypes[t]) return OPTIMI_ERR_DTYPE;  // bf16 and fp16 in one list
  }
  *low = low_dtype;
  *mixed = any_f32 && low_dtype != OPTIMI_F32;
  return 0;
}

// Validates the list and gets its tables to where the kernel reads them: into `plan` itself for
// a list of at most kFew tensors (nothing is uploaded), else into the group's device tables,
// (re)building the chunk map and tensor table and uploading what changed.
// `lists[a]` may be nullptr for an array the launch does not touch (`need` has its bit clear).
// `dtypes`: nullptr when every tensor has `dtype`; else every tensor's own dtype, `dtype` being
// the 16-bit one among them, and fp32 tensors have no array in `low_precision_only`.
int plan_list(optimi_group* g, int n_tensors, const void* const* const* lists, int n_arrays, uint32_t need,
              uint32_t low_precision_only, const int64_t* numel, const int* dtypes, int dtype, uint32_t flags,
              hipStream_t stream, ListPlan* plan) {
  if (!g) return OPTIMI_ERR_NULL;
  if (n_tensors < 0) return OPTIMI_ERR_SIZE;
  if (!valid_dtype(dtype)) return OPTIMI_ERR_DTYPE;
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev != g->device) return OPTIMI_ERR_DEVICE;

  plan->n_tensors = n_tensors;
  plan->mixed = dtypes != nullptr;
  plan->few = n_tensors <= kFew;
  std::memset(&plan->table, 0, sizeof(plan->table));
  std::vector<TensorEntry> fresh;
  TensorEntry* entries = plan->table.e;
  if (!plan->few) {
    try {
      fresh.resize((size_t)n_tensors);
    } catch (const std::bad_alloc&) {
      return OPTIMI_ERR_NOMEM;
    }
    entries = fresh.data();
  }
  int64_t n_chunks = 0;
  int rc = optimi_tables::build_entries(n_tensors, lists, n_arrays, need, numel, dtypes, dtype, low_precision_only,
                                        kMaxChunks, entries, &n_chunks);
  if (rc) return rc;
  plan->n_chunks = n_chunks;
  int64_t bytes = 0, off_grid = 0;
  for (int t = 0; t < n_tensors; ++t) {
    const bool f32 = (entries[t].flags & optimi_tables::kEntryF32) != 0;
    const int64_t b = numel[t] * (f32 ? 4 : 2) * popcount(f32 ? need & ~low_precision_only : need);
    bytes += b;
    if (!(entries[t].flags & optimi_tables::kEntryVec)) off_grid += b;
  }
  plan->misaligned = 2 * off_grid > bytes;
  plan->resident = (flags & OPTIMI_RESIDENT) && bytes <= kResidentBytes;
  if (plan->resident)
    for (int t = 0; t < n_tensors; ++t) entries[t].flags |= optimi_tables::kEntryCached;
  if (plan->few) {
    optimi_tables::finish_few(&plan->table, n_tensors);
    return 0;
  }

  // a group moved to another stream must not overwrite tables a previous launch still reads
  // (a capturing stream uploads nothing, see below, and takes no part in the group's events)
  bool capturing = false;
  rc = stream_capturing(stream, &capturing);
  if (rc) return rc;
  if (!capturing && g->launched && g->last_stream != stream) HIP_TRY(hipStreamWaitEvent(stream, g->last_launch, 0));

  // the chunk map is a function of where every tensor's chunks start and of how many there are
  bool same_map = g->map_first.size() == (size_t)n_tensors + 1 && g->map_first[(size_t)n_tensors] == n_chunks;
  for (int t = 0; same_map && t < n_tensors; ++t) same_map = g->map_first[(size_t)t] == fresh[(size_t)t].first_chunk;
  int hit = g->tables[g->table_cur].holds(fresh) ? g->table_cur : g->tables[1 - g->table_cur].holds(fresh) ? 1 - g->table_cur : -1;
  if (capturing && ((!same_map && n_chunks > 0) || hit < 0))
    return OPTIMI_ERR_CAPTURE;  // the tables must be on the device before the capture begins
  if (!same_map && n_chunks > 0) {
    g->map_first.clear();  // the cached map is void until the new one is on its way
    try {
      g->host_map.resize((size_t)n_chunks);
    } catch (const std::bad_alloc&) {
      return OPTIMI_ERR_NOMEM;
    }
    optimi_tables::build_chunk_map(fresh.data(), n_tensors, g->host_map.data());
    rc = g->chunk_map.reserve(sizeof(int32_t) * (size_t)n_chunks);
    if (rc) return rc;
    rc = staged_upload(g, g->chunk_map.ptr, g->host_map.data(), sizeof(int32_t) * (size_t)n_chunks, stream);
    if (rc) return rc;
    try {
      g->map_first.resize((size_t)n_tensors + 1);
    } catch (const std::bad_alloc&) {
      return OPTIMI_ERR_NOMEM;
    }
    for (int t = 0; t < n_tensors; ++t) g->map_first[(size_t)t] = fresh[(size_t)t].first_chunk;
    g->map_first[(size_t)n_tensors] = n_chunks;
  }

  if (hit < 0) {  // into the slot that the last launch did not read
    hit = 1 - g->table_cur;
    TableSlot& slot = g->tables[hit];
    slot.host.clear();  // void until the new table is on its way
    rc = slot.dev.reserve(sizeof(TensorEntry) * fresh.size());
    if (rc) return rc;
    rc = staged_upload(g, slot.dev.ptr, fresh.data(), sizeof(TensorEntry) * fresh.size(), stream);
    if (rc) return rc;
    slot.host.swap(fresh);
  }
  g->table_cur = hit;
  return 0;
}

int note_launch(optimi_group* g, hipStream_t stream) {
  HIP_TRY(hipGetLastError());
  bool capturing = false;
  int rc = stream_capturing(stream, &capturing);
  if (rc) return rc;
  if (capturing) return 0;  // the graph orders its own nodes; the group's event stays an eager one
  if (!g->last_launch) HIP_TRY(hipEventCreateWithFlags(&g->last_launch, hipEventDisableTiming));
  HIP_TRY(hipEventRecord(g->last_launch, stream));
  g->last_stream = stream;
  g->launched = true;
  return 0;
}

// After a list launch: a launch that used the group's device tables is recorded so that the
// next use of the group on another stream waits for it; a short list touched nothing of the group.
int finish_list(optimi_group* g, const ListPlan& plan, hipStream_t stream) {
  if (!plan.few) return note_launch(g, stream);
  HIP_TRY(hipGetLastError());
  return 0;
}

// Occupancy throttle.  HBM serves this read-modify-write mix best when a CU keeps only a
// certain number of wavefronts resident - fewer the more 16-byte-per-lane streams (loads plus
// stores) each wavefront carries; beyond it the achieved bandwidth drops by several per cent,
// below it the CU cannot cover the latency.  The cap is imposed with a dynamic-LDS request that
// no kernel touches.  A CU hands its 160 KiB of LDS out in 128 granules of 1280 bytes (measured:
// swept over the request size, the achieved bandwidth moves in steps exactly where the granule
// count changes), so a workgroup that asks for g granules leaves room for floor(128 / g)
// workgroups; reachable occupancies are therefore 32, 25, 21, 18, 16, 14, 12, 11, 10, 9, 8, ...
// The table holds the measured optimum in granules on MI355X with the write-through tile stores
// (7B-parameter lists):
//    3 streams  SGD without momentum, accumulate-only Lion and SGD      5 (6.81 TB/s; 6.56 at 4)
//    4          StableAdamW pass 2 without Kahan                        6 (5 to 7 within 0.5 %)
//    5, 6       StableAdamW pass 1 and 2, accumulate-only Adam, SGD     8 (16-bit pass 1, which also reduces and stores a
//                                                                         partial sum per workgroup: 7 - the 7B list
//                                                                         in 22.08 ms against 22.44 ms, the 1B list
//                                                                         in 4.00 ms against 4.07 ms)
//    7          Lion / SGD with Kahan, fp32 Adam                        11
//    9          Adam with Kahan                                         12
//    11         Ranger's Lookahead step, Adan without Kahan             12 (22.75 ms; 23.34 ms at 14)
//    13         Adan with Kahan                                         16
// and entries in between are interpolated.  fp32 Adan (also 11 streams) does best at 17 granules,
// 7 workgroups (a Llama-1B-shaped list: 8.12 ms at 16, 7.98 ms at 17 and 18).  16-bit list
// launches of fewer than kLongLaunch workgroups (the Llama-1B-shaped list) do best one granule
// lower, i.e. with one more workgroup resident.  Lists that live in the last-level cache follow
// the same table (16.8 M parameters: fp32 AdamW 68.9 us at 6 granules, 67.5 us at 10 and 11;
// bf16 AdamW 48.7 us at 6, 47.0 us at 12; fp32 Adan 131 us at 6, 120 us at 14).
// A launch whose tensors mostly have a buffer off the 16-byte grid (its accesses straddle
// segments and lines) does best two granules higher: on the 7B list with every parameter and
// gradient misaligned, AdamW 21.86 -> 20.84 ms, Lion 16.43 -> 16.00 ms, fp32 AdamW on the 1B list
// 5.79 -> 5.60 ms, StableAdamW and Adan 1 %.
// OPTIMI_HIP_WAVES overrides the number of wavefronts per CU for every kernel (nearest
// reachable count at or above it; 0 = no throttle); read once.
constexpr int kLdsGranule = 1280, kLdsGranules = 128;
constexpr int kMaxStreams = 2 * kMaxArrays;
constexpr int kBestGranules[kMaxStreams + 1] = {5, 5, 5, 5, 6, 8, 8, 11, 11, 12, 12, 12, 14, 16, 16};
constexpr int64_t kLongLaunch = (int64_t)1 << 22;  // workgroups

int forced_waves() {
#ifdef OPTIMI_TUNING
  if (const char* env = std::getenv("OPTIMI_HIP_WAVES")) return (int)std::strtol(env, nullptr, 10);
  return -1;
#endif
  static const int value = [] {
    const char* env = std::getenv("OPTIMI_HIP_WAVES");
    return env ? (int)std::strtol(env, nullptr, 10) : -1;
  }();
  return value;
}

struct LaunchShape {
  unsigned lds;  // dynamic LDS request in bytes (the occupancy throttle)
};

// `few`: the table travels as a kernel argument (per-tensor launches and short lists).  Such a
// workgroup reaches its loads sooner than one that first reads the chunk map and the tensor
// table from memory, so fewer of the resident wavefronts are idle at any time and the optimum
// sits a little lower: the table as it is for 7 streams and more (no extra workgroup for
// launches under kLongLaunch), 9 granules instead of 8 for 5 and 6 streams (measured on
// per-tensor launches over tensors that are cold when revisited, 4 M to 45 M elements).
// `request` > 0: the caller names the granules itself (the traffic probe's sweep).
template <class Op>
LaunchShape launch_shape(int64_t workgroups, bool few, bool misaligned, int request = 0) {
  constexpr int streams = (popcount(Op::kLoad) + popcount(Op::kStore)) * kUnroll;
  // the traffic probe stands in for a 16-bit step with as many streams, whatever its own vector type
  constexpr bool f32 = std::is_same<typename Op::DT, F32>::value && !is_probe<Op>::value;
  LaunchShape shape;
  if (request > 0) {
    shape.lds = (unsigned)((request > 51 ? 51 : request) * kLdsGranule - 128);
    return shape;
  }
  int granules = kBestGranules[streams < kMaxStreams ? streams : kMaxStreams];
  if (f32 && streams == 11) granules = 17;
  if (!few && !f32 && streams >= 7 && workgroups < kLongLaunch) granules -= 1;
  if (few && (streams == 5 || streams == 6)) granules = 9;
  if (!few && !f32 && Op::kReduce) granules = 7;
  if (misaligned) granules += 2;
#ifdef OPTIMI_TUNING
  {  // raw request for the kernels with this many streams only, tuning builds only
    char name[32];
    std::snprintf(name, sizeof(name), "OPTIMI_HIP_LDS_S%d", streams);
    if (const char* env = std::getenv(name)) {
      shape.lds = (unsigned)std::strtol(env, nullptr, 10);
      return shape;
    }
  }
  if (const char* env = std::getenv("OPTIMI_HIP_LDS")) {  // raw request, tuning builds only
    shape.lds = (unsigned)std::strtol(env, nullptr, 10);
    return shape;
  }
#endif
  const int forced = forced_waves();
  if (forced == 0) {
    shape.lds = 0;
    return shape;
  }
  if (forced > 0) {
    const int wgs = forced / (kThreads / 64) > 0 ? forced / (kThreads / 64) : 1;
    granules = kLdsGranules / wgs;
  }
  if (granules < 1) granules = 1;
  if (granules > 51) granules = 51;  // a workgroup may ask for 64 KiB at most
  // a little under the granule boundary: the kernel's own static LDS (a few bytes in the
  // reducing kernels) is added to the request and must not tip it into the next granule
  shape.lds = (unsigned)(granules * kLdsGranule - 128);
  return shape;
}

const FewTable kNoTable = {};

std::atomic<int64_t> kernel_launches{0};  // every kernel this library has launched in this process
std::atomic<int64_t> resident_launches{0};  // list launches among them that read with cached loads

// A grid holds fewer than 2^32 threads: a launch of 2^26 or more 64-lane workgroups is refused by
// the runtime when the count is an exact multiple of 2^26 and otherwise runs only the count
// modulo 2^26 without any error (measured: 2^26 + 16 workgroups ran 16).  Lists beyond that -
// more than 64 GiB per array - are stepped by several launches of whole chunks, each told where
// it starts.  The limit is a variable so that tests can exercise the split on small lists.
constexpr int64_t kGridWorkgroups = ((int64_t)1 << 32) / kThreads - kSub;
std::atomic<int64_t> launch_workgroup_limit{kGridWorkgroups};

// `s_f32`: the same scalars formed for fp32 tensors; read only when the plan is a mixed list.
template <class Op>
void launch_list(optimi_group* g, const ListPlan& plan, const typename Op::Scalars& s, hipStream_t stream,
                 double* partials = nullptr, const typename Op::Scalars* s_f32 = nullptr, int granules = 0) {
  const int64_t workgroups = plan.n_chunks * kSub;
  const LaunchShape shape = launch_shape<Op>(workgroups, plan.few, plan.misaligned, granules);
  if (plan.resident) ++resident_launches;
  const int64_t limit = launch_workgroup_limit.load();
  for (int64_t first = 0; first < workgroups; first += limit) {
    const dim3 grid((unsigned)(workgroups - first < limit ? workgroups - first : limit));
    ++kernel_launches;
    if constexpr (!std::is_same<typename Op::DT, F32>::value) {
      if (plan.mixed) {
        if (plan.few)
          mixed_kernel<Op, typename Op::F32Partner, false><<<grid, dim3(kThreads), shape.lds, stream>>>(
              nullptr, nullptr, plan.table, s, *s_f32, partials, first);
        else
          mixed_kernel<Op, typename Op::F32Partner, true><<<grid, dim3(kThreads), shape.lds, stream>>>(
              (const TensorEntry*)g->tables[g->table_cur].dev.ptr, (const int32_t*)g->chunk_map.ptr, kNoTable, s, *s_f32, partials, first);
        continue;
      }
    }
    if (plan.few)
      step_kernel<Op, false><<<grid, dim3(kThreads), shape.lds, stream>>>(nullptr, nullptr, plan.table, s, partials, first);
    else
      step_kernel<Op, true><<<grid, dim3(kThreads), shape.lds, stream>>>(
          (const TensorEntry*)g->tables[g->table_cur].dev.ptr, (const int32_t*)g->chunk_map.ptr, kNoTable, s, partials, first);
  }
}

inline FewTable table_of_one(const TensorEntry& e) {
  FewTable one = {};
  one.e[0] = e;
  one.e[0].first_chunk = 0;
  optimi_tables::finish_few(&one, 1);
  return one;
}

template <class Op>
void launch_single(const TensorEntry& e, const typename Op::Scalars& s, double* partials, hipStream_t stream) {
  const int64_t chunk = chunk_elems<typename Op::DT>();
  const int64_t workgroups = (e.numel + chunk - 1) / chunk * kSub;
  const LaunchShape shape = launch_shape<Op>(workgroups, true, !(e.flags & optimi_tables::kEntryVec));
  const FewTable one = table_of_one(e);
  const int64_t limit = launch_workgroup_limit.load();
  for (int64_t first = 0; first < workgroups; first += limit) {
    ++kernel_launches;
    step_kernel<Op, false><<<dim3((unsigned)(workgroups - first < limit ? workgroups - first : limit)), dim3(kThreads), shape.lds,
                             stream>>>(nullptr, nullptr, one, s, partials, first);
  }
}

// Calls fn(Op{}) for the Op selected by dtype x kahan x update x weight-decay mode.  NWD is
// the number of decay modes the Op family has (modes 0..NWD-1); an accumulate-only step never
// decays, and only bf16 has a Kahan branch.
template <template <class, bool, bool, int> class OpT, int NWD, class Fn>
void dispatch(int dtype, bool kahan, bool update, int wd, Fn&& fn) {
  auto pick_wd = [&](auto dt, auto kh) {
    using DT = decltype(dt);
    constexpr bool K = decltype(kh)::value;
    if (wd == 1) fn(OpT<DT, K, true, 1>{});
    else if (wd == 2 && NWD > 2) fn(OpT<DT, K, true, (NWD > 2 ? 2 : 0)>{});
    else fn(OpT<DT, K, true, 0>{});
  };
  if (dtype == OPTIMI_BF16) {
    if (!update) fn(OpT<BF16, false, false, 0>{});
    else if (kahan) pick_wd(BF16{}, std::true_type{});
    else pick_wd(BF16{}, std::false_type{});
  } else if (dtype == OPTIMI_F16) {
    if (!update) fn(OpT<F16, false, false, 0>{});
    else if (kahan) pick_wd(F16{}, std::true_type{});
    else pick_wd(F16{}, std::false_type{});
  } else {
    if (!update) fn(OpT<F32, false, false, 0>{});
    else pick_wd(F32{}, std::false_type{});
  }
}

// Same selection, handing the choices over as tag types so the caller can add further
// compile-time parameters of its own: fn(DT{}, bool_c<kahan>, bool_c<update>, int_c<wd>).
template <bool B> using bool_c = std::integral_constant<bool, B>;
template <int I> using int_c = std::integral_constant<int, I>;

template <class Fn>
void dispatch_tags(int dtype, bool kahan, bool update, int wd, Fn&& fn) {
  auto pick_wd = [&](auto dt, auto kh) {
    if (wd == 1) fn(dt, kh, bool_c<true>{}, int_c<1>{});
    else if (wd == 2) fn(dt, kh, bool_c<true>{}, int_c<2>{});
    else fn(dt, kh, bool_c<true>{}, int_c<0>{});
  };
  if (dtype == OPTIMI_BF16) {
    if (!update) fn(BF16{}, bool_c<false>{}, bool_c<false>{}, int_c<0>{});
    else if (kahan) pick_wd(BF16{}, bool_c<true>{});
    else pick_wd(BF16{}, bool_c<false>{});
  } else if (dtype == OPTIMI_F16) {
    if (!update) fn(F16{}, bool_c<false>{}, bool_c<false>{}, int_c<0>{});
    else if (kahan) pick_wd(F16{}, bool_c<true>{});
    else pick_wd(F16{}, bool_c<false>{});
  } else {
    if (!update) fn(F32{}, bool_c<false>{}, bool_c<false>{}, int_c<0>{});
    else pick_wd(F32{}, bool_c<false>{});
  }
}

int single_entry(TensorEntry& e, const void* const* ptrs, int n_arrays, uint32_t need, int64_t numel, int dtype) {
  if (numel < 0) return OPTIMI_ERR_SIZE;
  if (!valid_dtype(dtype)) return OPTIMI_ERR_DTYPE;
  if (numel > chunk_elems_rt(dtype) * ((int64_t)0x7fffffff / kSub)) return OPTIMI_ERR_SIZE;
  std::memset(&e, 0, sizeof(e));
  e.numel = numel;
  e.flags = optimi_tables::kEntryVec | (dtype == OPTIMI_F32 ? optimi_tables::kEntryF32 : 0u);
  const int eb = elem_bytes(dtype);
  for (int a = 0; a < n_arrays; ++a) {
    if (!(need & bit(a))) continue;
    if (!ptrs[a] && numel > 0) return OPTIMI_ERR_NULL;
    uintptr_t u = (uintptr_t)ptrs[a];
    if (u % (uintptr_t)eb) return OPTIMI_ERR_ALIGN;
    if (u % 16) e.flags &= ~optimi_tables::kEntryVec;
    e.ptr[a] = const_cast<void*>(ptrs[a]);
  }
  return 0;
}

// ---- scalar packs ------------------------------------------------------------------
AdamScalars adam_scalars(int dtype, double lr, double beta1_comp, double beta2_hat, double beta2_comp,
                         double weight_decay, double eps) {
  AdamScalars s;
  s.l1 = make_lerp(beta1_comp);
  s.wd = S(weight_decay);
  s.wd_alpha = Sd(weight_decay, dtype);
  s.b2h = S(beta2_hat);
  s.b2c = S(beta2_comp);
  s.eps_d = Sd(eps, dtype);
  s.neg_lr = S(-lr);
  s.neg_lr_d = Sd(-lr, dtype);
  return s;
}
int adam_wd_mode(double weight_decay, uint32_t flags) {
  return (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? ((flags & OPTIMI_DECOUPLE_WD) ? 1 : 2) : 0;
}
uint32_t adam_need(bool kahan, bool update) {
  return update ? (bit(0) | bit(1) | bit(2) | bit(3) | (kahan ? bit(4) : 0)) : (bit(1) | bit(2) | bit(3));
}

LionScalars lion_scalars(int dtype, double lr, double beta1_comp, double beta2_comp, double weight_decay) {
  LionScalars s;
  s.l1 = make_lerp(beta1_comp);
  s.l2 = make_lerp(beta2_comp);
  s.wd = S(weight_decay);
  s.neg_lr_d = Sd(-lr, dtype);
  return s;
}
int lion_wd_mode(double weight_decay, uint32_t flags) { return (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? 1 : 0; }
uint32_t lion_need(bool kahan, bool update) {
  return update ? (bit(0) | bit(1) | bit(2) | (kahan ? bit(3) : 0)) : (bit(1) | bit(2));
}

AdanScalars adan_scalars(int dtype, double lr, double beta1_comp, double beta2, double beta2_comp, double beta3_hat,
                         double beta3_comp, double eps, double weight_decay) {
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
  return s;
}
int adan_wd_mode(double weight_decay, uint32_t flags) {
  return (weight_decay != 0 && (flags & OPTIMI_UPDATE)) ? ((flags & OPTIMI_ADAM_WD) ? 1 : 2) : 0;
}
uint32_t adan_need(bool kahan, bool update) {
  return bit(1) | bit(2) | bit(3) | bit(4) | bit(5) | (update ? (bit(0) | (kahan ? bit(6) : 0)) : 0);
}

SgdScalars sgd_scalars(int dtype, double lr, double momentum, double weight_decay) {
  SgdScalars s;
  s.damp = make_lerp(1 - momentum);
  s.wd = S(weight_decay);
  s.wd_alpha = Sd(weight_decay, dtype);
  s.momentum = S(momentum);
  s.neg_lr_d = Sd(-lr, dtype);
  return s;
}
inline int sgd_mom_mode(double momentum, uint32_t flags) { return momentum != 0 ? ((flags & OPTIMI_DAMPENING) ? 2 : 1) : 0; }
uint32_t sgd_need(bool kahan, bool update, int mom) {
  return bit(1) | (mom ? bit(2) : 0) | (update ? (bit(0) | (kahan ? bit(3) : 0)) : 0);
}
uint32_t ranger_need(bool kahan, bool update, bool la) { return adam_need(kahan, update) | ((update && la) ? bit(5) : 0); }

// Launches the SGD variant chosen by dtype x kahan x update x decay mode x momentum mode.
template <class Launch>
void sgd_dispatch(int dtype, bool kahan, bool update, int wd, int mom, Launch&& launch) {
  dispatch_tags(dtype, kahan, update, wd, [&](auto dt, auto kh, auto up, auto w) {
    using DT = decltype(dt);
    constexpr bool K = decltype(kh)::value, U = decltype(up)::value;
    constexpr int W = decltype(w)::value;
    if (mom == 1) launch(SgdOp<DT, K, U, W, 1>{});
    else if (mom == 2) launch(SgdOp<DT, K, U, W, 2>{});
    else launch(SgdOp<DT, K, U, W, 0>{});
  });
}

// Launches the Ranger variant of a step that synchronises with the slow weights: ... x rectified
// or not.  (A Ranger step without the Lookahead sync, and every accumulate-only one, is the RAdam
// step - optimi/ranger.py:402-473 - and runs RAdam's kernels.)
template <class Launch>
void ranger_dispatch(int dtype, bool kahan, int wd, bool rectify, Launch&& launch) {
  dispatch_tags(dtype, kahan, true, wd, [&](auto dt, auto kh, auto up, auto w) {
    using DT = decltype(dt);
    constexpr bool K = decltype(kh)::value;
    constexpr int W = decltype(w)::value;
    (void)up;
    if (rectify) launch(RangerOp<DT, K, W, 0>{});
    else launch(RangerOp<DT, K, W, 1>{});
  });
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
  return dtype != OPTIMI_F32 && (flags & OPTIMI_KAHAN) && (flags & OPTIMI_UPDATE);
}

// The device scratch one StableAdamW step needs beyond the caller's tensors: one double per
// pass-1 workgroup and the per-tensor scalars the finalize kernel hands to pass 2.
struct StableScratch {
  double* partials;
  TensorScalars* tensor_scalars;
};

template <class DT>
int64_t stable_partials(int64_t numel) {  // pass-1 workgroups of one tensor
  const int64_t chunk = chunk_elems<DT>();
  return (numel + chunk - 1) / chunk * kSub;
}

// `scratch` is written before it is read within the call (every pass-1 workgroup stores its
// partial, finalize stores the scalars), so it needs no clearing between calls.
// `plan`: the list to step, or nullptr to step the one tensor `single`.
template <class DT>
int stable_run(const ListPlan* plan, optimi_group* g, const TensorEntry& single, const StableScratch& scratch,
               int dtype, double lr, double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay,
               double eps, double max_lr, uint32_t flags, hipStream_t stream) {
  const bool update = (flags & OPTIMI_UPDATE) != 0;
  const bool kahan = kahan_on(dtype, flags);
  StableP1Scalars s1 = stable_p1_scalars(dtype, beta1_comp, beta2_hat, beta2_comp, eps);
  const StableP1Scalars s1_f32 = stable_p1_scalars(OPTIMI_F32, beta1_comp, beta2_hat, beta2_comp, eps);
  if (!update) {
    if (plan) launch_list<StablePass1Op<DT, false>>(g, *plan, s1, stream, nullptr, &s1_f32);
    else launch_single<StablePass1Op<DT, false>>(single, s1, nullptr, stream);
    return 0;
  }
  FinalizeArgs fa;
  fa.lr = lr;
  fa.weight_decay = weight_decay;
  fa.max_lr = max_lr;
  fa.decouple_lr = (flags & OPTIMI_DECOUPLE_LR) ? 1u : 0u;
  StableP2Scalars s2;
  s2.per_tensor = scratch.tensor_scalars;
  s2.eps_d = Sd(eps, dtype);
  s2.neg_lr = 0.0f;
  s2.wd = 0.0f;
  StableP2Scalars s2_f32 = s2;
  s2_f32.eps_d = Sd(eps, OPTIMI_F32);
  const bool wd = weight_decay != 0;
  ++kernel_launches;  // the finalize kernel below
  if (plan) {
    launch_list<StablePass1Op<DT, true>>(g, *plan, s1, stream, scratch.partials, &s1_f32);
    if (plan->few)
      stable_finalize_kernel<DT, false><<<dim3((unsigned)plan->n_tensors), dim3(kReduceThreads), 0, stream>>>(
          nullptr, plan->table, scratch.partials, scratch.tensor_scalars, fa);
    else
      stable_finalize_kernel<DT, true><<<dim3((unsigned)plan->n_tensors), dim3(kReduceThreads), 0, stream>>>(
          (const TensorEntry*)g->tables[g->table_cur].dev.ptr, kNoTable, scratch.partials, scratch.tensor_scalars, fa);
    if (kahan && wd) launch_list<StablePass2Op<DT, true, 1>>(g, *plan, s2, stream, nullptr, &s2_f32);
    else if (kahan) launch_list<StablePass2Op<DT, true, 0>>(g, *plan, s2, stream, nullptr, &s2_f32);
    else if (wd) launch_list<StablePass2Op<DT, false, 1>>(g, *plan, s2, stream, nullptr, &s2_f32);
    else launch_list<StablePass2Op<DT, false, 0>>(g, *plan, s2, stream, nullptr, &s2_f32);
  } else {
    launch_single<StablePass1Op<DT, true>>(single, s1, scratch.partials, stream);
    stable_finalize_kernel<DT, false><<<dim3(1), dim3(kReduceThreads), 0, stream>>>(
        nullptr, table_of_one(single), scratch.partials, scratch.tensor_scalars, fa);
    if (kahan && wd) launch_single<StablePass2Op<DT, true, 1>>(single, s2, nullptr, stream);
    else if (kahan) launch_single<StablePass2Op<DT, true, 0>>(single, s2, nullptr, stream);
    else if (wd) launch_single<StablePass2Op<DT, false, 1>>(single, s2, nullptr, stream);
    else launch_single<StablePass2Op<DT, false, 0>>(single, s2, nullptr, stream);
  }
  return 0;
}

// The group's own scratch, grown to what this step needs (a whole list, or one tensor).
template <class DT>
int group_scratch(optimi_group* g, const ListPlan* plan, int64_t single_numel, uint32_t flags, StableScratch* out) {
  out->partials = nullptr;
  out->tensor_scalars = nullptr;
  if (!(flags & OPTIMI_UPDATE)) return 0;  // the accumulate-only step reduces nothing
  const int64_t n_partials = plan ? plan->n_chunks * kSub : stable_partials<DT>(single_numel);
  int rc = g->partials.reserve(sizeof(double) * (size_t)n_partials);
  if (rc) return rc;
  rc = g->tensor_scalars.reserve(sizeof(TensorScalars) * (size_t)(plan ? plan->n_tensors : 1));
  if (rc) return rc;
  out->partials = (double*)g->partials.ptr;
  out->tensor_scalars = (TensorScalars*)g->tensor_scalars.ptr;
  return 0;
}

template <class DT>
int stable_group_run(const ListPlan* plan, optimi_group* g, const TensorEntry& single, int dtype, double lr,
                     double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps,
                     double max_lr, uint32_t flags, hipStream_t stream) {
  StableScratch scratch;
  int rc = group_scratch<DT>(g, plan, single.numel, flags, &scratch);
  if (rc) return rc;
  return stable_run<DT>(plan, g, single, scratch, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr,
                        flags, stream);
}

// ---- fixed scratch of the allocation-free entry point ---------------------------------------
// One array per GPU, part of the loaded code object, so it exists from the moment the library
// is loaded on a device until the process ends and no call ever allocates it.  Layout: the
// per-tensor scalars in the first 256 bytes, then the pass-1 partials.  `scratch` itself is only
// a host-side handle for hipGetSymbolAddress; kernels get the address that call returns for the
// device they run on.
constexpr size_t kScratchHead = 256;
constexpr size_t kScratchBytes = OPTIMI_NOALLOC_SCRATCH_BYTES;
constexpr int64_t kScratchPartials = (int64_t)((kScratchBytes - kScratchHead) / sizeof(double));
static_assert(kScratchBytes % 256 == 0 && sizeof(TensorScalars) <= kScratchHead, "scratch layout");
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_addr[kMaxDevices] = {};

// Address of the current device's copy of `scratch`; resolved once per device.
int device_scratch(void** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return OPTIMI_ERR_DEVICE;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_addr[dev]) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p || ((uintptr_t)p % 256)) return OPTIMI_ERR_ALIGN;
    scratch_addr[dev] = p;
  }
  *out = scratch_addr[dev];
  return 0;
}


// ---- whole-list steps ------------------------------------------------------------------------
// One function per optimizer behind both of its list entry points.  `dtypes` is nullptr for a
// list of one dtype (`dtype`); for a mixed list it holds every tensor's dtype.

// Sorts out the dtype arguments of a list call: afterwards `*dtype` is the dtype of the list's
// 16-bit tensors (or fp32) and `*dtypes` is null unless fp32 and 16-bit tensors are both there.
int resolve_dtypes(int n_tensors, const int** dtypes, int* dtype) {
  if (!*dtypes) return valid_dtype(*dtype) ? 0 : OPTIMI_ERR_DTYPE;
  if (n_tensors < 0) return OPTIMI_ERR_SIZE;
  bool mixed = false;
  int rc = list_dtypes(n_tensors, *dtypes, dtype, &mixed);
  if (rc) return rc;
  if (!mixed) *dtypes = nullptr;
  return 0;
}

int adam_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
              void* const* exp_avg_sq, void* const* kahan_comp, const int64_t* numel, const int* dtypes, int dtype,
              double lr, double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps,
              uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[5] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 5, adam_need(kahan, update), bit(4), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const AdamScalars s = adam_scalars(dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  const AdamScalars s_f32 = adam_scalars(OPTIMI_F32, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  dispatch<AdamOp, 3>(dtype, kahan, update, adam_wd_mode(weight_decay, flags),
                      [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); });
  return finish_list(g, plan, stream);
}

int lion_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
              void* const* kahan_comp, const int64_t* numel, const int* dtypes, int dtype, double lr, double beta1_comp,
              double beta2_comp, double weight_decay, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[4] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 4, lion_need(kahan, update), bit(3), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const LionScalars s = lion_scalars(dtype, lr, beta1_comp, beta2_comp, weight_decay);
  const LionScalars s_f32 = lion_scalars(OPTIMI_F32, lr, beta1_comp, beta2_comp, weight_decay);
  dispatch<LionOp, 2>(dtype, kahan, update, lion_wd_mode(weight_decay, flags),
                      [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); });
  return finish_list(g, plan, stream);
}

int stableadamw_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
                     void* const* exp_avg_sq, void* const* kahan_comp, const int64_t* numel, const int* dtypes, int dtype,
                     double lr, double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps,
                     double max_lr, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  if ((flags & OPTIMI_DECOUPLE_LR) && weight_decay != 0 && !(max_lr > 0)) return OPTIMI_ERR_ARG;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[5] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 5, adam_need(kahan, update), bit(4), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  // the reduction scratch is the group's: a previous launch on another stream may still read it
  if (plan.few && g->launched && g->last_stream != stream) {
    bool capturing = false;
    rc = stream_capturing(stream, &capturing);
    if (rc) return rc;
    if (!capturing) HIP_TRY(hipStreamWaitEvent(stream, g->last_launch, 0));
  }
  TensorEntry none;
  std::memset(&none, 0, sizeof(none));
  rc = dtype == OPTIMI_BF16
           ? stable_group_run<BF16>(&plan, g, none, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
       : dtype == OPTIMI_F16
           ? stable_group_run<F16>(&plan, g, none, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
           : stable_group_run<F32>(&plan, g, none, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream);
  if (rc) return rc;
  return note_launch(g, stream);
}

int adan_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
              void* const* exp_avg_diff, void* const* exp_avg_sq, void* const* prev_grad, void* const* kahan_comp,
              const int64_t* numel, const int* dtypes, int dtype, double lr, double beta1_comp, double beta2,
              double beta2_comp, double beta3_hat, double beta3_comp, double eps, double weight_decay, uint32_t flags,
              hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* const* lists[7] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_diff, (const void* const*)exp_avg_sq,
                                 (const void* const*)prev_grad, (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 7, adan_need(kahan, update), bit(6), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const AdanScalars s = adan_scalars(dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay);
  const AdanScalars s_f32 = adan_scalars(OPTIMI_F32, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay);
  dispatch<AdanOp, 3>(dtype, kahan, update, adan_wd_mode(weight_decay, flags),
                      [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); });
  return finish_list(g, plan, stream);
}

int sgd_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
             void* const* kahan_comp, const int64_t* numel, const int* dtypes, int dtype, double lr, double momentum,
             double weight_decay, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const int mom = sgd_mom_mode(momentum, flags);
  if (!update && !mom) return 0;  // nothing to accumulate into
  const void* const* lists[4] = {(const void* const*)param, grad, (const void* const*)exp_avg, (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 4, sgd_need(kahan, update, mom), bit(3), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const SgdScalars s = sgd_scalars(dtype, lr, momentum, weight_decay);
  const SgdScalars s_f32 = sgd_scalars(OPTIMI_F32, lr, momentum, weight_decay);
  sgd_dispatch(dtype, kahan, update, adam_wd_mode(weight_decay, flags), mom,
               [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); });
  return finish_list(g, plan, stream);
}

int radam_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
               void* const* exp_avg_sq, void* const* kahan_comp, const int64_t* numel, const int* dtypes, int dtype,
               double lr, double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps,
               double rect, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const bool rectify = (flags & OPTIMI_RECTIFY) != 0;
  const void* const* lists[5] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 5, adam_need(kahan, update), bit(4), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const double step_lr = rectify ? lr * rect : lr;
  const AdamScalars s = adam_scalars(dtype, step_lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  const AdamScalars s_f32 = adam_scalars(OPTIMI_F32, step_lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  const int wd = adam_wd_mode(weight_decay, flags);
  auto launch = [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); };
  if (rectify || !update) dispatch<AdamOp, 3>(dtype, kahan, update, wd, launch);
  else dispatch<RAdamEarlyOp, 3>(dtype, kahan, update, wd, launch);
  return finish_list(g, plan, stream);
}

int ranger_list(optimi_group* g, int n_tensors, void* const* param, const void* const* grad, void* const* exp_avg,
                void* const* exp_avg_sq, void* const* la_param, void* const* kahan_comp, const int64_t* numel,
                const int* dtypes, int dtype, double lr, double beta1_comp, double beta2_hat, double beta2_comp,
                double weight_decay, double eps, double rect, double alpha, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  int rc = resolve_dtypes(n_tensors, &dtypes, &dtype);
  if (rc) return rc;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const bool rectify = (flags & OPTIMI_RECTIFY) != 0, la = (flags & OPTIMI_LOOKAHEAD) != 0;
  const void* const* lists[6] = {(const void* const*)param, grad, (const void* const*)exp_avg,
                                 (const void* const*)exp_avg_sq, (const void* const*)kahan_comp,
                                 (const void* const*)la_param};
  ListPlan plan;
  rc = plan_list(g, n_tensors, lists, 6, ranger_need(kahan, update, la), bit(4), numel, dtypes, dtype, flags, stream, &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  const double step_lr = rectify ? lr * rect : lr;
  RangerScalars s, s_f32;
  s.a = adam_scalars(dtype, step_lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  s.alpha_d = Sd(alpha, dtype);
  s_f32.a = adam_scalars(OPTIMI_F32, step_lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  s_f32.alpha_d = Sd(alpha, OPTIMI_F32);
  const int wd = adam_wd_mode(weight_decay, flags);
  if (update && la) {
    ranger_dispatch(dtype, kahan, wd, rectify, [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, &s_f32); });
  } else {  // the RAdam step
    auto launch = [&](auto op) { launch_list<decltype(op)>(g, plan, s.a, stream, nullptr, &s_f32.a); };
    if (rectify || !update) dispatch<AdamOp, 3>(dtype, kahan, update, wd, launch);
    else dispatch<RAdamEarlyOp, 3>(dtype, kahan, update, wd, launch);
  }
  return finish_list(g, plan, stream);
}

// Calls fn(ProbeOp<NR, NW>{}) for 1 <= NW <= NR <= kMaxArrays.
template <int NR, class Fn, int... W>
void probe_pick_write(int n_write, Fn&& fn, std::integer_sequence<int, W...>) {
  (void)std::initializer_list<int>{(n_write == W + 1 ? (fn(ProbeOp<NR, W + 1>{}), 0) : 0)...};
}
template <class Fn, int... R>
void probe_pick(int n_read, int n_write, Fn&& fn, std::integer_sequence<int, R...>) {
  (void)std::initializer_list<int>{
      (n_read == R + 1 ? (probe_pick_write<R + 1>(n_write, fn, std::make_integer_sequence<int, R + 1>{}), 0) : 0)...};
}

int probe_list(optimi_group* g, int n_tensors, void* const* const* arrays, const int64_t* bytes, int n_read, int n_write,
               int granules, uint32_t flags, hipStream_t stream) {
  if (!g) return OPTIMI_ERR_NULL;
  if (n_tensors < 0) return OPTIMI_ERR_SIZE;
  if (n_write < 1 || n_write > n_read || n_read > kMaxArrays) return OPTIMI_ERR_ARG;
  if (granules < 0 || granules > 51) return OPTIMI_ERR_ARG;
  if (n_tensors > 0 && (!arrays || !bytes)) return OPTIMI_ERR_NULL;
  const void* const* lists[kMaxArrays] = {};
  std::vector<int64_t> numel;
  try {
    numel.resize((size_t)n_tensors);
  } catch (const std::bad_alloc&) {
    return OPTIMI_ERR_NOMEM;
  }
  for (int a = 0; a < n_read; ++a) {
    if (n_tensors > 0 && !arrays[a]) return OPTIMI_ERR_NULL;
    lists[a] = (const void* const*)arrays[a];
  }
  for (int t = 0; t < n_tensors; ++t) {
    if (bytes[t] < 0 || bytes[t] % 16) return OPTIMI_ERR_SIZE;
    numel[(size_t)t] = bytes[t] / 4;
    for (int a = 0; a < n_read; ++a) {
      if (!arrays[a][t] && bytes[t] > 0) return OPTIMI_ERR_NULL;
      if ((uintptr_t)arrays[a][t] % 16) return OPTIMI_ERR_ALIGN;
    }
  }
  ListPlan plan;
  int rc = plan_list(g, n_tensors, lists, kMaxArrays, (1u << n_read) - 1u, 0u, numel.data(), nullptr, OPTIMI_F32, flags, stream,
                     &plan);
  if (rc) return rc;
  if (plan.n_chunks == 0) return 0;
  ProbeScalars s;
  s.salt = 0x9e3779b9u;
  s.mask = (flags & OPTIMI_PROBE_SCRAMBLE) ? 0xffffffffu : 0u;
  probe_pick(n_read, n_write,
             [&](auto op) { launch_list<decltype(op)>(g, plan, s, stream, nullptr, nullptr, granules); },
             std::make_integer_sequence<int, kMaxArrays>{});
  return finish_list(g, plan, stream);
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
    case OPTIMI_ERR_DTYPE: return "optimi_hip: unsupported dtype (expected OPTIMI_F32, OPTIMI_BF16 or OPTIMI_F16)";
    case OPTIMI_ERR_ALIGN: return "optimi_hip: buffer not aligned to its element size";
    case OPTIMI_ERR_DEVICE: return "optimi_hip: group used on a different device than it was created on";
    case OPTIMI_ERR_NOMEM: return "optimi_hip: host allocation failed";
    case OPTIMI_ERR_ARG: return "optimi_hip: inconsistent scalar argument";
    case OPTIMI_ERR_CAPTURE: return "optimi_hip: the stream is capturing a HIP graph and this list's tables are not on the device yet (step the same list once before the capture)";
    case OPTIMI_ERR_LIMIT: return "optimi_hip: tensor has more elements than the fixed scratch of the allocation-free entry point covers (OPTIMI_NOALLOC_MAX_NUMEL)";
    default: break;
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "optimi_hip: unknown status";
}

int optimi_hip_version(void) { return kAbiVersion; }

int64_t optimi_hip_chunk_elems(int dtype) {
  if (!valid_dtype(dtype)) return OPTIMI_ERR_DTYPE;
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
  g->tables[0].dev.release();
  g->tables[1].dev.release();
  g->chunk_map.release();
  g->partials.release();
  g->tensor_scalars.release();
  delete g;
  return rc;
}

int optimi_hip_adam_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                          const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                          double beta2_comp, double weight_decay, double eps, uint32_t flags, optimi_stream_t stream) {
  return adam_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, nullptr, dtype, lr, beta1_comp,
                   beta2_hat, beta2_comp, weight_decay, eps, flags, (hipStream_t)stream);
}

int optimi_hip_adam_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                const int64_t* numel, const int* dtype, double lr, double beta1_comp, double beta2_hat,
                                double beta2_comp, double weight_decay, double eps, uint32_t flags,
                                optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return adam_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, dtype, OPTIMI_F32, lr, beta1_comp,
                   beta2_hat, beta2_comp, weight_decay, eps, flags, (hipStream_t)stream);
}

int optimi_hip_lion_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                          optimi_stream_t stream) {
  return lion_list(g, n_tensors, param, grad, exp_avg, kahan_comp, numel, nullptr, dtype, lr, beta1_comp, beta2_comp,
                   weight_decay, flags, (hipStream_t)stream);
}

int optimi_hip_lion_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                                double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                                optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return lion_list(g, n_tensors, param, grad, exp_avg, kahan_comp, numel, dtype, OPTIMI_F32, lr, beta1_comp, beta2_comp,
                   weight_decay, flags, (hipStream_t)stream);
}

int optimi_hip_stableadamw_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                 void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                 const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                                 double beta2_comp, double weight_decay, double eps, double max_lr, uint32_t flags,
                                 optimi_stream_t stream) {
  return stableadamw_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, nullptr, dtype, lr,
                          beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, (hipStream_t)stream);
}

int optimi_hip_stableadamw_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                       void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                       const int64_t* numel, const int* dtype, double lr, double beta1_comp,
                                       double beta2_hat, double beta2_comp, double weight_decay, double eps,
                                       double max_lr, uint32_t flags, optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return stableadamw_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, dtype, OPTIMI_F32, lr,
                          beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, (hipStream_t)stream);
}

int optimi_hip_adan_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_diff, void* const* exp_avg_sq,
                          void* const* prev_grad, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2, double beta2_comp, double beta3_hat, double beta3_comp,
                          double eps, double weight_decay, uint32_t flags, optimi_stream_t stream) {
  return adan_list(g, n_tensors, param, grad, exp_avg, exp_avg_diff, exp_avg_sq, prev_grad, kahan_comp, numel, nullptr,
                   dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags,
                   (hipStream_t)stream);
}

int optimi_hip_adan_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* exp_avg_diff, void* const* exp_avg_sq,
                                void* const* prev_grad, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                                double lr, double beta1_comp, double beta2, double beta2_comp, double beta3_hat,
                                double beta3_comp, double eps, double weight_decay, uint32_t flags,
                                optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return adan_list(g, n_tensors, param, grad, exp_avg, exp_avg_diff, exp_avg_sq, prev_grad, kahan_comp, numel, dtype,
                   OPTIMI_F32, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags,
                   (hipStream_t)stream);
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
  AdamScalars s = adam_scalars(dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  dispatch<AdamOp, 3>(dtype, kahan, update, adam_wd_mode(weight_decay, flags), [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
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
  LionScalars s = lion_scalars(dtype, lr, beta1_comp, beta2_comp, weight_decay);
  dispatch<LionOp, 2>(dtype, kahan, update, lion_wd_mode(weight_decay, flags), [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
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
  if (g->launched && g->last_stream != stream) {
    bool capturing = false;
    rc = stream_capturing(stream, &capturing);
    if (rc) return rc;
    if (!capturing) HIP_TRY(hipStreamWaitEvent(stream, g->last_launch, 0));
  }
  rc = dtype == OPTIMI_BF16
           ? stable_group_run<BF16>(nullptr, g, e, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
       : dtype == OPTIMI_F16
           ? stable_group_run<F16>(nullptr, g, e, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
           : stable_group_run<F32>(nullptr, g, e, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream);
  if (rc) return rc;
  return note_launch(g, stream);
}

int optimi_hip_stableadamw_single_noalloc(void* param, const void* grad, void* exp_avg, void* exp_avg_sq,
                                          void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                                          double beta2_hat, double beta2_comp, double weight_decay, double eps,
                                          double max_lr, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if ((flags & OPTIMI_DECOUPLE_LR) && weight_decay != 0 && !(max_lr > 0)) return OPTIMI_ERR_ARG;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const void* ptrs[5] = {param, grad, exp_avg, exp_avg_sq, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 5, adam_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel > OPTIMI_NOALLOC_MAX_NUMEL(dtype)) return OPTIMI_ERR_LIMIT;
  if (numel == 0) return 0;
  void* base = nullptr;
  rc = device_scratch(&base);
  if (rc) return rc;
  StableScratch sc;
  sc.tensor_scalars = (TensorScalars*)base;
  sc.partials = (double*)((unsigned char*)base + kScratchHead);
  const int64_t n_partials = dtype == OPTIMI_F32 ? stable_partials<F32>(numel) : stable_partials<BF16>(numel);
  if (n_partials > kScratchPartials) return OPTIMI_ERR_LIMIT;  // the macro and the layout must agree
  rc = dtype == OPTIMI_BF16
           ? stable_run<BF16>(nullptr, nullptr, e, sc, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
       : dtype == OPTIMI_F16
           ? stable_run<F16>(nullptr, nullptr, e, sc, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream)
           : stable_run<F32>(nullptr, nullptr, e, sc, dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags, stream);
  if (rc) return rc;
  HIP_TRY(hipGetLastError());
  return 0;
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
  AdanScalars s = adan_scalars(dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay);
  dispatch<AdanOp, 3>(dtype, kahan, update, adan_wd_mode(weight_decay, flags), [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_sgd_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                         void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                         double momentum, double weight_decay, uint32_t flags, optimi_stream_t stream) {
  return sgd_list(g, n_tensors, param, grad, exp_avg, kahan_comp, numel, nullptr, dtype, lr, momentum, weight_decay,
                  flags, (hipStream_t)stream);
}

int optimi_hip_sgd_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                               void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                               double lr, double momentum, double weight_decay, uint32_t flags,
                               optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return sgd_list(g, n_tensors, param, grad, exp_avg, kahan_comp, numel, dtype, OPTIMI_F32, lr, momentum, weight_decay,
                  flags, (hipStream_t)stream);
}

int optimi_hip_sgd_single(void* param, const void* grad, void* exp_avg, void* kahan_comp, int64_t numel, int dtype,
                          double lr, double momentum, double weight_decay, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const int mom = sgd_mom_mode(momentum, flags);
  const void* ptrs[4] = {param, grad, exp_avg, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 4, sgd_need(kahan, update, mom), numel, dtype);
  if (rc) return rc;
  if (numel == 0 || (!update && !mom)) return 0;
  SgdScalars s = sgd_scalars(dtype, lr, momentum, weight_decay);
  sgd_dispatch(dtype, kahan, update, adam_wd_mode(weight_decay, flags), mom, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_radam_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                           void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                           const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                           double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                           optimi_stream_t stream) {
  return radam_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, nullptr, dtype, lr, beta1_comp,
                    beta2_hat, beta2_comp, weight_decay, eps, rect, flags, (hipStream_t)stream);
}

int optimi_hip_radam_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                 void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                 const int64_t* numel, const int* dtype, double lr, double beta1_comp, double beta2_hat,
                                 double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                                 optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return radam_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, kahan_comp, numel, dtype, OPTIMI_F32, lr, beta1_comp,
                    beta2_hat, beta2_comp, weight_decay, eps, rect, flags, (hipStream_t)stream);
}

int optimi_hip_radam_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan_comp,
                            int64_t numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                            double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                            optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const bool rectify = (flags & OPTIMI_RECTIFY) != 0;
  const void* ptrs[5] = {param, grad, exp_avg, exp_avg_sq, kahan_comp};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 5, adam_need(kahan, update), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  AdamScalars s = adam_scalars(dtype, rectify ? lr * rect : lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  const int wd = adam_wd_mode(weight_decay, flags);
  if (rectify || !update) dispatch<AdamOp, 3>(dtype, kahan, update, wd, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  else dispatch<RAdamEarlyOp, 3>(dtype, kahan, update, wd, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_ranger_multi(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                            void* const* exp_avg, void* const* exp_avg_sq, void* const* la_param,
                            void* const* kahan_comp, const int64_t* numel, int dtype, double lr, double beta1_comp,
                            double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                            double alpha, uint32_t flags, optimi_stream_t stream) {
  return ranger_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, la_param, kahan_comp, numel, nullptr, dtype, lr,
                     beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, rect, alpha, flags, (hipStream_t)stream);
}

int optimi_hip_ranger_multi_mixed(optimi_group* g, int n_tensors, void* const* param, const void* const* grad,
                                  void* const* exp_avg, void* const* exp_avg_sq, void* const* la_param,
                                  void* const* kahan_comp, const int64_t* numel, const int* dtype, double lr,
                                  double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay,
                                  double eps, double rect, double alpha, uint32_t flags, optimi_stream_t stream) {
  if (!dtype && n_tensors > 0) return OPTIMI_ERR_NULL;
  return ranger_list(g, n_tensors, param, grad, exp_avg, exp_avg_sq, la_param, kahan_comp, numel, dtype, OPTIMI_F32, lr,
                     beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, rect, alpha, flags, (hipStream_t)stream);
}

int optimi_hip_ranger_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* la_param,
                             void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                             double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                             double alpha, uint32_t flags, optimi_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const bool update = (flags & OPTIMI_UPDATE) != 0, kahan = kahan_on(dtype, flags);
  const bool rectify = (flags & OPTIMI_RECTIFY) != 0, la = (flags & OPTIMI_LOOKAHEAD) != 0;
  const void* ptrs[6] = {param, grad, exp_avg, exp_avg_sq, kahan_comp, la_param};
  TensorEntry e;
  int rc = single_entry(e, ptrs, 6, ranger_need(kahan, update, la), numel, dtype);
  if (rc) return rc;
  if (numel == 0) return 0;
  RangerScalars s;
  s.a = adam_scalars(dtype, rectify ? lr * rect : lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps);
  s.alpha_d = Sd(alpha, dtype);
  const int wd = adam_wd_mode(weight_decay, flags);
  if (update && la) {
    ranger_dispatch(dtype, kahan, wd, rectify, [&](auto op) { launch_single<decltype(op)>(e, s, nullptr, stream); });
  } else {  // the RAdam step
    auto launch = [&](auto op) { launch_single<decltype(op)>(e, s.a, nullptr, stream); };
    if (rectify || !update) dispatch<AdamOp, 3>(dtype, kahan, update, wd, launch);
    else dispatch<RAdamEarlyOp, 3>(dtype, kahan, update, wd, launch);
  }
  HIP_TRY(hipGetLastError());
  return 0;
}

int optimi_hip_copy_probe(void* dst, const void* src, int64_t bytes, optimi_stream_t stream_) {
  if (!dst || !src) return OPTIMI_ERR_NULL;
  if (bytes < 0 || bytes % 16) return OPTIMI_ERR_SIZE;
  if (((uintptr_t)dst % 16) || ((uintptr_t)src % 16)) return OPTIMI_ERR_ALIGN;
  const int64_t n_vec = bytes / 16;
  if (n_vec == 0) return 0;
  // fewer than 2^32 threads per grid (see launch_workgroup_limit): just under 64 GiB per launch
  constexpr int64_t kVecPerLaunch = (((int64_t)1 << 32) / 256 - 1) * 256;
  for (int64_t first = 0; first < n_vec; first += kVecPerLaunch) {
    const int64_t n = n_vec - first < kVecPerLaunch ? n_vec - first : kVecPerLaunch;
    ++kernel_launches;
    copy_probe_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream_>>>((u32x4*)dst + first,
                                                                                                 (const u32x4*)src + first, n);
    HIP_TRY(hipGetLastError());
  }
  return 0;
}

int64_t optimi_hip_launch_limit(int64_t workgroups) {
  const int64_t before = launch_workgroup_limit.load();
  if (workgroups > 0) {
    int64_t w = workgroups / kSub * kSub;  // whole chunks
    if (w < kSub) w = kSub;
    if (w > kGridWorkgroups) w = kGridWorkgroups;
    launch_workgroup_limit.store(w);
  } else if (workgroups < 0) {
    launch_workgroup_limit.store(kGridWorkgroups);
  }
  return before;
}

int optimi_hip_stream_probe(optimi_group* g, int n_tensors, void* const* const* arrays, const int64_t* bytes, int n_read,
                            int n_write, int granules, uint32_t flags, optimi_stream_t stream) {
  return probe_list(g, n_tensors, arrays, bytes, n_read, n_write, granules, flags, (hipStream_t)stream);
}

int64_t optimi_hip_launch_count(void) { return kernel_launches.load(); }

int64_t optimi_hip_resident_bytes(void) { return kResidentBytes; }

int64_t optimi_hip_upload_count(void) { return table_uploads.load(); }

int64_t optimi_hip_resident_launch_count(void) { return resident_launches.load(); }

}  // extern "C"
