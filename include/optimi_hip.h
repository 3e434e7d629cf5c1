/*
 * optimi_hip.h — C ABI of the MI355X (gfx950) fused optimizer-step library.
 *
 * The reference (warner-benjamin/optimi) has no FFI: its accelerated backend is a set
 * of Triton kernels launched from Python, one launch per tensor.  Each entry point
 * below takes the place of one of those launchers and keeps its argument meaning:
 * pointers to the parameter, gradient and state buffers, the element count, and the
 * step scalars already formed by the functional dispatcher (debiased betas, the
 * weight-decay factor).  Scalars arrive as doubles, exactly as the Python floats the
 * reference passes, and are narrowed inside the library the way the reference's
 * PyTorch for-loop path narrows them, because that path defines the results.
 *
 * Conventions
 *   - every function returns 0 on success, a negative optimi_status for a rejected
 *     argument, or a positive hipError_t value for a HIP runtime failure;
 *     optimi_hip_error_string() explains either.  Nothing throws.
 *   - all buffers are device memory of the current HIP device, contiguous, and of
 *     the one dtype named by `dtype` (the `_multi_mixed` entry points take a dtype per
 *     tensor).  The gradient is never written.
 *   - work is enqueued on `stream` (a hipStream_t; NULL = the default stream) and
 *     the call returns without waiting for it.
 *   - `kahan_comp` may be NULL whenever the Kahan branch is not taken (fp32 tensors,
 *     OPTIMI_KAHAN unset, or OPTIMI_UPDATE unset).  "Low precision" below means bf16 or fp16.
 *   - buffers need only be aligned to their element size.  Tensors whose buffers are all
 *     16-byte aligned take the streaming path; others run the same 16-byte vectors through
 *     element-aligned accesses (about 10 % slower).
 */
#ifndef OPTIMI_HIP_H
#define OPTIMI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* optimi_stream_t; /* hipStream_t */

enum optimi_dtype { OPTIMI_F32 = 0, OPTIMI_BF16 = 1, OPTIMI_F16 = 2 };

enum optimi_flags {
  OPTIMI_KAHAN = 1,       /* kahan_sum: only acts on bf16/fp16 tensors (optimi/adam.py:384)       */
  OPTIMI_UPDATE = 2,      /* update_parameters; unset = accumulate-only step (optimi/adam.py:308) */
  OPTIMI_DECOUPLE_WD = 4, /* Adam: decoupled decay p*=factor; unset = L2 (optimi/adam.py:373-377) */
  OPTIMI_ADAM_WD = 8,     /* Adan: Adam-style decay before the step (optimi/adan.py:447-448)      */
  OPTIMI_DECOUPLE_LR = 16,/* StableAdamW: fully decoupled decay (optimi/stableadamw.py:453-457)   */
  OPTIMI_DAMPENING = 32,  /* SGD: momentum buffer is an EMA, lerp(m, g, 1-momentum) (optimi/sgd.py:352-353) */
  OPTIMI_RECTIFY = 64,    /* RAdam/Ranger: rho > 5, take the rectified Adam step (optimi/radam.py:269-277) */
  OPTIMI_LOOKAHEAD = 128, /* Ranger: this step synchronises with the slow weights, step % k == 0
                             (optimi/ranger.py:452, 471)                                           */
  OPTIMI_RESIDENT = 256,  /* whole-list entry points, a hint: the list was stepped a moment ago and nothing
                             else has gone through the GPU's last-level cache since (a loop of optimizer
                             steps with no forward or backward pass in between).  If its arrays also total
                             at most optimi_hip_resident_bytes(), they are read with cached loads, which
                             then hit.  Without the hint every list is read with streaming loads: after a
                             backward pass nothing of it is left in the cache, and streaming loads are the
                             faster ones on data that has to come from memory.  Results do not depend on
                             it.  No counterpart in the reference.                                  */
  OPTIMI_PROBE_SCRAMBLE = 512 /* optimi_hip_stream_probe only: the written arrays get new bits (a mix of
                             everything that was read) instead of keeping theirs                    */
};

enum optimi_status {
  OPTIMI_OK = 0,
  OPTIMI_ERR_NULL = -1,      /* a required pointer is NULL                         */
  OPTIMI_ERR_SIZE = -2,      /* negative element or tensor count, or beyond limits */
  OPTIMI_ERR_DTYPE = -3,     /* dtype is not an optimi_dtype                       */
  OPTIMI_ERR_ALIGN = -4,     /* a buffer is not aligned to its element size        */
  OPTIMI_ERR_DEVICE = -5,    /* group used on a device other than the one it was made on */
  OPTIMI_ERR_NOMEM = -6,     /* host allocation failed                             */
  OPTIMI_ERR_ARG = -7,       /* inconsistent scalar argument (e.g. max_lr <= 0 with OPTIMI_DECOUPLE_LR) */
  OPTIMI_ERR_LIMIT = -8,     /* numel above OPTIMI_NOALLOC_MAX_NUMEL in the allocation-free entry point */
  OPTIMI_ERR_CAPTURE = -9    /* `stream` is capturing a HIP graph and the list's tables would have to be uploaded */
};

/* Text for a status returned by any function of this header. */
const char* optimi_hip_error_string(int status);

/* ABI version of the loaded library (major * 1000 + minor). */
int optimi_hip_version(void);

/* Elements one workgroup covers for `dtype`; tensors are cut into chunks of this size. */
int64_t optimi_hip_chunk_elems(int dtype);

/* ---------------------------------------------------------------------------------
 * Group handle.  Owns what a whole-list launch needs besides the caller's tensors:
 * the device-side tensor table (pointers, sizes), the chunk map, StableAdamW's
 * reduction partials and per-tensor scalars, and a small pinned staging ring.  None
 * of it is optimizer state; it can be dropped and rebuilt at any time.  The group keeps the
 * tensor tables of its two most recent distinct lists on the device (gradients that alternate
 * between two sets of buffers find theirs every time) and uploads one only when the pointers and
 * sizes of a call match neither; the chunk map depends on the sizes alone.  A list of at most
 * 16 tensors needs no tables at all (its pointers travel as kernel arguments).  A group
 * belongs to the device that was current when it was created and must be used by
 * one thread and one stream at a time.  Under HIP graph capture a whole-list call uploads
 * nothing and keeps the group's own stream bookkeeping out of the graph: a list of more than 16
 * tensors must have been stepped once, with the same pointers and sizes, before the capture
 * begins (and that step must have completed), otherwise the call returns OPTIMI_ERR_CAPTURE;
 * StableAdamW's reduction scratch must have been sized by such a step as well.  (No counterpart in the reference: it plays
 * the role of the Python loop in optimi/adam.py:551-583.)
 * ------------------------------------------------------------------------------- */
typedef struct optimi_group optimi_group;
int optimi_hip_group_create(optimi_group** out);
int optimi_hip_group_destroy(optimi_group* group);

/* ---------------------------------------------------------------------------------
 * Whole-list steps: one launch covers every tensor of the list.
 * Arrays of `n_tensors` host pointers to device buffers; numel[i] elements each.
 * ------------------------------------------------------------------------------- */

/* Adam / AdamW over a list.  Replaces _triton_adam (optimi/adam.py:533-583); results
 * follow _single_param_adam (optimi/adam.py:354-396).  weight_decay is the formed
 * factor 1-lr*wd when OPTIMI_DECOUPLE_WD is set, the raw coefficient otherwise, 0 = none. */
int optimi_hip_adam_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                          const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                          double beta2_comp, double weight_decay, double eps, uint32_t flags,
                          optimi_stream_t stream);

/* Lion over a list.  Replaces _triton_lion (optimi/lion.py:453-492); results follow
 * _single_param_lion (optimi/lion.py:301-338).  weight_decay is the formed factor, 0 = none. */
int optimi_hip_lion_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                          optimi_stream_t stream);

/* StableAdamW over a list.  Replaces _triton_stableadamw (optimi/stableadamw.py:657-725);
 * results follow _single_param_stableadamw (optimi/stableadamw.py:421-472).  Three launches:
 * moments + per-chunk partial sums of g^2/max(v,eps^2); one workgroup per tensor that turns
 * the partials into that tensor's clipped lr and decay factor on the device; the update.
 * weight_decay is the raw coefficient; max_lr is read only with OPTIMI_DECOUPLE_LR. */
int optimi_hip_stableadamw_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                 void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                 const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                                 double beta2_comp, double weight_decay, double eps, double max_lr, uint32_t flags,
                                 optimi_stream_t stream);

/* Adan over a list.  Replaces _triton_adan (optimi/adan.py:652-711); results follow
 * _single_param_adan (optimi/adan.py:405-469).  prev_grad holds the negated previous
 * gradient.  weight_decay is the formed factor 1+lr*wd (or 1-lr*wd with OPTIMI_ADAM_WD), 0 = none. */
int optimi_hip_adan_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                          void* const* exp_avg, void* const* exp_avg_diff, void* const* exp_avg_sq,
                          void* const* prev_grad, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                          double beta1_comp, double beta2, double beta2_comp, double beta3_hat, double beta3_comp,
                          double eps, double weight_decay, uint32_t flags, optimi_stream_t stream);

/* SGD over a list.  Replaces _triton_sgd (optimi/sgd.py:501-543); results follow _single_param_sgd
 * (optimi/sgd.py:329-372).  exp_avg may be NULL when momentum == 0.  weight_decay as for Adam.
 * OPTIMI_DAMPENING selects the dampened momentum update. */
int optimi_hip_sgd_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                         void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, int dtype, double lr,
                         double momentum, double weight_decay, uint32_t flags, optimi_stream_t stream);

/* RAdam over a list.  Replaces _triton_radam (optimi/radam.py:567-628); results follow
 * _single_param_radam (optimi/radam.py:368-417).  With OPTIMI_RECTIFY the step is
 * -lr*rect*m/(sqrt(v)+eps); without it (the first steps) it is -lr*m and `rect` is ignored. */
int optimi_hip_radam_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                           void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                           const int64_t* numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                           double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                           optimi_stream_t stream);

/* Ranger over a list.  Replaces _triton_ranger (optimi/ranger.py:674-745); results follow
 * _single_param_ranger (optimi/ranger.py:402-473): the RAdam step, then with OPTIMI_LOOKAHEAD the
 * Lookahead interpolation la += alpha*(p - la), p = la.  la_param is read only on such steps. */
int optimi_hip_ranger_multi(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                            void* const* exp_avg, void* const* exp_avg_sq, void* const* la_param,
                            void* const* kahan_comp, const int64_t* numel, int dtype, double lr, double beta1_comp,
                            double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                            double alpha, uint32_t flags, optimi_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Whole-list steps over a list of mixed dtypes: the same steps, still one launch, for a
 * parameter group that holds fp32 tensors beside tensors of one 16-bit dtype (a model kept
 * in bf16 whose embeddings or norms stay fp32).  The reference's launchers loop over the
 * tensors of a group whatever their dtypes (optimi/adam.py:551-583 and the same loop in
 * lion.py, stableadamw.py, adan.py, sgd.py, radam.py, ranger.py); these entry points keep such a
 * group in one launch.  They differ from their `_multi` namesakes in one argument: `dtype`
 * is an array with every tensor's own dtype.  bf16 and fp16 in one list is OPTIMI_ERR_DTYPE.
 * OPTIMI_KAHAN applies to the 16-bit tensors only; kahan_comp[i] of an fp32 tensor is ignored
 * and may be NULL.  Every tensor gets the bits its dtype's `_multi` call would give it.  A
 * list that turns out to hold one dtype is stepped exactly as by `_multi`.
 * ------------------------------------------------------------------------------- */
int optimi_hip_adam_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                const int64_t* numel, const int* dtype, double lr, double beta1_comp, double beta2_hat,
                                double beta2_comp, double weight_decay, double eps, uint32_t flags,
                                optimi_stream_t stream);
int optimi_hip_lion_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                                double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                                optimi_stream_t stream);
int optimi_hip_stableadamw_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                       void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                       const int64_t* numel, const int* dtype, double lr, double beta1_comp,
                                       double beta2_hat, double beta2_comp, double weight_decay, double eps,
                                       double max_lr, uint32_t flags, optimi_stream_t stream);
int optimi_hip_adan_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                void* const* exp_avg, void* const* exp_avg_diff, void* const* exp_avg_sq,
                                void* const* prev_grad, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                                double lr, double beta1_comp, double beta2, double beta2_comp, double beta3_hat,
                                double beta3_comp, double eps, double weight_decay, uint32_t flags,
                                optimi_stream_t stream);
int optimi_hip_sgd_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                               void* const* exp_avg, void* const* kahan_comp, const int64_t* numel, const int* dtype,
                               double lr, double momentum, double weight_decay, uint32_t flags,
                               optimi_stream_t stream);
int optimi_hip_radam_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                 void* const* exp_avg, void* const* exp_avg_sq, void* const* kahan_comp,
                                 const int64_t* numel, const int* dtype, double lr, double beta1_comp, double beta2_hat,
                                 double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                                 optimi_stream_t stream);
int optimi_hip_ranger_multi_mixed(optimi_group* group, int n_tensors, void* const* param, const void* const* grad,
                                  void* const* exp_avg, void* const* exp_avg_sq, void* const* la_param,
                                  void* const* kahan_comp, const int64_t* numel, const int* dtype, double lr,
                                  double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay,
                                  double eps, double rect, double alpha, uint32_t flags, optimi_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Per-tensor steps for gradient release: pointers travel as kernel arguments, no table.
 * ------------------------------------------------------------------------------- */

/* Replaces _single_param_triton_adam (optimi/adam.py:585-630). */
int optimi_hip_adam_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan_comp,
                           int64_t numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                           double beta2_comp, double weight_decay, double eps, uint32_t flags, optimi_stream_t stream);

/* Replaces _single_param_triton_lion (optimi/lion.py:494-530). */
int optimi_hip_lion_single(void* param, const void* grad, void* exp_avg, void* kahan_comp, int64_t numel, int dtype,
                           double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags,
                           optimi_stream_t stream);

/* Replaces _single_param_triton_stableadamw (optimi/stableadamw.py:727-791).  `group`
 * supplies the reduction workspace (the reference keeps a one-float `mean_square` tensor
 * in the optimizer state for this, optimi/stableadamw.py:129-130). */
int optimi_hip_stableadamw_single(optimi_group* group, void* param, const void* grad, void* exp_avg, void* exp_avg_sq,
                                  void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                                  double beta2_hat, double beta2_comp, double weight_decay, double eps, double max_lr,
                                  uint32_t flags, optimi_stream_t stream);

/* The same step as optimi_hip_stableadamw_single for callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference.  It takes no group: the reduction partials and the
 * per-tensor scalars live in a fixed array of OPTIMI_NOALLOC_SCRATCH_BYTES that is part of
 * the library's device code (one copy per GPU, held until the process ends), so the call
 * makes no hipMalloc/hipFree and no other allocating call; the first call on a device only
 * looks the array's address up (hipGetSymbolAddress), so make one call outside a capture first.
 * A tensor with more than OPTIMI_NOALLOC_MAX_NUMEL(dtype) elements is rejected with
 * OPTIMI_ERR_LIMIT.  Every call on a GPU uses that GPU's one array: calls that may overlap
 * on one GPU (different streams, different threads) race and must be ordered by the caller.
 * Results are bit-identical to optimi_hip_stableadamw_single. */
#define OPTIMI_NOALLOC_SCRATCH_BYTES (4u * 1024u * 1024u + 256u)
#define OPTIMI_NOALLOC_MAX_NUMEL(dtype) ((dtype) == OPTIMI_F32 ? (int64_t)134217728 : (int64_t)268435456)
int optimi_hip_stableadamw_single_noalloc(void* param, const void* grad, void* exp_avg, void* exp_avg_sq,
                                          void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                                          double beta2_hat, double beta2_comp, double weight_decay, double eps,
                                          double max_lr, uint32_t flags, optimi_stream_t stream);

/* Replaces _single_param_triton_adan (optimi/adan.py:713-770). */
int optimi_hip_adan_single(void* param, const void* grad, void* exp_avg, void* exp_avg_diff, void* exp_avg_sq,
                           void* prev_grad, void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                           double beta2, double beta2_comp, double beta3_hat, double beta3_comp, double eps,
                           double weight_decay, uint32_t flags, optimi_stream_t stream);

/* Replaces _single_param_triton_sgd (optimi/sgd.py:545-584). */
int optimi_hip_sgd_single(void* param, const void* grad, void* exp_avg, void* kahan_comp, int64_t numel, int dtype,
                          double lr, double momentum, double weight_decay, uint32_t flags, optimi_stream_t stream);

/* Replaces _single_param_triton_radam (optimi/radam.py:630-686). */
int optimi_hip_radam_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* kahan_comp,
                            int64_t numel, int dtype, double lr, double beta1_comp, double beta2_hat,
                            double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags,
                            optimi_stream_t stream);

/* Replaces _single_param_triton_ranger (optimi/ranger.py:747-810). */
int optimi_hip_ranger_single(void* param, const void* grad, void* exp_avg, void* exp_avg_sq, void* la_param,
                             void* kahan_comp, int64_t numel, int dtype, double lr, double beta1_comp,
                             double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                             double alpha, uint32_t flags, optimi_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Measurement aid (no counterpart in the reference): a plain 16-byte-per-lane copy of
 * `bytes` bytes (a multiple of 16, both pointers 16-byte aligned).  Benchmarks use it as
 * the practical bandwidth ceiling and to scale hardware byte counters.
 * ------------------------------------------------------------------------------- */
int optimi_hip_copy_probe(void* dst, const void* src, int64_t bytes, optimi_stream_t stream);

/* Measurement aid (no counterpart in the reference; nothing of the optimizers calls it): the
 * memory traffic of a step without its arithmetic.  Array a of tensor i is arrays[a][i], bytes[i]
 * bytes long (a multiple of 16, every pointer 16-byte aligned); arrays 0 .. n_read-1 are read and
 * arrays 0 .. n_write-1 are also written in place, 1 <= n_write <= n_read <= 7 (OPTIMI_ERR_ARG
 * otherwise) - AdamW with Kahan summation is 5 read / 4 written, Lion 4 / 3, StableAdamW's two
 * passes 3 / 2 and 4 / 2, Adan 7 / 6.  The launch is the optimizers' own: the same kernel,
 * 64-lane tiles, streaming loads, write-through tile stores, tensor table / chunk map and
 * occupancy throttle as a 16-bit step with n_read + n_write streams, so bytes moved / duration
 * is the ceiling of that access mix on the machine at hand.  `granules` = 0 takes the occupancy
 * the library would choose for such a step; 1 .. 51 requests that many 1280-byte LDS granules
 * per workgroup instead (a CU holds floor(128 / granules) workgroups).  `flags`: 0, OPTIMI_RESIDENT,
 * OPTIMI_PROBE_SCRAMBLE.  Every stored vector depends on every loaded one (as the parameter, the
 * first array an optimizer stores, depends on all of its inputs).  The written arrays keep their
 * contents: each is stored back as it was read (the bandwidth of this memory depends a little on
 * the data, so the probe leaves the step's own data in place); with OPTIMI_PROBE_SCRAMBLE they
 * are overwritten with a mix of everything that was read, which is how the tests see what the
 * probe touched. */
int optimi_hip_stream_probe(optimi_group* group, int n_tensors, void* const* const* arrays, const int64_t* bytes,
                            int n_read, int n_write, int granules, uint32_t flags, optimi_stream_t stream);

/* Measurement aid (no counterpart in the reference): the number of step, reduction and probe
 * kernels this library has launched in this process so far, every entry point and every thread
 * counted (the small copy that brings a changed tensor table to the device is not).  Tests and
 * benchmarks take differences of it to see how many launches a step costs. */
int64_t optimi_hip_launch_count(void);

/* The largest total size, in bytes, of the arrays a whole-list launch works on for which
 * OPTIMI_RESIDENT is honoured (see there).  A caller that steps several lists per optimizer step
 * compares the sum over all of them with this before passing the hint: a short list of a large
 * model has left the cache by the time it is stepped again.  No counterpart in the reference. */
int64_t optimi_hip_resident_bytes(void);

/* Measurement aids (no counterpart in the reference), counted like optimi_hip_launch_count:
 * how many tensor tables and chunk maps have been copied to the device (a list of more than 16
 * tensors whose pointers and sizes are those of one of the group's two most recent distinct lists
 * uploads nothing: gradients may alternate between two sets of buffers), and
 * how many of the kernels launched for lists read their tensors with cached loads. */
int64_t optimi_hip_upload_count(void);
int64_t optimi_hip_resident_launch_count(void);

/* Test aid (no counterpart in the reference).  A HIP grid holds fewer than 2^32 threads, i.e.
 * fewer than 2^26 of this library's 64-lane workgroups, which is 64 GiB per array; a longer list
 * or tensor (up to 2^31 / 16 chunks of 16 KiB per array, and 2^22 - 1 tensors: OPTIMI_ERR_SIZE
 * beyond) is stepped by several launches, each starting where the previous one ended.  This call
 * sets the number of workgroups one launch may hold - rounded down to whole chunks (16
 * workgroups), at least one chunk, at most the hardware's limit - so that tests can run the
 * split on small lists; 0 changes nothing, a negative value restores the hardware's limit.
 * Returns the limit that was in force before.  Results never depend on it. */
int64_t optimi_hip_launch_limit(int64_t workgroups);

#ifdef __cplusplus
}
#endif
#endif /* OPTIMI_HIP_H */
