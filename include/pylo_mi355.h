/*
 * pylo_mi355.h -- C ABI of the MI355X (gfx950) fused learned-optimizer step.
 *
 * The library replaces the three CUDA extension modules of the reference
 * (pylo/csrc/celo2_kernel.cu, velo_kernel.cu, learned_optimizer.cu) and the
 * per-tensor accumulator updates their Python callers perform around them
 * (pylo/optim/ELO_CELO2_cuda.py:179-202,235-286, velo_cuda.py:502-546,668-755,
 * AdafacLO_cuda.py:291-407).  One "plan" describes a fixed list of parameter
 * tensors; one *_step call advances every tensor of the plan by one optimizer
 * step with a constant number of kernel launches.
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on failure;
 *     pylo_mi355_last_error() then returns a thread-local message;
 *   - all device buffers are caller-owned fp32, contiguous, 16-byte aligned;
 *     nothing is allocated on the device by the library (the caller passes a
 *     workspace of pylo_mi355_plan_workspace_bytes() bytes, 256-byte aligned);
 *   - `stream` is a hipStream_t (NULL = the null stream); calls only enqueue
 *     work and never synchronise the device;
 *   - a plan must not be used from two host threads, or on two streams, at once.
 */
#ifndef PYLO_MI355_H
#define PYLO_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PYLO_MI355_ABI_VERSION 1
#define PYLO_MAX_DIMS 8

/* optimizer kinds */
#define PYLO_KIND_CELO2 0   /* ELO_CELO2_CUDA / CELO2_CUDA (celo2_kernel.cu)           */
#define PYLO_KIND_VELO 1    /* VeLO_CUDA (velo_kernel.cu)                              */
#define PYLO_KIND_ADAFAC 2  /* AdafacLO_CUDA / ELO_CUDA / MuLO_CUDA (learned_optimizer.cu) */

/* PyloTensorShape.flags */
#define PYLO_F_ADAM 1 /* CELO2: update with AdamW on mom[0] / rms (1-D tensors, is_embedding groups;
                         ELO_CELO2_cuda.py:246-253) */

typedef struct PyloPlan PyloPlan; /* opaque, host memory owned by the library */

typedef struct {
  int32_t ndim; /* 0..PYLO_MAX_DIMS (0 = scalar, treated as one element) */
  int32_t flags;
  int64_t shape[PYLO_MAX_DIMS];
} PyloTensorShape;

/* Accumulator decays (already clipped to [0,1]); 1-beta is formed in fp32 by the library,
   as `1 - beta` is in ELO_CELO2_naive.py:145-153 / Velo_naive.py:419-420. */
typedef struct {
  float beta_m[3];
  float beta_rms;
  float beta_fac[3];
} PyloDecays;

/* Per-tensor, per-step arguments.  Pointers are device pointers; the table itself is host
   memory and is copied by the call. */
typedef struct {
  const float* grad; /* NULL: the tensor is skipped this step (p.grad is None)               */
  float* param;      /* (n)                                                                  */
  float* mom;        /* (3, n)  momentum accumulators, decay axis leading                    */
  float* rms;        /* (n)     second-moment accumulator                                    */
  float* fac_r;      /* (3, n/size(dr)) row accumulator (mean of g^2 over the largest dim)   */
  float* fac_c;      /* (3, n/size(dc)) column accumulator (mean over the 2nd-largest dim)   */
  float* fac_v;      /* (3, n)  VeLO / AdafacLO non-factored accumulator, else NULL          */
  float* step_out;   /* (n)     CELO2: raw per-element step (celo2_kernel.cu:280), else NULL */
  float lr;          /* VeLO / AdafacLO: lr applied in-kernel; CELO2 AdamW branch: adam lr   */
  float weight_decay;/* VeLO / AdafacLO: p -= wd*lr*p after the update; CELO2 AdamW: adam wd */
  float clip_norm;   /* CELO2: global-norm clip threshold, 0 = clipping off for this tensor  */
  float clip_val;    /* element-wise clamp of the gradient (1000 in the reference), 0 = off  */
  float exp_mult;
  float step_mult;
  float bc1;         /* CELO2 AdamW: 1 - beta1^t                                             */
  float bc2;         /* CELO2 AdamW: 1 - beta2^t                                             */
} PyloTensorArgs;

int pylo_mi355_abi_version(void);
const char* pylo_mi355_last_error(void);

/* Bytes of device workspace a plan over these tensors needs. */
int pylo_mi355_plan_workspace_bytes(int kind, const PyloTensorShape* shapes, int n_tensors,
                                    size_t* bytes_out);

/* Builds the launch tables for `n_tensors` tensors and uploads them into `workspace`
   (synchronously, on `stream`).  The workspace must stay alive and untouched by the caller
   for the life of the plan. */
int pylo_mi355_plan_create(int kind, const PyloTensorShape* shapes, int n_tensors, void* workspace,
                           size_t workspace_bytes, void* stream, PyloPlan** plan_out);
int pylo_mi355_plan_destroy(PyloPlan* plan);

/* Number of launches one step enqueues, and the factored dims chosen for tensor i
   (dc = 2nd-largest dim, dr = largest; -1/-1 when not factored). */
int pylo_mi355_plan_num_launches(const PyloPlan* plan);
int pylo_mi355_plan_factored_dims(const PyloPlan* plan, int tensor, int* dc, int* dr);

/* Optional per-launch timing, for benchmarks (no counterpart in the reference).  Between begin and
   end every *_step call records one HIP event before its first launch and one after each launch,
   on the call's stream, for at most `max_steps` calls.  end synchronises the last event and
   writes steps x num_launches durations in milliseconds (row-major) into ms_out. */
int pylo_mi355_plan_timing_begin(PyloPlan* plan, int max_steps);
int pylo_mi355_plan_timing_end(PyloPlan* plan, float* ms_out, int capacity, int* steps_out);

/* Names of the launches of one step, in launch order (static strings). */
const char* pylo_mi355_plan_launch_name(const PyloPlan* plan, int launch);

/*
 * ELO-CELO2 / CELO2 step (replaces celo2_cuda_kernel.celo2_kernel, pylo/csrc/celo2_kernel.cu:284-350,
 * plus the accumulator updates of ELO_CELO2_cuda.py:154-202,235-253).
 *
 * For every tensor with a gradient:  g <- clamp(g * clip_scale, +-clip_val) with
 * clip_scale = clip_norm / max(||all grads||_2, clip_norm); mom/rms EMAs; then
 *   - PYLO_F_ADAM tensors: AdamW on mom[0] / rms, parameter updated in place;
 *   - other (>=2-D) tensors: fac_r / fac_c EMAs, 30 features, per-channel RMS normalisation
 *     over the tensor, the 30->8->8->3 MLP; step_out = o0 * exp(o1 * exp_mult).  The parameter
 *     is NOT touched (Newton-Schulz, normalise and apply follow, ELO_CELO2_cuda.py:288-296).
 * `mlp` is a device pointer to 347 floats: w_in (30,8) | b_in 8 | w_h (8,8) | b_h 8 | w_out (8,3) | b_out 3,
 * weights stored (in, out) as in pylo/models/CELO2_MLP.py:72-86.
 */
int pylo_mi355_celo2_step(PyloPlan* plan, const PyloTensorArgs* args, const PyloDecays* decays,
                          const float* mlp, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PYLO_MI355_H */
