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
 *   - all device buffers are caller-owned, contiguous, 16-byte aligned and fp32,
 *     except `grad` and `param` of tensors whose PyloTensorShape carries a
 *     PYLO_F_STORE_* tag; nothing is allocated on the device by the library
 *     (the caller passes a workspace of pylo_mi355_plan_workspace_bytes()
 *     bytes, 256-byte aligned);
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

#define PYLO_MI355_ABI_VERSION 9
#define PYLO_MAX_DIMS 8
#define PYLO_MAX_GROUPS 8   /* parameter groups with their own step counter (VeLO) */

/* optimizer kinds */
#define PYLO_KIND_CELO2 0   /* ELO_CELO2_CUDA / CELO2_CUDA (celo2_kernel.cu)           */
#define PYLO_KIND_VELO 1    /* VeLO_CUDA (velo_kernel.cu)                              */
#define PYLO_KIND_ADAFAC 2  /* AdafacLO_CUDA / ELO_CUDA / MuLO_CUDA (learned_optimizer.cu) */

/* PyloTensorShape.flags */
#define PYLO_F_ADAM 1 /* CELO2: update with AdamW on mom[0] / rms (1-D tensors, is_embedding groups;
                         ELO_CELO2_cuda.py:246-253) */
#define PYLO_F_ADAM_INDEP 2 /* CELO2: AdamW with the tensor's own moments (CELO2_cuda.py:234-253): `mom`
                               points to exp_avg (n), `rms` to exp_avg_sq (n); betas and eps come from
                               PyloDecays.adam_*; bc1 / bc2 carry 1 - beta^adam_step of the tensor */

#define PYLO_F_NAN_TO_NUM 4 /* AdafacLO kind: the (clip-scaled) gradient passes through torch.nan_to_num
                              (ELO_cuda.py:208-211): NaN -> 0; give the tensor clip_val = FLT_MAX so that
                              +-inf map to +-FLT_MAX as torch maps them */
#define PYLO_F_WD_PRESTEP 8 /* AdafacLO kind: p -= lr * (step + weight_decay * p) against the pre-step
                               parameter (ELO_naive.py:236-237; ELO_cuda.py:244-247,285-286) instead of
                               the two-stage AdafacLO update */

#define PYLO_F_GLOBAL_NORM 16 /* AdafacLO kind: the tensor's gradient is summed into the global norm of the
                                 call; required on every tensor of a plan whose steps pass clip_norm > 0
                                 (CELO2 plans always take the norm over all their tensors) */
#define PYLO_F_TENSOR_NORM 32 /* AdafacLO kind: clip_norm > 0 bounds the norm of this tensor's gradient alone, as
                                 torch.nn.utils.clip_grad_norm_(p, clip_norm) does on one parameter
                                 (AdafacLO_naive.py:199-200, AdafacLO_cuda.py:214-215): the step sees
                                 g * min(1, clip_norm / (||g||_2 + 1e-6)).  The gradient buffer itself is not
                                 modified (the reference scales p.grad in place).  On every tensor of the plan or
                                 on none; not with PYLO_F_GLOBAL_NORM or PYLO_F_NAN_TO_NUM; clip_val must be 0 */

#define PYLO_F_NO_ORTHOGONALIZE 64 /* CELO2 kind: the tensor is never passed to
                                 pylo_mi355_celo2_orthogonalize_finish with PYLO_ARG_ORTHOGONALIZE (its group does not
                                 orthogonalise, or the caller does that itself): no Newton-Schulz workspace is
                                 reserved for it.  That workspace is 12 bytes per element of every other 2-D
                                 MLP tensor (two fp16 planes of X in both orientations, twice for the one the
                                 update product writes), three times the tensor's fp32 size, and makes up most
                                 of what pylo_mi355_plan_workspace_bytes reports for an ELO-CELO2 plan */

/* Storage type of the tensor's `grad` and `param` buffers (bits 8-9 of PyloTensorShape.flags).  The reference's
   kernels are instantiated for float, double and half (AT_DISPATCH_FLOATING_TYPES_AND_HALF,
   celo2_kernel.cu:314,328, velo_kernel.cu:405,427, learned_optimizer.cu:338,364): they widen every value to
   float on load (celo2_kernel.cu:70-75), compute in float and narrow on store (:280).  Here likewise: the
   gradient and the parameter are widened exactly to fp32 when read, every accumulator (mom, rms, fac_*,
   step_out) stays fp32 as the reference's classes keep them (ELO_CELO2_cuda.py:167-177), all arithmetic is
   that of an fp32 tensor holding the widened values (fp64 values are rounded to fp32 first, as
   static_cast<float> does), and the updated parameter is rounded to nearest-even into its storage type.
   bf16 is an addition (the reference's dispatch has no bf16 case).  Mixed plans are fine: the tag is per
   tensor. */
#define PYLO_F_STORE_F32 0
#define PYLO_F_STORE_F16 0x100
#define PYLO_F_STORE_BF16 0x200
#define PYLO_F_STORE_F64 0x300
#define PYLO_F_STORE_MASK 0x300

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
  float adam_beta1, adam_beta2, adam_eps; /* PYLO_F_ADAM_INDEP tensors only (CELO2_cuda.py:113-114) */
} PyloDecays;

/* Per-tensor, per-step arguments.  Pointers are device pointers; the table itself is host
   memory and is copied by the call. */
typedef struct {
  const float* grad; /* NULL: the tensor is skipped this step (p.grad is None); elements of the
                        tensor's storage type (PYLO_F_STORE_*), fp32 without a tag            */
  float* param;      /* (n)     of the tensor's storage type                                  */
  float* mom;        /* (3, n)  momentum accumulators, decay axis leading                    */
  float* rms;        /* (n)     second-moment accumulator                                    */
  float* fac_r;      /* (3, n/size(dr)) row accumulator (mean of g^2 over the largest dim)   */
  float* fac_c;      /* (3, n/size(dc)) column accumulator (mean over the 2nd-largest dim)   */
  float* fac_v;      /* (3, n)  VeLO / AdafacLO non-factored accumulator, else NULL          */
  float* step_out;   /* (n)     CELO2: raw per-element step (celo2_kernel.cu:280), else NULL */
  float lr;          /* VeLO / AdafacLO: lr applied in-kernel; CELO2 AdamW branch: adam lr   */
  float weight_decay;/* VeLO / AdafacLO: p -= wd*lr*p after the update; CELO2 AdamW: adam wd */
  float clip_norm;   /* CELO2, AdafacLO kind (ELO_cuda.py:153-161): global-norm clip threshold over
                        the gradients of the call, 0 = clipping off for this tensor; on tensors
                        flagged PYLO_F_TENSOR_NORM: the bound on the tensor's own gradient norm
                        (AdafacLO_cuda.py:214-215)                                              */
  float clip_val;    /* element-wise clamp of the gradient (1000 in the reference), 0 = off  */
  float exp_mult;
  float step_mult;
  float bc1;         /* CELO2 AdamW: 1 - beta1^t; AdafacLO kind: the tensor's step counter when
                        the call passes step < 0                                             */
  float bc2;         /* CELO2 AdamW: 1 - beta2^t                                             */
  int32_t group;     /* VeLO: index into PyloVeloStep.frac (the tensor's parameter group)    */
  int32_t flags;     /* PYLO_ARG_* bits, 0 for the step calls                                */
} PyloTensorArgs;

/* PyloTensorArgs.flags, pylo_mi355_celo2_orthogonalize_finish: `step_out` holds the tensor's raw step and the
   call orthogonalises it first (the group's `orthogonalize`, ELO_CELO2_cuda.py:288-292) */
#define PYLO_ARG_ORTHOGONALIZE 1

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

/* ---- Steps that a HIP graph can replay.  No counterpart in the reference, whose step() waits for
 * the device once per step or per tensor (ELO_CELO2_cuda.py:154-162, velo_cuda.py:747) and counts
 * steps on the host (ELO_CELO2_cuda.py:224, AdafacLO_cuda.py:304-305). ------------------------- */

/* The plan's own argument tables: pinned host memory, `n_tensors` records each, slot 0..3.  A step /
   finish call whose `args` IS such a pointer does no host-side staging (no comparison with the
   previous table, no events, no waits): it enqueues one small kernel that reads the table when it
   RUNS.  Recorded into a HIP graph, every replay therefore takes the table's contents at that moment.
   The caller must not write a table while a run that reads it may be in flight.  A slot that has been
   handed out is no longer used for staging ordinary calls (which need at least one free slot). */
#define PYLO_ARG_TABLES 4
int pylo_mi355_plan_arg_table(PyloPlan* plan, int slot, PyloTensorArgs** table_out);

/* Step counters kept on the device.  With `counters` set, every *_step call on the plan first runs a
   small kernel that advances them and derives from them what the host otherwise supplies per step:
     CELO2 kind    counters[t] += 1 for every tensor (a PYLO_F_ADAM_INDEP tensor: only when it has a
                   gradient), then bc1 / bc2 of an AdamW tensor's record = 1 - beta1^counters[t] /
                   1 - beta2^counters[t];
     VeLO kind     frac of group g = tanh((counters[g] / num_steps - ts) * 10), then counters[g] += 1;
                   PyloVeloStep.frac is ignored; `counters` holds PYLO_MAX_GROUPS entries;
     AdafacLO kind bc1 of record t = counters[t], then counters[t] += 1 when tensor t has a gradient;
                   the call's `step` is ignored.
   `counters` is device memory owned by the caller (int32, one per tensor except for VeLO); NULL
   switches the mechanism off. */
typedef struct {
  int32_t* counters;
  double beta1, beta2; /* CELO2 kind */
  double num_steps;    /* VeLO kind  */
} PyloDeviceSteps;
int pylo_mi355_plan_device_steps(PyloPlan* plan, const PyloDeviceSteps* steps);

/*
 * ELO-CELO2 / CELO2 step (replaces celo2_cuda_kernel.celo2_kernel, pylo/csrc/celo2_kernel.cu:284-350,
 * plus the accumulator updates of ELO_CELO2_cuda.py:154-202,235-253).
 *
 * For every tensor with a gradient:  g <- clamp(g * clip_scale, +-clip_val) with
 * clip_scale = clip_norm / max(||all grads||_2, clip_norm); mom/rms EMAs; then
 *   - PYLO_F_ADAM tensors: AdamW on mom[0] / rms, parameter updated in place;
 *   - other tensors: fac_r / fac_c EMAs, 30 features, per-channel RMS normalisation over the last
 *     two dims (the whole tensor when it is 2-D; one set of normalisers per slice when it has more
 *     dims, ELO_CELO2_naive.py:217-218), the 30->8->8->3 MLP; step_out = o0 * exp(o1 * exp_mult).
 *     The parameter is NOT touched (Newton-Schulz, normalise and apply follow,
 *     ELO_CELO2_cuda.py:288-296).  A tensor of fewer than two dims without an AdamW flag takes the
 *     same path with the per-element accumulator fac_v and the first nine feature groups
 *     (use_adamw_for_1d=False, ELO_CELO2_naive.py:166-169,180-191).
 * `mlp` is a device pointer to 347 floats: w_in (30,8) | b_in 8 | w_h (8,8) | b_h 8 | w_out (8,3) | b_out 3,
 * weights stored (in, out) as in pylo/models/CELO2_MLP.py:72-86.
 */
int pylo_mi355_celo2_step(PyloPlan* plan, const PyloTensorArgs* args, const PyloDecays* decays,
                          const float* mlp, void* stream);

/*
 * ELO-CELO2 finishing pass (replaces the last two lines of the per-tensor loop in
 * ELO_CELO2_cuda.py:288-296 / CELO2_naive.py:54-56): for every non-ADAM tensor with a gradient,
 * with x = the step after Newton-Schulz (read from `step_out`, same shape as the parameter, contiguous):
 *     step = x * rsqrt(1e-9 + mean(x^2 over the tensor)) * step_mult      (step_mult carries rmsmult)
 *     param <- param - lr * (step + weight_decay * param)
 * Fields read per tensor: grad (only as "takes part" flag), param, step_out, lr, weight_decay,
 * step_mult.  PYLO_F_ADAM tensors are skipped; tensors of fewer than two dims on the MLP path are
 * handled like matrices (their normaliser is over the whole vector).  A tensor with more than two dims
 * has one normaliser per slice of its last two dims (ELO_CELO2_naive.py:217-218,235): where a slice fits (X
 * twice and two m x m fp32 matrices in 128 KB of LDS: every convolution kernel) its slices are normalised and
 * applied by launches of their own, each slice held in registers or LDS by the lanes that own it; larger slices
 * are units of the tensor-wide launches like whole tensors.  pylo_mi355_plan_finish_supported is 1 for every
 * tensor that these calls take (all but PYLO_F_ADAM ones).
 * Three launches: sum of squares per 8192-element block, per-tensor scale (fixed-order fp64 sum),
 * update.  16 bytes per element.
 */
int pylo_mi355_celo2_finish(PyloPlan* plan, const PyloTensorArgs* args, void* stream);
int pylo_mi355_plan_finish_supported(const PyloPlan* plan, int tensor);

/*
 * Newton-Schulz and the finishing pass in one call (replaces `step = newton_schulz(step, ...)` of the
 * per-tensor loop, ELO_CELO2_cuda.py:288-292 / CELO2_naive.py:59-73, for all tensors at once, followed by
 * what pylo_mi355_celo2_finish does).  For every tensor with PYLO_ARG_ORTHOGONALIZE in `flags`, with
 * X = step_out / (||step_out||_F + ns_eps) and (c0, c1, c2) = ns_coeffs, `ns_iters` times
 *     A = X X^T (the Gram matrix over the smaller dim);  X <- c0 X + (c1 A + c2 A A) X
 * as matrix-pipe products of the library's own that compute the symmetric A and c0 I + c1 A + c2 A A once per
 * pair of tiles -- by default on the fp16 matrix instructions at fp32 accuracy (every matrix is held as two fp16
 * planes of its entries times a power of two chosen from bounds that follow from `ns_coeffs`, three fp16 products
 * per fp32 product, fp32 accumulation; what is dropped is below 2^-22 of a term, under the rounding that the fp32
 * accumulation adds; two iterations share one Gram product and one update, A' = B' A B' and
 * X'' = (B'' B') X, which costs about 1e-6 of B' in accuracy whatever the spectrum of X -- PYLO_MI355_NS_PAIRS=0
 * in the environment keeps one of each per iteration, PYLO_MI355_NS_CHAINS="3,2" lets three and then two
 * iterations share them, faster and up to ten times less accurate), with PYLO_MI355_NS_F32=1 in the environment at plan
 * creation on the fp32 matrix instructions; then every tensor is normalised and applied as by pylo_mi355_celo2_finish (tensors without the
 * flag from `step_out` as it stands).  `step_out` of a flagged tensor is overwritten (with the orthogonalised
 * step).  A tensor can carry the flag when pylo_mi355_plan_orthogonalize_supported says so: two dims (any two;
 * the fp32 instructions: the last and the smaller dim multiples of 4) and no PYLO_F_NO_ORTHOGONALIZE in its
 * shape flags.  The function returns 1 for a tensor whose matrices go through these products (a tensor with
 * more than two dims: one matrix per slice of the last two dims, each with its own norm; the fp32 instructions
 * take 2-D tensors only) -- `ns_iters` = 0 with the flag is refused for those, the division by the norm alone
 * being the caller's -- and 2 for a tensor with more than two dims whose slices are small enough to be
 * orthogonalised in the launch that normalises and applies them (fp32 FMA in registers or LDS; `ns_iters` may
 * be 0 there; `step_out` is left as it was).  0: orthogonalised by the caller and passed without the flag.  The plan's workspace holds the operand planes:
 * 12 bytes per element of every such tensor (X as two fp16 planes in both orientations, the orientation
 * that the update product writes twice) plus 20 bytes per element of its m x m matrices -- 2.1 GB for a
 * GPT-2-small set, all tensors resident at once; pylo_mi355_plan_workspace_bytes reports the total.  The
 * products of groups of tensors run on streams of the plan's own next to the caller's (forked and joined
 * with events, default priority); the call returns with the caller's stream waiting for them.
 */
int pylo_mi355_celo2_orthogonalize_finish(PyloPlan* plan, const PyloTensorArgs* args, const float* ns_coeffs,
                                          int ns_iters, float ns_eps, void* stream);
int pylo_mi355_plan_orthogonalize_supported(const PyloPlan* plan, int tensor);

/*
 * VeLO step (replaces velo_cuda_kernel.velo_kernel_simple, pylo/csrc/velo_kernel.cu:370-457, for every
 * tensor at once, plus velo_cuda.py:183-211 (loss features), :213-252 (per-tensor LSTM features),
 * pylo/models/VeLO_RNN.py:43-66,110-135 (mixing + LSTM cell + heads), pylo/models/VeLO_MLP.py:92-126
 * (bank mixing) and velo_cuda.py:502-546 (accumulator updates)).
 *
 * All weight matrices are device pointers, fp32, stored (in, out) -- i.e. the transpose of the
 * torch.nn.Linear weights of pylo/models/VeLO_RNN.py (lstm_wt additionally with the gates innermost,
 * see the field); `bank` is (n_bank, 159): per entry
 * W_in (4,30) | b_in 4 | W_h (4,4) | b_h 4 | W_out (3,4) | b_out 3, each (out, in) as in VeLO_MLP.py:63-77.
 */
typedef struct {
  const float* mix2_wt;   /* (30, H)   mix_layer2.weight^T        */
  const float* mix2_b;    /* (H)                                  */
  const float* fmix_wt;   /* (30, H)   final_mix_layer.weight^T   */
  const float* fmix_b;    /* (H)                                  */
  const float* lstm_wt;   /* (2H, H, 4) lstm.linear.weight^T with the four gates (i, g, f, o) of a
                             unit adjacent: [k][u][q] = weight[q*H + u][k] */
  const float* lstm_b;    /* (4H)                                 */
  const float* ctrl_wt;   /* (H, K)    rnn_to_controls.weight^T   */
  const float* ctrl_b;    /* (K)                                  */
  const float* lr_w;      /* (H)       step_size.weight           */
  const float* lr_b;      /* (1)                                  */
  const float* bank;      /* (K, 159)                             */
  int32_t hidden;         /* H, multiple of 64                    */
  int32_t n_bank;         /* K                                    */
} PyloVeloNets;

typedef struct {
  float* lstm_h;             /* (T, H) hidden state, row r belongs to tensor T-1-r; updated in place */
  float* lstm_c;             /* (T, H) cell state; updated in place                                   */
  float* loss_means;         /* (10)  loss EMAs, updated in place (velo_cuda.py:183-198)              */
  float* loss_running_min;   /* (10)  updated in place                                                */
  const float* loss_decays;  /* (10)                                                                  */
  int32_t* loss_iteration;   /* (1)   updated in place                                                */
  const float* loss;         /* (1)   this step's loss, device scalar                                 */
  float* controls_out;       /* optional (T, K): the control vectors, NULL to skip                    */
  float* lr_mult_out;        /* optional (T): learning-rate multipliers, NULL to skip                 */
  float frac[PYLO_MAX_GROUPS][9]; /* tanh((step/num_steps - ts) * 10) per group (velo_cuda.py:155-162) */
} PyloVeloStep;

/* Every tensor of the plan must have a gradient.  For each tensor: g <- clamp(g, +-clip_val);
   mom / rms / fac_r / fac_c (or fac_v) EMAs; 30 features normalised over the whole tensor (eps 1e-5);
   the tensor's own 30->4->4->3 MLP;  p -= lr * lr_mult * sqrt(mean p^2 + 1e-9) * o0 * exp(o1 * exp_mult)
   * step_mult;  then p -= weight_decay * lr * p. */
int pylo_mi355_velo_step(PyloPlan* plan, const PyloTensorArgs* args, const PyloDecays* decays,
                         const PyloVeloNets* nets, const PyloVeloStep* step, void* stream);

/* The per-tensor LSTM reads sums over every tensor's parameter, momentum and rms values as they stand
   BEFORE the step (velo_cuda.py:213-252).  From its second step on a plan does not read the tensors for
   them: the apply items of step t sum up the values they write, which are the values step t+1 starts from,
   so the LSTM of step t+1 runs ahead of its statistics pass (next to the gradient sums, on a stream of the
   plan's own) and statistics and apply items run as one launch.  That holds as long as nobody else writes
   `param`, `mom` or `rms` of a tensor between two steps of the plan.  A caller who does (loads a checkpoint
   into them, edits parameters in place, swaps a state tensor) calls this first; the next step then takes the
   sums from the tensors again, each pass a launch of its own.  No counterpart in the reference, which
   recomputes everything every step. */
int pylo_mi355_plan_invalidate_statistics(PyloPlan* plan);

/* The guard of those carried sums.  A step that runs on them also takes the sum of p^2 of every tensor from
   the tensor itself (its statistics items read the parameter anyway) and holds it against the carried one.
   Where they differ by more than 1e-3 relative -- the parameter was written by somebody else since the last
   step and the plan was not told -- the LSTM of that step has already run on the stale sum: the tensor's
   step of that call is NaN (loud, like the fused pass's bounded wait) and the plan's flag is raised.  This
   call returns 0, or 1 + the index of a tensor the guard caught since the last
   pylo_mi355_plan_invalidate_statistics; it reads pinned host memory that the kernel writes when it catches a
   mismatch and does not wait for the GPU, so it may lag the step that raised the flag by the steps still in
   flight.  Writes
   that leave sum p^2 within 1e-3 also leave the LSTM's input feature within that, and are not flagged; the
   sums over `mom` and `rms` are not guarded (the Python class watches those tensors' identity and version
   counters).  No counterpart in the reference, which recomputes everything every step. */
int pylo_mi355_plan_statistics_stale(const PyloPlan* plan);

/*
 * AdafacLO step (replaces cuda_lo.learned_optimizer_kernel, pylo/csrc/learned_optimizer.cu:303-394, for
 * every tensor at once, plus the accumulator updates of AdafacLO_cuda.py:291-373 and the weight decay
 * of :406-407).  `net` is a device pointer to 2466 floats, every matrix stored (in, out):
 *   w1 (30,32): first-layer rows for the 30-channel feature order g, clip(g), p, m0..2, rms, m_k*rs,
 *               rs, g*rf_k*cf_k, g*rs, fac_r_k, fac_c_k, rsqrt(fac_r_k), rsqrt(fac_c_k), m_k*rf_k*cf_k
 *               (AdafacLO has no clip(g) / g*rs channel: rows 1 and 14 are zero);
 *   b1 32 | w_time (11,32): rows of the 11 tanh time features | w_h (32,32) | b_h 32 | w_o (32,2) | b_o 2
 * (pylo_amd.models.pack_metamlp builds it from a MetaMLP).  `step` is the 0-based step counter fed to
 * the time features (AdafacLO_cuda.py:400) of every tensor; a negative `step` takes each tensor's own
 * counter from its `bc1` field (the reference keeps one per parameter, AdafacLO_cuda.py:304-305, and
 * parameters that sat steps out lag behind).  Tensors without gradient are skipped.
 *   p -= lr * o0 * exp(o1 * exp_mult) * step_mult;  then p -= weight_decay * lr * p.
 * ELO_CUDA (pylo/optim/ELO_cuda.py:179-288) runs on the same call: raw decays in `decays`, step_mult = 1,
 * clip_norm > 0 for global-norm clipping, and the tensor flags PYLO_F_NAN_TO_NUM | PYLO_F_WD_PRESTEP.
 * AdafacLO_CUDA's max_grad_norm (AdafacLO_cuda.py:214-215): clip_norm = max_grad_norm on a plan whose tensors
 * carry PYLO_F_TENSOR_NORM.
 */
int pylo_mi355_adafac_step(PyloPlan* plan, const PyloTensorArgs* args, const PyloDecays* decays,
                           const float* net, float step, void* stream);

/* ---- Single-tensor calls with the argument lists of the reference's extension functions ------------
 * For callers that keep the reference's per-tensor loop (its optimizer classes update the accumulators
 * and form row_factor / col_factor with tensor operations, then call one function per tensor).  All
 * pointers are device pointers to contiguous fp32 data of the shapes the reference passes; `shape` /
 * `ndim` describe the parameter (the reference reads them off the tensor); dc / dr are the factored
 * dims (ignored when vector_like != 0).  `second_moment` must arrive zeroed and is accumulated into
 * (30 / 28 / 30 floats).  Factor vectors of tensors with more than two dims are addressed as
 * velo_kernel.cu:109-120 does, which for up to two dims is the `col_idx + k * num_cols` form of
 * celo2_kernel.cu:67-84 / learned_optimizer.cu:55-72.  Launches go to `stream` (the reference uses
 * the legacy default stream).  The plans above are the fast path: these calls cost two launches per
 * tensor and leave the accumulator updates to the caller. */

/* celo2_cuda_kernel.celo2_kernel (pylo/csrc/celo2_kernel.cu:284-357): step_out = o0 * exp(o1 * exp_mult)
   of the 30 -> 8 -> 8 -> 3 MLP (weights stored (in, out)) on features normalised with eps 1e-9; p is
   not modified. */
int pylo_mi355_celo2_kernel(const float* g, const float* p, const float* m, const float* v,
                            const float* fac_r, const float* fac_c, const float* row_factor,
                            const float* col_factor, float* second_moment, const float* w_in,
                            const float* b_in, const float* w_h, const float* b_h, const float* w_out,
                            const float* b_out, float* step_out, float exp_mult, const int64_t* shape,
                            int ndim, int dc, int dr, int vector_like, void* stream);

/* pylo_mi355_celo2_kernel without the `second_moment` argument.  No counterpart in the reference: it is
   for callers that cannot allocate device memory -- code under HIP graph capture, tight serving loops,
   harnesses that forbid hipMalloc -- and so cannot supply (and zero) that buffer per call.  The per-channel
   sums live in a 256-byte device array inside the library (one copy per GPU, held until the process ends)
   that the call clears with a small kernel before it accumulates into it; the call itself allocates and
   frees nothing.  Limit: tensors of up to 2^31 - 1 elements, as for pylo_mi355_celo2_kernel (the array does
   not grow with the tensor); larger ones are refused with an error.  Every call on a GPU shares that GPU's
   array: calls that may overlap on one GPU (two streams, two threads) race on the sums and must be
   serialised by the caller.  The GPU used is the calling thread's current device. */
int pylo_mi355_celo2_kernel_noalloc(const float* g, const float* p, const float* m, const float* v,
                                    const float* fac_r, const float* fac_c, const float* row_factor,
                                    const float* col_factor, const float* w_in, const float* b_in,
                                    const float* w_h, const float* b_h, const float* w_out, const float* b_out,
                                    float* step_out, float exp_mult, const int64_t* shape, int ndim, int dc,
                                    int dr, int vector_like, void* stream);

/* cuda_lo.learned_optimizer_kernel (pylo/csrc/learned_optimizer.cu:303-404): 28 features (eps 1e-5) +
   11 tanh(step / ts - 1) features, 39 -> 32 -> 32 -> 2 MLP with (out, in) weights;
   p -= lr * o0 * exp(o1 * exp_mult) * step_mult.  `weight_decay` is accepted and unused, as in the
   reference (its callers apply the decay themselves). */
int pylo_mi355_learned_optimizer_kernel(const float* g, float* p, const float* m, const float* v,
                                        const float* fac_r, const float* fac_c, const float* row_factor,
                                        const float* col_factor, float* second_moment,
                                        const float* input_weights, const float* input_bias,
                                        const float* hidden_weights, const float* hidden_bias,
                                        const float* output_weights, const float* output_bias, float lr,
                                        float step_mult, float exp_mult, float epsilon, float step,
                                        float weight_decay, const int64_t* shape, int ndim, int dc, int dr,
                                        int vector_like, void* stream);

/* velo_cuda_kernel.velo_kernel_simple (pylo/csrc/velo_kernel.cu:370-462; note the factor arguments
   come in a different order than above): 30 features (eps 1e-5), 30 -> 4 -> 4 -> 3 MLP with (out, in)
   weights; p -= lr * sqrt(mean p^2 + 1e-9) * o0 * exp(o1 * exp_mult) * step_mult, then
   p -= weight_decay * lr * p when weight_decay > 0. */
int pylo_mi355_velo_kernel_simple(const float* grad, float* param, const float* momentum, const float* rms,
                                  const float* row_factor, const float* col_factor, const float* fac_vec_row,
                                  const float* fac_vec_col, float* second_moment, const float* input_weights,
                                  const float* input_bias, const float* hidden_weights, const float* hidden_bias,
                                  const float* output_weights, const float* output_bias, float lr,
                                  float step_mult, float exp_mult, float epsilon, float weight_decay,
                                  const int64_t* shape, int ndim, int dc, int dr, int vector_like, void* stream);

/* The three calls above for arrays of another element type: what the reference's
   AT_DISPATCH_FLOATING_TYPES_AND_HALF over p.scalar_type() selects (celo2_kernel.cu:314,328,
   learned_optimizer.cu:338,364, velo_kernel.cu:405,427).  `dtype` is one of PYLO_F_STORE_*; every array holds
   elements of that type except `second_moment`, which is float as in the reference
   (second_moment.data_ptr<float>(), celo2_kernel.cu:324).  Values are widened to float on load, the arithmetic is
   float, results are rounded to nearest-even on store (celo2_kernel.cu:70-75,280).  PYLO_F_STORE_BF16 is an
   addition: the reference's dispatch has no bfloat16 case. */
int pylo_mi355_celo2_kernel_typed(int dtype, const void* g, const void* p, const void* m, const void* v,
                                  const void* fac_r, const void* fac_c, const void* row_factor,
                                  const void* col_factor, float* second_moment, const void* w_in, const void* b_in,
                                  const void* w_h, const void* b_h, const void* w_out, const void* b_out,
                                  void* step_out, float exp_mult, const int64_t* shape, int ndim, int dc, int dr,
                                  int vector_like, void* stream);
int pylo_mi355_learned_optimizer_kernel_typed(int dtype, const void* g, void* p, const void* m, const void* v,
                                              const void* fac_r, const void* fac_c, const void* row_factor,
                                              const void* col_factor, float* second_moment,
                                              const void* input_weights, const void* input_bias,
                                              const void* hidden_weights, const void* hidden_bias,
                                              const void* output_weights, const void* output_bias, float lr,
                                              float step_mult, float exp_mult, float epsilon, float step,
                                              float weight_decay, const int64_t* shape, int ndim, int dc, int dr,
                                              int vector_like, void* stream);
int pylo_mi355_velo_kernel_simple_typed(int dtype, const void* grad, void* param, const void* momentum,
                                        const void* rms, const void* row_factor, const void* col_factor,
                                        const void* fac_vec_row, const void* fac_vec_col, float* second_moment,
                                        const void* input_weights, const void* input_bias,
                                        const void* hidden_weights, const void* hidden_bias,
                                        const void* output_weights, const void* output_bias, float lr,
                                        float step_mult, float exp_mult, float epsilon, float weight_decay,
                                        const int64_t* shape, int ndim, int dc, int dr, int vector_like,
                                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PYLO_MI355_H */
